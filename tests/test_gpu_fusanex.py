"""Fusanex on the hybrid engine (registry -> FusanexModel -> ModelWorker -> vox_hybrid_*) against the float64 restatement in
oracle/fusanex_ref.py, on small configurations with random checkpoints made here.

fp32 engine: logits within 2e-4 of the oracle (relative RMS over the vocabulary); bf16 engine: 4e-2.  A schedule may change
rounding only, so every schedule of the same tokens is held to the same bar against the same whole-sequence oracle.  Attention
cases use a large score scale (a nearly one-hot softmax), so a key that is wrongly seen or lost, or a query temperature that
changes one position early or late, moves the logits by far more than the bar; the sensitivity tests check such claims on
the oracle itself.
"""
import pytest
import torch

from oracle import fusanex_ref as FR
from tests import fusanex_util as F
from tests import hybrid_util as U

pytestmark = pytest.mark.gpu

F32_BAR, BF16_BAR = 2e-4, 4e-2


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


def tokens(n, vocab, seed):
    return torch.randint(0, vocab, (n,), generator=torch.Generator().manual_seed(seed)).tolist()


def check(cfg, S, toks, cuts, dtype=torch.float32, bar=None, quantile=None, **kw):
    want = FR.forward(cfg, S, toks)
    d = U.Driver(cfg, S, dtype=dtype, **kw)
    try:
        got = d.run_cut("r", toks, cuts)
    finally:
        d.close()
    err = U.rel_err(got, want, quantile)
    assert err < (bar or (F32_BAR if dtype == torch.float32 else BF16_BAR)), err
    return got


SHARP = dict(scale=2.5)      # q, k of unit RMS times their weights, scores times 2.5: a nearly one-hot softmax

MECHANISMS = {
    "rglru": [F.rglru()],
    "rglru_one_block_one_tap": [F.rglru(width=20, blocks=1, conv=1)],
    "rglru_wide_long_conv": [F.rglru(width=40, blocks=5, conv=6)],
    "attention_alone": [F.parallel(right_scale=0.0, **SHARP)],
    "attention_mha_no_temperature": [F.parallel(heads=3, kv_heads=3, dim=4, vdim=4, right_scale=0.0, q_temp=False, **SHARP)],
    "attention_one_kv_head_every_1": [F.parallel(heads=5, kv_heads=1, dim=12, vdim=20, every=1, coef=1.5, right_scale=0.0, **SHARP)],
    "shift_decay_alone": [F.parallel(left_scale=0.0)],
    "shift_decay_one_head": [F.parallel(left_scale=0.0, rheads=1, rdim=20, right_scale=1.0)],
    "parallel_both": [F.parallel(**SHARP)],
    "moe": [F.rglru(mlp=F.moe())],
    "moe_top1_no_identity_no_shared": [F.rglru(mlp=F.moe(experts=3, identity=0, top=1, shared=None))],
    "moe_top3_two_identity": [F.rglru(mlp=F.moe(experts=4, identity=2, top=3, ff=20, limit=0.7, shared=(6, 2.0)))],
    "moe_identity_only_choice": [F.rglru(mlp=F.moe(experts=2, identity=3, top=2))],
}


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_mechanism_alone_whole_prompt(name):
    cfg = F.config(MECHANISMS[name])
    S = F.random_checkpoint(cfg, seed=1, identity_bias=0.15)
    check(cfg, S, tokens(70, 40, 2), [70])


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_mechanism_alone_token_by_token(name):
    cfg = F.config(MECHANISMS[name])
    S = F.random_checkpoint(cfg, seed=3, identity_bias=0.15)
    check(cfg, S, tokens(45, 40, 4), [])


@pytest.mark.parametrize("groups,embed_scale", [(1, 1.0), (3, 7.0), (24, 0.5)])
def test_norm_groups_and_embedding_scale(groups, embed_scale):
    cfg = F.config([F.rglru(mlp=F.moe()), F.parallel(mlp=F.moe())], groups=groups, embed_scale=embed_scale)
    S = F.random_checkpoint(cfg, seed=5)
    check(cfg, S, tokens(30, 40, 6), [22, 2])


def stack(sharp=True):
    sc = SHARP if sharp else {}
    layers = [F.parallel(mlp=F.moe(), **sc), F.rglru(width=32, blocks=4, conv=4, mlp=F.moe(experts=6, identity=2, top=2)),
              F.rglru(width=18, blocks=2, conv=2, mlp=None), F.parallel(heads=6, kv_heads=2, dim=16, vdim=8, every=9, rheads=3, rdim=12,
                                                                        mlp=F.moe(experts=3, identity=1, top=3, shared=None), **sc)]
    return F.config(layers, width=36, vocab=64, groups=3)


@pytest.mark.parametrize("order", [(0, 1, 2, 3), (1, 2, 0, 3), (3, 0), (2, 1)])
def test_stack_in_other_orders(order):
    cfg = stack()
    cfg["layers"] = [cfg["layers"][i] for i in order]
    S = F.random_checkpoint(cfg, seed=7, identity_bias=0.1)
    check(cfg, S, tokens(90, 64, 8), [90])


@pytest.mark.parametrize("cuts", [[2, 2, 2, 2, 3, 5, 2, 30, 2, 17], [31, 2, 1, 1, 2, 40], [7] * 13, [64, 2, 2], [9, 12, 9, 30]])
def test_portions(cuts):
    """Portions cut inside pages (8 tokens), shorter than the convolution, below and above the row count at which the routed
    feed-forward changes from per-entry products to per-expert tiles; the rest of the sequence token by token."""
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=9, identity_bias=0.1)
    check(cfg, S, tokens(100, 64, 10), cuts)


def test_bf16_schedules():
    cfg = stack(sharp=False)
    S = F.random_checkpoint(cfg, seed=11)
    toks = tokens(96, 64, 12)
    a = check(cfg, S, toks, [96], dtype=torch.bfloat16, quantile=0.95)
    b = check(cfg, S, toks, [5, 2, 40, 3], dtype=torch.bfloat16, quantile=0.95)
    # a routed choice that bf16 rounding flips changes a position by more than rounding in either schedule alike
    assert U.rel_err(a, b.double(), 0.9) < BF16_BAR


def test_first_tokens_and_single_token():
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=13)
    for n in (1, 2, 3):
        check(cfg, S, tokens(n, 64, 14 + n), [n])
    check(cfg, S, tokens(5, 64, 19), [1, 1, 3])


def test_mixed_batch_matches_each_alone():
    """Four unequal requests share steps (portions beside single tokens); every request's logits equal its oracle's."""
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=21, identity_bias=0.1)
    seqs = {"a": tokens(75, 64, 22), "b": tokens(33, 64, 23), "c": tokens(9, 64, 24), "d": tokens(50, 64, 25)}
    want = {k: FR.forward(cfg, S, v) for k, v in seqs.items()}
    plan = {"a": [20, 1, 1, 30, 2, 1, 1, 19], "b": [1, 1, 1, 10, 20], "c": [2, 2, 2, 2, 1], "d": [3, 40, 1, 1, 1, 1, 1, 1, 1]}
    d = U.Driver(cfg, S)
    try:
        got = {k: [] for k in seqs}
        done = {k: 0 for k in seqs}
        step = 0
        while any(done[k] < len(seqs[k]) for k in seqs):
            portions = []
            for k in seqs:
                # request c joins late, request b skips every third step
                if done[k] >= len(seqs[k]) or (k == "c" and step < 2) or (k == "b" and step % 3 == 2):
                    continue
                n = plan[k].pop(0) if plan[k] else 1
                portions.append((k, seqs[k][done[k]:done[k] + n]))
                done[k] += len(portions[-1][1])
            if portions:
                for k, lg in d.feed(portions).items():
                    got[k].append(lg)
            step += 1
        for k in seqs:
            assert U.rel_err(torch.cat(got[k], 0), want[k]) < F32_BAR, k
    finally:
        d.close()


def test_long_step_shared_by_requests():
    """A step of more than 64 rows (the recurrent unit cuts every request's rows into chunks that run side by side, the routed
    feed-forward runs expert by expert) shared by a long portion, a short one, and single decoded tokens."""
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=61, identity_bias=0.1)
    seqs = {"a": tokens(150, 64, 62), "b": tokens(40, 64, 63), "c": tokens(12, 64, 64)}
    want = {k: FR.forward(cfg, S, v) for k, v in seqs.items()}
    d = U.Driver(cfg, S, pages=64)
    try:
        got = {k: [] for k in seqs}
        steps = [[("c", 0, 10)], [("a", 0, 97), ("b", 0, 3), ("c", 10, 11)], [("a", 97, 98), ("b", 3, 40), ("c", 11, 12)], [("a", 98, 150)]]
        for st in steps:
            out = d.feed([(k, seqs[k][lo:hi]) for k, lo, hi in st])
            for k, lg in out.items():
                got[k].append(lg)
        for k in seqs:
            assert U.rel_err(torch.cat(got[k], 0), want[k]) < F32_BAR, k
    finally:
        d.close()


def test_identity_outputs_only():
    """A router with identity outputs only and no shared expert: the feed-forward adds the normed input itself."""
    cfg = F.config([F.rglru(mlp=F.moe(experts=0, identity=2, top=1, shared=None)), F.parallel(mlp=F.moe(experts=0, identity=3, top=2, shared=(6, 1.0)))])
    S = F.random_checkpoint(cfg, seed=65)
    check(cfg, S, tokens(30, 40, 66), [20, 2])


def test_pages_and_slots_are_reused():
    """6 pages and 2 state slots serve six requests, two at a time: stale K / V, recurrent state, convolution history or a
    previous owner's last input must not leak into the next owner."""
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=27)
    d = U.Driver(cfg, S, pages=6, slots=2, page_size=8, max_batch=2)
    try:
        for rnd in range(3):
            x, y = tokens(24, 64, 28 + rnd), tokens(17, 64, 38 + rnd)
            gx = [d.feed([("x", x[:10])])["x"]]
            o = d.feed([("x", x[10:]), ("y", y[:16])])
            gx.append(o["x"])
            gy = [o["y"], d.feed([("y", y[16:])])["y"]]
            assert d.worker.empty_pages.qsize() == 0 and d.worker.empty_state_slots.qsize() == 0
            d.end("x"); d.end("y")
            assert d.worker.empty_pages.qsize() == 6 and d.worker.empty_state_slots.qsize() == 2
            assert U.rel_err(torch.cat(gx, 0), FR.forward(cfg, S, x)) < F32_BAR
            assert U.rel_err(torch.cat(gy, 0), FR.forward(cfg, S, y)) < F32_BAR
    finally:
        d.close()


def far_key_case():
    """One attention layer with a sharp softmax and a temperature that steps every 7 positions; the recurrent side is off, so the
    logits at a position hang on single keys that may lie hundreds of tokens back."""
    cfg = F.config([F.parallel(heads=2, kv_heads=1, dim=16, vdim=16, scale=4.0, coef=0.8, every=7, right_scale=0.0)], width=16, vocab=32)
    return cfg, F.random_checkpoint(cfg, seed=31, gain=2.0)


def test_far_keys_prompt_and_decoding():
    cfg, S = far_key_case()
    toks = tokens(300, 32, 32)
    check(cfg, S, toks, [300], max_rows=320)
    check(cfg, S, toks, [200], page_size=16, max_rows=320)            # 100 decoded one by one over 200+ keys (segmented attention)
    check(cfg, S, toks, [3, 61, 2, 67, 2, 100], page_size=4, pages=128, max_rows=320)


def planted_pair(cfg, S):
    """(a, b): the token a whose query (head 0 of the first layer, position-free part) prefers the key of token b over the key of
    every other token by the widest margin."""
    Sd = {k: v.double() for k, v in S.items()}
    m = cfg["layers"][0]["mixer"]["left"]
    x = Sd["embed"] * cfg["embedding"]["scale"]
    n = FR.grouped_rms_norm(x, Sd["l0.norm1"], cfg["norm"]["groups"], cfg["norm"]["eps"])
    q = FR.unit_rms((n @ Sd["l0.mix.left.q"].T).view(-1, m["heads"], m["dim"]), cfg["norm"]["eps"])[:, 0] * Sd["l0.mix.left.q.norm"]
    k = FR.unit_rms((n @ Sd["l0.mix.left.k"].T).view(-1, m["kv_heads"], m["dim"]), cfg["norm"]["eps"])[:, 0] * Sd["l0.mix.left.k.norm"]
    sc = q @ k.T
    top2 = sc.topk(2, dim=-1)
    a = int((top2.values[:, 0] - top2.values[:, 1]).argmax())
    return a, int(top2.indices[a, 0])


def test_planted_far_key_is_found():
    """A token whose key the last tokens' queries prefer to every other is planted once, at position 3: an attention that loses it
    (a page dropped, a segment skipped) changes the output grossly.  Checked in a prompt, in decoding and across page borders."""
    cfg, S = far_key_case()
    a, b = planted_pair(cfg, S)
    toks = [t if t != b else (b + 1) % 32 for t in tokens(260, 32, 33)]
    toks[3] = b
    toks[250:] = [a] * 10
    want = FR.forward(cfg, S, toks)
    hidden = list(toks)
    hidden[3] = (b + 1) % 32
    assert U.rel_err(FR.forward(cfg, S, hidden)[250:], want[250:]) > 100 * F32_BAR      # the planted key matters
    for cuts, ps in (([260], 8), ([240], 8), ([2, 250], 64), ([100, 100], 32)):
        d = U.Driver(cfg, S, page_size=ps, pages=2048 // ps, max_rows=320)
        try:
            got = d.run_cut("r", toks, cuts)
        finally:
            d.close()
        assert U.rel_err(got, want) < F32_BAR, (cuts, ps)


def test_temperature_edge_sensitivity():
    """The bar is meaningful: a query temperature whose step comes one position early or late moves the oracle's own logits by
    far more than the bar, and so does a lost bonus term or a lost convolution tap."""
    cfg, S = far_key_case()
    toks = tokens(60, 32, 34)
    base = FR.forward(cfg, S, toks)
    real_floor = torch.floor
    try:
        for delta in (-1.0, 1.0):
            # the oracle's temperature is the only caller of torch.floor: floor((p + 1 + delta) / every) instead
            every = cfg["layers"][0]["mixer"]["left"]["q_temp"]["every"]
            torch.floor = lambda v: real_floor(v + delta / every)
            assert U.rel_err(FR.forward(cfg, S, toks), base) > 50 * F32_BAR
    finally:
        torch.floor = real_floor
    cfg2 = F.config([F.parallel(left_scale=0.0), F.rglru(conv=3)])
    S2 = F.random_checkpoint(cfg2, seed=35)
    base2 = FR.forward(cfg2, S2, toks[:40])
    no_bonus = dict(S2, **{"l0.mix.right.u": torch.zeros_like(S2["l0.mix.right.u"])})
    assert U.rel_err(FR.forward(cfg2, no_bonus, toks[:40]), base2) > 50 * F32_BAR
    conv = S2["l1.mix.conv"].clone()
    conv[:, 0] = 0
    assert U.rel_err(FR.forward(cfg2, dict(S2, **{"l1.mix.conv": conv}), toks[:40]), base2) > 50 * F32_BAR


@pytest.mark.parametrize("page_size", [4, 16, 64])
def test_keys_at_page_borders(page_size):
    cfg, S = far_key_case()
    toks = tokens(2 * page_size + 3, 32, 36)
    # the prompt ends one before, at, and one after a page border; then decoding crosses the next border
    for first in (page_size - 1, page_size, page_size + 1):
        check(cfg, S, toks, [first], page_size=page_size, pages=16)


def test_routed_choice_covers_every_expert_and_identity():
    """The test's routing is not degenerate: over the prompt every expert and every identity output is chosen at least once, and
    dropping the identity outputs' contribution would be seen."""
    cfg = F.config([F.rglru(mlp=F.moe(experts=4, identity=2, top=2))])
    S = F.random_checkpoint(cfg, seed=41, identity_bias=0.15)
    toks = tokens(120, 40, 42)
    Sd = {k: v.double() for k, v in S.items()}
    res = []
    FR.forward(cfg, S, toks, residuals=res)
    x0 = Sd["embed"][torch.tensor(toks)] * cfg["embedding"]["scale"]
    n2 = FR.grouped_rms_norm(x0, Sd["l0.norm2"], cfg["norm"]["groups"], cfg["norm"]["eps"])
    P = {k[len("l0.mlp."):]: v for k, v in Sd.items() if k.startswith("l0.mlp.")}
    chosen, w = FR.route(P, n2, cfg["layers"][0]["mlp"]["router"])
    assert set(chosen.flatten().tolist()) == set(range(6))
    assert torch.allclose(w.sum(-1), torch.ones(120, dtype=torch.float64))
    check(cfg, S, toks, [50, 9, 2])


def test_slow_decay_channels():
    """Channels whose decay a is within 1e-4 of 1 (a very negative lambda): 1 - a^2 must not be formed by a subtraction of rounded
    values — a relative error of 1e-7 in a would be one of 1e-3 in the input's weight sqrt(1 - a^2)."""
    cfg = F.config([F.rglru(width=24, blocks=3, conv=2)], width=24)
    S = F.random_checkpoint(cfg, seed=47)
    lam = S["l0.mix.lam"].float()
    lam[::2] = -11.0
    S["l0.mix.lam"] = lam.to(torch.bfloat16)
    toks = tokens(150, 40, 48)
    check(cfg, S, toks, [150], bar=2e-5)
    check(cfg, S, toks, [70, 3], bar=2e-5)


def test_long_decoding():
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=43)
    check(cfg, S, tokens(330, 64, 44), [10], pages=48)


def test_wide_sizes():
    """Sizes beyond one wave per head or block: 160 value columns, 96 key dims, a group of 5 query heads, 72 key dims of the
    matrix state, 80-channel gate blocks, odd width and vocabulary."""
    layers = [F.parallel(heads=5, kv_heads=1, dim=96, vdim=160, every=16, rheads=2, rdim=72, mlp=F.moe(experts=9, identity=3, top=4, ff=100, shared=(130, 1.0))),
              F.rglru(width=160, blocks=2, conv=4, mlp=F.moe(experts=3, identity=0, top=2, ff=70))]
    cfg = F.config(layers, width=100, vocab=131, groups=5)
    S = F.random_checkpoint(cfg, seed=45, lora=20)
    toks = tokens(80, 131, 46)
    check(cfg, S, toks, [37, 2, 30])
    check(cfg, S, toks, [80], dtype=torch.bfloat16, quantile=0.95)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_matrix_core_sizes(dtype):
    """Sizes at which every product takes its matrix-core or 16-byte form (widths and inner sizes that are multiples of 32), with
    prompt portions of 130 / 9 / 2 / 33 rows and decoding: the row-tile, tile and per-expert gathered forms against the same oracle."""
    layers = [F.parallel(heads=8, kv_heads=2, dim=32, vdim=64, every=50, rheads=3, rdim=64, mlp=F.moe(experts=6, identity=1, top=3, ff=96, shared=(160, 1.0))),
              F.rglru(width=512, blocks=4, conv=3, mlp=F.moe(experts=6, identity=1, top=3, ff=96, shared=(160, 1.0))),
              F.parallel(heads=4, kv_heads=4, dim=64, vdim=32, every=64, rheads=6, rdim=32, mlp=F.moe(experts=4, identity=0, top=2, ff=128, shared=None))]
    cfg = F.config(layers, width=384, vocab=500, groups=6, embed_scale=4.0)
    S = F.random_checkpoint(cfg, seed=71, lora=32)
    toks = tokens(190, 500, 72)
    q = None if dtype == torch.float32 else 0.95
    check(cfg, S, toks, [130, 9, 2, 33], dtype=dtype, quantile=q, page_size=64, pages=8, max_rows=192)
    check(cfg, S, toks, [190], dtype=dtype, quantile=q, page_size=64, pages=8, max_rows=192)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_sizes(dtype):
    """Sizes that defeat every vector path: width 18, key dims 10 / 5, value dims 6 / 7, 3 query heads per K/V head, matrix-state
    heads of 3 and 5 dims, gate blocks of 7 and 3 channels, a 37-entry vocabulary, expert widths 5 and 9, norm groups of 9 and 1."""
    layers = [F.parallel(heads=3, kv_heads=1, dim=10, vdim=6, every=3, rheads=3, rdim=5, mlp=F.moe(experts=3, identity=1, top=2, ff=5, shared=(7, 1.0))),
              F.rglru(width=21, blocks=3, conv=5, mlp=F.moe(experts=2, identity=1, top=1, ff=9, shared=None)),
              F.parallel(heads=2, kv_heads=2, dim=5, vdim=7, every=2, rheads=1, rdim=3), F.rglru(width=9, blocks=3, conv=2)]
    cfg = F.config(layers, width=18, vocab=37, groups=2)
    S = F.random_checkpoint(cfg, seed=51, lora=3)
    toks = tokens(75, 37, 52)
    q = None if dtype == torch.float32 else 0.9
    check(cfg, S, toks, [75], dtype=dtype, quantile=q)
    check(cfg, S, toks, [9, 2, 33, 5], dtype=dtype, quantile=q)


def test_greedy_generation_through_the_scheduler():
    """Requests enter through the scheduler's transport, are prefilled in portions next to decoding requests and generate greedily;
    the ids equal the oracle's greedy continuation (fp32 engine)."""
    import json

    from vox_serve_amd.model import get_model_class
    from vox_serve_amd.model.fusanex import config_from_dict
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=53)
    n_new = 12
    model = get_model_class("fusanex")("fusanex-test", weights=S, config=config_from_dict(cfg), dtype=torch.float32, max_batch_size=4, page_size=8,
                                       max_num_pages=64, max_seq_len=512, max_prefill_tokens=64, state_slots=4, max_tokens=n_new)
    worker = ModelWorker(model=model, max_batch_size=4, max_num_pages=64, page_size=8, greedy=True, prefill_chunk_tokens=16)
    sched = Scheduler(worker, max_batch_size=4)
    prompts = {"p0": tokens(37, 64, 54), "p1": tokens(5, 64, 55), "p2": tokens(50, 64, 56)}
    try:
        for rid, p in prompts.items():
            sched.transport.requests.put(encode_request(rid, " ".join(map(str, p)), is_streaming=False))
        reqs = {}
        for _ in range(400):
            sched._step()
            for r in sched.active_requests:
                reqs[r.request_id] = r
            if not sched.active_requests and not sched.transport.pending():
                break
        assert set(reqs) == set(prompts)
        for rid, p in prompts.items():
            seq = list(p)
            for _ in range(n_new):
                seq.append(int(FR.forward(cfg, S, seq)[-1].argmax()))
            got = [int(t[0, 0]) for t in reqs[rid].lm_output_tokens]
            assert got == seq[len(p):], (rid, got, seq[len(p):])
        done = []
        while not sched.transport.results.empty():
            done.append(sched.transport.results.get())
        assert sum(b"|COMPLETION|" in m and json.loads(m.split(b"|", 2)[2])["status"] == "completed" for m in done) == 3
        assert worker.empty_pages.qsize() == 64 and worker.empty_state_slots.qsize() == 4
    finally:
        model.engine.close()


def test_top_k_sampling_and_async_scheduling():
    """Stochastic sampling goes through the library's sampler (every id is one of the oracle's five most likely continuations of
    the request's own prefix; the same seed repeats the ids), and the pipelined scheduler loop generates the greedy ids."""
    from vox_serve_amd.model import get_model_class
    from vox_serve_amd.model.fusanex import config_from_dict
    from vox_serve_amd.sampling import SamplingConfig
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg = stack(sharp=False)
    S = F.random_checkpoint(cfg, seed=91)
    prompts = {"a": tokens(21, 64, 92), "b": tokens(9, 64, 93)}

    def generate(sampling, n_new, greedy, async_scheduling):
        model = get_model_class("fusanex")("fusanex-test", weights=S, config=config_from_dict(cfg), dtype=torch.float32, max_batch_size=2,
                                           page_size=8, max_num_pages=32, max_seq_len=256, max_prefill_tokens=64, state_slots=2,
                                           max_tokens=n_new, sampling=sampling)
        worker = ModelWorker(model=model, max_batch_size=2, max_num_pages=32, page_size=8, seed=7, greedy=greedy, prefill_chunk_tokens=16)
        sched = Scheduler(worker, max_batch_size=2, async_scheduling=async_scheduling)
        seen = {}
        orig = sched._prepare_requests

        def spy():
            orig()
            for r in sched.active_requests:
                seen[r.request_id] = r
        sched._prepare_requests = spy
        try:
            for rid, p in prompts.items():
                sched.transport.requests.put(encode_request(rid, " ".join(map(str, p)), is_streaming=False))
            sched.run_until_idle(max_steps=400)
            assert worker.empty_pages.qsize() == 32 and worker.empty_state_slots.qsize() == 2
            return {rid: [int(t[0, 0]) for t in seen[rid].lm_output_tokens][:n_new] for rid in prompts}
        finally:
            model.engine.close()
    first = generate(SamplingConfig(top_k=5, temperature=0.8, max_tokens=8), 8, False, False)
    for rid, p in prompts.items():
        assert len(first[rid]) == 8
        seq = list(p)
        for tok in first[rid]:
            top = FR.forward(cfg, S, seq)[-1].topk(5).indices.tolist()
            assert tok in top, (rid, tok, top)
            seq.append(tok)
    assert generate(SamplingConfig(top_k=5, temperature=0.8, max_tokens=8), 8, False, False) == first
    got = generate(None, 7, True, True)
    for rid, p in prompts.items():
        seq = list(p)
        for _ in range(7):
            seq.append(int(FR.forward(cfg, S, seq)[-1].argmax()))
        assert got[rid] == seq[len(p):], (rid, got[rid], seq[len(p):])


def test_checkpoint_folder_through_the_registry(tmp_path):
    """config.json + model.safetensors in a folder: `load_checkpoint_dir` picks the design by the config's architecture."""
    import json

    from safetensors.torch import save_file

    from vox_serve_amd.model import load_checkpoint_dir
    from vox_serve_amd.requests import Request
    from vox_serve_amd.worker.base import ModelWorker
    cfg = stack()
    S = F.random_checkpoint(cfg, seed=57)
    (tmp_path / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in S.items()}, str(tmp_path / "model.safetensors"))
    model = load_checkpoint_dir(str(tmp_path), dtype=torch.float32, max_batch_size=2, page_size=8, max_num_pages=16, max_seq_len=128,
                                max_prefill_tokens=64, max_logit_rows=66, state_slots=2)
    try:
        worker = ModelWorker(model=model, max_batch_size=2, max_num_pages=16, page_size=8, greedy=True)
        toks = tokens(20, 64, 58)
        req = Request(request_id="r", prompt_open=True)
        req.input_tokens, req._preprocessed, req.step_budget = torch.tensor(toks).view(-1, 1), True, len(toks)
        li = worker.prepare_lm_inputs([req], [])
        li["logit_rows"] = list(range(20))
        worker.run_lm_prefill([req], li)
        got = model.engine.out_logits[1:21].to("cpu", torch.float32)
        assert U.rel_err(got, FR.forward(cfg, S, toks)) < F32_BAR
    finally:
        model.engine.close()
