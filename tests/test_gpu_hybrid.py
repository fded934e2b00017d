"""The hybrid-mixer engine (vox_hybrid_* through ModelWorker and the Sirodra plugin) against the float64 restatement in
oracle/hybrid_ref.py, on small configurations with random checkpoints made here.

fp32 engine: logits within 2e-4 of the oracle (relative RMS over the vocabulary); bf16 engine: 4e-2.  What a schedule may
change is rounding only, so every schedule of the same tokens is held to the same bar against the same whole-sequence oracle.
Attention cases use a large score scale: the softmax is nearly one-hot, so one key that is wrongly seen or not seen (a
window's or a pooled block's edge, a page border, a far block) moves the logits by orders of magnitude more than the bar —
`test_window_edge_sensitivity` checks that claim on the oracle itself.
"""
import pytest
import torch

from oracle import hybrid_ref as HR
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
    want = HR.forward(cfg, S, toks)
    d = U.Driver(cfg, S, dtype=dtype, **kw)
    try:
        got = d.run_cut("r", toks, cuts)
    finally:
        d.close()
    err = U.rel_err(got, want, quantile)
    assert err < (bar or (F32_BAR if dtype == torch.float32 else BF16_BAR)), err
    return got


SHARP = dict(scale=3.0)      # scores of unit-RMS q, k times 3: dim 16 -> logits of magnitude 48, a one-hot softmax

MECHANISMS = {
    "hgrn2": [U.hgrn2()],
    "hgrn2_ff": [U.hgrn2(heads=3, dim=4, vdim=8, ff=24)],
    "mlstm": [U.mlstm()],
    "mlstm_hard_gates": [U.mlstm(heads=1, dim=16, vdim=8, cap=30.0)],
    "attention": [U.attention(**SHARP)],
    "attention_no_rot_mha": [U.attention(heads=2, kv_heads=2, dim=8, vdim=24, window=5, pool=3, rot=0, **SHARP)],
    "attention_full_rot_scaled": [U.attention(heads=6, kv_heads=1, dim=8, vdim=8, window=7, pool=5, rot=8, base=50.0, factor=4.0, ff=40, **SHARP)],
    "attention_window1_pool1": [U.attention(heads=1, kv_heads=1, dim=4, vdim=4, window=1, pool=1, rot=2, **SHARP)],
}


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_mechanism_alone_whole_prompt(name):
    cfg = U.config(MECHANISMS[name], width=24, vocab=40)
    S = U.random_checkpoint(cfg, seed=1)
    check(cfg, S, tokens(70, 40, 2), [70])


@pytest.mark.parametrize("name", list(MECHANISMS))
def test_mechanism_alone_token_by_token(name):
    cfg = U.config(MECHANISMS[name], width=24, vocab=40)
    S = U.random_checkpoint(cfg, seed=3)
    check(cfg, S, tokens(60, 40, 4), [])


def stack(loop=(1, 3, 2), sharp=True):
    sc = SHARP if sharp else {}
    layers = [U.hgrn2(heads=2, dim=8, vdim=12), U.attention(heads=4, kv_heads=2, dim=16, vdim=8, window=9, pool=4, rot=8, ff=48, **sc),
              U.mlstm(heads=3, dim=8, vdim=8), U.attention(heads=2, kv_heads=1, dim=8, vdim=16, window=4, pool=3, rot=4, factor=2.0, **sc),
              U.hgrn2(heads=1, dim=16, vdim=16, ff=32)]
    return U.config(layers, width=40, vocab=64, loop=loop)


@pytest.mark.parametrize("loop", [(1, 3, 2), (0, 5, 3), (2, 3, 1), None])
def test_stack_with_loops(loop):
    cfg = stack(loop)
    S = U.random_checkpoint(cfg, seed=5)
    check(cfg, S, tokens(90, 64, 6), [90])


@pytest.mark.parametrize("cuts", [[2, 2, 2, 2, 3, 5, 2, 30, 2, 17], [31, 2, 1, 1, 2, 40], [7] * 13, [64, 2, 2]])
def test_portions(cuts):
    """Portions cut inside pages (8 tokens), windows and pooled blocks; the rest of the sequence token by token."""
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=7)
    check(cfg, S, tokens(100, 64, 8), cuts)


def test_bf16_schedules():
    """bf16 rounding under a one-hot softmax is not small: the bf16 bar is taken with ordinary score scales."""
    cfg = stack(sharp=False)
    S = U.random_checkpoint(cfg, seed=9)
    toks = tokens(96, 64, 10)
    a = check(cfg, S, toks, [96], dtype=torch.bfloat16)
    b = check(cfg, S, toks, [5, 2, 40, 3], dtype=torch.bfloat16)
    assert U.rel_err(a, b.double()) < BF16_BAR


def test_first_tokens_and_single_token():
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=11)
    for n in (1, 2, 3):
        check(cfg, S, tokens(n, 64, 12 + n), [n])


def test_mixed_batch_matches_each_alone():
    """Four unequal requests share steps (portions beside single tokens); every request's logits equal its oracle's."""
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=13)
    seqs = {"a": tokens(75, 64, 14), "b": tokens(33, 64, 15), "c": tokens(9, 64, 16), "d": tokens(50, 64, 17)}
    want = {k: HR.forward(cfg, S, v) for k, v in seqs.items()}
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
                out = d.feed(portions)
                for k, lg in out.items():
                    got[k].append(lg)
            step += 1
        for k in seqs:
            assert U.rel_err(torch.cat(got[k], 0), want[k]) < F32_BAR, k
    finally:
        d.close()


def test_pages_and_slots_are_reused():
    """A pool of 6 pages and 2 state slots serves six requests one after the other and two at a time: stale K / V, pooled
    entries or recurrent state of an earlier owner must not leak."""
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=19)
    d = U.Driver(cfg, S, pages=6, slots=2, page_size=8, max_batch=2)
    try:
        for rnd in range(3):
            x, y = tokens(24, 64, 20 + rnd), tokens(17, 64, 30 + rnd)
            gx = [d.feed([("x", x[:10])])["x"]]
            o = d.feed([("x", x[10:]), ("y", y[:16])])
            gx.append(o["x"])
            gy = [o["y"], d.feed([("y", y[16:])])["y"]]
            assert d.worker.empty_pages.qsize() == 6 - 3 - 3 and d.worker.empty_state_slots.qsize() == 0
            d.end("x"); d.end("y")
            assert d.worker.empty_pages.qsize() == 6 and d.worker.empty_state_slots.qsize() == 2
            assert U.rel_err(torch.cat(gx, 0), HR.forward(cfg, S, x)) < F32_BAR
            assert U.rel_err(torch.cat(gy, 0), HR.forward(cfg, S, y)) < F32_BAR
    finally:
        d.close()


def test_out_of_pages_defers_before_any_state_changes():
    from vox_serve_amd.worker.base import OutOfPages
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=21)
    d = U.Driver(cfg, S, pages=3, slots=1, page_size=8, max_batch=2)
    try:
        d.feed([("x", tokens(20, 64, 1))])
        with pytest.raises(OutOfPages):
            d.feed([("x", tokens(8, 64, 2))])
        assert d.live["x"].kv_token_len == 20 and d.live["x"].prefill_cursor == 20
        with pytest.raises(OutOfPages):
            d.feed([("z", tokens(2, 64, 3))])              # pages would do for nobody, and the one state slot is taken
    finally:
        d.close()


def far_key_case():
    """One attention layer whose pooled history matters: window 4, blocks of 4, 200 tokens -> up to 49 pooled keys, sharp softmax."""
    cfg = U.config([U.attention(heads=2, kv_heads=1, dim=16, vdim=16, window=4, pool=4, rot=8, base=1000.0, scale=4.0)], width=16, vocab=32)
    return cfg, U.random_checkpoint(cfg, seed=23, gain=2.0)


def test_far_keys_prompt_and_decoding():
    cfg, S = far_key_case()
    toks = tokens(200, 32, 24)
    check(cfg, S, toks, [200])
    check(cfg, S, toks, [150], page_size=16)            # the last 50 decoded one by one, pooled blocks far behind them
    check(cfg, S, toks, [3, 61, 2, 67], page_size=4)    # a page per pooled block


def test_window_edge_sensitivity():
    """The bar is meaningful: moving the window or the pooled-block rule by one token changes the oracle's own logits by far
    more than the bar (so an engine that is one off cannot pass the tests above)."""
    cfg, S = far_key_case()
    toks = tokens(120, 32, 25)
    base = HR.forward(cfg, S, toks)
    for dw, dp in ((1, 0), (-1, 0)):
        c2 = U.config([dict(cfg["layers"][0], mixer=dict(cfg["layers"][0]["mixer"], mask={"size": 4 + dw, "pool": 4 + dp}))], width=16, vocab=32)
        assert U.rel_err(HR.forward(c2, S, toks), base) > 50 * F32_BAR


@pytest.mark.parametrize("page_size,pool", [(8, 3), (8, 8), (4, 8), (16, 5)])
def test_pool_blocks_across_page_borders(page_size, pool):
    """Pooled blocks that straddle pages, equal a page, or span several pages."""
    cfg = U.config([U.attention(heads=2, kv_heads=2, dim=8, vdim=8, window=3, pool=pool, rot=4, scale=4.0), U.hgrn2()], width=16, vocab=32)
    S = U.random_checkpoint(cfg, seed=27, gain=2.0)
    toks = tokens(90, 32, 28)
    check(cfg, S, toks, [11, 2, 29], page_size=page_size, pages=32)


def test_many_keys_few_rows():
    """More than 256 visible keys (window 150 + up to 135 pooled blocks of 2): steps of few rows split the keys over several
    blocks and merge; prompts of many rows do not.  Both against the same oracle, sharp softmax."""
    toks = tokens(420, 40, 42)
    for scale, dtype, q in ((2.0, torch.float32, None), (None, torch.bfloat16, 0.9)):
        cfg = U.config([U.attention(heads=4, kv_heads=2, dim=16, vdim=24, window=150, pool=2, rot=8, scale=scale), U.mlstm()], width=24, vocab=40)
        S = U.random_checkpoint(cfg, seed=41)
        # (bf16: the mLSTM's normaliser max(|n.q|, exp(-m)) amplifies rounding at a few positions, in every schedule alike: 90 % bar)
        a = check(cfg, S, toks, [420], pages=64, max_rows=512, dtype=dtype, quantile=q)
        b = check(cfg, S, toks, [330, 3, 2, 20], pages=64, max_rows=512, dtype=dtype, quantile=q)   # 20-, 3- and 1-row steps over 280+ keys
        assert U.rel_err(b, a.double(), 0.9) < (F32_BAR if dtype == torch.float32 else BF16_BAR)


def test_long_decoding():
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=29)
    check(cfg, S, tokens(330, 64, 30), [10], pages=48)


def test_wide_sizes():
    """Sizes beyond one wave per head: 160 value columns, 96 key dims, a group of 5 query heads, odd width and vocabulary."""
    layers = [U.hgrn2(heads=2, dim=40, vdim=160), U.attention(heads=5, kv_heads=1, dim=96, vdim=160, window=20, pool=7, rot=32, ff=100),
              U.mlstm(heads=2, dim=72, vdim=96)]
    cfg = U.config(layers, width=100, vocab=131, loop=(0, 2, 2))
    S = U.random_checkpoint(cfg, seed=31)
    toks = tokens(80, 131, 32)
    check(cfg, S, toks, [37, 2, 30])
    check(cfg, S, toks, [80], dtype=torch.bfloat16)


def test_large_recurrent_dims():
    """Key dims beyond 256 per head: the scans keep 32 dims per wave instead of 16, and stage fewer tokens per tile."""
    cfg = U.config([U.hgrn2(heads=1, dim=300, vdim=24), U.mlstm(heads=2, dim=272, vdim=16)], width=32, vocab=40)
    S = U.random_checkpoint(cfg, seed=55)
    toks = tokens(50, 40, 56)
    check(cfg, S, toks, [50])
    check(cfg, S, toks, [17, 2, 20])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_odd_sizes(dtype):
    """Sizes that defeat every vector path: width 18, key dims 10 / 5 / 3, value dims 6 / 7 / 5, 3 query heads per K/V head,
    6 of 10 dims rotated, a 37-entry vocabulary, a window of 11 and blocks of 5 on pages of 8."""
    layers = [U.hgrn2(heads=3, dim=5, vdim=7, ff=13), U.attention(heads=3, kv_heads=1, dim=10, vdim=6, window=11, pool=5, rot=6, ff=0),
              U.mlstm(heads=1, dim=3, vdim=5), U.attention(heads=2, kv_heads=2, dim=6, vdim=9, window=2, pool=7, rot=2, factor=3.0)]
    cfg = U.config(layers, width=18, vocab=37, loop=(1, 4, 2))
    S = U.random_checkpoint(cfg, seed=51)
    toks = tokens(75, 37, 52)
    q = None if dtype == torch.float32 else 0.9
    check(cfg, S, toks, [75], dtype=dtype, quantile=q)
    check(cfg, S, toks, [9, 2, 33, 5], dtype=dtype, quantile=q)


def test_greedy_generation_through_the_scheduler():
    """Requests enter through the scheduler's transport, are prefilled in portions next to decoding requests and generate greedily;
    the ids equal the oracle's greedy continuation (fp32 engine)."""
    import json

    from vox_serve_amd.model.sirodra import SirodraModel, config_from_dict
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=33)
    n_new = 12
    model = SirodraModel("sirodra-test", S, config_from_dict(cfg), dtype=torch.float32, max_batch_size=4, page_size=8, max_num_pages=64,
                         max_seq_len=512, max_prefill_tokens=64, state_slots=4, max_tokens=n_new)
    worker = ModelWorker(model=model, max_batch_size=4, max_num_pages=64, page_size=8, greedy=True, prefill_chunk_tokens=16)
    sched = Scheduler(worker, max_batch_size=4)
    prompts = {"p0": tokens(37, 64, 34), "p1": tokens(5, 64, 35), "p2": tokens(50, 64, 36)}
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
                seq.append(int(HR.forward(cfg, S, seq)[-1].argmax()))
            got = [int(t[0, 0]) for t in reqs[rid].lm_output_tokens]
            assert got == seq[len(p):], (rid, got, seq[len(p):])
        done = []
        while not sched.transport.results.empty():
            done.append(sched.transport.results.get())
        assert sum(b"|COMPLETION|" in m and json.loads(m.split(b"|", 2)[2])["status"] == "completed" for m in done) == 3
        assert worker.empty_pages.qsize() == 64 and worker.empty_state_slots.qsize() == 4
    finally:
        model.engine.close()


def test_top_k_sampling_through_the_scheduler():
    """Stochastic sampling goes through the library's sampler: every generated id is one of the oracle's five most likely
    continuations of the request's own prefix, and a second run with the same seed repeats the ids."""
    from vox_serve_amd.model.sirodra import SirodraModel, config_from_dict
    from vox_serve_amd.sampling import SamplingConfig
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg = stack(sharp=False)
    S = U.random_checkpoint(cfg, seed=61)
    prompts = {"a": tokens(21, 64, 62), "b": tokens(9, 64, 63)}

    def generate():
        model = SirodraModel("sirodra-test", S, config_from_dict(cfg), dtype=torch.float32, max_batch_size=2, page_size=8, max_num_pages=32,
                             max_seq_len=256, max_prefill_tokens=64, state_slots=2, max_tokens=10,
                             sampling=SamplingConfig(top_k=5, temperature=0.8, max_tokens=10))
        worker = ModelWorker(model=model, max_batch_size=2, max_num_pages=32, page_size=8, seed=7)
        sched = Scheduler(worker, max_batch_size=2)
        try:
            for rid, p in prompts.items():
                sched.transport.requests.put(encode_request(rid, " ".join(map(str, p)), is_streaming=False))
            reqs = {}
            for _ in range(200):
                sched._step()
                for r in sched.active_requests:
                    reqs[r.request_id] = r
                if not sched.active_requests and not sched.transport.pending():
                    break
            return {rid: [int(t[0, 0]) for t in reqs[rid].lm_output_tokens] for rid in prompts}
        finally:
            model.engine.close()
    first = generate()
    for rid, p in prompts.items():
        assert len(first[rid]) == 10
        seq = list(p)
        for tok in first[rid]:
            top = HR.forward(cfg, S, seq)[-1].topk(5).indices.tolist()
            assert tok in top, (rid, tok, top)
            seq.append(tok)
    assert generate() == first


def test_async_scheduling_generates_the_same_ids():
    """The pipelined scheduler loop (a step is launched before the previous step's ids are read; a finished request gets one surplus
    row that is dropped) generates the oracle's greedy ids too."""
    from vox_serve_amd.model.sirodra import SirodraModel, config_from_dict
    from vox_serve_amd.scheduler.base import Scheduler, encode_request
    from vox_serve_amd.worker.base import ModelWorker
    cfg = stack()
    S = U.random_checkpoint(cfg, seed=71)
    n_new = 9
    model = SirodraModel("sirodra-test", S, config_from_dict(cfg), dtype=torch.float32, max_batch_size=4, page_size=8, max_num_pages=64,
                         max_seq_len=512, max_prefill_tokens=64, state_slots=4, max_tokens=n_new)
    worker = ModelWorker(model=model, max_batch_size=4, max_num_pages=64, page_size=8, greedy=True, prefill_chunk_tokens=20)
    sched = Scheduler(worker, max_batch_size=4, async_scheduling=True)
    prompts = {"p0": tokens(30, 64, 72), "p1": tokens(3, 64, 73), "p2": tokens(41, 64, 74)}
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
        sched.run_until_idle(max_steps=500)
        assert set(seen) == set(prompts)
        for rid, p in prompts.items():
            seq = list(p)
            for _ in range(n_new):
                seq.append(int(HR.forward(cfg, S, seq)[-1].argmax()))
            got = [int(t[0, 0]) for t in seen[rid].lm_output_tokens]
            assert got[:n_new] == seq[len(p):], (rid, got, seq[len(p):])
        assert worker.empty_pages.qsize() == 64 and worker.empty_state_slots.qsize() == 4
    finally:
        model.engine.close()
