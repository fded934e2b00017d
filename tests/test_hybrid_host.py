"""Host-side pieces of the hybrid-mixer (Sirodra) path that need no GPU: the config reader, the layer schedule, the fused weight
layout, the worker's portion / page / state-slot bookkeeping (against a stand-in engine), and sanity properties of the float64
oracle's own mechanisms."""
import math

import pytest
import torch

from oracle import hybrid_ref as HR
from tests import hybrid_util as U


def test_config_reader_and_schedule():
    from vox_serve_amd.model.sirodra import config_from_dict
    cfg = U.config([U.hgrn2(heads=3, dim=4, vdim=6), U.attention(heads=6, kv_heads=3, dim=8, vdim=10, window=7, pool=3, rot=4, base=77.0, factor=2.5, scale=0.3, ff=20),
                    U.mlstm(heads=2, dim=6, vdim=4, cap=9.0)], width=12, vocab=31, loop=(1, 3, 2), eps=3e-6)
    c = config_from_dict(cfg)
    assert (c.width, c.vocab, c.loop) == (12, 31, (1, 3, 2)) and abs(c.eps - 3e-6) < 1e-12
    a = c.layers[1]
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.pool, a.rot_dims, a.rot_base, a.rot_factor, a.scale, a.ff) == \
        ("attention", 6, 3, 8, 10, 7, 3, 4, 77.0, 2.5, 0.3, 20)
    assert c.layers[2].gate_cap == 9.0 and c.layers[0].ff == 0
    assert [m.n_in for m in c.layers] == [2 * 12 + 18, 48 + 3 * 18 + 6, 2 * 12 + 2 * 8 + 4]
    assert c.runs() == [(0, False), (1, True), (2, False), (1, True), (2, False)]
    assert c.runs() == HR.run_order(cfg)
    for loop in (None, (0, 3, 1), (0, 1, 3), (2, 3, 2)):
        cc = U.config(cfg["layers"], width=12, vocab=31, loop=loop)
        assert config_from_dict(cc).runs() == HR.run_order(cc)
    with pytest.raises(ValueError):
        config_from_dict(dict(cfg, architecture="Other"))
    bad = U.config([dict(U.hgrn2(), type="conv")])
    with pytest.raises(ValueError):
        config_from_dict(bad)


def test_fused_weight_layout():
    from vox_serve_amd.model.sirodra import config_from_dict, pack_weights, synth_weights
    cfg = U.config([U.hgrn2(heads=3, dim=4, vdim=6), U.attention(heads=6, kv_heads=3, dim=8, vdim=10, ff=20), U.mlstm(heads=2, dim=6, vdim=4)],
                   width=12, vocab=31, loop=(0, 2, 2))
    c = config_from_dict(cfg)
    S = U.random_checkpoint(cfg, seed=1)
    assert set(synth_weights(c)) == set(S) and all(synth_weights(c)[k].shape == S[k].shape for k in S)
    W = pack_weights(S, c)
    for m, lw in zip(c.layers, W["layers"]):
        assert tuple(lw["w_in"].shape) == (m.n_in, 12)
    a = W["layers"][1]
    assert torch.equal(a["w_in"][48:48 + 24], S["l1.mix.k"]) and torch.equal(a["w_in"][-6:], S["l1.mix.g"])
    assert torch.equal(a["b_in"][:48], S["l1.mix.q.b"].float()) and float(a["b_in"][-6:].abs().sum()) == 0.0      # the gate has no bias
    m_ = W["layers"][2]
    assert torch.equal(m_["w_in"][-4:-2], S["l2.mix.i"]) and torch.equal(m_["b_in"][-2:], S["l2.mix.f.b"].float())
    assert float(m_["b_in"][:-4].abs().sum()) == 0.0
    h = W["layers"][0]
    assert torch.equal(h["w_in"][12:24], S["l0.mix.f"]) and torch.equal(h["b_in"][12:24], S["l0.mix.f.b"].float())
    assert W["loop_in"] is S["loop.in"] and W["layers"][0]["w_up"] is None


def test_rotary_frequencies_fp32():
    from vox_serve_amd.engine_hybrid import rotary_frequencies
    f = rotary_frequencies(8, 100.0, 4.0)
    assert f.dtype == torch.float32 and f.shape == (4,)
    assert torch.allclose(f.double(), torch.tensor([100.0 ** (-2 * i / 8) / 4.0 for i in range(4)], dtype=torch.float64), rtol=1e-6)


class _FakeEngine:
    needs_state_slots, state_slots, max_rows, max_batch, max_out = True, 2, 16, 4, 8


class _FakeModel:
    needs_input_masks = needs_input_features = use_repetition_penalty = False
    supports_input_streaming = False
    model_name = "fake"

    def __init__(self):
        self.engine = _FakeEngine()


def _req(rid, toks, budget=None, open_=False):
    from vox_serve_amd.requests import Request
    r = Request(request_id=rid, prompt_open=open_)
    r.input_tokens, r._preprocessed, r.step_budget = torch.tensor(toks).view(-1, 1), True, budget
    return r


def test_worker_portions_pages_and_slots():
    from vox_serve_amd.worker.base import ModelWorker, OutOfPages
    w = ModelWorker(model=_FakeModel(), max_batch_size=4, max_num_pages=5, page_size=4)
    a, b = _req("a", list(range(11)), budget=5), _req("b", [7, 8, 9])
    li = w.prepare_lm_inputs([a, b], [])
    assert li["qo_indptr"] == [0, 5, 8] and li["position_ids"].tolist() == [0, 1, 2, 3, 4, 0, 1, 2]
    assert li["input_ids"].view(-1).tolist() == [0, 1, 2, 3, 4, 7, 8, 9]
    assert (a.kv_pages, b.kv_pages, a.kv_last_page_len, b.kv_last_page_len) == ([0, 1], [2], 1, 3)
    assert (a.state_slot, b.state_slot) == (0, 1) and not a.done_lm_prefill and b.done_lm_prefill and b.next_position_id == 3
    q_req, kvlen, page, slot = w._token_plan(li)
    assert q_req == [0] * 5 + [1] * 3 and kvlen == [1, 2, 3, 4, 5, 1, 2, 3] and page == [0, 0, 0, 0, 1, 2, 2, 2] and slot == [0, 1, 2, 3, 0, 0, 1, 2]
    # second portion of a (2 tokens, inside page 1) beside a decode row of b
    a.step_budget = 2
    b.input_tokens = torch.tensor([[5]])
    li = w.prepare_lm_inputs([a, b], [])
    assert li["qo_indptr"] == [0, 2, 3] and li["position_ids"].tolist() == [5, 6, 3] and a.kv_pages == [0, 1] and a.prefill_cursor == 7
    q_req, kvlen, page, slot = w._token_plan(li)
    assert kvlen == [6, 7, 4] and page == [1, 1, 2] and slot == [1, 2, 3]
    # the rest of a needs a third page; a new request finds no state slot and is deferred before anything changes
    a.step_budget = None
    c = _req("c", [1, 2])
    with pytest.raises(OutOfPages):
        w.prepare_lm_inputs([a, c], [])
    assert a.prefill_cursor == 7 and w.empty_pages.qsize() == 2 and c.state_slot is None
    li = w.prepare_lm_inputs([a], [])
    assert li["position_ids"].tolist() == [7, 8, 9, 10] and a.kv_pages == [0, 1, 3] and a.done_lm_prefill and a.next_position_id == 11
    # pages exhausted: a 9-token prompt needs 3 pages, 1 is free
    w.free_kv_cache(b)
    assert w.empty_state_slots.qsize() == 1 and w.empty_pages.qsize() == 2 and b.state_slot is None
    with pytest.raises(OutOfPages):
        w.prepare_lm_inputs([_req("d", list(range(9)))], [])
    w.free_kv_cache(a)
    assert w.empty_state_slots.qsize() == 2 and w.empty_pages.qsize() == 5
    # an open prompt never completes by itself; the worker's chunk size bounds a portion; the engine's row capacity too
    w.prefill_chunk_tokens = 3
    e = _req("e", list(range(8)), open_=True)
    assert w.prepare_lm_inputs([e], [])["qo_indptr"] == [0, 3]
    w.prefill_chunk_tokens = None
    assert w.prepare_lm_inputs([e], [])["qo_indptr"] == [0, 5] and not e.done_lm_prefill and e.prefill_cursor == 8
    with pytest.raises(ValueError):
        w.prepare_lm_inputs([e], [])                      # nothing left to run
    w.free_kv_cache(e)
    big = _req("f", list(range(40)))
    w2 = ModelWorker(model=_FakeModel(), max_batch_size=4, max_num_pages=32, page_size=4)
    assert w2.prepare_lm_inputs([big, _req("g", [1])], [])["qo_indptr"] == [0, 15, 16]     # 16 rows: 15 + the other request's one


def test_oracle_visible_keys():
    assert HR.visible_keys(0, 4, 3) == ([], [0])
    assert HR.visible_keys(5, 4, 3) == ([], [2, 3, 4, 5])                 # block 0 = tokens 0..2 ends at 2 > 5 - 4
    assert HR.visible_keys(6, 4, 3) == ([0], [3, 4, 5, 6])                # ... ends at 2 <= 6 - 4: seen, with nothing unseen between
    assert HR.visible_keys(8, 4, 3) == ([0], [5, 6, 7, 8])                # tokens 3, 4 are in no seen block and outside the window
    assert HR.visible_keys(9, 4, 3) == ([0, 1], [6, 7, 8, 9])
    assert HR.visible_keys(7, 1, 1) == (list(range(7)), [7])


def test_oracle_attention_reduces_to_plain_causal_softmax():
    """A window longer than the sequence, no rotation: ordinary causal attention on unit-RMS q, k."""
    torch.manual_seed(0)
    m = {"heads": 2, "kv_heads": 1, "dim": 4, "vdim": 3, "mask": {"size": 100, "pool": 5}, "rot": {"dims": 0}, "scale": 0.7}
    h = torch.randn(9, 6, dtype=torch.float64)
    P = {k: torch.randn(s, dtype=torch.float64) for k, s in
         {"q": (8, 6), "q.b": (8,), "k": (4, 6), "k.b": (4,), "v": (3, 6), "v.b": (3,), "g": (2, 6), "o": (6, 6)}.items()}
    got = HR.pooled_window_attention(P, h, m, 1e-6)
    q = HR.unit_rms((h @ P["q"].T + P["q.b"]).view(9, 2, 4), 1e-6)
    k = HR.unit_rms((h @ P["k"].T + P["k.b"]).view(9, 1, 4), 1e-6)
    v = (h @ P["v"].T + P["v.b"]).view(9, 1, 3)
    sc = torch.einsum("thd,sd->hts", q, k[:, 0]) * 0.7
    sc = sc.masked_fill(torch.triu(torch.ones(9, 9, dtype=torch.bool), 1), -math.inf)
    y = torch.einsum("hts,se->the", torch.softmax(sc, -1), v[:, 0]) * torch.sigmoid(h @ P["g"].T).unsqueeze(-1)
    assert torch.allclose(got, y.reshape(9, 6) @ P["o"].T, atol=1e-12)


def test_oracle_mlstm_matches_unstabilised_form():
    """With moderate gates the running maximum only rescales numerator and denominator: the plain (overflow-prone) recurrence
    C_t = f C + i k v^T, n_t = f n + i k, y = C^T q / (max(|n.q|, 1) + 1e-6 e^{m}) e^{0} agrees once both are written in the same scale."""
    torch.manual_seed(1)
    m = {"heads": 1, "dim": 3, "vdim": 2, "gate_cap": 8.0}
    h = torch.randn(7, 5, dtype=torch.float64)
    P = {k: torch.randn(s, dtype=torch.float64) for k, s in
         {"q": (3, 5), "k": (3, 5), "v": (2, 5), "g": (2, 5), "i": (1, 5), "i.b": (1,), "f": (1, 5), "f.b": (1,), "norm": (2,), "o": (5, 2)}.items()}
    got = HR.mlstm_mixer(P, h, m, 1e-6)
    q, k, v = (h @ P["q"].T) / math.sqrt(3), h @ P["k"].T, h @ P["v"].T
    li = 8.0 * torch.tanh((h @ P["i"].T + P["i.b"]) / 8.0)
    lf = torch.nn.functional.logsigmoid(8.0 * torch.tanh((h @ P["f"].T + P["f.b"]) / 8.0))
    C, n, mx, ys = torch.zeros(3, 2, dtype=torch.float64), torch.zeros(3, dtype=torch.float64), 0.0, []
    for t in range(7):
        C = torch.exp(lf[t]) * C + torch.exp(li[t]) * torch.outer(k[t], v[t])       # true scale
        n = torch.exp(lf[t]) * n + torch.exp(li[t]) * k[t]
        mx = max(float(lf[t]) + mx, float(li[t]))
        ys.append((C.T @ q[t]) * math.exp(-mx) / (max(abs(float(n @ q[t])) * math.exp(-mx), math.exp(-mx)) + 1e-6))
    y = HR.unit_rms(torch.stack(ys).view(7, 1, 2), 1e-6).reshape(7, 2) * P["norm"] * torch.sigmoid(h @ P["g"].T)
    assert torch.allclose(got, y @ P["o"].T, atol=1e-10)


def test_oracle_rotary_keeps_norm_and_pairs():
    x = torch.randn(5, 2, 8, dtype=torch.float64)
    y = HR.rotary_interleaved(x, 4, 10.0, 2.0)
    assert torch.equal(y[..., 4:], x[..., 4:]) and torch.equal(y[0], x[0])
    assert torch.allclose((y[..., :2] ** 2).sum(-1), (x[..., :2] ** 2).sum(-1))
    ang = 3 * 10.0 ** (-2.0 / 4) / 2.0                                    # position 3, pair 1
    assert torch.allclose(y[3, :, 2], x[3, :, 2] * math.cos(ang) - x[3, :, 3] * math.sin(ang))


def test_oracle_hgrn2_lower_bound_and_state():
    """lower = 1 freezes the state at zero (nothing is ever written); lower = 0 and a saturated forget bias keeps the first write."""
    cfg = U.config([U.hgrn2(heads=1, dim=2, vdim=2)], width=4, vocab=6)
    S = {k: v.double() for k, v in U.random_checkpoint(cfg, seed=2).items()}
    S["l0.mix.lower"] = torch.ones(2, dtype=torch.float64)
    x = HR.forward(cfg, S, [1, 2, 3])
    S0 = dict(S); S0["l0.mix.o"] = torch.zeros_like(S["l0.mix.o"])
    assert torch.allclose(x, HR.forward(cfg, S0, [1, 2, 3]))
