"""Host-side pieces of the Fusanex path that need no GPU: the config reader, the fused weight layout, the registry entry, and
identities of the oracle itself (causality, routing weights, the closed form of a constant-gate recurrence)."""
import math

import pytest
import torch

from oracle import fusanex_ref as FR
from tests import fusanex_util as F


def small():
    return F.config([F.parallel(mlp=F.moe()), F.rglru(width=30, blocks=5, conv=3, mlp=F.moe(experts=3, identity=0, top=1, shared=None)),
                     F.rglru(mlp=None)], width=24, groups=4, embed_scale=2.5)


def test_config_reader_takes_every_size_and_constant():
    from vox_serve_amd.model.fusanex import config_from_dict
    c = config_from_dict(small())
    assert (c.width, c.vocab, c.norm_kind, c.norm_groups, c.embed_scale) == (24, 40, "rms_groups", 4, 2.5)
    a, r1, r2 = c.layers
    assert (a.kind, a.heads, a.kv_heads, a.dim, a.vdim, a.block) == ("causal_attention", 4, 2, 8, 12, "parallel")
    assert (a.q_temp_coef, a.q_temp_every, a.v_unit_rms, a.out_scale) == (0.4, 5, True, 1.1)
    assert (a.side.kind, a.side.heads, a.side.dim, a.side.vdim, a.side.out_scale) == ("shift_decay", 2, 8, 8, 0.7)
    assert (a.moe.experts, a.moe.identity, a.moe.top, a.moe.ff, a.moe.limit, a.moe.shared_ff, a.moe.shared_limit) == (5, 1, 2, 12, 1.5, 10, 0.8)
    assert (r1.kind, r1.heads, r1.dim, r1.conv_taps, r1.rec_scale) == ("rglru", 5, 6, 3, 8.0)
    assert r1.moe.shared_ff == 0 and r2.moe is None
    assert [i for i, _ in c.runs()] == [0, 1, 2]
    bad = small()
    bad["layers"][1]["mixer"]["blocks"] = 4
    with pytest.raises(ValueError):
        config_from_dict(bad)
    bad = small()
    bad["architecture"] = "Other"
    with pytest.raises(ValueError):
        config_from_dict(bad)


def test_pack_weights_layout():
    from vox_serve_amd.model.fusanex import config_from_dict, pack_weights
    cfg = small()
    S = F.random_checkpoint(cfg, seed=3, lora=7)
    c = config_from_dict(cfg)
    w = pack_weights(S, c)
    a, r1, r2 = w["layers"]
    assert tuple(a["w_in"].shape) == (c.layers[0].n_in, 24) and torch.equal(a["w_in"][32:48], S["l0.mix.left.k"])
    assert c.layers[0].side.lora == 7 and tuple(a["side"]["w_in"].shape) == (c.layers[0].side.n_in, 24) == (4 * 16 + 7, 24)
    assert torch.equal(a["side"]["shift_mu"][4], S["l0.mix.right.mu.w"].float()) and tuple(a["side"]["bonus"].shape) == (16,)
    assert tuple(a["moe"]["w_gate_up"].shape) == (5, 24, 24) and torch.equal(a["moe"]["w_gate_up"][2, 12:], S["l0.mlp.e2.up"])
    assert tuple(a["moe"]["w_down"].shape) == (5, 24, 12) and tuple(a["moe"]["shared_gate_up"].shape) == (20, 24)
    assert tuple(r1["w_gates"].shape) == (5, 12, 6) and torch.equal(r1["w_gates"][3, 6:], S["l1.mix.ri"][3])
    assert torch.equal(r1["b_gates"][2, :6], S["l1.mix.ra.b"][2].float()) and tuple(r1["w_in"].shape) == (60, 24)
    assert "shared_gate_up" not in r1["moe"] and "moe" not in r2


def test_synthetic_weights_fit_the_reader():
    from vox_serve_amd.model.fusanex import config_from_dict, pack_weights, synth_weights
    c = config_from_dict(small())
    w = pack_weights(synth_weights(c, lora=5), c)
    assert c.layers[0].side.lora == 5 and len(w["layers"]) == 3


def test_registry_names_the_design():
    from vox_serve_amd.model import MODEL_REGISTRY, get_model_class
    assert "fusanex" in MODEL_REGISTRY and get_model_class("Fusanex") is MODEL_REGISTRY["fusanex"]


def test_oracle_is_causal_and_deterministic():
    cfg = small()
    S = F.random_checkpoint(cfg, seed=5)
    toks = torch.randint(0, 40, (30,), generator=torch.Generator().manual_seed(6)).tolist()
    full = FR.forward(cfg, S, toks)
    assert torch.allclose(FR.forward(cfg, S, toks[:17]), full[:17], atol=1e-12)
    other = list(toks)
    other[20] = (other[20] + 1) % 40
    assert torch.allclose(FR.forward(cfg, S, other)[:20], full[:20], atol=1e-12)
    assert not torch.allclose(FR.forward(cfg, S, other)[20:], full[20:], atol=1e-6)


def test_oracle_routing_weights_and_identity():
    g = torch.Generator().manual_seed(7)
    n = torch.randn(50, 8, generator=g, dtype=torch.float64)
    P = {"router": torch.randn(6, 8, generator=g, dtype=torch.float64), "correction": torch.tensor([0, 0, 0, 0, 5.0, 5.0], dtype=torch.float64)}
    r = {"experts": 4, "identity": 2, "top": 2}
    chosen, w = FR.route(P, n, r)
    assert set(chosen.flatten().tolist()) == {4, 5}                       # the correction decides the choice ...
    s = torch.softmax(n @ P["router"].T, -1)
    assert torch.allclose(w, torch.gather(s, 1, chosen) / torch.gather(s, 1, chosen).sum(-1, keepdim=True))   # ... but not the weights
    # only identity outputs chosen and no shared expert: the feed-forward returns its input
    out = FR.moe_ff(P, n, {"router": r, "expert": {"ff": 4, "limit": 1.0}})
    assert torch.allclose(out, n)


def test_oracle_recurrence_closed_form():
    """With gates that do not depend on the input (zero gate matrices) the recurrent unit is a geometric series."""
    C, T = 4, 12
    P = {"y": torch.zeros(C, 3, dtype=torch.float64), "y.b": torch.full((C,), 2.0, dtype=torch.float64),
         "x": torch.zeros(C, 3, dtype=torch.float64), "x.b": torch.ones(C, dtype=torch.float64),
         "conv": torch.tensor([[0.0, 1.0]] * C, dtype=torch.float64), "conv.b": torch.zeros(C, dtype=torch.float64),
         "ra": torch.zeros(1, C, C, dtype=torch.float64), "ra.b": torch.zeros(1, C, dtype=torch.float64),
         "ri": torch.zeros(1, C, C, dtype=torch.float64), "ri.b": torch.zeros(1, C, dtype=torch.float64),
         "lam": torch.zeros(C, dtype=torch.float64), "o": torch.eye(C, dtype=torch.float64)}
    out = FR.rglru_mixer(P, torch.zeros(T, 3, dtype=torch.float64), {"width": C, "blocks": 1, "conv": 2})
    a = math.exp(-8.0 * 0.5 * math.log(2.0))
    b = math.sqrt(1.0 - a * a) * 0.5
    y = float(FR.gelu_tanh(torch.tensor(2.0, dtype=torch.float64)))
    want = torch.tensor([b * (1 - a ** (t + 1)) / (1 - a) * y for t in range(T)], dtype=torch.float64)
    assert torch.allclose(out[:, 0], want, atol=1e-12)


def test_oracle_shift_reads_the_previous_token():
    """mu = 1 makes every projection of the matrix-state mixer read the previous token only: the first token's output is zero
    and token t's output does not depend on token t."""
    cfg = F.config([F.parallel(left_scale=0.0)], width=16)
    S = F.random_checkpoint(cfg, seed=9)
    for s in "rkvgw":
        S["l0.mix.right.mu." + s] = torch.ones(16, dtype=torch.bfloat16)
    Sd = {k[len("l0.mix.right."):]: v.double() for k, v in S.items() if k.startswith("l0.mix.right.")}
    g = torch.Generator().manual_seed(10)
    n = torch.randn(6, 16, generator=g, dtype=torch.float64)
    out = FR.shifted_state_mixer(Sd, n, cfg["layers"][0]["mixer"]["right"], 1e-5)
    assert torch.allclose(out[0], torch.zeros(16, dtype=torch.float64))
    n2 = n.clone()
    n2[5] += 1.0
    assert torch.allclose(FR.shifted_state_mixer(Sd, n2, cfg["layers"][0]["mixer"]["right"], 1e-5), out)
