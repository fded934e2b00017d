"""Fusanex: a decoder-only language model on the hybrid engine (`engine_hybrid.HybridEngine`).

A checkpoint is a folder with `config.json` and `model.safetensors`.  config.json:
  architecture "Fusanex"; vocab, width; embedding.scale; norm.eps, norm.groups;
  layers[i] = {type: "rglru" | "parallel", mixer: {...}, mlp: null | {kind: "moe", router: {experts, identity, top},
               expert: {ff, limit}, shared: {ff, limit}}}.
Tensors (bf16, linear weights [out, in]): embed, head, final.norm, and per layer l<i>.norm1, l<i>.norm2, l<i>.mix.*, l<i>.mlp.*.

x0 = embed[token] * embedding.scale.  Every layer is parallel: x += mixer(norm1 x) + moe(norm2 x), both norms of the same x; a
norm divides each of `groups` equal slices of the vector by its own root mean square and multiplies by a weight.  The mixers:
  rglru     y = gelu_tanh(Wy n + b), u = causal conv over `conv` taps of (Wx n + b); per block of channels r, i = sigmoid of a
            square matrix times the block's u (+ bias); a = exp(-8 r softplus(lam)); S <- a S + sqrt(1 - a^2) i u; out = Wo (S y).
  parallel  left_scale * left + right_scale * right, both reading the same normed input:
            left   grouped-query softmax attention over all earlier tokens, no rotation: q, k RMS-normed per head with a shared
                   weight, q times 1 + coef ln(floor((p + 1) / every) + 1) at position p, v divided by its RMS per head;
            right  token-shift mixes n + (n_prev - n) mu_s for s = r, k, v, g, w; decay w = exp(-exp(W2 tanh(W1 mix_w) + w0));
                   o = (S + diag(u) k v^T)^T r, S <- diag(w) S + k v^T; unit RMS per head, weight, silu gate, projection.
The feed-forward routes every token to `top` of experts + identity outputs by softmax score (+ a correction for the choice only),
weights renormalised over the chosen; experts are clamped gated units g * sigmoid(1.702 g) * (u + 1); identity outputs pass their
input through; a shared expert of the same form is always added.
The plugin fuses each mixer's projections into the engine's row order at load time.
"""
from typing import Dict

import torch

from ..engine_hybrid import HybridCfg, MixerCfg, MoECfg
from .hybrid_lm import HybridLM

ARCHITECTURE = "Fusanex"
RGLRU_DECAY_SCALE = 8.0         # a = exp(-8 r softplus(lam))
EXPERT_SIGMOID_SLOPE = 1.702    # g * sigmoid(1.702 g)
SHIFT_ORDER = ("r", "k", "v", "g", "w")


def _moe_from_dict(i: int, mlp) -> MoECfg:
    if mlp is None:
        return None
    if mlp.get("kind", "moe") != "moe":
        raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not part of this design")
    r, e, sh = mlp["router"], mlp["expert"], mlp.get("shared")
    return MoECfg(experts=int(r["experts"]), identity=int(r.get("identity", 0)), top=int(r["top"]), ff=int(e["ff"]), limit=float(e["limit"]),
                  shared_ff=int(sh["ff"]) if sh else 0, shared_limit=float(sh["limit"]) if sh else 0.0, act_alpha=EXPERT_SIGMOID_SLOPE)


def config_from_dict(d: dict) -> HybridCfg:
    if d.get("architecture") != ARCHITECTURE:
        raise ValueError(f"not a {ARCHITECTURE} config: architecture = {d.get('architecture')!r}")
    layers = []
    for i, l in enumerate(d["layers"]):
        t, m = l["type"], l["mixer"]
        moe = _moe_from_dict(i, l.get("mlp"))
        if t == "rglru":
            C, B = int(m["width"]), int(m["blocks"])
            if C % B:
                raise ValueError(f"layer {i}: {B} blocks do not divide {C} channels")
            layers.append(MixerCfg("rglru", B, C // B, C // B, conv_taps=int(m["conv"]), rec_scale=RGLRU_DECAY_SCALE, block="parallel", moe=moe))
        elif t == "parallel":
            a, r = m["left"], m["right"]
            qt = a.get("q_temp") or {}
            right = MixerCfg("shift_decay", int(r["heads"]), int(r["dim"]), int(r["dim"]), out_scale=float(m.get("right_scale", 1.0)))
            layers.append(MixerCfg("causal_attention", int(a["heads"]), int(a["dim"]), int(a["vdim"]), kv_heads=int(a["kv_heads"]),
                                   scale=float(a["scale"]), q_temp_coef=float(qt.get("coef", 0.0)), q_temp_every=int(qt.get("every", 1)),
                                   v_unit_rms=True, out_scale=float(m.get("left_scale", 1.0)), block="parallel", side=right, moe=moe))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
    nm = d["norm"]
    return HybridCfg(int(d["width"]), int(d["vocab"]), float(nm["eps"]), layers, None, norm_kind="rms_groups",
                     norm_groups=int(nm.get("groups", 1)), embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)))


def pack_weights(S: Dict[str, torch.Tensor], cfg: HybridCfg) -> Dict:
    """Checkpoint tensors -> the engine's fused layout.  Sizes a config does not give (the decay bottleneck) come from the shapes."""
    layers = []
    for i, m in enumerate(cfg.layers):
        p = f"l{i}.mix."
        lw = dict(norm1=S[f"l{i}.norm1"], norm2=S.get(f"l{i}.norm2"))
        if m.kind == "rglru":
            C = m.heads * m.dim
            lw.update(w_in=torch.cat([S[p + "y"], S[p + "x"]], 0).contiguous(),
                      b_in=torch.cat([S[p + "y.b"].float(), S[p + "x.b"].float()]), w_out=S[p + "o"],
                      conv_w=S[p + "conv"], conv_b=S[p + "conv.b"],
                      w_gates=torch.cat([S[p + "ra"], S[p + "ri"]], 1).contiguous(),       # [blocks][2*bs][bs]
                      b_gates=torch.cat([S[p + "ra.b"].float(), S[p + "ri.b"].float()], 1).contiguous(), lam=S[p + "lam"])
            assert lw["conv_w"].shape == (C, m.conv_taps), (i, tuple(lw["conv_w"].shape))
        else:
            a, r, sm = p + "left.", p + "right.", m.side
            lw.update(w_in=torch.cat([S[a + "q"], S[a + "k"], S[a + "v"]], 0).contiguous(), w_out=S[a + "o"],
                      q_norm=S[a + "q.norm"], k_norm=S[a + "k.norm"])
            sm.lora = int(S[r + "w1"].shape[0])
            lw["side"] = dict(w_in=torch.cat([S[r + n] for n in ("r", "k", "v", "g", "w1")], 0).contiguous(), w_out=S[r + "o"],
                              shift_mu=torch.stack([S[r + "mu." + n].float() for n in SHIFT_ORDER]).contiguous(),
                              w_decay2=S[r + "w2"], decay0=S[r + "w0"], bonus=S[r + "u"].reshape(-1), head_norm=S[r + "norm"])
        if m.moe is not None:
            e, q = m.moe, f"l{i}.mlp."
            if lw["norm2"] is None:
                raise KeyError(f"layer {i}: norm2 missing")
            mw = dict(router=S[q + "router"], correction=S.get(q + "correction"))
            if e.experts:
                mw["w_gate_up"] = torch.stack([torch.cat([S[f"{q}e{j}.gate"], S[f"{q}e{j}.up"]], 0) for j in range(e.experts)]).contiguous()
                mw["w_down"] = torch.stack([S[f"{q}e{j}.down"] for j in range(e.experts)]).contiguous()
            if e.shared_ff:
                mw["shared_gate_up"] = torch.cat([S[q + "shared.gate"], S[q + "shared.up"]], 0).contiguous()
                mw["shared_down"] = S[q + "shared.down"]
            lw["moe"] = mw
        layers.append(lw)
    return dict(embedding=S["embed"], head=S["head"], final_norm=S["final.norm"], loop_in=None, layers=layers)


def synth_weights(cfg: HybridCfg, seed: int = 0, lora: int = 32) -> Dict[str, torch.Tensor]:
    """Random checkpoint tensors (bf16, the checkpoint's names) for a config: benchmarks."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def lin(*shape):
        return (torch.randn(*shape, generator=g) / shape[-1] ** 0.5).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": torch.randn(cfg.vocab, W, generator=g).to(torch.bfloat16), "head": lin(cfg.vocab, W), "final.norm": vec(W, 1.0)}
    for i, m in enumerate(cfg.layers):
        p = f"l{i}."
        S[p + "norm1"], S[p + "norm2"] = vec(W, 1.0), vec(W, 1.0)
        if m.kind == "rglru":
            C, B, bs = m.heads * m.dim, m.heads, m.dim
            S.update({p + "mix.y": lin(C, W), p + "mix.y.b": vec(C), p + "mix.x": lin(C, W), p + "mix.x.b": vec(C),
                      p + "mix.conv": lin(C, m.conv_taps), p + "mix.conv.b": vec(C), p + "mix.ra": lin(B, bs, bs), p + "mix.ra.b": vec(B * bs).view(B, bs),
                      p + "mix.ri": lin(B, bs, bs), p + "mix.ri.b": vec(B * bs).view(B, bs), p + "mix.lam": vec(C, -1.0, 1.0), p + "mix.o": lin(W, C)})
        else:
            a, r, sm = p + "mix.left.", p + "mix.right.", m.side
            H, G, d, e, HD = m.heads, m.kv_heads, m.dim, m.vdim, sm.heads * sm.dim
            S.update({a + "q": lin(H * d, W), a + "k": lin(G * d, W), a + "v": lin(G * e, W), a + "q.norm": vec(d, 1.0), a + "k.norm": vec(d, 1.0),
                      a + "o": lin(W, H * e)})
            S.update({r + "mu." + n: torch.rand(W, generator=g).to(torch.bfloat16) for n in SHIFT_ORDER})
            S.update({r + "r": lin(HD, W), r + "k": lin(HD, W), r + "v": lin(HD, W), r + "g": lin(HD, W), r + "w1": lin(lora, W),
                      r + "w2": lin(HD, lora), r + "w0": vec(HD, -1.0, 1.0), r + "u": vec(HD, 0.0, 0.5).view(sm.heads, sm.dim),
                      r + "norm": vec(HD, 1.0), r + "o": lin(W, HD)})
        if m.moe is not None:
            e, q = m.moe, p + "mlp."
            for j in range(e.experts):
                S.update({f"{q}e{j}.gate": lin(e.ff, W), f"{q}e{j}.up": lin(e.ff, W), f"{q}e{j}.down": lin(W, e.ff)})
            S[q + "router"], S[q + "correction"] = lin(e.experts + e.identity, W), vec(e.experts + e.identity, 0.0, 0.02)
            if e.shared_ff:
                S.update({q + "shared.gate": lin(e.shared_ff, W), q + "shared.up": lin(e.shared_ff, W), q + "shared.down": lin(W, e.shared_ff)})
    return S


class FusanexModel(HybridLM):
    """The text-only plugin of `hybrid_lm.HybridLM` with this design's config reader and weight packer."""

    default_name = "fusanex"
    config_from_dict = staticmethod(config_from_dict)
    pack_weights = staticmethod(pack_weights)
