"""Sirodra: a decoder-only language model of mixed token mixers on the hybrid engine (`engine_hybrid.HybridEngine`).

A checkpoint is a folder with `config.json` and `model.safetensors`.  config.json:
  architecture "Sirodra"; vocab, width; norm.eps;
  layers[i] = {type: "hgrn2" | "attention" | "mlstm", mixer: {...sizes...}, mlp: null | {kind: "dense", ff}};
  loop = {start, stop, times} (optional): layers start..stop-1 run `times` times with the same weights; before the first
  layer of every pass x <- loop.in [x; x0], x0 being the embedding output.
Tensors (bf16, linear weights [out, in]): embed, head, final.norm, loop.in, and per layer l<i>.norm1, l<i>.norm2,
l<i>.mix.<name>[.b], l<i>.mlp.up / .down.

Every layer is pre-norm with a weight-only layer norm:  x += mixer(norm1 x);  x += down(gelu(up(norm2 x))) when it has a
feed-forward.  The mixers:
  hgrn2      q = silu(Wq h), v = Wv h, forget f = lower + (1 - lower) * sigmoid(Wf h + b): S <- diag(f) S + (1 - f) v^T, o = S^T q,
             per-head RMS norm with a shared weight, output projection.
  mlstm      q = Wq h / sqrt(dim), k, v; log gates i = cap*tanh(./cap), f = logsigmoid(cap*tanh(./cap)); stabilised by a running
             maximum that starts at 0; o = S^T q / (max(|n.q|, exp(-m)) + 1e-6); unit RMS per head, weight, sigmoid gate, projection.
  attention  grouped-query, biased q/k/v, interleaved rotary on the first rot.dims dims with linearly scaled positions, unit RMS
             of q and k per head, a window of mask.size tokens plus one mean key/value per block of mask.pool tokens that lies
             wholly before the window, one softmax over both, a sigmoid gate per head, projection.
The plugin fuses each mixer's input projections into one matrix (the engine's row order) at load time; forward, sampling and
the next-step feedback are one native call per step.  There is no audio side: generated ids are the output.
"""
from typing import Dict

import torch

from ..engine_hybrid import HybridCfg, MixerCfg
from .hybrid_lm import HybridLM

ARCHITECTURE = "Sirodra"


def config_from_dict(d: dict) -> HybridCfg:
    if d.get("architecture") != ARCHITECTURE:
        raise ValueError(f"not a {ARCHITECTURE} config: architecture = {d.get('architecture')!r}")
    layers = []
    for i, l in enumerate(d["layers"]):
        t, m, mlp = l["type"], l["mixer"], l.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: feed-forward kind {mlp.get('kind')!r} is not part of this design")
        ff = int(mlp["ff"]) if mlp is not None else 0
        if t == "hgrn2":
            layers.append(MixerCfg("hgrn2", int(m["heads"]), int(m["dim"]), int(m["vdim"]), ff=ff))
        elif t == "mlstm":
            layers.append(MixerCfg("mlstm", int(m["heads"]), int(m["dim"]), int(m["vdim"]), gate_cap=float(m["gate_cap"]), ff=ff))
        elif t == "attention":
            rot = m.get("rot") or {}
            layers.append(MixerCfg("attention", int(m["heads"]), int(m["dim"]), int(m["vdim"]), kv_heads=int(m["kv_heads"]),
                                   window=int(m["mask"]["size"]), pool=int(m["mask"]["pool"]), rot_dims=int(rot.get("dims", 0)),
                                   rot_base=float(rot.get("base", 10000.0)),
                                   rot_factor=float((rot.get("scaling") or {}).get("factor", 1.0)), scale=float(m["scale"]), ff=ff))
        else:
            raise ValueError(f"layer {i}: unknown mixer type {t!r}")
    lp = d.get("loop")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else None
    return HybridCfg(int(d["width"]), int(d["vocab"]), float(d["norm"]["eps"]), layers, loop)


def pack_weights(S: Dict[str, torch.Tensor], cfg: HybridCfg) -> Dict:
    """Checkpoint tensors -> the engine's fused layout."""
    def cat_bias(p, names, sizes):
        if not any(p + n + ".b" in S for n in names):
            return None
        return torch.cat([S[p + n + ".b"].float() if p + n + ".b" in S else torch.zeros(k) for n, k in zip(names, sizes)])
    layers = []
    for i, m in enumerate(cfg.layers):
        p = f"l{i}.mix."
        names = {"hgrn2": ("q", "f", "v"), "attention": ("q", "k", "v", "g"), "mlstm": ("q", "k", "v", "g", "i", "f")}[m.kind]
        mats = [S[p + n] for n in names]
        lw = dict(norm1=S[f"l{i}.norm1"], norm2=S.get(f"l{i}.norm2"), w_in=torch.cat(mats, 0).contiguous(),
                  b_in=cat_bias(p, names, [t.shape[0] for t in mats]), w_out=S[p + "o"], lower=S.get(p + "lower"),
                  head_norm=S.get(p + "norm"), w_up=S.get(f"l{i}.mlp.up"), w_down=S.get(f"l{i}.mlp.down"))
        if m.ff and (lw["w_up"] is None or lw["norm2"] is None):
            raise KeyError(f"layer {i}: feed-forward tensors missing")
        layers.append(lw)
    return dict(embedding=S["embed"], head=S["head"], final_norm=S["final.norm"], loop_in=S.get("loop.in"), layers=layers)


def synth_weights(cfg: HybridCfg, seed: int = 0, scale: float = 1.0) -> Dict[str, torch.Tensor]:
    """Random checkpoint tensors (bf16, the checkpoint's names) for a config: benchmarks and tests."""
    g = torch.Generator().manual_seed(seed)
    W = cfg.width

    def lin(o, i):
        return (torch.randn(o, i, generator=g) * (scale / i ** 0.5)).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.1):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": (torch.randn(cfg.vocab, W, generator=g)).to(torch.bfloat16), "head": lin(cfg.vocab, W), "final.norm": vec(W, 1.0)}
    if cfg.loop:
        S["loop.in"] = lin(W, 2 * W)
    for i, m in enumerate(cfg.layers):
        p = f"l{i}."
        S[p + "norm1"] = vec(W, 1.0)
        h, d, v = m.heads, m.dim, m.vdim
        if m.kind == "hgrn2":
            S.update({p + "mix.q": lin(h * d, W), p + "mix.f": lin(h * d, W), p + "mix.f.b": vec(h * d, 1.0, 1.0),
                      p + "mix.lower": torch.rand(h * d, generator=g).mul(0.9).to(torch.bfloat16), p + "mix.v": lin(h * v, W),
                      p + "mix.norm": vec(v, 1.0), p + "mix.o": lin(W, h * v)})
        elif m.kind == "mlstm":
            S.update({p + "mix.q": lin(h * d, W), p + "mix.k": lin(h * d, W), p + "mix.v": lin(h * v, W), p + "mix.g": lin(h * v, W),
                      p + "mix.o": lin(W, h * v), p + "mix.norm": vec(h * v, 1.0), p + "mix.i": lin(h, W), p + "mix.i.b": vec(h, 0.0, 1.0),
                      p + "mix.f": lin(h, W), p + "mix.f.b": vec(h, 3.0, 1.0)})
        else:
            G = m.kv_heads
            S.update({p + "mix.q": lin(h * d, W), p + "mix.q.b": vec(h * d), p + "mix.k": lin(G * d, W), p + "mix.k.b": vec(G * d),
                      p + "mix.v": lin(G * v, W), p + "mix.v.b": vec(G * v), p + "mix.g": lin(h, W), p + "mix.o": lin(W, h * v)})
        if m.ff:
            S.update({p + "norm2": vec(W, 1.0), p + "mlp.up": lin(m.ff, W), p + "mlp.down": lin(W, m.ff)})
    return S


class SirodraModel(HybridLM):
    """The text-only plugin of `hybrid_lm.HybridLM` with this design's config reader and weight packer."""

    default_name = "sirodra"
    config_from_dict = staticmethod(config_from_dict)
    pack_weights = staticmethod(pack_weights)
