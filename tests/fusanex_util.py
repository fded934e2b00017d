"""Small Fusanex configurations and random checkpoints for the tests (the checkpoint's config.json layout and tensor names)."""
import math

import torch


def moe(experts=5, identity=1, top=2, ff=12, limit=1.5, shared=(10, 0.8)):
    m = {"kind": "moe", "router": {"experts": experts, "identity": identity, "top": top}, "expert": {"ff": ff, "limit": limit}}
    if shared:
        m["shared"] = {"ff": shared[0], "limit": shared[1]}
    return m


def rglru(width=24, blocks=3, conv=3, mlp=None):
    return {"type": "rglru", "mixer": {"width": width, "blocks": blocks, "conv": conv}, "mlp": mlp}


def parallel(heads=4, kv_heads=2, dim=8, vdim=12, scale=None, coef=0.4, every=5, rheads=2, rdim=8, left_scale=1.1, right_scale=0.7, mlp=None,
             q_temp=True):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if q_temp:
        left["q_temp"] = {"coef": coef, "every": every}
    return {"type": "parallel", "mixer": {"left": left, "right": {"heads": rheads, "dim": rdim}, "left_scale": left_scale,
                                          "right_scale": right_scale}, "mlp": mlp}


def config(layers, width=24, vocab=40, groups=2, eps=1e-5, embed_scale=3.0):
    return {"architecture": "Fusanex", "vocab": vocab, "width": width, "embedding": {"scale": embed_scale},
            "norm": {"eps": eps, "groups": groups}, "layers": layers}


def random_checkpoint(cfg, seed=0, gain=1.0, lora=6, identity_bias=0.0):
    """bf16 tensors under the checkpoint's names.  gain > 1 sharpens every projection; identity_bias is added to the choice
    correction of the identity outputs (so that they are chosen often)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * (s * gain / math.sqrt(shape[-1]))).to(torch.bfloat16)

    def vec(n, mean=0.0, std=0.2):
        return (mean + std * torch.randn(n, generator=g)).to(torch.bfloat16)
    S = {"embed": (torch.randn(cfg["vocab"], W, generator=g) * 0.5).to(torch.bfloat16), "head": mat(cfg["vocab"], W), "final.norm": vec(W, 1.0)}
    for i, L in enumerate(cfg["layers"]):
        m, p = L["mixer"], f"l{i}."
        S[p + "norm1"] = vec(W, 1.0)
        q = p + "mix."
        if L["type"] == "rglru":
            C, B = m["width"], m["blocks"]
            bs = C // B
            S.update({q + "y": mat(C, W), q + "y.b": vec(C), q + "x": mat(C, W), q + "x.b": vec(C), q + "conv": mat(C, m["conv"], s=1.5),
                      q + "conv.b": vec(C), q + "ra": mat(B, bs, bs, s=2.0), q + "ra.b": vec(C, 0.0, 1.0).view(B, bs), q + "ri": mat(B, bs, bs, s=2.0),
                      q + "ri.b": vec(C, 0.0, 1.0).view(B, bs), q + "lam": vec(C, -1.5, 1.5), q + "o": mat(W, C)})
        else:
            a, r = m["left"], m["right"]
            H, G, d, e, HD = a["heads"], a["kv_heads"], a["dim"], a["vdim"], r["heads"] * r["dim"]
            S.update({q + "left.q": mat(H * d, W), q + "left.k": mat(G * d, W), q + "left.v": mat(G * e, W), q + "left.q.norm": vec(d, 1.0, 0.3),
                      q + "left.k.norm": vec(d, 1.0, 0.3), q + "left.o": mat(W, H * e)})
            S.update({q + "right.mu." + n: torch.rand(W, generator=g).to(torch.bfloat16) for n in "rkvgw"})
            S.update({q + "right.r": mat(HD, W), q + "right.k": mat(HD, W), q + "right.v": mat(HD, W), q + "right.g": mat(HD, W, s=2.0),
                      q + "right.w1": mat(lora, W, s=2.0), q + "right.w2": mat(HD, lora, s=2.0), q + "right.w0": vec(HD, -1.0, 1.0),
                      q + "right.u": vec(HD, 0.3, 0.5).view(r["heads"], r["dim"]), q + "right.norm": vec(HD, 1.0), q + "right.o": mat(W, HD)})
        if L["mlp"]:
            S[p + "norm2"] = vec(W, 1.0)
            r, f, q = L["mlp"]["router"], L["mlp"]["expert"]["ff"], p + "mlp."
            nE = r["experts"] + r["identity"]
            for j in range(r["experts"]):
                S.update({f"{q}e{j}.gate": mat(f, W, s=2.0), f"{q}e{j}.up": mat(f, W, s=2.0), f"{q}e{j}.down": mat(W, f)})
            S[q + "router"] = mat(nE, W, s=2.0)
            corr = 0.05 * torch.randn(nE, generator=g)
            if r["identity"]:
                corr[-r["identity"]:] += identity_bias
            S[q + "correction"] = corr.to(torch.bfloat16)
            sh = L["mlp"].get("shared")
            if sh:
                S.update({q + "shared.gate": mat(sh["ff"], W, s=2.0), q + "shared.up": mat(sh["ff"], W, s=2.0), q + "shared.down": mat(W, sh["ff"])})
    return S
