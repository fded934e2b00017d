"""Slow float64 restatement of the hybrid-mixer decoder (Sirodra), one function per mechanism, whole sequences only.

Test infrastructure: nothing under vox_serve_amd/ imports this, and this imports nothing from there.  The model is a dict
config (the checkpoint's config.json layout) and a dict of tensors under the checkpoint's names.
Notation: T tokens, h [T, width] the normed layer input, heads H, key width d, value width e.
"""
import math

import torch

F64 = torch.float64


def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    dev = x - mu
    return dev / torch.sqrt((dev * dev).mean(-1, keepdim=True) + eps) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def hgrn2_mixer(P, h, m, eps):
    """S_t = diag(f_t) S_{t-1} + (1 - f_t) (x) v_t ; y_t = S_t^T q_t ; f bounded below by `lower`."""
    T, H, d, e = h.shape[0], m["heads"], m["dim"], m["vdim"]
    q = h @ P["q"].T
    q = (q * torch.sigmoid(q)).view(T, H, d)
    v = (h @ P["v"].T).view(T, H, e)
    low = P["lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ P["f"].T + P["f.b"])).view(T, H, d)
    S = torch.zeros(H, d, e, dtype=F64)
    y = []
    for t in range(T):
        S = f[t].unsqueeze(-1) * S + (1.0 - f[t]).unsqueeze(-1) * v[t].unsqueeze(1)
        y.append((S * q[t].unsqueeze(-1)).sum(1))
    y = unit_rms(torch.stack(y), eps) * P["norm"]
    return y.reshape(T, H * e) @ P["o"].T


def mlstm_mixer(P, h, m, eps):
    """Matrix-memory LSTM with exponential gating, kept finite by a running maximum of the log gates (initially 0)."""
    T, H, d, e, cap = h.shape[0], m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ P["q"].T).view(T, H, d) / math.sqrt(d)
    k = (h @ P["k"].T).view(T, H, d)
    v = (h @ P["v"].T).view(T, H, e)
    log_i = cap * torch.tanh((h @ P["i"].T + P["i.b"]) / cap)
    log_f = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ P["f"].T + P["f.b"]) / cap))
    C = torch.zeros(H, d, e, dtype=F64)
    n = torch.zeros(H, d, dtype=F64)
    mx = torch.zeros(H, dtype=F64)
    y = []
    for t in range(T):
        new = torch.maximum(log_f[t] + mx, log_i[t])
        keep, write = torch.exp(log_f[t] + mx - new), torch.exp(log_i[t] - new)
        C = keep[:, None, None] * C + write[:, None, None] * (k[t].unsqueeze(-1) * v[t].unsqueeze(1))
        n = keep[:, None] * n + write[:, None] * k[t]
        mx = new
        top = (C * q[t].unsqueeze(-1)).sum(1)
        bottom = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        y.append(top / bottom[:, None])
    y = unit_rms(torch.stack(y), eps).reshape(T, H * e) * P["norm"] * torch.sigmoid(h @ P["g"].T)
    return y @ P["o"].T


def rotary_interleaved(x, n_rot, base, factor):
    """x [T, heads, d]: dims (2i, 2i+1), i < n_rot/2, turn by angle t * base^(-2i/n_rot) / factor; the rest stays."""
    T = x.shape[0]
    out = x.clone()
    for i in range(n_rot // 2):
        ang = torch.arange(T, dtype=F64) * (base ** (-2.0 * i / n_rot) / factor)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        a, b = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = a * c - b * s
        out[..., 2 * i + 1] = b * c + a * s
    return out


def visible_keys(t, window, pool):
    """(pooled block indices, token indices) position t attends to: the last `window` tokens, and every block of `pool`
    consecutive tokens that ends at or before t - window."""
    toks = [j for j in range(t + 1) if t - j < window]
    blocks = [b for b in range((t + 1) // pool + 1) if b * pool + pool - 1 <= t - window]
    return blocks, toks


def pooled_window_attention(P, h, m, eps, cache_round=None):
    """cache_round: what the K / V cache does to a stored value (e.g. bf16 rounding); pooled entries average the stored values."""
    T, H, G, d, e = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m.get("rot") or {}
    n_rot, base, factor = rot.get("dims", 0), rot.get("base", 10000.0), (rot.get("scaling") or {}).get("factor", 1.0)
    q = (h @ P["q"].T + P["q.b"]).view(T, H, d)
    k = (h @ P["k"].T + P["k.b"]).view(T, G, d)
    v = (h @ P["v"].T + P["v.b"]).view(T, G, e)
    q = unit_rms(rotary_interleaved(q, n_rot, base, factor), eps)
    k = unit_rms(rotary_interleaved(k, n_rot, base, factor), eps)
    if cache_round is not None:
        k, v = cache_round(k), cache_round(v)
    window, pool = m["mask"]["size"], m["mask"]["pool"]
    gate = torch.sigmoid(h @ P["g"].T)
    y = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        blocks, toks = visible_keys(t, window, pool)
        for hh in range(H):
            g = hh // (H // G)
            K = [k[b * pool:(b + 1) * pool, g].mean(0) for b in blocks] + [k[j, g] for j in toks]
            V = [v[b * pool:(b + 1) * pool, g].mean(0) for b in blocks] + [v[j, g] for j in toks]
            K, V = torch.stack(K), torch.stack(V)
            w = torch.softmax((K @ q[t, hh]) * m["scale"], 0)
            y[t, hh] = (w @ V) * gate[t, hh]
    return y.reshape(T, H * e) @ P["o"].T


def dense_ff(P, h):
    z = h @ P["up"].T
    return (0.5 * z * (1.0 + torch.erf(z / math.sqrt(2.0)))) @ P["down"].T


MIXERS = {"hgrn2": hgrn2_mixer, "mlstm": mlstm_mixer, "attention": pooled_window_attention}


def run_order(cfg):
    n, lp = len(cfg["layers"]), cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    order = [(i, False) for i in range(lp["start"])]
    for _ in range(lp["times"]):
        order += [(i, i == lp["start"]) for i in range(lp["start"], lp["stop"])]
    return order + [(i, False) for i in range(lp["stop"], n)]


def forward(cfg, S, tokens, residuals=None, cache_round=None):
    """tokens: list of ids -> logits [T, vocab] (float64).  S: checkpoint tensors (any float dtype)."""
    S = {k: v.to(F64) for k, v in S.items()}
    eps = cfg["norm"]["eps"]
    x0 = S["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    for i, reenter in run_order(cfg):
        if reenter:
            x = torch.cat([x, x0], -1) @ S["loop.in"].T
        L = cfg["layers"][i]
        P = {k[len(f"l{i}.mix."):]: v for k, v in S.items() if k.startswith(f"l{i}.mix.")}
        h = layer_norm(x, S[f"l{i}.norm1"], eps)
        if L["type"] == "attention":
            x = x + pooled_window_attention(P, h, L["mixer"], eps, cache_round)
        else:
            x = x + MIXERS[L["type"]](P, h, L["mixer"], eps)
        if L.get("mlp") is not None:
            F = {"up": S[f"l{i}.mlp.up"], "down": S[f"l{i}.mlp.down"]}
            x = x + dense_ff(F, layer_norm(x, S[f"l{i}.norm2"], eps))
        if residuals is not None:
            residuals.append(x.clone())
    return layer_norm(x, S["final.norm"], eps) @ S["head"].T
