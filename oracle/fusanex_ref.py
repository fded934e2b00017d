"""Slow float64 restatement of the Fusanex decoder, one function per mechanism, whole sequences only.

Test infrastructure: nothing under vox_serve_amd/ imports this, and this imports nothing from there.  The model is a dict
config (the checkpoint's config.json layout) and a dict of tensors under the checkpoint's names.
Notation: T tokens, n [T, width] a normed layer input, heads H, key / value heads G, key width d, value width e.

The design: x_0 = embedding * scale; every layer adds mixer(norm1 x) + moe(norm2 x) to x, both branches reading the same x;
norms are RMS norms taken over `groups` equal slices of the vector; the mixer is either a real-gated linear recurrent unit
behind a short causal convolution, or the scaled sum of a softmax attention (no rotation; normed q / k / v and a query
temperature that grows with the logarithm of the position) and a matrix-state recurrence with token shift and a
data-dependent decay per key channel.
"""
import math

import torch

F64 = torch.float64


def grouped_rms_norm(x, w, groups, eps):
    """Each of `groups` consecutive slices of the last axis is divided by its own sqrt(mean square + eps); then times w."""
    T, W = x.shape
    p = x.view(T, groups, W // groups)
    return (p / torch.sqrt((p * p).mean(-1, keepdim=True) + eps)).reshape(T, W) * w


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def causal_conv(x, taps, bias):
    """x [T, C], taps [C, K] (last column weighs the current token), zeros before the sequence."""
    T, C = x.shape
    K = taps.shape[1]
    pad = torch.cat([torch.zeros(K - 1, C, dtype=x.dtype), x], 0)
    out = bias.expand(T, C).clone()
    for j in range(K):
        out = out + pad[j:j + T] * taps[:, j]
    return out


def rglru_mixer(P, n, m):
    """Gated branch y; recurrent branch u = conv(Wx n); per block of channels two sigmoid gates from block-diagonal matrices;
    a = exp(-8 r softplus(lam));  S_t = a S_{t-1} + sqrt(1 - a^2) (i u_t);  out = Wo (S y)."""
    T = n.shape[0]
    C, B = m["width"], m["blocks"]
    y = gelu_tanh(n @ P["y"].T + P["y.b"])
    u = causal_conv(n @ P["x"].T + P["x.b"], P["conv"], P["conv.b"])
    ub = u.view(T, B, C // B)
    r = torch.sigmoid(torch.einsum("boi,tbi->tbo", P["ra"], ub) + P["ra.b"]).reshape(T, C)
    i = torch.sigmoid(torch.einsum("boi,tbi->tbo", P["ri"], ub) + P["ri.b"]).reshape(T, C)
    a = torch.exp(-8.0 * r * torch.nn.functional.softplus(P["lam"]))
    S = torch.zeros(C, dtype=F64)
    out = []
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] * a[t]) * (i[t] * u[t])
        out.append(S * y[t])
    return torch.stack(out) @ P["o"].T


def softmax_attention(P, n, m, eps, cache_round=None):
    """Causal grouped-query attention without rotation.  q, k: RMS norm per head with a shared weight; q also times
    1 + coef * ln(floor((p + 1) / every) + 1) at position p; v: unit RMS per head (that is what the cache keeps)."""
    T, H, G, d, e = n.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((n @ P["q"].T).view(T, H, d), eps) * P["q.norm"]
    k = unit_rms((n @ P["k"].T).view(T, G, d), eps) * P["k.norm"]
    v = unit_rms((n @ P["v"].T).view(T, G, e), eps)
    qt = m.get("q_temp")
    if qt:
        pos = torch.arange(T, dtype=F64)
        q = q * (1.0 + qt["coef"] * torch.log(torch.floor((pos + 1.0) / qt["every"]) + 1.0))[:, None, None]
    if cache_round is not None:
        k, v = cache_round(k), cache_round(v)
    out = torch.zeros(T, H, e, dtype=F64)
    for t in range(T):
        for hh in range(H):
            g = hh // (H // G)
            w = torch.softmax((k[:t + 1, g] @ q[t, hh]) * m["scale"], 0)
            out[t, hh] = w @ v[:t + 1, g]
    return out.reshape(T, H * e) @ P["o"].T


def shifted_state_mixer(P, n, m, eps):
    """Token shift: every projection reads n_t + (n_{t-1} - n_t) mu (n_{-1} = 0).  Decay w = exp(-exp(W2 tanh(W1 .) + w0)) per
    head and key channel.  o_t = (S + diag(u) k v^T)^T r;  S <- diag(w) S + k v^T.  Then unit RMS per head, a weight, a silu
    gate and the output projection."""
    T, H, d = n.shape[0], m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, n.shape[1], dtype=F64), n[:-1]], 0)

    def mix(s):
        return n + (prev - n) * P["mu." + s]
    r = (mix("r") @ P["r"].T).view(T, H, d)
    k = (mix("k") @ P["k"].T).view(T, H, d)
    v = (mix("v") @ P["v"].T).view(T, H, d)
    z = mix("g") @ P["g"].T
    gate = z * torch.sigmoid(z)
    w = torch.exp(-torch.exp(torch.tanh(mix("w") @ P["w1"].T) @ P["w2"].T + P["w0"])).view(T, H, d)
    S = torch.zeros(H, d, d, dtype=F64)
    out = []
    for t in range(T):
        kv = k[t].unsqueeze(-1) * v[t].unsqueeze(1)
        out.append(((S + P["u"].unsqueeze(-1) * kv) * r[t].unsqueeze(-1)).sum(1))
        S = w[t].unsqueeze(-1) * S + kv
    o = unit_rms(torch.stack(out), eps).reshape(T, H * d) * P["norm"] * gate
    return o @ P["o"].T


def parallel_mixer(P, n, m, eps, cache_round=None):
    left = {k[len("left."):]: v for k, v in P.items() if k.startswith("left.")}
    right = {k[len("right."):]: v for k, v in P.items() if k.startswith("right.")}
    return m["left_scale"] * softmax_attention(left, n, m["left"], eps, cache_round) + \
        m["right_scale"] * shifted_state_mixer(right, n, m["right"], eps)


def clamped_glu_expert(P, n, limit):
    g = torch.clamp(n @ P["gate"].T, max=limit)
    u = torch.clamp(n @ P["up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ P["down"].T


def route(P, n, r):
    """-> (chosen [T, top] expert indices, weights [T, top]).  Softmax over real and identity experts alike; the choice adds
    a per-expert correction to the scores, the weights do not."""
    s = torch.softmax(n @ P["router"].T, -1)
    chosen = torch.topk(s + P["correction"], r["top"], dim=-1).indices
    w = torch.gather(s, 1, chosen)
    return chosen, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(P, n, mlp):
    """Experts e < `experts` are clamped gated units; the last `identity` router outputs return their input.  A shared expert
    of the same form runs for every token."""
    r = mlp["router"]
    E = r["experts"]
    chosen, w = route(P, n, r)
    out = torch.zeros_like(n)
    for t in range(n.shape[0]):
        for c, wt in zip(chosen[t].tolist(), w[t]):
            if c >= E:
                out[t] += wt * n[t]
            else:
                Pe = {k[len(f"e{c}."):]: v for k, v in P.items() if k.startswith(f"e{c}.")}
                out[t] += wt * clamped_glu_expert(Pe, n[t:t + 1], mlp["expert"]["limit"])[0]
    if mlp.get("shared"):
        Ps = {k[len("shared."):]: v for k, v in P.items() if k.startswith("shared.")}
        out = out + clamped_glu_expert(Ps, n, mlp["shared"]["limit"])
    return out


def forward(cfg, S, tokens, residuals=None, cache_round=None):
    """tokens: list of ids -> logits [T, vocab] (float64).  S: checkpoint tensors (any float dtype)."""
    S = {k: v.to(F64) for k, v in S.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = S["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, L in enumerate(cfg["layers"]):
        P = {k[len(f"l{i}.mix."):]: v for k, v in S.items() if k.startswith(f"l{i}.mix.")}
        n1 = grouped_rms_norm(x, S[f"l{i}.norm1"], groups, eps)
        if L["type"] == "rglru":
            add = rglru_mixer(P, n1, L["mixer"])
        elif L["type"] == "parallel":
            add = parallel_mixer(P, n1, L["mixer"], eps, cache_round)
        else:
            raise ValueError(L["type"])
        if L.get("mlp") is not None:
            F = {k[len(f"l{i}.mlp."):]: v for k, v in S.items() if k.startswith(f"l{i}.mlp.")}
            add = add + moe_ff(F, grouped_rms_norm(x, S[f"l{i}.norm2"], groups, eps), L["mlp"])
        x = x + add
        if residuals is not None:
            residuals.append(x.clone())
    return grouped_rms_norm(x, S["final.norm"], groups, eps) @ S["head"].T
