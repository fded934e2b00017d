"""Prefill and decode throughput of the hybrid-mixer engine (Sirodra design, random weights) at layer sizes of a real model,
beside the single-stack LM engine (llama-style: grouped-query attention + SwiGLU) at the same width, depth and parameter
count per layer.  Both engines are driven directly (plan upload + one native step), bf16, one GPU.

    python tools/bench_sirodra.py [--sizes 1024,2048] [--prompt 512,2048] [--batch 1,8] [--steps 30] [--warmup 5]

Sirodra layers per block of three: HGRN2 (heads = width/128, 128 x 128 state per head), pooled-window attention (heads =
width/128, 4 query heads per K/V head, window 1024, blocks of 16, 64 rotated dims) with a dense feed-forward of 4 x width,
mLSTM (heads = width/128, 64 key dims, 128 value dims).  The comparison stack has the same number of layers, each with
attention + a SwiGLU of 8/3 x width (the same 8 width^2 feed-forward parameters).  Prints one JSON object.
"""
import argparse
import json
import os
import sys
import time

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
import numpy as np
import torch


def sirodra_cfg(width, blocks, vocab):
    from vox_serve_amd.engine_hybrid import HybridCfg, MixerCfg
    h = width // 128
    layers = []
    for _ in range(blocks):
        layers += [MixerCfg("hgrn2", h, 128, 128),
                   MixerCfg("attention", h, 128, 128, kv_heads=max(1, h // 4), window=1024, pool=16, rot_dims=64, rot_base=10000.0,
                            rot_factor=1.0, scale=128 ** -0.5, ff=4 * width),
                   MixerCfg("mlstm", h, 64, 128, gate_cap=15.0)]
    return HybridCfg(width, vocab, 1e-5, layers, None)


def layer_bytes(cfg):
    """bf16 weight bytes one decode step streams (all layers + head)."""
    n = cfg.vocab * cfg.width
    for m in cfg.layers:
        n += m.n_in * cfg.width + cfg.width * m.heads * m.vdim + 2 * m.ff * cfg.width
    return 2 * n


def time_steps(fn, steps, warmup):
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / steps


def bench_hybrid(width, blocks, vocab, prompts, batches, ctx, steps, warmup, dev):
    from vox_serve_amd.model.sirodra import pack_weights, synth_weights
    cfg = sirodra_cfg(width, blocks, vocab)
    return bench_hybrid_cfg(cfg, pack_weights(synth_weights(cfg), cfg), layer_bytes(cfg), prompts, batches, ctx, steps, warmup, dev)


def bench_hybrid_cfg(cfg, packed, wbytes, prompts, batches, ctx, steps, warmup, dev):
    """Any design of the hybrid engine: `packed` = the engine's weight layout, wbytes = weight bytes a one-row decode step streams."""
    from vox_serve_amd.engine_hybrid import HybridEngine
    vocab = cfg.vocab
    ps = 128
    maxp, maxb = max(prompts), max(batches)
    pages = max((maxp + ps - 1) // ps, maxb * ((ctx + 64 + ps - 1) // ps)) + 1
    eng = HybridEngine(cfg, packed, dtype=torch.bfloat16, max_batch=maxb, page_size=ps, max_pages=pages,
                       max_seq_len=max(maxp, ctx + 64) + ps, max_prefill_rows=maxp, state_slots=maxb, device=dev)
    out = {"weight_bytes_per_step": wbytes, "prefill": {}, "decode": {}}
    sc = eng.sampling_cfg(greedy=True)
    rng = np.random.default_rng(0)
    for n in prompts:
        eng.row_ids[:n, 0] = torch.from_numpy(rng.integers(0, vocab, n).astype(np.int32)).to(dev)
        npg = (n + ps - 1) // ps
        eng.upload_plan(pos=np.arange(n), kvlen=np.arange(1, n + 1), page=np.arange(n) // ps, slot=np.arange(n) % ps, q_req=np.zeros(n),
                        last_rows=[n - 1], indptr=[0, npg], indices=np.arange(npg), req_rows=[0, n], state=[0])
        dt = time_steps(lambda: eng.step(n, 1, 1, sc, feedback=False, max_kvlen=n), max(3, steps // 5), 2)
        out["prefill"][str(n)] = {"ms": dt * 1e3, "tokens_per_s": n / dt}
    for B in batches:
        # every request has `ctx` tokens behind it (cache contents are whatever the pages hold: timing only)
        per = (ctx + 64 + ps - 1) // ps
        kv = [ctx] * B

        def step():
            for b in range(B):
                kv[b] += 1
            npg = [(k + ps - 1) // ps for k in kv]
            eng.upload_plan(pos=[k - 1 for k in kv], kvlen=kv, page=[b * per + npg[b] - 1 for b in range(B)], slot=[(k - 1) % ps for k in kv],
                            q_req=np.arange(B), last_rows=np.arange(B), indptr=np.concatenate([[0], np.cumsum(npg)]),
                            indices=sum([[b * per + j for j in range(npg[b])] for b in range(B)], []), req_rows=np.arange(B + 1),
                            state=np.arange(B))
            eng.frame(B, max(kv), sc, feedback=True)
        dt = time_steps(step, steps, warmup)
        kv[:] = [ctx] * B
        out["decode"][str(B)] = {"ms": dt * 1e3, "tokens_per_s": B / dt, "weight_GBps": wbytes / dt / 1e9}
    eng.close()
    return out


def bench_stack(width, n_layers, vocab, prompts, batches, ctx, steps, warmup, dev):
    from vox_serve_amd.engine import LMCfg, LMEngine, StackCfg
    h = width // 128
    ffn = (8 * width // 3 + 255) // 256 * 256
    st = StackCfg(width, n_layers, h, max(1, h // 4), 128, ffn, eps=1e-5, rope_theta=1e4, qk_norm=False, qkv_bias=False)
    g = torch.Generator().manual_seed(0)
    w = lambda o, i: (torch.randn(o, i, generator=g) * (i ** -0.5)).to(torch.bfloat16)
    ones = lambda n: torch.ones(n, dtype=torch.bfloat16)
    qkv = (h + 2 * st.kv_heads) * 128
    layers = [dict(wqkv=w(qkv, width), wo=w(width, h * 128), wgate=w(ffn, width), wup=w(ffn, width), wdown=w(width, ffn), ln1=ones(width),
                   ln2=ones(width)) for _ in range(n_layers)]
    ps = 128
    maxp, maxb = max(prompts), max(batches)
    pages = max((maxp + ps - 1) // ps, maxb * ((ctx + 64 + ps - 1) // ps)) + 1
    eng = LMEngine(LMCfg(st, vocab, vocab, 1, 0, 8192), layers, ones(width), w(vocab, width), w(vocab, width), None, max_batch=maxb, page_size=ps,
                   max_pages=pages, max_seq_len=max(maxp, ctx + 64) + ps, max_prefill_rows=maxp, device=dev)
    wbytes = 2 * (vocab * width + n_layers * (qkv * width + width * h * 128 + 3 * ffn * width))
    out = {"weight_bytes_per_step": wbytes, "prefill": {}, "decode": {}}
    sc = eng.sampling_cfg(greedy=True)
    rng = np.random.default_rng(0)
    for n in prompts:
        eng.row_ids[:n, 0] = torch.from_numpy(rng.integers(0, vocab, n).astype(np.int32)).to(dev)
        npg = (n + ps - 1) // ps
        eng.upload_plan(pos=np.arange(n), kvlen=np.arange(1, n + 1), page=np.arange(n) // ps, slot=np.arange(n) % ps, q_req=np.zeros(n),
                        last_rows=[n - 1], indptr=[0, npg], indices=np.arange(npg))
        dt = time_steps(lambda: eng.prefill(n, 1, n, sc, feedback=False, use_graph=False), max(3, steps // 5), 2)
        out["prefill"][str(n)] = {"ms": dt * 1e3, "tokens_per_s": n / dt}
    for B in batches:
        per = (ctx + 64 + ps - 1) // ps
        kv = [ctx] * B

        def step():
            for b in range(B):
                kv[b] += 1
            npg = [(k + ps - 1) // ps for k in kv]
            eng.upload_plan(pos=[k - 1 for k in kv], kvlen=kv, page=[b * per + npg[b] - 1 for b in range(B)], slot=[(k - 1) % ps for k in kv],
                            indptr=np.concatenate([[0], np.cumsum(npg)]),
                            indices=sum([[b * per + j for j in range(npg[b])] for b in range(B)], []))
            eng.frame(B, max(kv), sc, feedback=True)
        dt = time_steps(step, steps, warmup)
        kv[:] = [ctx] * B
        out["decode"][str(B)] = {"ms": dt * 1e3, "tokens_per_s": B / dt, "weight_GBps": wbytes / dt / 1e9}
    eng.close()
    return out


def run(sizes=(1024, 2048), prompts=(512, 2048), batches=(1, 8), blocks=4, vocab=32000, ctx=1024, steps=30, warmup=5, device="cuda:0",
        only=None):
    res = {"workload": "Sirodra layer pattern (HGRN2 | pooled-window attention + dense FF | mLSTM) x %d blocks vs a llama-style stack of the "
                       "same depth, bf16, random weights, decode context %d" % (blocks, ctx), "sizes": {}}
    for W in sizes:
        ent = {}
        if only in (None, "sirodra"):
            ent["sirodra"] = bench_hybrid(W, blocks, vocab, prompts, batches, ctx, steps, warmup, device)
        if only in (None, "stack"):
            ent["stack"] = bench_stack(W, 3 * blocks, vocab, prompts, batches, ctx, steps, warmup, device)
        res["sizes"][str(W)] = ent
    return res


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--sizes", default="1024,2048")
    ap.add_argument("--prompt", default="512,2048")
    ap.add_argument("--batch", default="1,8")
    ap.add_argument("--blocks", type=int, default=4)
    ap.add_argument("--steps", type=int, default=30)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--only", default=None, choices=[None, "sirodra", "stack"])
    a = ap.parse_args()
    ints = lambda s: tuple(int(x) for x in s.split(","))
    print(json.dumps(run(ints(a.sizes), ints(a.prompt), ints(a.batch), a.blocks, steps=a.steps, warmup=a.warmup, only=a.only)))
