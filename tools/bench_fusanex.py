"""Prefill and decode throughput of the Fusanex design (random weights) at layer sizes of a real model, beside the framework's
closest existing model, Sirodra, on the same engine at the same width and number of layers.  bf16, one GPU; both are driven
directly (plan upload + one native step).

    python tools/bench_fusanex.py [--sizes 1024,2048] [--prompt 512,2048] [--batch 1,8] [--steps 30] [--warmup 5]

Fusanex layers per block of three: a parallel mixer (attention: heads = width/128 of 128 dims, 4 query heads per K/V head;
matrix state: width/64 heads of 64 dims, decay bottleneck 64) and two gated linear recurrent units (width channels in blocks of
128, 4 taps); every layer has a routed feed-forward of 8 experts (+ 2 identity outputs), 2 per token, expert width = width,
and a shared expert of width `width` (9 width^2 active feed-forward parameters per token; Sirodra's dense one has 8 width^2 in
one layer of three).  Prints one JSON object.
"""
import argparse
import json
import os
import sys

sys.path.insert(0, os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
from tools.bench_sirodra import bench_hybrid, bench_hybrid_cfg


def fusanex_cfg(width, blocks, vocab, experts=8, top=2):
    from vox_serve_amd.engine_hybrid import HybridCfg, MixerCfg, MoECfg
    h = width // 128

    def moe():
        return MoECfg(experts=experts, identity=2, top=top, ff=width, limit=7.0, shared_ff=width, shared_limit=7.0)
    layers = []
    for _ in range(blocks):
        right = MixerCfg("shift_decay", width // 64, 64, 64, out_scale=1.0)
        layers += [MixerCfg("causal_attention", h, 128, 128, kv_heads=max(1, h // 4), scale=128 ** -0.5, q_temp_coef=0.1, q_temp_every=512,
                            v_unit_rms=True, block="parallel", side=right, moe=moe()),
                   MixerCfg("rglru", width // 128, 128, 128, conv_taps=4, block="parallel", moe=moe()),
                   MixerCfg("rglru", width // 128, 128, 128, conv_taps=4, block="parallel", moe=moe())]
    return HybridCfg(width, vocab, 1e-5, layers, None, norm_kind="rms_groups", norm_groups=4, embed_scale=1.0)


def step_bytes(cfg, lora):
    """bf16 weight bytes a one-row decode step streams: all mixers, the chosen experts, the shared expert, router (fp32), head."""
    W = cfg.width
    n = cfg.vocab * W
    for m in cfg.layers:
        n += m.n_in * W + W * m.heads * m.vdim
        if m.kind == "rglru":
            n += 2 * m.heads * m.dim * m.dim
        if m.side is not None:
            n += (4 * m.side.heads * m.side.dim + lora) * W + m.side.heads * m.side.dim * lora + W * m.side.heads * m.side.dim
        e = m.moe
        n += 3 * e.top * e.ff * W + 3 * e.shared_ff * W + 2 * (e.experts + e.identity) * W
    return 2 * n


def run(sizes=(1024, 2048), prompts=(512, 2048), batches=(1, 8), blocks=4, vocab=32000, ctx=1024, steps=30, warmup=5, device="cuda:0", only=None):
    from vox_serve_amd.model.fusanex import pack_weights, synth_weights
    res = {"workload": "Fusanex layer pattern (attention || matrix state | RG-LRU | RG-LRU, each with a routed feed-forward) x %d blocks vs the "
                       "Sirodra pattern of the same depth, bf16, random weights, decode context %d" % (blocks, ctx), "sizes": {}}
    for W in sizes:
        ent = {}
        if only in (None, "fusanex"):
            cfg = fusanex_cfg(W, blocks, vocab)
            packed = pack_weights(synth_weights(cfg, lora=64), cfg)
            ent["fusanex"] = bench_hybrid_cfg(cfg, packed, step_bytes(cfg, 64), prompts, batches, ctx, steps, warmup, device)
        if only in (None, "sirodra"):
            ent["sirodra"] = bench_hybrid(W, blocks, vocab, prompts, batches, ctx, steps, warmup, device)
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
    ap.add_argument("--only", default=None, choices=[None, "fusanex", "sirodra"])
    a = ap.parse_args()
    ints = lambda s: tuple(int(x) for x in s.split(","))
    print(json.dumps(run(ints(a.sizes), ints(a.prompt), ints(a.batch), a.blocks, steps=a.steps, warmup=a.warmup, only=a.only)))
