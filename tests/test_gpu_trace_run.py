"""bin/trace_run as a user runs it: a checkpoint folder, steps on standard input, logits files out.  A small Fusanex checkpoint made
here, a schedule of four requests in mixed steps (portions beside single tokens, wanted places, requests that end and whose pages and
slot the next one takes), both dtypes, against the float64 oracle."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from oracle import fusanex_ref as FR
from tests import fusanex_util as F
from tests import hybrid_util as U

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module", autouse=True)
def _gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")


@pytest.mark.parametrize("dtype,bar", [("float32", 2e-4), ("bfloat16", 4e-2)])
def test_trace_replay(tmp_path, dtype, bar):
    from safetensors.torch import save_file
    layers = [F.rglru(width=48, blocks=3, conv=3, mlp=F.moe()), F.parallel(heads=4, kv_heads=2, dim=16, vdim=8, every=11, mlp=F.moe(experts=3, identity=1, top=2))]
    cfg = F.config(layers, width=32, vocab=50, groups=4)
    S = F.random_checkpoint(cfg, seed=81)
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in S.items()}, str(model / "model.safetensors"))
    g = torch.Generator().manual_seed(82)
    seqs = {k: torch.randint(0, 50, (n,), generator=g).tolist() for k, n in (("a", 100), ("b", 70), ("c", 3), ("d", 90), ("e", 64))}
    want = {k: FR.forward(cfg, S, v) for k, v in seqs.items()}
    # at most 4 live requests and 5 pages of 64 tokens: e starts only after b and c have ended and takes their pages and a used slot
    plan = [[("a", 60), ("c", 1)], [("a", 1), ("b", 30), ("c", 2)], [("a", 1), ("b", 40), ("d", 2)], [("a", 38), ("d", 1), ("e", 63)],
            [("d", 87), ("e", 1)]]
    at = {k: 0 for k in seqs}
    lines, asked = [], []
    for n, step in enumerate(plan):
        entries, end, rows = [], [], []
        for k, cnt in step:
            lo, hi = at[k], at[k] + cnt
            wanted = sorted({0, cnt - 1, cnt // 2})
            entries.append({"id": k, "tokens": seqs[k][lo:hi], "want": wanted})
            rows += [(k, lo + w) for w in wanted]
            at[k] = hi
            if hi == len(seqs[k]):
                end.append(k)
        lines.append(json.dumps({"step": n, "entries": entries, "end": end}))
        asked.append(rows)
    lines.append(json.dumps({"step": len(plan), "entries": [], "end": []}))        # a step in which nothing runs
    assert all(at[k] == len(seqs[k]) for k in seqs)
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model), "--dtype", dtype, "--out", str(out),
                        "--max-tokens", str(5 * 64)], input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert p.returncode == 0, p.stderr[-2000:]
    done = [ln for ln in p.stdout.splitlines() if ln.startswith("done ")]
    assert done == [f"done {n}" for n in range(len(plan) + 1)]
    assert not (out / f"{len(plan)}.f32").exists()
    worst = 0.0
    for n, rows in enumerate(asked):
        got = torch.from_numpy(np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), 50).copy())
        ref = torch.stack([want[k][i] for k, i in rows])
        worst = max(worst, U.rel_err(got, ref))
    assert worst < bar, worst
