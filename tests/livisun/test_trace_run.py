"""bin/trace_run on a checkpoint folder written by the test: config.json picks the model class,
the steps run through the engine, the logits files match the oracle."""
import json
import os
import subprocess

import numpy as np
import torch
from safetensors.torch import save_file

from replisense_rfq_amd.models.config import LayeredConfig
from replisense_rfq_amd.models.weights import init_layered_weights

from . import oracle
from .common import TAPS4, tokens

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))


def test_trace_run_cli(tmp_path):
    cfg = TAPS4
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    full = init_layered_weights(LayeredConfig.from_json(cfg), "cpu", torch.float32, seed=3)["full"]
    save_file({k: v.to(torch.bfloat16).contiguous() for k, v in full.items()},
              str(model / "model.safetensors"))
    a, b = tokens(70, cfg["vocab"], 1), tokens(9, cfg["vocab"], 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:40], "want": [0, 39]},
                                {"id": "b", "tokens": b[:2], "want": []}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": a[40:41], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[2:], "want": [6]},
                                {"id": "a", "tokens": a[41:], "want": [28]}], "end": ["a", "b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": b, "want": [8]}], "end": ["a"]},   # name reused
    ]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", str(model), "--dtype",
                        "float32", "--out", str(out), "--max-tokens", "192", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.split("\n") if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    ra, rb = oracle.forward(cfg, full, a), oracle.forward(cfg, full, b)
    want = {0: [ra[0], ra[39]], 1: [ra[40]], 2: [rb[8], ra[69]], 3: [rb[8]]}
    for n, rows in want.items():
        got = np.fromfile(out / f"{n}.f32", dtype="<f4").reshape(len(rows), cfg["vocab"])
        for g, r in zip(got, rows):
            assert float(np.abs(g - r.numpy()).max() / r.abs().max()) < 2e-4
