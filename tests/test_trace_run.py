"""bin/trace_run as a program: a model folder (config.json + model.safetensors in bfloat16) is loaded
through the checkpoint loader and the registry, JSON steps go in on stdin, logits come back as files
and every step answers 'done <n>'.  Runs on the CPU path in float32 here (--device cpu); the GPU runs
of the same program are covered by the engine tests."""
import json
import os
import subprocess
import sys

import numpy as np
import torch
from safetensors.torch import save_file

import oracle_tudilix as O
from test_tudilix import cfg_a, rel_err

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_trace_run_replays_a_schedule(tmp_path):
    cfg = cfg_a()
    sd = {k: torch.from_numpy(v).to(torch.bfloat16) for k, v in O.make_weights(cfg, seed=21).items()}
    model = tmp_path / "model"
    model.mkdir()
    (model / "config.json").write_text(json.dumps(cfg))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model / "model.safetensors"))
    rng = np.random.default_rng(3)
    toks = {"a": rng.integers(0, cfg["vocab"], 50).tolist(), "b": rng.integers(0, cfg["vocab"], 21).tolist()}
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": toks["a"][:30], "want": [0, 29]}], "end": []},
        {"step": 1, "entries": [{"id": "a", "tokens": toks["a"][30:31], "want": [0]},
                                {"id": "b", "tokens": toks["b"][:20], "want": [19]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": toks["b"][20:], "want": []}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": toks["a"][31:], "want": [18]}], "end": ["a"]},
    ]
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "128", "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    assert not (out / "2.f32").exists()                       # nothing wanted in step 2
    ref = {n: O.forward(cfg, {k: v.float() for k, v in sd.items()}, t)[0] for n, t in toks.items()}
    got = {i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, cfg["vocab"]) for i in (0, 1, 3)}
    assert rel_err(got[0], ref["a"][[0, 29]]) < 3e-5
    assert rel_err(got[1], np.stack([ref["a"][30], ref["b"][19]])) < 3e-5
    assert rel_err(got[3], ref["a"][[49]]) < 3e-5
