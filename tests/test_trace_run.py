"""bin/trace_run end to end on the CPU: a model directory written here (config.json + model.safetensors of
a small random Gezavik, Sigudra, Tukedra or Purozen model), a few steps on standard input, logits files against the plain
oracle.  The runner picks the model class by the directory's config.json."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import gezavik_oracle as oracle
from financial_chatbot_llm_amd.models.configs import layered_config
from financial_chatbot_llm_amd.models.gezavik import GezavikModel
from test_gezavik import random_weights, small_config, tokens

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_cli(tmp_path, dtype):
    from safetensors.torch import save_file
    cfgd = small_config("AmaM", width=64, vocab=120, heads=2)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfgd))
    sd = random_weights(GezavikModel(layered_config(cfgd, "t"), device="cpu"), 3)
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model_dir / "model.safetensors"))
    a, b = tokens(75, 120, 1), tokens(9, 120, 2)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[66:67], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "a", "tokens": a[67:], "want": [7]}, {"id": "b", "tokens": b[2:], "want": [6]}],
         "end": ["a", "b"]},
    ]
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", "192", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    assert not (out_dir / "1.f32").exists() or np.fromfile(out_dir / "1.f32", "<f4").size == 120
    wa = oracle.forward(cfgd, sd, a, torch.float64)
    wb = oracle.forward(cfgd, sd, b, torch.float64)
    tol = 3e-4 if dtype == "float32" else 6e-2

    def ok(got, want):
        want = want.float().numpy()
        assert np.abs(got - want).max() / np.abs(want).max() < tol

    g0 = np.fromfile(out_dir / "0.f32", "<f4").reshape(2, 120)
    ok(g0[0], wa[0]); ok(g0[1], wa[65])
    ok(np.fromfile(out_dir / "1.f32", "<f4").reshape(1, 120)[0], wa[66])
    g2 = np.fromfile(out_dir / "2.f32", "<f4").reshape(2, 120)
    ok(g2[0], wa[74]); ok(g2[1], wb[8])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_cli_sigudra(tmp_path, dtype):
    """The same runner on a Sigudra directory whose config.json carries no ranks (the tensors give them):
    a request admitted beside a running one, a request that sits out a step, a slot given back and reused."""
    import copy

    import sigudra_oracle
    import test_sigudra as ts
    from financial_chatbot_llm_amd.models.sigudra import SigudraModel
    from safetensors.torch import save_file
    full = ts.small_config("pGdg", width=64, vocab=120)
    sd = ts.random_weights(SigudraModel(layered_config(full, "t"), device="cpu"), 3)
    cfgd = copy.deepcopy(full)
    for l in cfgd["layers"]:
        l["mixer"].pop("decay_rank", None)
        l["mixer"].pop("gate_rank", None)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfgd))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model_dir / "model.safetensors"))
    a, b, c = tokens(75, 120, 1), tokens(9, 120, 2), tokens(3, 120, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[66:67], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[2:], "want": [6]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [0, 2]}, {"id": "a", "tokens": a[67:], "want": [7]}], "end": ["a", "c"]},
    ]
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", "192", "--max-seqs", "2", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    want = {k: sigudra_oracle.forward(cfgd, sd, t) for k, t in (("a", a), ("b", b), ("c", c))}
    tol = 3e-4 if dtype == "float32" else 8e-2

    def ok(got, w):
        w = w.float().numpy()
        assert np.abs(got - w).max() / np.abs(w).max() < tol

    g0 = np.fromfile(out_dir / "0.f32", "<f4").reshape(2, 120)
    ok(g0[0], want["a"][0]); ok(g0[1], want["a"][65])
    ok(np.fromfile(out_dir / "1.f32", "<f4").reshape(1, 120)[0], want["a"][66])
    ok(np.fromfile(out_dir / "2.f32", "<f4").reshape(1, 120)[0], want["b"][8])
    g3 = np.fromfile(out_dir / "3.f32", "<f4").reshape(3, 120)
    ok(g3[0], want["c"][0]); ok(g3[1], want["c"][2]); ok(g3[2], want["a"][74])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_cli_tukedra(tmp_path, dtype):
    """The same runner on a Tukedra directory: portions cut inside a block of the mask, a request admitted
    beside a running one, a slot and pages given back and used again."""
    import test_tukedra as tt
    import tukedra_oracle
    from financial_chatbot_llm_amd.models.tukedra import TukedraModel
    from safetensors.torch import save_file
    cfgd = tt.small_config("aLrl", width=64, vocab=120)
    sd = tt.random_weights(TukedraModel(layered_config(cfgd, "t"), device="cpu"), 3)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfgd))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model_dir / "model.safetensors"))
    a, b, c = tokens(75, 120, 1), tokens(9, 120, 2), tokens(3, 120, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 36, 37, 65]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[66:67], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[2:], "want": [6]}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "c", "tokens": c, "want": [0, 2]}, {"id": "a", "tokens": a[67:], "want": [6, 7]}], "end": ["a", "c"]},
    ]
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", "192", "--max-seqs", "2", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(4)]
    want = {k: tukedra_oracle.forward(cfgd, sd, t) for k, t in (("a", a), ("b", b), ("c", c))}
    tol = 3e-4 if dtype == "float32" else 8e-2

    def ok(got, w):
        w = w.float().numpy()
        assert np.abs(got - w).max() / np.abs(w).max() < tol

    g0 = np.fromfile(out_dir / "0.f32", "<f4").reshape(4, 120)
    for i, at in enumerate((0, 36, 37, 65)):
        ok(g0[i], want["a"][at])
    ok(np.fromfile(out_dir / "1.f32", "<f4").reshape(1, 120)[0], want["a"][66])
    ok(np.fromfile(out_dir / "2.f32", "<f4").reshape(1, 120)[0], want["b"][8])
    g3 = np.fromfile(out_dir / "3.f32", "<f4").reshape(4, 120)
    ok(g3[0], want["c"][0]); ok(g3[1], want["c"][2]); ok(g3[2], want["a"][73]); ok(g3[3], want["a"][74])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_cli_purozen(tmp_path, dtype):
    """The same runner on a Purozen directory (no ``head`` tensor: the embedding table projects to the
    vocabulary): portions cut inside a window, a step in which nothing is wanted, a request admitted beside
    a running one, a slot and pages given back and used again."""
    import purozen_oracle
    import test_purozen as tp
    from financial_chatbot_llm_amd.models.purozen import PurozenModel
    from safetensors.torch import save_file
    cfgd = tp.small_config("apal", width=64, vocab=120)
    sd = tp.random_weights(PurozenModel(layered_config(cfgd, "t"), device="cpu"), 3)
    model_dir, out_dir = tmp_path / "model", tmp_path / "out"
    model_dir.mkdir()
    (model_dir / "config.json").write_text(json.dumps(cfgd))
    save_file({k: v.contiguous() for k, v in sd.items()}, str(model_dir / "model.safetensors"))
    a, b, c = tokens(75, 120, 1), tokens(9, 120, 2), tokens(3, 120, 4)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 36, 37, 65]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:2], "want": []}, {"id": "a", "tokens": a[66:67], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[2:7], "want": []}], "end": []},
        {"step": 3, "entries": [{"id": "b", "tokens": b[7:], "want": [1]}], "end": ["b"]},
        {"step": 4, "entries": [{"id": "c", "tokens": c, "want": [0, 2]}, {"id": "a", "tokens": a[67:], "want": [6, 7]}], "end": ["a", "c"]},
    ]
    p = subprocess.run([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", str(model_dir), "--dtype", dtype,
                        "--out", str(out_dir), "--max-tokens", "192", "--max-seqs", "2", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == [f"done {i}" for i in range(5)]
    assert not (out_dir / "2.f32").exists()
    want = {k: purozen_oracle.forward(cfgd, sd, t) for k, t in (("a", a), ("b", b), ("c", c))}
    tol = 3e-4 if dtype == "float32" else 8e-2

    def ok(got, w):
        assert np.abs(got - w).max() / np.abs(w).max() < tol

    g0 = np.fromfile(out_dir / "0.f32", "<f4").reshape(4, 120)
    for i, at in enumerate((0, 36, 37, 65)):
        ok(g0[i], want["a"][at])
    ok(np.fromfile(out_dir / "1.f32", "<f4").reshape(1, 120)[0], want["a"][66])
    ok(np.fromfile(out_dir / "3.f32", "<f4").reshape(1, 120)[0], want["b"][8])
    g4 = np.fromfile(out_dir / "4.f32", "<f4").reshape(4, 120)
    ok(g4[0], want["c"][0]); ok(g4[1], want["c"][2]); ok(g4[2], want["a"][73]); ok(g4[3], want["a"][74])
