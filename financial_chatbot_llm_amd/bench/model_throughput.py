"""Prefill and decode throughput of a layered hybrid decoder beside a Llama twin of equal size.

    python bench.py --model-throughput gezavik [--mt-widths 1024,2048,4096]
    python bench.py --model-throughput sigudra          # beside Gezavik, its closest relative here
    python bench.py --model-throughput tukedra          # beside Sigudra, its closest relative here
    python bench.py --model-throughput purozen          # beside a dense-feed-forward Sigudra of equal size
    python -m financial_chatbot_llm_amd.bench.model_throughput --mt-only gezavik-w2048

For each width a Gezavik model (random weights, 8 layers: latent attention and Mamba-2 mixers, dense
and routed feed-forwards, sizes in the range of a real model's layers) and a Llama model of the same
width, depth, vocabulary and ACTIVE parameter count (its FFN width is fitted) run the same two
workloads through the real engine (scheduler, pages, state slots, hipGraph decode):

* prefill: ``--mt-prompts`` prompts of ``--mt-prompt-len`` tokens, one sampled token each;
* decode: ``--mt-batch`` sequences behind ``--mt-ctx``-token prompts, ``--mt-steps`` timed steps.

One JSON line per model and workload; random weights, synthetic token ids.
"""
from __future__ import annotations

import argparse
import json
import time
from typing import Dict, List

import torch

PATTERN = "aMmAmMaM"


def _gezavik_params(cfgd: Dict) -> Dict[str, int]:
    """(total, active per token) parameter counts of a layered config dict."""
    W, V = cfgd["width"], cfgd["vocab"]
    total = active = 2 * V * W
    for l in cfgd["layers"]:
        m = l["mixer"]
        if l["type"] == "mamba2":
            inner = m["heads"] * m["vdim"]
            n = W * (2 * inner + 2 * m["groups"] * m["state"] + m["heads"]) + inner * W
        else:
            H, dq = m["heads"], m["dim"] + m["rot_dim"]
            n = W * (m["q_rank"] + m["kv_rank"] + m["rot_dim"] + H) + m["q_rank"] * H * dq \
                + m["kv_rank"] * H * (m["dim"] + m["vdim"]) + H * m["vdim"] * W
        total += n
        active += n
        f = l["mlp"]
        if f is None:
            continue
        if f["kind"] == "dense":
            total += 2 * W * f["ff"]
            active += 2 * W * f["ff"]
        else:
            e = 3 * W * f["expert"]["ff"]
            sh = 3 * W * f["shared"]["ff"] if f.get("shared") else 0
            r = f["router"]
            total += r["experts"] * e + sh + (r["experts"] + r.get("identity", 0)) * W
            active += r["top"] * e + sh
    return {"total": total, "active": active}


def register(width: int, vocab: int = 32768) -> List[str]:
    """Register ``gezavik-w<width>`` and its Llama twin ``llama-eq-w<width>``; returns the two names."""
    from ..models.configs import REGISTRY, ModelConfig, layered_config
    from ..models.gezavik import example_config
    cfgd = example_config(width=width, vocab=vocab, heads=max(width // 128, 2), pattern=PATTERN, scale_up=True)
    g, l = f"gezavik-w{width}", f"llama-eq-w{width}"
    REGISTRY[g] = layered_config(cfgd, g)
    p = _gezavik_params(cfgd)
    L, heads = len(cfgd["layers"]), max(width // 128, 2)
    kvh = max(heads // 4, 1)
    attn = width * (heads + 2 * kvh) * 128 + heads * 128 * width
    ff = max(256, int((p["active"] - 2 * vocab * width - L * attn) / (3 * width * L)) // 256 * 256)
    REGISTRY[l] = ModelConfig(l, "llama", vocab, width, L, heads, kvh, 128, ff, max_position=8192,
                              bos_token_id=0, eos_token_ids=())
    return [g, l]


def register_sigudra(width: int, vocab: int = 32768) -> List[str]:
    """Register ``sigudra-w<width>`` (8 layers ``dGPgDpdG``: delta rule, gated linear attention and
    windowed attention beside a gated LRU; dense and routed feed-forwards) and the Gezavik model of the
    same width, depth and vocabulary; returns the two names."""
    from ..models.configs import REGISTRY, layered_config
    from ..models.sigudra import example_config
    name = f"sigudra-w{width}"
    REGISTRY[name] = layered_config(example_config(width=width, vocab=vocab, pattern="dGPgDpdG", scale_up=True), name)
    return [name, register(width, vocab)[0]]


def register_tukedra(width: int, vocab: int = 32768) -> List[str]:
    """Register ``tukedra-w<width>`` (8 layers ``lLRalLrA``: lightning and retention scans, chunk-masked
    attention; dense and routed feed-forwards; two residual streams) and the Sigudra model of the same
    width, depth and vocabulary (within 2 % of the same parameter count); returns the two names."""
    from ..models.configs import REGISTRY, layered_config
    from ..models.tukedra import example_config
    name = f"tukedra-w{width}"
    REGISTRY[name] = layered_config(example_config(width=width, vocab=vocab, pattern="lLRalLrA", scale_up=True), name)
    return [name, register_sigudra(width, vocab)[0]]


def register_purozen(width: int, vocab: int = 32768) -> List[str]:
    """Register ``purozen-w<width>`` (8 layers ``paalpaal``: sigmoid attention beside a minimal GRU, windowed
    attention with kept first tokens and blended values, position-free latent attention; plain GeLU
    feed-forwards of 4 x width; gated residual updates) and ``sigudra-dense-w<width>``, the Sigudra model of
    the same width, depth and vocabulary with dense feed-forwards only (``pgpdpgpd``: windowed attention
    beside a gated LRU, matrix-state scans; within 3 % of the same parameter count); returns the two names."""
    from ..models.configs import REGISTRY, layered_config
    from ..models.purozen import example_config
    from ..models.sigudra import example_config as sigudra_config
    name, twin = f"purozen-w{width}", f"sigudra-dense-w{width}"
    REGISTRY[name] = layered_config(example_config(width=width, vocab=vocab, pattern="paalpaal", scale_up=True), name)
    REGISTRY[twin] = layered_config(sigudra_config(width=width, vocab=vocab, pattern="pgpdpgpd", scale_up=True), twin)
    return [name, twin]


def _tokens(n: int, vocab: int, seed: int) -> List[int]:
    g = torch.Generator().manual_seed(seed)
    return torch.randint(5, vocab - 300, (n,), generator=g).tolist()


def measure(name: str, a) -> List[Dict]:
    from ..config import EngineConfig
    from ..engine import LLMEngine, SamplingParams
    from ..models.configs import get_model_config
    mc = get_model_config(name)
    cfg = EngineConfig(model=name, device="cuda", max_num_seqs=a.mt_batch, max_model_len=4096,
                       max_num_batched_tokens=a.mt_step_tokens, graph_batch_sizes=(a.mt_batch,),
                       enable_prefix_caching=False, kv_mem_fraction=0.3)
    eng = LLMEngine(cfg)
    eng.warmup()
    V = mc.vocab_size
    info = {"model": name, "width": mc.hidden_size, "layers": mc.num_layers,
            "params_b": round(eng.model.num_bytes() / 2 / 1e9, 3)}
    out = []
    # prefill (one warm-up round, then timed)
    for rnd in range(2):
        seqs = [eng.add_request(f"p{rnd}-{i}", _tokens(a.mt_prompt_len, V, 100 * rnd + i),
                                SamplingParams(temperature=0.0, max_tokens=1, ignore_eos=True)) for i in range(a.mt_prompts)]
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        while any(not s.finished for s in seqs):
            eng.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
    ntok = a.mt_prompts * a.mt_prompt_len
    out.append({**info, "workload": "prefill", "prompts": a.mt_prompts, "prompt_len": a.mt_prompt_len,
                "step_tokens": a.mt_step_tokens, "tokens_per_s": round(ntok / dt, 1), "ms": round(1e3 * dt, 2)})
    # decode
    sp = SamplingParams(temperature=0.7, max_tokens=a.mt_steps + 16, ignore_eos=True, seed=1)
    seqs = [eng.add_request(f"d{i}", _tokens(a.mt_ctx, V, 1000 + i), sp) for i in range(a.mt_batch)]
    while any(s.num_computed < len(s.prompt_ids) for s in seqs):
        eng.step()
    for _ in range(6):
        eng.step()
    torch.cuda.synchronize()
    g0 = eng.runner.stats["graph_steps"]
    t0 = time.perf_counter()
    for _ in range(a.mt_steps):
        eng.step()
    torch.cuda.synchronize()
    dt = time.perf_counter() - t0
    out.append({**info, "workload": "decode", "batch": a.mt_batch, "ctx": a.mt_ctx, "steps": a.mt_steps,
                "graph_steps": eng.runner.stats["graph_steps"] - g0, "ms_per_step": round(1e3 * dt / a.mt_steps, 3),
                "tokens_per_s": round(a.mt_batch * a.mt_steps / dt, 1)})
    for s in seqs:
        eng.abort(s.request_id)
    del eng
    torch.cuda.empty_cache()
    return out


def add_arguments(ap: argparse.ArgumentParser) -> None:
    ap.add_argument("--mt-widths", default="1024,2048,4096")
    ap.add_argument("--mt-prompts", type=int, default=8)
    ap.add_argument("--mt-prompt-len", type=int, default=2048)
    ap.add_argument("--mt-step-tokens", type=int, default=4096)
    ap.add_argument("--mt-batch", type=int, default=64)
    ap.add_argument("--mt-ctx", type=int, default=1024)
    ap.add_argument("--mt-steps", type=int, default=64)
    ap.add_argument("--mt-only", default="", help="run only this registered name (e.g. gezavik-w2048)")


def run(a) -> int:
    names: List[str] = []
    design = getattr(a, "model_throughput", "") or "gezavik"
    for w in (int(x) for x in a.mt_widths.split(",") if x):
        names += {"sigudra": register_sigudra, "tukedra": register_tukedra, "purozen": register_purozen}.get(design, register)(w)
    if a.mt_only:
        names = [n for n in names if n == a.mt_only]
    for n in names:
        for rec in measure(n, a):
            print(json.dumps(rec), flush=True)
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--model-throughput", default="gezavik", choices=["gezavik", "sigudra", "tukedra", "purozen"])
    add_arguments(ap)
    return run(ap.parse_args(argv))


if __name__ == "__main__":
    raise SystemExit(main())
