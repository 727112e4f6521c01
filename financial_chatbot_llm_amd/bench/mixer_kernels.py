"""Times the sequence-mixer kernels (``ops.mixers``) at the layer shapes of a hybrid decoder.

    python -m financial_chatbot_llm_amd.bench.mixer_kernels [--width 2048] [--design gezavik|sigudra|tukedra|purozen]

Two step shapes: a prefill step of two 2048-token prompts and a decode step of 64 single rows at
depth 1024.  Shapes follow ``models.gezavik.example_config(scale_up=True)``: Mamba-2 with inner =
2 * width, 64-wide heads, state 128, 2 groups, 4 taps; latent attention with width / 128 heads,
kv_rank 256, rot_dim 32, window 1024.  One JSON line per kernel and shape (microseconds, and the
arithmetic or byte rate the time corresponds to).  ``--design sigudra``: the kernels of that design at
``models.sigudra.example_config(scale_up=True)`` shapes (width / 128 heads of key and value size 128
for the delta rule and the windowed attention with 4 query heads per key/value head, 64-wide keys for
gated linear attention, a gated LRU as wide as the model, window 1024).  ``--design tukedra``: that
design's kernels at ``models.tukedra.example_config(scale_up=True)`` shapes (width / 128 heads; lightning
128 x 128 with the SiLU at staging, retention 64 x 128 on rotated f32 q and k, chunk-masked attention with
128-wide heads, 4 query heads per key/value head and blocks of 2048 positions; two residual streams).
``--design purozen``: that design's kernels at ``models.purozen.example_config(scale_up=True)`` shapes
(width / 128 heads of 128 with 4 query heads per key/value head: sigmoid-weight attention over the whole
prefix, softmax attention with 64 rotated entries, window 1024 and 4 kept first tokens; a minimal GRU as
wide as the model; position-free latent attention of rank 256; the gated residual update; plain GeLU).
"""
from __future__ import annotations

import argparse
import json

import torch

from ..ops import mixers as mx


def _time(f, n: int = 20) -> float:
    for _ in range(3):
        f()
    torch.cuda.synchronize()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    a.record()
    for _ in range(n):
        f()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / n * 1e3


def _steps(dev):
    for name, lens, start in (("prefill 2x2048", [2048, 2048], 0), ("decode 64x1 at 1024", [1] * 64, 1024)):
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        pos = torch.cat([torch.arange(start, start + n) for n in lens]).to(torch.int32).to(dev)
        yield name, lens, start, cu, pos, torch.arange(len(lens), dtype=torch.int32, device=dev)


def sigudra(width: int) -> int:
    dev = "cuda"
    H, D, P, K, window = max(width // 128, 2), 128, 128, 4, 1024
    G = max(H // 4, 1)
    out = lambda **kw: print(json.dumps(kw), flush=True)  # noqa: E731
    for name, lens, start, cu, pos, slot in _steps(dev):
        S, T, ml = len(lens), sum(lens), max(lens)
        # delta rule: convolution over q | k | v, then the scan
        C = 2 * H * D + H * P
        inp = torch.randn(T, C, device=dev).bfloat16()
        cw = torch.randn(C, K, device=dev)
        cst = torch.zeros(S, K - 1, C, device=dev)
        us = _time(lambda: mx.conv_act(inp, cw, None, cst, cu, slot, pos, ml, "silu"))
        out(shape=name, kernel="conv_act", us=round(us, 1), TB_per_s=round(T * C * 6 / us / 1e6, 2))
        u = mx.conv_act(inp, cw, None, cst, cu, slot, pos, ml, "silu")
        a_ = torch.randn(T, H * D, device=dev)
        ab, Al = torch.zeros(H * D, device=dev), torch.zeros(H, device=dev)
        beta = torch.randn(T, H, device=dev).bfloat16()
        st = torch.zeros(S, H, D, P, device=dev)
        nq = H * D
        us = _time(lambda: mx.matrix_scan(u[:, :nq], u[:, nq:2 * nq], u[:, 2 * nq:], a_, ab, st, cu, slot, pos, H, H, D, P,
                                          "delta", A_log=Al, beta=beta, max_len=ml), 5)
        out(shape=name, kernel="matrix_scan delta", us=round(us, 1), f32_TFLOP_per_s=round(T * H * D * P * 9 / us / 1e6, 2),
            state_TB_per_s=round(S * H * D * P * 8 / us / 1e6, 2))
        Dg = 64
        qkv = torch.randn(T, 2 * H * Dg + H * P, device=dev).bfloat16() * 0.1
        ag = torch.randn(T, H * Dg, device=dev) + 3
        stg = torch.zeros(S, H, Dg, P, device=dev)
        us = _time(lambda: mx.matrix_scan(qkv[:, :H * Dg], qkv[:, H * Dg:2 * H * Dg], qkv[:, 2 * H * Dg:], ag,
                                          ab[:H * Dg], stg, cu, slot, pos, H, H, Dg, P, "gla", tau=16.0, max_len=ml), 5)
        out(shape=name, kernel="matrix_scan gla", us=round(us, 1), f32_TFLOP_per_s=round(T * H * Dg * P * 5 / us / 1e6, 2),
            state_TB_per_s=round(S * H * Dg * P * 8 / us / 1e6, 2))
        o = torch.randn(T, H * P, device=dev)
        gt = torch.randn(T, H * P, device=dev).bfloat16()
        nw = torch.ones(P, device=dev)
        us = _time(lambda: mx.head_norm_gate(o, nw, 1e-5, gt, H, "sigmoid", torch.bfloat16))
        out(shape=name, kernel="head_norm_gate", us=round(us, 1), TB_per_s=round(T * H * P * 8 / us / 1e6, 2))
        # gated LRU
        R, Bk = width, max(width // 256, 1)
        uu = torch.randn(T, R, device=dev)
        z = torch.randn(Bk, T, 2 * R // Bk, device=dev)
        rb, lam = torch.zeros(R, device=dev), torch.zeros(R, device=dev)
        y = torch.randn(T, R, device=dev).bfloat16()
        sl = torch.zeros(S, R, device=dev)
        us = _time(lambda: mx.lru_scan(uu, z, Bk, rb, rb, lam, y, rb, sl, cu, slot, pos, torch.bfloat16, max_len=ml))
        out(shape=name, kernel="lru_scan", us=round(us, 1), TB_per_s=round(T * R * 16 / us / 1e6, 2))
        # windowed attention
        pages = (start + ml + 63) // 64
        cache = torch.randn(S * pages * 64, G * (D + P), device=dev).bfloat16()
        bt = torch.arange(S * pages, dtype=torch.int32, device=dev).view(S, pages).contiguous()
        q = torch.randn(T, H * D, device=dev).bfloat16() * .1
        k = torch.randn(T, G * D, device=dev).bfloat16()
        v = torch.randn(T, G * P, device=dev).bfloat16()
        qw, kw = torch.ones(H * D, device=dev), torch.ones(G * D, device=dev)
        slots = (bt[:, None, :].expand(S, ml, pages).reshape(-1, pages).gather(1, (pos // 64).long()[:, None])[:, 0] * 64
                 + pos % 64).to(torch.int32)
        us = _time(lambda: mx.qk_norm_write(q, k, v, qw, kw, 1e-5, slots, cache))
        out(shape=name, kernel="qk_norm_write", us=round(us, 1),
            TB_per_s=round(T * (2 * H * D + 2 * G * (D + P)) * 2 / us / 1e6, 2))
        gate = torch.randn(T, H, device=dev).bfloat16()
        us = _time(lambda: mx.window_attend(q, cache, cu, pos, bt, window, 0.1, ml, H, G, D, P, gate=gate), 5)
        pairs = sum(min(p + 1, window) for n in lens for p in range(start, start + n))
        out(shape=name, kernel="window_attend", us=round(us, 1),
            bf16_TFLOP_per_s=round(pairs * H * 2 * (D + P) / us / 1e6, 1),
            cache_TB_per_s=round(S * min(start + ml, window + ml) * G * (D + P) * 2 / us / 1e6, 2))
        x = torch.randn(T, width, device=dev)
        aa = torch.randn(T, width, device=dev).bfloat16()
        w = torch.ones(width, device=dev)
        us = _time(lambda: mx.post_norm_add(x, aa, w, 1e-5, torch.bfloat16))
        out(shape=name, kernel="post_norm_add", us=round(us, 1), TB_per_s=round(T * width * 12 / us / 1e6, 2))
    return 0


def tukedra(width: int) -> int:
    dev = "cuda"
    H, D, P, size, S2 = max(width // 128, 2), 128, 128, 2048, 2
    G = max(H // 4, 1)
    out = lambda **kw: print(json.dumps(kw), flush=True)  # noqa: E731
    for name, lens, start, cu, pos, slot in _steps(dev):
        S, T, ml = len(lens), sum(lens), max(lens)
        # lightning: one launch, SiLU while the rows are staged
        qkv = torch.randn(T, 2 * H * D + H * P, device=dev).bfloat16() * 0.3
        decay = torch.linspace(0.9, 0.999, H, device=dev)
        st = torch.zeros(S, H, D, P, device=dev)
        us = _time(lambda: mx.decay_scan(qkv[:, :H * D], qkv[:, H * D:2 * H * D], qkv[:, 2 * H * D:], decay, st, cu, slot, pos,
                                         H, D, P, act="silu", max_len=ml), 5)
        out(shape=name, kernel="decay_scan lightning", us=round(us, 1), f32_TFLOP_per_s=round(T * H * D * P * 5 / us / 1e6, 2),
            state_TB_per_s=round(S * H * D * P * 8 / us / 1e6, 2))
        # retention: rotation of q and k into f32, then the scan
        Dr = 64
        freq, ms = mx.rope_freqs(Dr, 10000.0, device=dev)
        q2 = torch.randn(T, 2 * H * Dr + H * P, device=dev).bfloat16() * 0.3
        us = _time(lambda: mx.rope_heads(q2[:, :H * Dr], q2[:, H * Dr:2 * H * Dr], H, H, Dr, freq, pos, "half", ms,
                                         k_scale=Dr ** -0.5, q_dtype=torch.float32, k_dtype=torch.float32))
        out(shape=name, kernel="rope_heads retention", us=round(us, 1), TB_per_s=round(T * 2 * H * Dr * 6 / us / 1e6, 2))
        qf, kf = mx.rope_heads(q2[:, :H * Dr], q2[:, H * Dr:2 * H * Dr], H, H, Dr, freq, pos, "half", ms, k_scale=Dr ** -0.5,
                               q_dtype=torch.float32, k_dtype=torch.float32)
        st2 = torch.zeros(S, H, Dr, P, device=dev)
        us = _time(lambda: mx.decay_scan(qf, kf, q2[:, 2 * H * Dr:], decay, st2, cu, slot, pos, H, Dr, P, max_len=ml), 5)
        out(shape=name, kernel="decay_scan retention", us=round(us, 1), f32_TFLOP_per_s=round(T * H * Dr * P * 5 / us / 1e6, 2),
            state_TB_per_s=round(S * H * Dr * P * 8 / us / 1e6, 2))
        o = torch.randn(T, H * P, device=dev)
        gt = torch.randn(T, H * P, device=dev).bfloat16()
        nw = torch.ones(H * P, device=dev)
        us = _time(lambda: mx.head_norm_gate(o, nw, 1e-5, gt, 1, "sigmoid", torch.bfloat16))
        out(shape=name, kernel="head_norm_gate all heads", us=round(us, 1), TB_per_s=round(T * H * P * 8 / us / 1e6, 2))
        us = _time(lambda: mx.head_norm_gate(o, None, 1e-5, gt, H, "silu", torch.bfloat16))
        out(shape=name, kernel="head_norm_gate per head", us=round(us, 1), TB_per_s=round(T * H * P * 8 / us / 1e6, 2))
        # attention: rotation + per-head norm + cache write, then the chunk-masked attention
        pages = (start + ml + 63) // 64
        cache = torch.randn(S * pages * 64, 2 * G * D, device=dev).bfloat16()
        bt = torch.arange(S * pages, dtype=torch.int32, device=dev).view(S, pages).contiguous()
        qk = torch.randn(T, (H + G) * D, device=dev).bfloat16()
        fa, ma = mx.rope_freqs(64, 10000.0, {"factor": 4.0, "fast": 32.0, "original": 4096, "slow": 1.0}, device=dev)
        slots = (bt[:, None, :].expand(S, ml, pages).reshape(-1, pages).gather(1, (pos // 64).long()[:, None])[:, 0] * 64
                 + pos % 64).to(torch.int32)
        us = _time(lambda: mx.rope_heads(qk[:, :H * D], qk[:, H * D:], H, G, D, fa, pos, "pairs", ma, norm_eps=1e-5,
                                         k_out=cache, slots=slots, v=qk[:, H * D:]))
        out(shape=name, kernel="rope_heads attention", us=round(us, 1),
            TB_per_s=round(T * (2 * H * D + 3 * G * D) * 2 / us / 1e6, 2))
        qn, _ = mx.rope_heads(qk[:, :H * D], qk[:, H * D:], H, G, D, fa, pos, "pairs", ma, norm_eps=1e-5, k_out=cache,
                              slots=slots, v=qk[:, H * D:])
        us = _time(lambda: mx.window_attend(qn, cache, cu, pos, bt, size, 1.0, ml, H, G, D, P, chunked=True), 5)
        pairs = sum(p % size + 1 for n in lens for p in range(start, start + n))
        keys = sum(max(p % size + 1 for p in range(start, start + n)) for n in lens)
        out(shape=name, kernel="window_attend chunked", us=round(us, 1),
            bf16_TFLOP_per_s=round(pairs * H * 2 * (D + P) / us / 1e6, 1),
            cache_TB_per_s=round(keys * G * (D + P) * 2 / us / 1e6, 3))
        x = torch.randn(T, S2, width, device=dev)
        y = torch.randn(T, width, device=dev).bfloat16()
        mix, wo, wi = torch.eye(S2, device=dev), torch.ones(S2, device=dev), torch.ones(S2, device=dev) / S2
        w = torch.ones(width, device=dev)
        us = _time(lambda: mx.hyper_mix(x, y, mix, wo, wi, w, 1e-5, torch.bfloat16))
        out(shape=name, kernel="hyper_mix 2 streams", us=round(us, 1), TB_per_s=round(T * width * (8 * S2 + 4) / us / 1e6, 2))
    return 0


def purozen(width: int) -> int:
    dev = "cuda"
    H, D, P, window, keep, R = max(width // 128, 2), 128, 128, 1024, 4, 256
    G = max(H // 4, 1)
    out = lambda **kw: print(json.dumps(kw), flush=True)  # noqa: E731
    for name, lens, start, cu, pos, slot in _steps(dev):
        S, T, ml = len(lens), sum(lens), max(lens)
        pages = (start + ml + 63) // 64
        bt = torch.arange(S * pages, dtype=torch.int32, device=dev).view(S, pages).contiguous()
        slots = (bt[:, None, :].expand(S, ml, pages).reshape(-1, pages).gather(1, (pos // 64).long()[:, None])[:, 0] * 64
                 + pos % 64).to(torch.int32)
        # sigmoid attention: cache write, then weights sigmoid(score + bias) over the whole prefix
        cache = torch.randn(S * pages * 64, G * (D + P), device=dev).bfloat16()
        qkv = torch.randn(T, (H + 2 * G) * D, device=dev).bfloat16() * .1
        q, k, v = qkv[:, :H * D], qkv[:, H * D:(H + G) * D], qkv[:, (H + G) * D:]
        us = _time(lambda: mx.qk_norm_write(q, k, v, None, None, 1e-5, slots, cache))
        out(shape=name, kernel="qk_norm_write (cache write only)", us=round(us, 1),
            TB_per_s=round(T * 2 * G * (D + P) * 2 / us / 1e6, 2))
        qc = mx.qk_norm_write(q, k, v, None, None, 1e-5, slots, cache)
        pb = torch.full((H,), -4.0, device=dev)
        us = _time(lambda: mx.window_attend(qc, cache, cu, pos, bt, 1 << 30, D ** -0.5, ml, H, G, D, P, head_bias=pb), 5)
        pairs = sum(p + 1 for n in lens for p in range(start, start + n))
        out(shape=name, kernel="window_attend sigmoid, causal", us=round(us, 1),
            bf16_TFLOP_per_s=round(pairs * H * 2 * (D + P) / us / 1e6, 1),
            cache_TB_per_s=round(S * (start + ml) * G * (D + P) * 2 / us / 1e6, 3))
        us = _time(lambda: mx.window_attend(qc, cache, cu, pos, bt, 1 << 30, D ** -0.5, ml, H, G, D, P), 5)
        out(shape=name, kernel="window_attend softmax, causal (same walk)", us=round(us, 1),
            bf16_TFLOP_per_s=round(pairs * H * 2 * (D + P) / us / 1e6, 1),
            cache_TB_per_s=round(S * (start + ml) * G * (D + P) * 2 / us / 1e6, 3))
        # minimal GRU as wide as the model
        zxg = torch.randn(T, 3 * width, device=dev).bfloat16()
        zb = torch.zeros(width, device=dev)
        st = torch.zeros(S, width, device=dev)
        us = _time(lambda: mx.mingru_scan(zxg[:, :width], zxg[:, width:2 * width], zxg[:, 2 * width:], zb, zb, st, cu, slot, pos,
                                          torch.bfloat16, max_len=ml))
        out(shape=name, kernel="mingru_scan", us=round(us, 1), TB_per_s=round(T * width * (8 + 24 + 2) / us / 1e6, 2))
        # attention: rotation + per-head norm + blended values + cache write, then window + kept first tokens
        freq, ms = mx.rope_freqs(64, 10000.0, {"factor": 2.0}, device=dev)
        v1 = torch.randn(T, G * P, device=dev).bfloat16()
        us = _time(lambda: mx.rope_heads(q, k, H, G, D, freq, pos, "half", ms, norm_eps=1e-5, k_out=cache, slots=slots, v=v,
                                         v_mix=v1, v_lam=0.3))
        out(shape=name, kernel="rope_heads + value blend", us=round(us, 1),
            TB_per_s=round(T * (2 * H * D + 2 * G * D + 3 * G * P) * 2 / us / 1e6, 2))
        qn, _ = mx.rope_heads(q, k, H, G, D, freq, pos, "half", ms, norm_eps=1e-5, k_out=cache, slots=slots, v=v, v_mix=v1,
                              v_lam=0.3)
        us = _time(lambda: mx.window_attend(qn, cache, cu, pos, bt, window, 1.0, ml, H, G, D, P, keep_first=keep), 5)
        pairs = sum(min(p + 1, window) + (keep if p >= window + keep else 0) for n in lens for p in range(start, start + n))
        out(shape=name, kernel="window_attend window + kept", us=round(us, 1),
            bf16_TFLOP_per_s=round(pairs * H * 2 * (D + P) / us / 1e6, 1),
            cache_TB_per_s=round(S * min(start + ml, window + ml + keep) * G * (D + P) * 2 / us / 1e6, 3))
        # latent attention without positions, plain causal
        lcache = torch.randn(S * pages * 64, R, device=dev).bfloat16()
        kvp = torch.randn(T, R, device=dev).bfloat16()
        nw = torch.ones(R, device=dev)
        nof = torch.zeros(0, device=dev)
        us = _time(lambda: mx.latent_prep(kvp, nw, 1e-5, nof, 0, pos, slots, lcache, q, H, D, D, R, 0))
        out(shape=name, kernel="latent_prep (no rotation)", us=round(us, 1), TB_per_s=round(T * R * 4 / us / 1e6, 2))
        ql = torch.randn(T, H, R, device=dev).bfloat16() * .1
        qr = torch.empty(T, H, 0, device=dev, dtype=torch.bfloat16)
        us = _time(lambda: mx.latent_attend(ql, qr, lcache, cu, pos, bt, 1 << 30, 0.1, ml), 5)
        pairs = sum(p + 1 for n in lens for p in range(start, start + n))
        out(shape=name, kernel="latent_attend causal", us=round(us, 1),
            bf16_TFLOP_per_s=round(pairs * H * 2 * 2 * R / us / 1e6, 1),
            cache_TB_per_s=round(S * (start + ml) * R * 2 / us / 1e6, 3))
        # gated residual update + next norm; plain GeLU on a column slice
        x = torch.randn(T, width, device=dev)
        ag = torch.randn(T, 2 * width, device=dev).bfloat16()
        w = torch.ones(width, device=dev)
        us = _time(lambda: mx.residual_norm(x, w, 1e-5, a=ag[:, :width], gate=ag[:, width:], gate_bias=zb))
        out(shape=name, kernel="residual_norm gated", us=round(us, 1), TB_per_s=round(T * width * 14 / us / 1e6, 2))
        up = torch.randn(T, 5 * width, device=dev).bfloat16()
        us = _time(lambda: mx.glu_act(up[:, :4 * width], None, "gelu_tanh"))
        out(shape=name, kernel="gelu_tanh", us=round(us, 1), TB_per_s=round(T * 4 * width * 4 / us / 1e6, 2))
    return 0


def main(argv=None) -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--width", type=int, default=2048)
    ap.add_argument("--design", default="gezavik", choices=["gezavik", "sigudra", "tukedra", "purozen"])
    a = ap.parse_args(argv)
    if a.design == "purozen":
        return purozen(a.width)
    if a.design == "sigudra":
        return sigudra(a.width)
    if a.design == "tukedra":
        return tukedra(a.width)
    dev = "cuda"
    H, P, Ns, G, K = 2 * a.width // 64, 64, 128, 2, 4
    C = H * P + 2 * G * Ns
    Ha, R, Dr, window = max(a.width // 128, 2), 256, 32, 1024
    for name, lens, start in (("prefill 2x2048", [2048, 2048], 0), ("decode 64x1 at 1024", [1] * 64, 1024)):
        S, T = len(lens), sum(lens)
        cu = torch.tensor([0] + torch.tensor(lens).cumsum(0).tolist(), dtype=torch.int32, device=dev)
        pos = torch.cat([torch.arange(start, start + n) for n in lens]).to(torch.int32).to(dev)
        slot = torch.arange(S, dtype=torch.int32, device=dev)
        inp = torch.randn(T, C, device=dev).bfloat16()
        cw, cb = torch.randn(C, K, device=dev), torch.randn(C, device=dev)
        cst = torch.zeros(S, K - 1, C, device=dev)
        us = _time(lambda: mx.conv_silu(inp, cw, cb, cst, cu, slot, pos, max(lens)))
        print(json.dumps({"shape": name, "kernel": "conv_silu", "us": round(us, 1),
                          "TB_per_s": round(T * C * 6 / us / 1e6, 2)}), flush=True)
        u = mx.conv_silu(inp, cw, cb, cst, cu, slot, pos, max(lens))
        dtr = torch.randn(T, H, device=dev).bfloat16()
        dtb, Al, Dd = torch.zeros(H, device=dev) - 3, torch.zeros(H, device=dev), torch.ones(H, device=dev)
        sst = torch.zeros(S, H, P, Ns, device=dev)
        us = _time(lambda: mx.ssm_scan(u, dtr, dtb, Al, Dd, sst, cu, slot, pos, H, P, Ns, G))
        print(json.dumps({"shape": name, "kernel": "ssm_scan", "us": round(us, 1),
                          "f32_TFLOP_per_s": round(T * H * P * Ns * 4 / us / 1e6, 2),
                          "state_TB_per_s": round(S * H * P * Ns * 8 / us / 1e6, 2)}), flush=True)
        pages = (start + max(lens) + 63) // 64
        cache = torch.randn(S * pages * 64, R + Dr, device=dev).bfloat16()
        bt = torch.arange(S * pages, dtype=torch.int32, device=dev).view(S, pages).contiguous()
        ql = torch.randn(T, Ha, R, device=dev).bfloat16() * .1
        qr = torch.randn(T, Ha, Dr, device=dev).bfloat16() * .1
        gate = torch.randn(T, Ha, device=dev).bfloat16()
        us = _time(lambda: mx.latent_attend(ql, qr, cache, cu, pos, bt, window, 0.1, max(lens), gate=gate), 5)
        pairs = sum(min(p + 1, window) for n in lens for p in range(start, start + n))
        print(json.dumps({"shape": name, "kernel": "latent_attend", "us": round(us, 1),
                          "bf16_TFLOP_per_s": round(pairs * Ha * 2 * (2 * R + Dr) / us / 1e6, 1),
                          "cache_TB_per_s": round(S * min(start + max(lens), window + max(lens)) * (R + Dr) * 2 / us / 1e6, 2)}),
              flush=True)
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
