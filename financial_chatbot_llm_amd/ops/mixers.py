"""Sequence-mixer ops of the hybrid decoders (``csrc/mixers``): a 32-bit residual stream with a fused
parallel-block update + RMS norm, grouped / gated RMS norms, the Mamba-2 causal convolution and
state-space scan over a flat batch of segments, latent attention over a paged latent cache with a
sliding window, clamped gated units, and biased top-k routing; and, for the sequential post-norm
decoders, a hashed token-pair embedding, layer norm on the sublayer output fused with the residual
add, matrix-state linear recurrences (gated linear attention, gated delta rule), a real-gated linear
recurrent unit, sliding-window attention with grouped key/value heads over a paged [k | v] row cache,
gated activations with a per-row scale and sigmoid top-k routing; and, for decoders with several
residual streams per token (hyper-connections), the fused stream update + read + RMS norm, a rotation
of projected heads (two pair layouts, scaled frequencies, per-head RMS norm), matrix-state recurrences
with one fixed decay per head, a chunked attention mask, top-k routing with a softmax over the chosen
logits, and the logit scale / soft cap; and, for pre-norm decoders with gated residual updates, a sigmoid
gate and two weighted outputs on the fused residual update, attention with kept first tokens beyond a
sliding window and with unnormalised sigmoid weights, a minimal gated recurrent unit, values blended
across layers at the cache write, and linearly scaled rotation frequencies.

Activations are bf16 or f32 (a model-wide choice); statistics, scores, softmax, recurrences and the
residual stream are f32 either way.  CUDA(HIP) tensors run the kernels of ``libpenny_mixers.so``
and fail loudly without it; CPU tensors run the fp32 PyTorch forms below (CI).

Batch layout: a step's rows are ``S`` segments, segment ``s`` owning rows ``cu[s]:cu[s+1]`` (a
prompt chunk, or a single decoded token), ``pos`` the position of every row, ``slot[s]`` the
segment's recurrent-state slot (< 0: padding, skipped) and ``bt[s]`` its cache page table.  A
segment whose first row is at position 0 starts from zero state whatever its slot holds.
"""
from __future__ import annotations

from typing import Optional, Tuple

import torch
import torch.nn.functional as F

from . import _native as N

PAGE = 64


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return 1
    if t.dtype == torch.bfloat16:
        return 0
    raise TypeError(f"mixer ops take bf16 or f32 tensors, got {t.dtype}")


def _rows(t: torch.Tensor) -> torch.Tensor:
    """A 2-D view whose last dimension is contiguous (column slices of a projection pass as is)."""
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError("expected a [rows, n] tensor with unit column stride")
    return t


# ----------------------------------------------------------------------------------------------
# residual stream
# ----------------------------------------------------------------------------------------------
def embed_f32(ids: torch.Tensor, table: torch.Tensor) -> torch.Tensor:
    """Token rows of ``table`` (bf16 or f32) as an f32 residual stream [T, W]."""
    T, (V, W) = ids.numel(), table.shape
    if N.use_native(table):
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
        N.mcall("mx_embed", N.ptr(ids.to(torch.int32).contiguous()), N.ptr(table), _dt(table), N.ptr(out), T, W, V,
                N.stream())
        return out
    return table[ids.long().clamp(0, V - 1)].float()


def residual_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float, a: Optional[torch.Tensor] = None,
                  b: Optional[torch.Tensor] = None, mult: float = 1.0,
                  out_dtype: torch.dtype = torch.bfloat16, mult_b: Optional[float] = None,
                  gate: Optional[torch.Tensor] = None, gate_bias: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x`` (f32 [T, W], in place) <- x + mult * (a + b) when a sublayer output is given, then
    y = x / sqrt(mean(x^2) + eps) * w in ``out_dtype`` (``w`` None: the update only).  ``mult_b``: b's own
    weight, the update is mult * a + mult_b * b.  ``gate`` ([T, W] column slice, the type of a) and
    ``gate_bias`` (f32 [W]): the update is multiplied element by element by sigmoid(gate + gate_bias)."""
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    ab = a if a is not None else b
    mult_b = mult if mult_b is None else mult_b
    if gate is not None and ab is None:
        raise ValueError("a gate needs a sublayer output to act on")
    if N.use_native(x):
        out = torch.empty((T, W), dtype=out_dtype, device=x.device) if w is not None else None
        if a is not None and b is not None:
            assert a.dtype == b.dtype
        if gate is not None:
            assert gate.dtype == ab.dtype and gate.shape[1] == W
        N.mcall("mx_residual_norm", N.ptr(x), N.ptr(_rows(a)) if a is not None else None,
                a.stride(0) if a is not None else 0, N.ptr(_rows(b)) if b is not None else None,
                b.stride(0) if b is not None else 0, _dt(ab) if ab is not None else 1, float(mult), float(mult_b),
                N.ptr(_rows(gate)) if gate is not None else None, gate.stride(0) if gate is not None else 0,
                N.ptr(gate_bias), N.ptr(w), float(eps), N.ptr(out), _dt(out) if out is not None else 1, T, W, N.stream())
        return out
    if ab is not None:
        s = torch.zeros_like(x)
        for t, m in ((a, mult), (b, mult_b)):
            if t is not None:
                s = s + m * t.float()
        if gate is not None:
            s = s * torch.sigmoid(gate.float() + (gate_bias.float() if gate_bias is not None else 0.0))
        x.add_(s)
    if w is None:
        return None
    return (x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def group_norm(inp: torch.Tensor, w: torch.Tensor, eps: float, groups: int = 1, gate: Optional[torch.Tensor] = None,
               out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """RMS norm of each of ``groups`` equal parts of every row of ``inp`` [T, n] (each part by its own
    root mean square), times ``w`` [n].  ``gate``: the row is multiplied by silu(gate) first."""
    T, n = inp.shape
    out_dtype = out_dtype or inp.dtype
    if n % groups:
        raise ValueError(f"{n} columns do not split into {groups} groups")
    if N.use_native(inp):
        out = torch.empty((T, n), dtype=out_dtype, device=inp.device)
        N.mcall("mx_group_norm", N.ptr(_rows(inp)), inp.stride(0), _dt(inp), N.ptr(_rows(gate)) if gate is not None else None,
                gate.stride(0) if gate is not None else 0, _dt(gate) if gate is not None else 1, N.ptr(w),
                float(eps), N.ptr(out), out.stride(0), _dt(out), T, groups, n // groups, N.stream())
        return out
    v = inp.float()
    if gate is not None:
        v = v * F.silu(gate.float())
    v = v.view(T, groups, n // groups)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    return (v.reshape(T, n) * w.float()).to(out_dtype)


# ----------------------------------------------------------------------------------------------
# activations
# ----------------------------------------------------------------------------------------------
def relu2(x: torch.Tensor) -> torch.Tensor:
    """relu(x)^2, rows may be a column slice of a wider projection."""
    T, n = x.shape
    if N.use_native(x):
        out = torch.empty((T, n), dtype=x.dtype, device=x.device)
        N.mcall("mx_relu2", N.ptr(_rows(x)), x.stride(0), N.ptr(out), out.stride(0), _dt(x), T, n, N.stream())
        return out
    return torch.relu(x.float()).square().to(x.dtype)


def glu_clamp(gate: torch.Tensor, up: torch.Tensor, limit: float, alpha: float) -> torch.Tensor:
    """g = min(gate, limit), u = clamp(up, -limit, limit): g * sigmoid(alpha * g) * (u + 1)."""
    T, n = gate.shape
    if N.use_native(gate):
        out = torch.empty((T, n), dtype=gate.dtype, device=gate.device)
        N.mcall("mx_glu_clamp", N.ptr(_rows(gate)), gate.stride(0), N.ptr(_rows(up)), up.stride(0), float(limit),
                float(alpha), N.ptr(out), out.stride(0), _dt(gate), T, n, N.stream())
        return out
    g = gate.float().clamp(max=limit)
    u = up.float().clamp(-limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)).to(gate.dtype)


# ----------------------------------------------------------------------------------------------
# routing
# ----------------------------------------------------------------------------------------------
def route_biased(z: torch.Tensor, bias: Optional[torch.Tensor], top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Scores s = softmax(z) over all entries (f32); the ``top`` entries with the largest s + bias are
    chosen, and their weights are the unbiased scores s (not renormalised).  Returns (weights f32
    [T, top], indices int32 [T, top])."""
    T, E = z.shape
    assert z.dtype == torch.float32
    if N.use_native(z):
        z = z.contiguous()
        w = torch.empty((T, top), dtype=torch.float32, device=z.device)
        i = torch.empty((T, top), dtype=torch.int32, device=z.device)
        N.mcall("mx_route_biased", N.ptr(z), N.ptr(bias), E, top, N.ptr(w), N.ptr(i), T, N.stream())
        return w, i
    s = torch.softmax(z, -1)
    c = s + bias.float() if bias is not None else s
    idx = torch.topk(c, top, dim=-1).indices
    return s.gather(1, idx), idx.to(torch.int32)


def moe_combine(ys: Optional[torch.Tensor], pos: torch.Tensor, idx: torch.Tensor, wts: torch.Tensor, h: torch.Tensor,
                shared: Optional[torch.Tensor], num_experts: int) -> torch.Tensor:
    """out[t] = sum_k wts[t, k] * src(t, k) (+ shared[t]): src is the token's own input ``h[t]`` for an
    identity expert (idx >= num_experts), else row ``pos[t, k]`` of the expert outputs ``ys``."""
    T, W = h.shape
    top = idx.shape[1]
    if N.use_native(h):
        out = torch.empty((T, W), dtype=h.dtype, device=h.device)
        N.mcall("mx_moe_combine", N.ptr(ys), N.ptr(pos.contiguous()), N.ptr(idx.contiguous()), N.ptr(wts.contiguous()),
                N.ptr(_rows(h)), h.stride(0), N.ptr(_rows(shared)) if shared is not None else None,
                shared.stride(0) if shared is not None else 0, num_experts, top, W, N.ptr(out), _dt(h), T, N.stream())
        return out
    acc = shared.float().clone() if shared is not None else torch.zeros((T, W), dtype=torch.float32)
    for k in range(top):
        e = idx[:, k].long()
        ident = e >= num_experts
        src = h.float().clone()
        if ys is not None and (~ident).any():
            rows = pos[:, k].long().clamp(0, ys.shape[0] - 1)
            src = torch.where(ident[:, None], src, ys.float()[rows])
        acc += wts[:, k:k + 1] * src
    return acc.to(h.dtype)


# ----------------------------------------------------------------------------------------------
# state-space mixer
# ----------------------------------------------------------------------------------------------
def conv_silu(inp: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor,
              cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, max_len: int) -> torch.Tensor:
    """Causal per-channel convolution + SiLU over every segment.  ``inp`` [T, C] (a column slice of the
    in-projection), ``w`` f32 [C, K] (last column: the current token's tap), ``state`` f32
    [slots, K-1, C]: the last K-1 inputs of each slot's sequence, read (unless the segment starts
    at position 0) and then replaced.  Returns f32 [T, C]."""
    T, C = inp.shape
    K = w.shape[1]
    S = cu.numel() - 1
    if N.use_native(inp):
        out = torch.empty((T, C), dtype=torch.float32, device=inp.device)
        N.mcall("mx_conv_silu", N.ptr(_rows(inp)), inp.stride(0), _dt(inp), N.ptr(w), N.ptr(bias), N.ptr(state),
                N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(out), S, int(max_len), C, K, N.stream())
        return out
    out = torch.zeros((T, C), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    x = inp.float()
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if sll[s] < 0 or b <= a:
            continue
        hist = torch.zeros((K - 1, C)) if pl[a] == 0 else state[sll[s]].clone()
        full = torch.cat([hist, x[a:b]])
        win = full.unfold(0, K, 1)                      # [n, C, K]
        acc = (win * w.float()[None]).sum(-1)
        if bias is not None:
            acc = acc + bias.float()
        out[a:b] = F.silu(acc)
        if K > 1:
            state[sll[s]] = full[-(K - 1):]
    return out


def ssm_scan(u: torch.Tensor, dt_raw: torch.Tensor, dt_bias: torch.Tensor, A_log: torch.Tensor, D: torch.Tensor,
             state: torch.Tensor, cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, heads: int, vdim: int,
             nstate: int, groups: int) -> torch.Tensor:
    """Mamba-2 recurrence, token by token, f32.  ``u`` f32 [T, H*P + 2*G*N] = [x | B | C] (after the
    convolution), ``dt_raw`` [T, H]; per head h of group h // (H / G):
    dt = softplus(dt_raw + dt_bias), S <- exp(-exp(A_log) dt) S + dt x B^T, y = S C + D x.
    ``state`` f32 [slots, H, P, N] is read (unless the segment starts at position 0) and replaced."""
    T, C = u.shape
    H, P, Ns, G = heads, vdim, nstate, groups
    S = cu.numel() - 1
    assert u.dtype == torch.float32 and u.is_contiguous() and C == H * P + 2 * G * Ns
    if N.use_native(u):
        y = torch.empty((T, H * P), dtype=torch.float32, device=u.device)
        N.mcall("mx_ssm_scan", N.ptr(u), C, N.ptr(_rows(dt_raw)), dt_raw.stride(0), _dt(dt_raw), N.ptr(dt_bias),
                N.ptr(A_log), N.ptr(D), N.ptr(state), N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(y), S, H, P, Ns, G, T,
                N.stream())
        return y
    y = torch.zeros((T, H * P), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    A = -torch.exp(A_log.float())
    rep = H // G
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if sll[s] < 0 or b <= a:
            continue
        St = torch.zeros((H, P, Ns)) if pl[a] == 0 else state[sll[s]].clone()
        dt = F.softplus(dt_raw[a:b].float() + dt_bias.float())          # [n, H]
        dec = torch.exp(A * dt)
        x = u[a:b, :H * P].view(-1, H, P)
        Bm = u[a:b, H * P:H * P + G * Ns].view(-1, G, Ns).repeat_interleave(rep, 1)
        Cm = u[a:b, H * P + G * Ns:].view(-1, G, Ns).repeat_interleave(rep, 1)
        for t in range(b - a):
            St = dec[t, :, None, None] * St + (dt[t, :, None] * x[t])[:, :, None] * Bm[t][:, None, :]
            y[a + t] = ((St * Cm[t][:, None, :]).sum(-1) + D.float()[:, None] * x[t]).reshape(-1)
        state[sll[s]] = St
    return y


# ----------------------------------------------------------------------------------------------
# latent attention
# ----------------------------------------------------------------------------------------------
def rope_inv_freq(dims: int, base: float, device=None) -> torch.Tensor:
    """f_i = base^(-2i / dims), i < dims / 2, f32."""
    i = torch.arange(0, dims, 2, dtype=torch.float32, device=device)
    return (1.0 / (base ** (i / dims))).contiguous()


def _rotate(v: torch.Tensor, ang: torch.Tensor, dims: int) -> torch.Tensor:
    """Interleaved-pair rotation of the first ``dims`` entries of the last axis; ``ang`` broadcasts
    against v[..., 0:dims:2]."""
    out = v.clone()
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    c, s = torch.cos(ang), torch.sin(ang)
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def latent_prep(kv: torch.Tensor, norm_w: torch.Tensor, eps: float, inv_freq: torch.Tensor, rot_dims: int,
                pos: torch.Tensor, slots: torch.Tensor, cache: torch.Tensor, q: torch.Tensor, heads: int,
                head_stride: int, rot_off: int, rank: int, rot_dim: int) -> torch.Tensor:
    """Per token: c = RMSnorm(kv[:rank]) * norm_w and the rotated shared key part rope(kv[rank:]) go to
    cache row ``slots[t]`` (< 0: no write; ``cache`` [rows, rank + rot_dim]); every head's rotated
    query part ``q[t, h*head_stride + rot_off : +rot_dim]`` is rotated into the returned
    [T, heads, rot_dim].  Angles are pos * inv_freq in f32, pairs interleaved."""
    T = kv.shape[0]
    R, Dr, H = rank, rot_dim, heads
    if N.use_native(kv):
        assert kv.dtype == cache.dtype == q.dtype
        q_rot = torch.empty((T, H, Dr), dtype=q.dtype, device=q.device)
        N.mcall("mx_latent_prep", N.ptr(_rows(kv)), kv.stride(0), N.ptr(norm_w), float(eps), N.ptr(inv_freq),
                int(rot_dims), N.ptr(pos), N.ptr(slots), N.ptr(cache), N.ptr(_rows(q)), q.stride(0), head_stride,
                rot_off, N.ptr(q_rot), _dt(kv), T, H, R, Dr, N.stream())
        return q_rot
    kvf = kv.float()
    c = kvf[:, :R]
    c = c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * norm_w.float()
    ang = pos.float()[:, None] * inv_freq.float()[None, :rot_dims // 2]
    kr = _rotate(kvf[:, R:R + Dr], ang, rot_dims)
    rows = torch.cat([c, kr], 1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, R + Dr)[slots[ok].long()] = rows[ok]
    qr = torch.stack([q[:, h * head_stride + rot_off:h * head_stride + rot_off + Dr] for h in range(H)], 1).float()
    return _rotate(qr, ang[:, None, :], rot_dims).to(q.dtype)


def latent_attend(q_lat: torch.Tensor, q_rot: torch.Tensor, cache: torch.Tensor, cu: torch.Tensor, pos: torch.Tensor,
                  bt: torch.Tensor, window: int, scale: float, max_len: int,
                  gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Windowed causal attention in the latent space.  ``q_lat`` [T, H, R], ``q_rot`` [T, H, Dr];
    cache rows [c | k_rot]; the query at position p sees the keys j of its own sequence with
    0 <= p - j < window; score = (q_lat . c_j + q_rot . k_rot_j) * scale, f32 softmax,
    out[t, h] = sum_j p_j c_j, times sigmoid(gate[t, h]) when a gate [T, H] is given."""
    T, H, R = q_lat.shape
    Dr = q_rot.shape[2]
    S = cu.numel() - 1
    if N.use_native(q_lat):
        assert q_lat.is_contiguous() and q_rot.is_contiguous() and bt.is_contiguous()
        out = torch.empty((T, H, R), dtype=q_lat.dtype, device=q_lat.device)
        # decode-size steps (one row per segment) walk each row's keys with several blocks so that a
        # small batch still fills the chip; the split depends only on static sizes (graph-safe)
        nsplit, ws = 1, None
        if max_len == 1 and q_lat.dtype == torch.bfloat16:
            tiles = (min(window, bt.shape[1] * PAGE) + 31) // 32 + 1
            nsplit = max(1, min(16, tiles // 2, 1024 // max(S * ((H + 63) // 64), 1)))
            if nsplit > 1:
                ws = torch.empty((T, H, nsplit, R + 2), dtype=torch.float32, device=q_lat.device)
        N.mcall("mx_latent_attend", N.ptr(q_lat), N.ptr(q_rot), N.ptr(cache), N.ptr(cu), N.ptr(pos), N.ptr(bt),
                bt.shape[1], N.ptr(_rows(gate)) if gate is not None else None,
                gate.stride(0) if gate is not None else 0, int(min(window, 1 << 30)), float(scale), N.ptr(out),
                _dt(q_lat), S, int(max_len), H, R, Dr, nsplit, N.ptr(ws), N.stream())
        return out
    out = torch.zeros((T, H, R), dtype=torch.float32)
    rows = cache.view(-1, R + Dr).float()
    cul, pl = cu.tolist(), pos.tolist()
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if b <= a:
            continue
        ctx = pl[b - 1] + 1
        pages = bt[s, :(ctx + PAGE - 1) // PAGE].long()
        keys = rows.view(-1, PAGE, R + Dr)[pages].reshape(-1, R + Dr)[:ctx]
        qq = torch.cat([q_lat[a:b].float(), q_rot[a:b].float()], -1)       # [n, H, D]
        sc = torch.einsum("nhd,jd->nhj", qq, keys) * scale
        p = pos[a:b].long()[:, None]
        j = torch.arange(ctx)[None]
        vis = (j <= p) & (j > p - window)
        sc = sc.masked_fill(~vis[:, None, :], float("-inf"))
        out[a:b] = torch.einsum("nhj,jr->nhr", torch.softmax(sc, -1), keys[:, :R])
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.to(q_lat.dtype)


# ----------------------------------------------------------------------------------------------
# sequential (post-norm) blocks: hashed pair embedding, layer norm on the sublayer output
# ----------------------------------------------------------------------------------------------
def embed_pairs(ids: torch.Tensor, table: torch.Tensor, pair_table: Optional[torch.Tensor], mul_prev: int, mul_cur: int,
                last_token: Optional[torch.Tensor], cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor,
                max_len: int) -> torch.Tensor:
    """f32 residual stream [T, W]: ``table[id]`` plus, with a ``pair_table`` [buckets + 1, W], its row
    ``(prev * mul_prev + id * mul_cur) mod buckets`` -- ``prev`` the token before in the same
    sequence -- or row ``buckets`` at position 0.  ``last_token`` int32 [slots] holds every slot's
    last token between steps (read by a segment's first row, then replaced by its last id)."""
    T, (V, W) = ids.numel(), table.shape
    S = cu.numel() - 1
    ids = ids.to(torch.int32).contiguous()
    if pair_table is None:
        return embed_f32(ids, table)
    B = pair_table.shape[0] - 1
    if N.use_native(table):
        out = torch.empty((T, W), dtype=torch.float32, device=table.device)
        N.mcall("mx_embed_pairs", N.ptr(ids), N.ptr(table), N.ptr(pair_table), _dt(table), int(mul_prev), int(mul_cur),
                B, N.ptr(last_token), N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(out), S, int(max_len), W, V, N.stream())
        return out
    out = table[ids.long().clamp(0, V - 1)].float()
    cul, sll, pl, idl = cu.tolist(), slot.tolist(), pos.tolist(), ids.tolist()
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if sll[s] < 0 or b <= a:
            continue
        for r in range(a, b):
            if pl[r] == 0:
                row = B
            else:
                prev = idl[r - 1] if r > a else int(last_token[sll[s]])
                row = (prev * mul_prev + idl[r] * mul_cur) % B
            out[r] += pair_table[row].float()
        last_token[sll[s]] = idl[b - 1]
    return out


def _ln(v: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    mu = v.mean(-1, keepdim=True)
    d = v - mu
    return d * torch.rsqrt(d.pow(2).mean(-1, keepdim=True) + eps) * w.float()


def layer_norm_out(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype: torch.dtype) -> torch.Tensor:
    """(x - mean) / sqrt(var + eps) * w of every f32 row, in ``out_dtype``."""
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    if N.use_native(x):
        out = torch.empty((T, W), dtype=out_dtype, device=x.device)
        N.mcall("mx_post_norm", N.ptr(x), None, 0, None, None, 0, None, 1, N.ptr(w), float(eps), N.ptr(out), _dt(out),
                T, W, N.stream())
        return out
    return _ln(x, w, eps).to(out_dtype)


def post_norm_add(x: torch.Tensor, a: torch.Tensor, w: torch.Tensor, eps: float, out_dtype: Optional[torch.dtype] = None,
                  b: Optional[torch.Tensor] = None, wa: Optional[torch.Tensor] = None,
                  wb: Optional[torch.Tensor] = None) -> Optional[torch.Tensor]:
    """``x`` (f32 [T, W], in place) <- x + LayerNorm(m) * w, the norm on the sublayer's output only.
    m = a, or with a second branch m = (RMSnorm(a) * wa + RMSnorm(b) * wb) / 2 (two mixers side by
    side).  Returns the new x rounded to ``out_dtype`` (the next sublayer's GEMM input) when one is
    given and differs from f32, else x itself."""
    T, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    want = out_dtype is not None and out_dtype != torch.float32
    if N.use_native(x):
        out = torch.empty((T, W), dtype=out_dtype, device=x.device) if want else None
        if b is not None:
            assert a.dtype == b.dtype
        N.mcall("mx_post_norm", N.ptr(x), N.ptr(_rows(a)), a.stride(0), N.ptr(wa), N.ptr(_rows(b)) if b is not None else None,
                b.stride(0) if b is not None else 0, N.ptr(wb), _dt(a), N.ptr(w), float(eps), N.ptr(out),
                _dt(out) if want else 1, T, W, N.stream())
        return out if want else x
    m = a.float()
    if b is not None:
        rms = lambda v: v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)  # noqa: E731
        m = 0.5 * (rms(m) * wa.float() + rms(b.float()) * wb.float())
    x.add_(_ln(m, w, eps))
    return x.to(out_dtype) if want else x


ACTS = {"none": 0, "silu": 1, "gelu_tanh": 2, "sigmoid": 3}


def _act(v: torch.Tensor, act: str) -> torch.Tensor:
    if act == "silu":
        return F.silu(v)
    if act == "gelu_tanh":
        return F.gelu(v, approximate="tanh")
    if act == "sigmoid":
        return torch.sigmoid(v)
    return v


def glu_act(gate: torch.Tensor, up: Optional[torch.Tensor], act: str,
            row_scale: Optional[torch.Tensor] = None) -> torch.Tensor:
    """act(s * gate) * (s * up) with ``s`` an optional f32 scale per row (a routed expert whose weight
    multiplies its INPUT: the scale commutes with the two projections); ``act``: silu | gelu_tanh | sigmoid.
    ``up`` None: act(s * gate) alone (a plain, ungated feed-forward)."""
    T, n = gate.shape
    if N.use_native(gate):
        out = torch.empty((T, n), dtype=gate.dtype, device=gate.device)
        N.mcall("mx_glu_act", N.ptr(_rows(gate)), gate.stride(0), N.ptr(_rows(up)) if up is not None else None,
                up.stride(0) if up is not None else 0, N.ptr(row_scale), ACTS[act], N.ptr(out), out.stride(0), _dt(gate),
                T, n, N.stream())
        return out
    g = gate.float()
    if row_scale is not None:
        g = g * row_scale[:, None]
    if up is None:
        return _act(g, act).to(gate.dtype)
    u = up.float() * (row_scale[:, None] if row_scale is not None else 1.0)
    return (_act(g, act) * u).to(gate.dtype)


ROUTE_SCORES = {"softmax": 0, "sigmoid": 1, "softmax_top": 2}


def route_scores(z: torch.Tensor, top: int, score: str = "sigmoid") -> Tuple[torch.Tensor, torch.Tensor]:
    """The ``top`` largest entries of each row of the f32 router logits ``z`` (ties: the lower index)
    and their scores: ``sigmoid`` (independent per expert) or ``softmax`` over all entries, neither
    renormalised, or ``softmax_top``: the softmax over the chosen logits only.
    Returns (weights f32 [T, top], indices int32 [T, top]), the largest first."""
    T, E = z.shape
    assert z.dtype == torch.float32
    if N.use_native(z):
        z = z.contiguous()
        w = torch.empty((T, top), dtype=torch.float32, device=z.device)
        i = torch.empty((T, top), dtype=torch.int32, device=z.device)
        N.mcall("mx_route_scores", N.ptr(z), E, top, ROUTE_SCORES[score], N.ptr(w), N.ptr(i), T, N.stream())
        return w, i
    if score == "softmax_top":
        # a stable sort: ties go to the lower index, as in the kernel
        idx = torch.sort(z, dim=-1, descending=True, stable=True).indices[:, :top]
        return torch.softmax(z.gather(1, idx), -1), idx.to(torch.int32)
    if score not in ROUTE_SCORES:
        raise ValueError(f"unknown routing score {score!r}")
    s = torch.sigmoid(z) if score == "sigmoid" else torch.softmax(z, -1)
    idx = torch.topk(s, top, dim=-1).indices
    return s.gather(1, idx), idx.to(torch.int32)


def conv_act(inp: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], state: torch.Tensor, cu: torch.Tensor,
             slot: torch.Tensor, pos: torch.Tensor, max_len: int, act: str = "silu",
             in_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """:func:`conv_silu` with the activation as a parameter (``silu`` | ``none``) and an optional
    bias ``in_bias`` [C] added to every input BEFORE the convolution (inputs before the sequence stay
    zero; the slot's history holds biased inputs)."""
    if act == "silu" and in_bias is None:
        return conv_silu(inp, w, bias, state, cu, slot, pos, max_len)
    T, C = inp.shape
    K = w.shape[1]
    S = cu.numel() - 1
    if N.use_native(inp):
        out = torch.empty((T, C), dtype=torch.float32, device=inp.device)
        N.mcall("mx_conv_act", N.ptr(_rows(inp)), inp.stride(0), _dt(inp), N.ptr(w), N.ptr(bias), N.ptr(in_bias),
                ACTS[act], N.ptr(state), N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(out), S, int(max_len), C, K, N.stream())
        return out
    out = torch.zeros((T, C), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    x = inp.float() + (in_bias.float() if in_bias is not None else 0.0)
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if sll[s] < 0 or b <= a:
            continue
        hist = torch.zeros((K - 1, C)) if pl[a] == 0 else state[sll[s]].clone()
        full = torch.cat([hist, x[a:b]])
        acc = (full.unfold(0, K, 1) * w.float()[None]).sum(-1)
        if bias is not None:
            acc = acc + bias.float()
        out[a:b] = _act(acc, act)
        if K > 1:
            state[sll[s]] = full[-(K - 1):]
    return out


# ----------------------------------------------------------------------------------------------
# matrix-state linear recurrences (gated linear attention, gated delta rule)
# ----------------------------------------------------------------------------------------------
def matrix_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, a: torch.Tensor, a_bias: torch.Tensor,
                state: torch.Tensor, cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, heads: int, kv_heads: int,
                dim: int, vdim: int, mode: str, tau: float = 1.0, A_log: Optional[torch.Tensor] = None,
                beta: Optional[torch.Tensor] = None, max_len: int = 0) -> torch.Tensor:
    """Token-by-token f32 recurrence over a [dim, vdim] state per head (``state`` f32
    [slots, H, dim, vdim], read unless the segment starts at position 0, then replaced), with one
    decay per head and key channel acting on the state's rows.  ``q``/``k`` [T, G*dim], ``v``
    [T, H*vdim] (column slices; head h reads q/k head h // (H/G)), ``a`` f32 [T, H*dim] the decay's
    pre-activation (the kernels overwrite it with the decays), ``a_bias`` f32 [H*dim].

    ``mode="gla"``:   g = sigmoid(a + a_bias)^(1/tau);  S <- g S + k v^T;  o = S^T (q dim^-1/2).
    ``mode="delta"``: q, k <- unit vectors (x / sqrt(sum x^2 + 1e-6)), q scaled by dim^-1/2;
                      g = exp(-exp(A_log[h]) softplus(a + a_bias));  b = sigmoid(beta[t, h]);
                      S <- g S;  u = b (v - S^T k);  S <- S + k u^T;  o = S^T q.
    ``max_len``: the longest segment when known (1 selects the kernels' single-row form).
    Returns o f32 [T, H*vdim]."""
    T = q.shape[0]
    H, G, D, P = heads, kv_heads, dim, vdim
    S = cu.numel() - 1
    delta = mode == "delta"
    assert a.dtype == torch.float32 and a.shape[1] == H * D and q.shape[1] == G * D and v.shape[1] == H * P
    assert q.dtype == k.dtype == v.dtype
    if N.use_native(q):
        out = torch.empty((T, H * P), dtype=torch.float32, device=q.device)
        aux = torch.empty((T, 2 * G + H), dtype=torch.float32, device=q.device) if delta else None
        N.mcall("mx_matrix_scan", N.ptr(_rows(q)), q.stride(0), N.ptr(_rows(k)), k.stride(0), N.ptr(_rows(v)), v.stride(0),
                _dt(q), N.ptr(_rows(a)), a.stride(0), N.ptr(a_bias), N.ptr(A_log) if delta else None,
                N.ptr(_rows(beta)) if delta else None, beta.stride(0) if delta else 0, _dt(beta) if delta else 1,
                float(tau), 1 if delta else 0, N.ptr(aux), N.ptr(state), N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(out), S, T,
                int(max_len), H, G, D, P, N.stream())
        return out
    out = torch.zeros((T, H * P), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    rep = H // G
    for s in range(S):
        r0, r1 = cul[s], cul[s + 1]
        if sll[s] < 0 or r1 <= r0:
            continue
        n = r1 - r0
        qq = q[r0:r1].float().view(n, G, D)
        kk = k[r0:r1].float().view(n, G, D)
        vv = v[r0:r1].float().view(n, H, P)
        z = a[r0:r1].float() + a_bias.float()
        if delta:
            qq = qq * torch.rsqrt(qq.pow(2).sum(-1, keepdim=True) + 1e-6)
            kk = kk * torch.rsqrt(kk.pow(2).sum(-1, keepdim=True) + 1e-6)
            g = torch.exp(-torch.exp(A_log.float()).repeat_interleave(D)[None] * F.softplus(z)).view(n, H, D)
            bt = torch.sigmoid(beta[r0:r1].float())
        else:
            g = torch.exp(-F.softplus(-z) / tau).view(n, H, D)
        qq = (qq * D ** -0.5).repeat_interleave(rep, 1)
        kk = kk.repeat_interleave(rep, 1)
        St = torch.zeros((H, D, P)) if pl[r0] == 0 else state[sll[s]].clone()
        for t in range(n):
            St = g[t][:, :, None] * St
            u = vv[t]
            if delta:
                u = bt[t][:, None] * (u - torch.einsum("hdp,hd->hp", St, kk[t]))
            St = St + kk[t][:, :, None] * u[:, None, :]
            out[r0 + t] = torch.einsum("hdp,hd->hp", St, qq[t]).reshape(-1)
        state[sll[s]] = St
    return out


def head_norm_gate(o: torch.Tensor, w: torch.Tensor, eps: float, gate: torch.Tensor, heads: int, act: str,
                   out_dtype: torch.dtype) -> torch.Tensor:
    """Every head's part of ``o`` [T, H*P] divided by its root mean square over P, times ``w`` [P]
    (shared by the heads; None: no weight), times act(gate) [T, H*P]; ``act``: sigmoid | silu.  With
    ``heads=1`` the whole row is normed at once with a weight per column."""
    T, n = o.shape
    P = n // heads
    if N.use_native(o):
        out = torch.empty((T, n), dtype=out_dtype, device=o.device)
        N.mcall("mx_head_norm_gate", N.ptr(_rows(o)), o.stride(0), _dt(o), N.ptr(w), float(eps), N.ptr(_rows(gate)),
                gate.stride(0), _dt(gate), ACTS[act], N.ptr(out), _dt(out), T, heads, P, N.stream())
        return out
    v = o.float().view(T, heads, P)
    v = v * torch.rsqrt(v.pow(2).mean(-1, keepdim=True) + eps)
    if w is not None:
        v = v * w.float()
    return (v.reshape(T, n) * _act(gate.float(), act)).to(out_dtype)


# ----------------------------------------------------------------------------------------------
# real-gated linear recurrent unit
# ----------------------------------------------------------------------------------------------
def lru_scan(u: torch.Tensor, z: torch.Tensor, blocks: int, r_bias: torch.Tensor, i_bias: torch.Tensor,
             lam: torch.Tensor, y: torch.Tensor, y_bias: Optional[torch.Tensor], state: torch.Tensor, cu: torch.Tensor,
             slot: torch.Tensor, pos: torch.Tensor, out_dtype: torch.dtype, max_len: int = 0) -> torch.Tensor:
    """Per channel, f32: r = sigmoid(zr + r_bias), i = sigmoid(zi + i_bias), a = exp(-8 r softplus(lam)),
    S <- a S + sqrt(1 - a^2) i u (also for a sequence's first token, from S = 0); returns
    S * gelu_tanh(y + y_bias) in ``out_dtype``.  ``u`` f32 [T, R] (the kernels reuse it as scratch);
    ``z`` f32 [blocks, T, 2 * R / blocks]:
    block b's gate pre-activations [zr | zi] as the batched block-diagonal product leaves them (the
    kernels overwrite it with the gates);
    ``y`` a column slice; ``state`` f32 [slots, R], read unless the segment starts at position 0,
    then replaced.  ``max_len``: the longest segment when known (1 selects the fused single-row kernel)."""
    T, R = u.shape
    S = cu.numel() - 1
    bs = R // blocks
    assert u.dtype == z.dtype == torch.float32 and u.is_contiguous() and z.is_contiguous()
    assert tuple(z.shape) == (blocks, T, 2 * bs)
    if N.use_native(u):
        out = torch.empty((T, R), dtype=out_dtype, device=u.device)
        N.mcall("mx_lru_scan", N.ptr(u), N.ptr(z), blocks, N.ptr(r_bias), N.ptr(i_bias), N.ptr(lam), N.ptr(_rows(y)),
                y.stride(0), _dt(y), N.ptr(y_bias), N.ptr(state), N.ptr(cu), N.ptr(slot), N.ptr(pos), N.ptr(out), _dt(out),
                S, R, T, int(max_len), N.stream())
        return out
    zr = z[:, :, :bs].transpose(0, 1).reshape(T, R)
    zi = z[:, :, bs:].transpose(0, 1).reshape(T, R)
    out = torch.zeros((T, R), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    a = torch.exp(-8.0 * torch.sigmoid(zr + r_bias.float()) * F.softplus(lam.float()))
    bx = torch.sqrt(1.0 - a * a) * torch.sigmoid(zi + i_bias.float()) * u
    yy = y.float() + (y_bias.float() if y_bias is not None else 0.0)
    for s in range(S):
        r0, r1 = cul[s], cul[s + 1]
        if sll[s] < 0 or r1 <= r0:
            continue
        St = torch.zeros(R) if pl[r0] == 0 else state[sll[s]].clone()
        for t in range(r0, r1):
            St = a[t] * St + bx[t]
            out[t] = St
        state[sll[s]] = St
    return (out * F.gelu(yy, approximate="tanh")).to(out_dtype)


# ----------------------------------------------------------------------------------------------
# minimal gated recurrent unit
# ----------------------------------------------------------------------------------------------
def mingru_scan(zp: torch.Tensor, xp: torch.Tensor, gp: torch.Tensor, z_bias: Optional[torch.Tensor],
                x_bias: Optional[torch.Tensor], state: torch.Tensor, cu: torch.Tensor, slot: torch.Tensor,
                pos: torch.Tensor, out_dtype: torch.dtype, max_len: int = 0) -> torch.Tensor:
    """Per channel, f32: z = sigmoid(zp + z_bias), u = xp + x_bias, candidate c = u + 1/2 where u >= 0 and
    sigmoid(u) below, S <- (1 - z) S + z c (gates from the current token only); returns S * silu(gp) in
    ``out_dtype``.  ``zp``, ``xp``, ``gp`` [T, R] are column slices of one projection; ``state`` f32
    [slots, R], read unless the segment starts at position 0, then replaced.  ``max_len``: the longest
    segment when known (1 selects the fused single-row kernel)."""
    T, R = zp.shape
    S = cu.numel() - 1
    assert xp.shape == zp.shape == gp.shape and zp.dtype == xp.dtype == gp.dtype
    if N.use_native(zp):
        out = torch.empty((T, R), dtype=out_dtype, device=zp.device)
        one = max_len == 1
        ab = None if one else torch.empty((T, 2 * R), dtype=torch.float32, device=zp.device)
        gy = None if one else torch.empty((T, R), dtype=torch.float32, device=zp.device)
        N.mcall("mx_mingru_scan", N.ptr(_rows(zp)), zp.stride(0), N.ptr(_rows(xp)), xp.stride(0), N.ptr(_rows(gp)),
                gp.stride(0), _dt(zp), N.ptr(z_bias), N.ptr(x_bias), N.ptr(ab), N.ptr(gy), N.ptr(state), N.ptr(cu),
                N.ptr(slot), N.ptr(pos), N.ptr(out), _dt(out), S, R, T, int(max_len), N.stream())
        return out
    a = zp.float() + (z_bias.float() if z_bias is not None else 0.0)
    u = xp.float() + (x_bias.float() if x_bias is not None else 0.0)
    keep, put = torch.sigmoid(-a), torch.sigmoid(a) * torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    out = torch.zeros((T, R), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    for s in range(S):
        r0, r1 = cul[s], cul[s + 1]
        if sll[s] < 0 or r1 <= r0:
            continue
        St = torch.zeros(R) if pl[r0] == 0 else state[sll[s]].clone()
        for t in range(r0, r1):
            St = keep[t] * St + put[t]
            out[t] = St
        state[sll[s]] = St
    return (out * F.silu(gp.float())).to(out_dtype)


# ----------------------------------------------------------------------------------------------
# sliding-window attention with grouped key/value heads over a paged row cache
# ----------------------------------------------------------------------------------------------
def qk_norm_write(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, qw: Optional[torch.Tensor],
                  kw: Optional[torch.Tensor], eps: float, slots: torch.Tensor, cache: torch.Tensor) -> torch.Tensor:
    """Per token: RMS norm of the WHOLE query projection (all heads at once) times ``qw`` -> returned
    [T, nq]; the same for the key projection with ``kw``; the normed keys and the values go to cache
    row ``slots[t]`` as [k | v] (< 0: no write).  ``qw``/``kw`` None: no norm (without ``qw`` the returned
    queries are ``q`` itself, a column slice: nothing is copied)."""
    T, nq = q.shape
    nk, nv = k.shape[1], v.shape[1]
    assert cache.shape[-1] == nk + nv
    if N.use_native(q):
        assert q.dtype == k.dtype == v.dtype == cache.dtype
        out = torch.empty((T, nq), dtype=q.dtype, device=q.device) if qw is not None else None
        N.mcall("mx_qk_norm_write", N.ptr(_rows(q)), q.stride(0), N.ptr(_rows(k)), k.stride(0), N.ptr(_rows(v)), v.stride(0),
                N.ptr(qw), N.ptr(kw), float(eps), N.ptr(slots), N.ptr(cache), N.ptr(out), _dt(q), T, nq, nk, nv, N.stream())
        return out if out is not None else q
    rms = lambda t, w: (t.float() * torch.rsqrt(t.float().pow(2).mean(-1, keepdim=True) + eps) * w.float()  # noqa: E731
                        if w is not None else t.float())
    rows = torch.cat([rms(k, kw), v.float()], 1).to(cache.dtype)
    ok = slots >= 0
    cache.view(-1, nk + nv)[slots[ok].long()] = rows[ok]
    return rms(q, qw).to(q.dtype) if qw is not None else q


def window_attend(q: torch.Tensor, cache: torch.Tensor, cu: torch.Tensor, pos: torch.Tensor, bt: torch.Tensor,
                  window: int, scale: float, max_len: int, heads: int, kv_heads: int, dim: int, vdim: int,
                  gate: Optional[torch.Tensor] = None, chunked: bool = False, keep_first: int = 0,
                  head_bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Causal softmax attention of ``q`` [T, H*dim] over the cache rows [k: G*dim | v: G*vdim] of each
    segment's pages: the query at position p sees keys j with 0 <= p - j < window, or -- ``chunked`` --
    the keys j <= p with floor(j / window) == floor(p / window) (blocks of ``window`` positions counted
    from the start of the sequence); with ``keep_first`` the keys j < keep_first of the sequence stay
    visible to every later query as well (at their true positions).  Query head h
    reads key/value head h // (H/G); score = q . k * scale, f32 softmax -- or, with ``head_bias`` (f32 [H]),
    no softmax: the weight of a visible key is sigmoid(score + head_bias[h]), not normalised over the keys.
    Head h's output is multiplied by sigmoid(gate[t, h]) when a gate [T, H] is given.  Returns [T, H*vdim]."""
    T = q.shape[0]
    H, G, D, P = heads, kv_heads, dim, vdim
    S = cu.numel() - 1
    Wr = G * (D + P)
    if head_bias is not None and (head_bias.dtype != torch.float32 or head_bias.numel() != H):
        raise ValueError("head_bias: one f32 value per query head")
    if N.use_native(q):
        assert bt.is_contiguous() and q.dtype == cache.dtype
        out = torch.empty((T, H * P), dtype=q.dtype, device=q.device)
        # decode-size steps (one row per segment) walk each row's keys with several blocks so that a
        # small batch still fills the chip; the split depends only on static sizes (graph-safe)
        nsplit, ws = 1, None
        if max_len == 1 and q.dtype == torch.bfloat16:
            tiles = (min(window + keep_first, bt.shape[1] * PAGE) + 31) // 32 + 1
            nsplit = max(1, min(16, tiles // 2, 1024 // max(S * G, 1)))
            if nsplit > 1:
                ws = torch.empty((T, H, nsplit, P + 2), dtype=torch.float32, device=q.device)
        N.mcall("mx_window_attend", N.ptr(_rows(q)), q.stride(0), N.ptr(cache), N.ptr(cu), N.ptr(pos), N.ptr(bt), bt.shape[1],
                N.ptr(_rows(gate)) if gate is not None else None, gate.stride(0) if gate is not None else 0,
                int(min(window, 1 << 30)), 1 if chunked else 0, int(keep_first), N.ptr(head_bias), float(scale), N.ptr(out),
                _dt(q), S, int(max_len), H, G, D, P, nsplit, N.ptr(ws), N.stream())
        return out
    out = torch.zeros((T, H, P), dtype=torch.float32)
    rows = cache.view(-1, Wr).float()
    cul, pl = cu.tolist(), pos.tolist()
    rep = H // G
    for s in range(S):
        a, b = cul[s], cul[s + 1]
        if b <= a:
            continue
        ctx = pl[b - 1] + 1
        pages = bt[s, :(ctx + PAGE - 1) // PAGE].long()
        kv = rows.view(-1, PAGE, Wr)[pages].reshape(-1, Wr)[:ctx]
        keys = kv[:, :G * D].view(ctx, G, D).repeat_interleave(rep, 1)
        vals = kv[:, G * D:].view(ctx, G, P).repeat_interleave(rep, 1)
        sc = torch.einsum("nhd,jhd->nhj", q[a:b].float().view(-1, H, D), keys) * scale
        p = pos[a:b].long()[:, None]
        j = torch.arange(ctx)[None]
        vis = (j <= p) & (((j // window == p // window) if chunked else (j > p - window)) | (j < keep_first))
        if head_bias is not None:
            wt = torch.sigmoid(sc + head_bias.float()[None, :, None]) * vis[:, None, :]
        else:
            wt = torch.softmax(sc.masked_fill(~vis[:, None, :], float("-inf")), -1)
        out[a:b] = torch.einsum("nhj,jhp->nhp", wt, vals)
    if gate is not None:
        out = out * torch.sigmoid(gate.float())[:, :, None]
    return out.reshape(T, H * P).to(q.dtype)


# ----------------------------------------------------------------------------------------------
# several residual streams per token (hyper-connections); logit scale and soft cap
# ----------------------------------------------------------------------------------------------
MAX_STREAMS = 16


def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float = 1.0, copies: int = 1) -> torch.Tensor:
    """``copies`` equal f32 streams [T, copies, W] of ``table[id] * scale``."""
    T, (V, W) = ids.numel(), table.shape
    if N.use_native(table):
        out = torch.empty((T, copies, W), dtype=torch.float32, device=table.device)
        N.mcall("mx_embed_scaled", N.ptr(ids.to(torch.int32).contiguous()), N.ptr(table), _dt(table), float(scale),
                int(copies), N.ptr(out), T, W, V, N.stream())
        return out
    row = table[ids.long().clamp(0, V - 1)].float() * scale
    return row[:, None, :].repeat(1, copies, 1).contiguous()


def hyper_mix(x: torch.Tensor, y: Optional[torch.Tensor], mix: Optional[torch.Tensor], w_out: Optional[torch.Tensor],
              w_in: torch.Tensor, w: Optional[torch.Tensor], eps: float,
              out_dtype: torch.dtype = torch.bfloat16) -> Optional[torch.Tensor]:
    """One pass over the streams ``x`` (f32 [T, S, W], in place) between two sublayers.  With the output
    ``y`` [T, W] of the sublayer that just ran: x_t <- sum_s mix[s, t] x_s + w_out[t] * y for every
    stream t at once (``mix`` f32 [S, S] indexed [from, to], ``w_out`` f32 [S]).  Then the next
    sublayer's input u = sum_t w_in[t] x_t and its RMS norm u / sqrt(mean(u^2) + eps) * w in
    ``out_dtype`` (``w`` None: the update only).  S = 1 with mix = w_out = w_in = 1 is the plain
    pre-norm residual sum."""
    T, S, W = x.shape
    assert x.dtype == torch.float32 and x.is_contiguous()
    if S > MAX_STREAMS:
        raise ValueError(f"at most {MAX_STREAMS} residual streams are supported, got {S}")
    if N.use_native(x):
        out = torch.empty((T, W), dtype=out_dtype, device=x.device) if w is not None else None
        N.mcall("mx_hyper_mix", N.ptr(x), N.ptr(_rows(y)) if y is not None else None, y.stride(0) if y is not None else 0,
                _dt(y) if y is not None else 1, N.ptr(mix), N.ptr(w_out), N.ptr(w_in), N.ptr(w), float(eps), N.ptr(out),
                _dt(out) if out is not None else 1, T, S, W, N.stream())
        return out
    if y is not None:
        new = torch.einsum("st,nsw->ntw", mix.float(), x) + w_out.float()[None, :, None] * y.float()[:, None, :]
        x.copy_(new)
    if w is None:
        return None
    u = torch.einsum("t,ntw->nw", w_in.float(), x)
    return (u * torch.rsqrt(u.pow(2).mean(-1, keepdim=True) + eps) * w.float()).to(out_dtype)


def logit_cap(logits: torch.Tensor, scale: float = 1.0, cap: float = 0.0) -> torch.Tensor:
    """``logits`` <- cap * tanh(logits * scale / cap) in place (``cap`` <= 0: the scale only)."""
    if scale == 1.0 and cap <= 0:
        return logits
    if N.use_native(logits):
        assert logits.is_contiguous()
        N.mcall("mx_logit_cap", N.ptr(logits), _dt(logits), float(scale), float(cap), logits.numel(), N.stream())
        return logits
    v = logits.float() * scale
    if cap > 0:
        v = cap * torch.tanh(v / cap)
    return logits.copy_(v.to(logits.dtype))


# ----------------------------------------------------------------------------------------------
# rotation of projected heads
# ----------------------------------------------------------------------------------------------
def rope_freqs(dims: int, base: float, scaling: Optional[dict] = None, device=None) -> Tuple[torch.Tensor, float]:
    """Frequencies f_i = base^(-2i / dims), i < dims / 2 (f32) and the factor on cos and sin.  With a
    ``scaling`` entry {factor, original, fast, slow} (YaRN): with turn(t) = dims ln(original / (2 pi t)) /
    (2 ln base), lo = max(floor(turn(fast)), 0), hi = min(ceil(turn(slow)), dims - 1) and
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) the frequency is f_i / factor * ramp_i +
    f_i (1 - ramp_i) and cos and sin are multiplied by 0.1 ln(factor) + 1.  A ``scaling`` entry with a factor
    only is linear scaling: every f_i is divided by the factor (positions are stretched), cos and sin unscaled."""
    import math
    i = torch.arange(dims // 2, dtype=torch.float64)
    f = float(base) ** (-2.0 * i / dims)
    m = 1.0
    if scaling and "original" not in scaling:      # linear scaling: every frequency divided by the factor
        f = f / float(scaling["factor"])
    elif scaling:
        factor, orig = float(scaling["factor"]), float(scaling["original"])
        turn = lambda t: dims * math.log(orig / (2 * math.pi * float(t))) / (2 * math.log(float(base)))  # noqa: E731
        lo = max(math.floor(turn(scaling["fast"])), 0)
        hi = min(math.ceil(turn(scaling["slow"])), dims - 1)
        ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
        f = f / factor * ramp + f * (1 - ramp)
        m = 0.1 * math.log(factor) + 1.0
    return f.to(torch.float32).to(device).contiguous(), m


def _rotate_heads(x: torch.Tensor, ang: torch.Tensor, rot: int, half: bool, m: float) -> torch.Tensor:
    """x f32 [T, H, D]; ang f32 [T, rot / 2]."""
    if rot == 0:
        return x
    c, s = (torch.cos(ang) * m)[:, None, :], (torch.sin(ang) * m)[:, None, :]
    out = x.clone()
    if half:
        a, b = x[..., :rot // 2], x[..., rot // 2:rot]
        out[..., :rot // 2] = a * c - b * s
        out[..., rot // 2:rot] = b * c + a * s
    else:
        a, b = x[..., 0:rot:2], x[..., 1:rot:2]
        out[..., 0:rot:2] = a * c - b * s
        out[..., 1:rot:2] = b * c + a * s
    return out


def rope_heads(q: torch.Tensor, k: torch.Tensor, heads: int, kv_heads: int, dim: int, freq: Optional[torch.Tensor],
               pos: torch.Tensor, layout: str = "pairs", mscale: float = 1.0, norm_eps: Optional[float] = None,
               q_scale: float = 1.0, k_scale: float = 1.0, q_dtype: Optional[torch.dtype] = None,
               k_out: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
               v: Optional[torch.Tensor] = None, k_dtype: Optional[torch.dtype] = None,
               v_mix: Optional[torch.Tensor] = None, v_lam: float = 0.0):
    """Per head of ``q`` [T, H*dim] and ``k`` [T, G*dim] (column slices): the first ``2 * len(freq)``
    entries are rotated by the angle pos * freq_i (f32), pair i being entries (2i, 2i+1) for
    ``layout="pairs"`` or (i, i + rot/2) for ``"half"``; (u, v) -> (u cos - v sin, v cos + u sin) with cos and
    sin times ``mscale``; then, with ``norm_eps``, the head is divided by its root mean square over
    ``dim`` (no weight); then times ``q_scale`` / ``k_scale``.  Returns (q', k'): q' [T, H*dim] in
    ``q_dtype``; k' [T, G*dim] in ``k_dtype`` -- or, with ``k_out`` (paged cache rows [rows, G*dim + nv])
    and ``slots`` [T], k' is written to row slots[t] (< 0: no write) followed by the raw values ``v``
    [T, nv], and None is returned for it; with ``v_mix`` ([T, nv]) the values written are
    (1 - v_lam) v + v_lam v_mix, blended in f32."""
    T = q.shape[0]
    H, G, D = heads, kv_heads, dim
    rot = 2 * freq.numel() if freq is not None else 0
    half = layout == "half"
    if layout not in ("pairs", "half") or rot > D:
        raise ValueError("rope_heads: layout is pairs | half and the rotated part must fit the head")
    q_dtype = q_dtype or q.dtype
    norm = norm_eps is not None
    if N.use_native(q):
        assert q.dtype == k.dtype and (v is None or v.dtype == q.dtype)
        qo = torch.empty((T, H * D), dtype=q_dtype, device=q.device)
        if k_out is None:
            ko = torch.empty((T, G * D), dtype=k_dtype or k.dtype, device=q.device)
            dst, sko, sl, nv = ko, G * D, None, 0
        else:
            nv = v.shape[1] if v is not None else 0
            assert k_out.shape[-1] >= G * D + nv and k_out.stride(-1) == 1 and slots is not None
            assert v_mix is None or (v is not None and v_mix.shape == v.shape and v_mix.dtype == v.dtype)
            ko, dst, sko, sl = None, k_out, k_out.shape[-1], slots
        N.mcall("mx_rope_heads", N.ptr(_rows(q)), q.stride(0), H, N.ptr(_rows(k)), k.stride(0), G, _dt(q), D, rot,
                1 if half else 0, N.ptr(freq), float(mscale), N.ptr(pos), 1 if norm else 0, float(norm_eps or 0.0),
                float(q_scale), float(k_scale), N.ptr(qo), _dt(qo), N.ptr(dst), sko, _dt(dst), N.ptr(sl),
                N.ptr(_rows(v)) if v is not None else None, v.stride(0) if v is not None else 0, nv,
                N.ptr(_rows(v_mix)) if v_mix is not None else None, v_mix.stride(0) if v_mix is not None else 0,
                float(v_lam), T, N.stream())
        return qo, ko
    ang = pos.float()[:, None] * freq.float()[None, :] if rot else None

    def prep(x, nh, sc):
        x = _rotate_heads(x.float().reshape(T, nh, D), ang, rot, half, mscale)
        if norm:
            x = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + norm_eps)
        return (x * sc).reshape(T, nh * D)

    qo = prep(q, H, q_scale).to(q_dtype)
    kk = prep(k, G, k_scale)
    if k_out is None:
        return qo, kk.to(k_dtype or k.dtype)
    vv = v.float() if v is not None else None
    if v_mix is not None:
        vv = (1.0 - v_lam) * vv + v_lam * v_mix.float()
    rows = torch.cat([kk] + ([vv] if vv is not None else []), 1).to(k_out.dtype)
    ok = slots >= 0
    k_out.view(-1, k_out.shape[-1])[slots[ok].long(), :rows.shape[1]] = rows[ok]
    return qo, None


# ----------------------------------------------------------------------------------------------
# matrix-state recurrence with one fixed decay per head
# ----------------------------------------------------------------------------------------------
def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, state: torch.Tensor,
               cu: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, heads: int, dim: int, vdim: int,
               act: str = "none", out_scale: float = 1.0, max_len: int = 0) -> torch.Tensor:
    """Token-by-token f32 recurrence over a [dim, vdim] state per head with a constant decay per head:
    S <- decay[h] S + act(k) act(v)^T, o = S^T act(q) * out_scale.  ``q``, ``k`` [T, H*dim] (one storage
    type) and ``v`` [T, H*vdim] (possibly another) are column slices; ``act``: none | silu, applied to
    all three; ``decay`` f32 [H]; ``state`` f32 [slots, H, dim, vdim], read unless the segment starts at
    position 0, then replaced.  Returns o f32 [T, H*vdim]."""
    T = q.shape[0]
    H, D, P = heads, dim, vdim
    S = cu.numel() - 1
    assert q.dtype == k.dtype and q.shape[1] == H * D and k.shape[1] == H * D and v.shape[1] == H * P
    assert decay.dtype == torch.float32 and decay.numel() == H and act in ("none", "silu")
    if N.use_native(q):
        out = torch.empty((T, H * P), dtype=torch.float32, device=q.device)
        N.mcall("mx_decay_scan", N.ptr(_rows(q)), q.stride(0), N.ptr(_rows(k)), k.stride(0), _dt(q), N.ptr(_rows(v)),
                v.stride(0), _dt(v), ACTS[act], N.ptr(decay), float(out_scale), N.ptr(state), N.ptr(cu), N.ptr(slot),
                N.ptr(pos), N.ptr(out), S, T, int(max_len), H, D, P, N.stream())
        return out
    out = torch.zeros((T, H * P), dtype=torch.float32)
    cul, sll, pl = cu.tolist(), slot.tolist(), pos.tolist()
    g = decay.float()[:, None, None]
    for s in range(S):
        r0, r1 = cul[s], cul[s + 1]
        if sll[s] < 0 or r1 <= r0:
            continue
        n = r1 - r0
        qq = _act(q[r0:r1].float(), act).view(n, H, D)
        kk = _act(k[r0:r1].float(), act).view(n, H, D)
        vv = _act(v[r0:r1].float(), act).view(n, H, P)
        St = torch.zeros((H, D, P)) if pl[r0] == 0 else state[sll[s]].clone()
        for t in range(n):
            St = g * St + kk[t][:, :, None] * vv[t][:, None, :]
            out[r0 + t] = (torch.einsum("hdp,hd->hp", St, qq[t]) * out_scale).reshape(-1)
        state[sll[s]] = St
    return out
