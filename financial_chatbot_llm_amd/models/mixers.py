"""Building blocks of layered (hybrid) decoders: sequence mixers and feed-forwards that read one
normed input ``h`` and return a sublayer output, with their sizes and constants as parameters.

* :class:`Mamba2Mixer` -- state-space duality layer (causal short convolution + selective scan with
  an f32 state per sequence slot, gated grouped RMS norm, output projection).
* :class:`LatentAttentionMixer` -- attention whose keys and values are up-projections of one cached
  latent per token plus one shared rotated key part; runs in the latent space over a paged latent
  cache with a sliding window and a per-head sigmoid output gate.
* :class:`ChannelDeltaMixer` -- gated delta rule with one decay per head and key channel (short
  convolutions on q, k, v; unit-norm q and k; low-rank decay and output-gate projections).
* :class:`GLAMixer` -- gated linear attention: the same matrix state with a plain k v^T write and a
  decay sigmoid(.)^(1/tau) per key channel.
* :class:`WindowAttentionMixer` -- softmax attention over a paged [keys | values] row cache with
  grouped key/value heads, RMS norm over the whole query / key projection, a sliding window, no
  positional rotation and a per-head sigmoid output gate.
* :class:`GatedLRUMixer` -- real-gated linear recurrent unit block (GeLU branch times a
  convolved, block-diagonally gated diagonal recurrence).
* :class:`ParallelMixer` -- two of the above side by side on the same input; the layer combines their
  RMS-normed outputs.
* :class:`LightningMixer` -- linear attention with one fixed decay per head on SiLU-activated q, k, v,
  an RMS norm over all heads and a sigmoid output gate.
* :class:`RetentionMixer` -- the same recurrence on rotated q and k (half-split pairs), a weightless RMS
  norm per head and a SiLU output gate.
* :class:`ChunkAttentionMixer` -- softmax attention whose values are the keys as projected; biased q / k
  projections, pairwise rotation with optionally scaled frequencies, weightless per-head RMS norm of q
  and k after the rotation, and a chunked mask (a query sees the keys of its own block of positions).
* :class:`SigmoidAttentionMixer` -- causal attention without positions and without softmax: independent
  sigmoid weights sigmoid(score + a bias per head), not normalised over the keys.
* :class:`MinGRUMixer` -- minimal gated recurrent unit: a diagonal recurrence whose update gate and
  candidate read only the current token, with a SiLU output gate.
* :class:`WeightedParallelMixer` -- two mixers side by side whose outputs are summed with fixed weights.
* :class:`SinkWindowAttentionMixer` -- softmax attention with half-split rotation on part of each head,
  weightless per-head RMS norm of q and k after the rotation, a sliding window that also keeps the first
  tokens of the sequence, and values blended with those of the model's first such layer.
* :class:`PlainLatentAttentionMixer` -- latent attention without positions: keys and values are
  up-projections of one cached normed latent per token, plain causal softmax.
* :class:`DenseFF` -- up, activation, down; optionally gated (act(gate) * up).
* :class:`TopSoftmaxRoutedFF` -- mixture of plain relu^2 experts, softmax over the chosen logits, plus a
  shared expert.
* :class:`RoutedFF` -- mixture of clamped gated experts with biased top-k choice, identity experts
  and an always-on shared expert.
* :class:`InputScaledRoutedFF` -- mixture of gated experts chosen by independent sigmoid scores, the
  score multiplying the expert's input.

A shape entry of ``None`` in ``shapes()`` is a size only the checkpoint's tensor gives (a low-rank
projection's rank).

Every block declares the rows it needs from a fused in-projection (``in_weight``): a layer stacks
its mixer's and its feed-forward's rows into ONE GEMM over ``h`` and hands each block its column
slice.  GEMMs are vendor matrix products (``F.linear`` / ``bmm``) on bf16 or f32 weights; everything
else runs on the kernels behind :mod:`..ops.mixers`.
"""
from __future__ import annotations

from typing import Callable, Dict, Optional

import torch
import torch.nn.functional as F

from ..ops import mixers as mx
from .common import AttentionMetadata

Getter = Callable[[str], torch.Tensor]

# steps with at most this many (token, expert) pairs run every expert over every row (no host sync:
# hipGraph-capturable, and a decode step streams all expert weights anyway); larger steps bucket
# the rows by expert and read the bucket sizes on the host once per layer
DENSE_MAX_PAIRS = 512


def _capturing(t: torch.Tensor) -> bool:
    return t.is_cuda and torch.cuda.is_current_stream_capturing()


class Mamba2Mixer:
    kind = "mamba2"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.P, self.N = int(spec["heads"]), int(spec["vdim"]), int(spec["state"])
        self.G, self.K = int(spec.get("groups", 1)), int(spec["conv"])
        self.norm_groups = int(spec.get("norm_groups", 1))
        self.inner = self.H * self.P
        self.C = self.inner + 2 * self.G * self.N          # convolved channels: x | B | C
        self.in_rows = 2 * self.inner + 2 * self.G * self.N + self.H   # z | x | B | C | dt
        self.width, self.eps = width, eps
        if self.H % self.G or self.inner % self.norm_groups:
            raise ValueError("mamba2: heads must split into groups and inner into norm_groups")
        if self.N > 256 or not 1 <= self.K <= 8:
            raise ValueError("mamba2: state <= 256 and 1 <= conv taps <= 8 are supported")

    def shapes(self) -> Dict[str, tuple]:
        return {"in": (self.in_rows, self.width), "conv": (self.C, self.K), "conv.b": (self.C,), "dt_bias": (self.H,),
                "A_log": (self.H,), "D": (self.H,), "norm": (self.inner,), "o": (self.width, self.inner)}

    def cache_spec(self):
        return ("state", self.K, self.C, self.H, self.P, self.N)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        f32 = lambda n: get(n).float().contiguous()  # noqa: E731
        self.conv_w, self.conv_b = f32("conv"), f32("conv.b")
        self.dt_bias, self.A_log, self.D, self.norm_w = f32("dt_bias"), f32("A_log"), f32("D"), f32("norm")
        self.o = get("o").to(dtype).contiguous()
        return get("in").to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.conv_w, self.conv_b, self.norm_w, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        _, conv_state, ssm_state = cache
        z = proj[:, :self.inner]
        xbc = proj[:, self.inner:self.inner + self.C]
        dt = proj[:, self.inner + self.C:self.inner + self.C + self.H]
        u = mx.conv_silu(xbc, self.conv_w, self.conv_b, conv_state, meta.seg_cu, meta.seg_state, positions,
                         meta.seg_max_len)
        y = mx.ssm_scan(u, dt, self.dt_bias, self.A_log, self.D, ssm_state, meta.seg_cu, meta.seg_state, positions,
                        self.H, self.P, self.N, self.G)
        # the gate comes before the norm: rms over silu(z) * y, in norm_groups equal parts
        yn = mx.group_norm(y, self.norm_w, self.eps, self.norm_groups, gate=z, out_dtype=proj.dtype)
        return F.linear(yn, self.o)


class LatentAttentionMixer:
    kind = "latent_attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.dn, self.dr, self.dv = int(spec["heads"]), int(spec["dim"]), int(spec["rot_dim"]), int(spec["vdim"])
        self.R, self.q_rank = int(spec["kv_rank"]), int(spec["q_rank"])
        rot = spec.get("rot") or {}
        self.rot_dims = int(rot.get("dims", self.dr))
        self.rot_base = float(rot.get("base", 10000.0))
        mask = spec.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 1 << 30      # no mask entry: plain causal
        self.scale = float(spec["scale"]) if "scale" in spec else (self.dn + self.dr) ** -0.5
        self.in_rows = self.q_rank + self.R + self.dr + self.H                # c_q | c, k_rot | gate
        self.width, self.eps = width, eps
        if self.rot_dims > self.dr or self.rot_dims % 2 or self.R > 512:
            raise ValueError("latent_attention: rot.dims must be even and <= rot_dim, kv_rank <= 512")

    def shapes(self) -> Dict[str, tuple]:
        H, dq = self.H, self.dn + self.dr
        return {"dq": (self.q_rank, self.width), "dq.norm": (self.q_rank,), "uq": (H * dq, self.q_rank),
                "dkv": (self.R + self.dr, self.width), "dkv.norm": (self.R,), "uk": (H * self.dn, self.R),
                "uv": (H * self.dv, self.R), "g": (H, self.width), "o": (self.width, H * self.dv)}

    def cache_spec(self):
        return ("latent", self.R + self.dr)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.dq_norm = get("dq.norm").float().contiguous()
        self.dkv_norm = get("dkv.norm").float().contiguous()
        self.uq = get("uq").to(dtype).contiguous()
        self.uk = get("uk").to(dtype).view(self.H, self.dn, self.R).contiguous()      # [H, dn, R]
        self.uv_t = get("uv").to(dtype).view(self.H, self.dv, self.R).transpose(1, 2).contiguous()  # [H, R, dv]
        self.o = get("o").to(dtype).contiguous()
        self.inv_freq = mx.rope_inv_freq(self.rot_dims, self.rot_base, device=self.uq.device)
        return torch.cat([get("dq"), get("dkv"), get("g")], 0).to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.uq, self.uk, self.uv_t, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        rows = cache[1]
        T = proj.shape[0]
        H, dn, dr, R = self.H, self.dn, self.dr, self.R
        a = self.q_rank
        cq = mx.group_norm(proj[:, :a], self.dq_norm, self.eps, 1)
        kv = proj[:, a:a + R + dr]
        gate = proj[:, a + R + dr:a + R + dr + H]
        q = F.linear(cq, self.uq)                                            # [T, H * (dn + dr)]
        # latent row + shared rotated key into the cache; every head's rotated query part
        q_rot = mx.latent_prep(kv, self.dkv_norm, self.eps, self.inv_freq, self.rot_dims, positions, meta.slots, rows,
                               q, H, dn + dr, dn, R, dr)
        # fold each head's key up-projection into its query: q_lat[h] = W_uk[h]^T q_nope[h]
        q_nope = q.view(T, H, dn + dr)[:, :, :dn]
        q_lat = torch.bmm(q_nope.transpose(0, 1), self.uk).transpose(0, 1).contiguous()   # [T, H, R]
        o_lat = mx.latent_attend(q_lat, q_rot, rows, meta.seg_cu, positions, meta.seg_bt, self.window, self.scale,
                                 meta.seg_max_len, gate=gate)
        o = torch.bmm(o_lat.transpose(0, 1), self.uv_t).transpose(0, 1).reshape(T, H * self.dv)
        return F.linear(o, self.o)


class DenseFF:
    """W_down act(W_up h), ``act`` = "relu2" (the square of relu) | gelu_tanh | silu; or, ``gated``,
    W_down (act(W_gate h) * (W_up h)) with ``act`` in silu | gelu_tanh."""

    def __init__(self, spec: Dict, width: int, act: str = "relu2", gated: bool = False):
        self.ff, self.width, self.act, self.gated = int(spec["ff"]), width, act, gated
        self.in_rows = self.ff * (2 if gated else 1)
        if act not in (("silu", "gelu_tanh") if gated else ("relu2", "silu", "gelu_tanh")):
            raise ValueError(f"unknown activation {act!r} for a {'gated' if gated else 'plain'} feed-forward")

    def shapes(self) -> Dict[str, tuple]:
        s = {"up": (self.ff, self.width), "down": (self.width, self.ff)}
        if self.gated:
            s["gate"] = (self.ff, self.width)
        return s

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.down = get("down").to(dtype).contiguous()
        if self.gated:
            return torch.cat([get("gate"), get("up")], 0).to(dtype)
        return get("up").to(dtype)

    def num_bytes(self) -> int:
        return self.down.numel() * self.down.element_size()

    def forward(self, h: torch.Tensor, proj: torch.Tensor, x32: Optional[torch.Tensor] = None) -> torch.Tensor:
        if self.gated:
            return F.linear(mx.glu_act(proj[:, :self.ff], proj[:, self.ff:2 * self.ff], self.act), self.down)
        up = proj[:, :self.ff]
        return F.linear(mx.relu2(up) if self.act == "relu2" else mx.glu_act(up, None, self.act), self.down)


class RoutedFF:
    """Mixture of ``experts`` clamped gated feed-forwards, ``top`` per token.

    Router logits z = W_r h in f32; scores s = softmax(z) over the experts and the ``identity``
    experts that follow them; the ``top`` largest s + correction are chosen and weighted by s itself.
    An identity expert returns its input.  Expert: g = min(W_g h, limit), u = clamp(W_u h, +-limit),
    W_d (g * sigmoid(alpha g) * (u + 1)).  A shared expert of the same form runs for every token."""

    def __init__(self, spec: Dict, width: int, alpha: float = 1.702):
        r = spec["router"]
        self.E, self.I, self.top = int(r["experts"]), int(r.get("identity", 0)), int(r["top"])
        self.F = int(spec["expert"]["ff"])
        self.limit = float(spec["expert"]["limit"])
        sh = spec.get("shared")
        self.Fs = int(sh["ff"]) if sh else 0
        self.limit_s = float(sh["limit"]) if sh else 0.0
        self.alpha, self.width = alpha, width
        self.in_rows = 2 * self.Fs                                            # shared gate | up

    def shapes(self) -> Dict[str, tuple]:
        s = {"router": (self.E + self.I, self.width), "correction": (self.E + self.I,)}
        for e in range(self.E):
            s.update({f"e{e}.gate": (self.F, self.width), f"e{e}.up": (self.F, self.width),
                      f"e{e}.down": (self.width, self.F)})
        if self.Fs:
            s.update({"shared.gate": (self.Fs, self.width), "shared.up": (self.Fs, self.width),
                      "shared.down": (self.width, self.Fs)})
        return s

    def load(self, get: Getter, dtype) -> Optional[torch.Tensor]:
        self.router = get("router").float().contiguous()
        self.correction = get("correction").float().contiguous()
        self.w13 = torch.stack([torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")], 0) for e in range(self.E)]).to(dtype)
        self.w2 = torch.stack([get(f"e{e}.down") for e in range(self.E)]).to(dtype).contiguous()
        if not self.Fs:
            return None
        self.down_s = get("shared.down").to(dtype).contiguous()
        return torch.cat([get("shared.gate"), get("shared.up")], 0).to(dtype)

    def num_bytes(self) -> int:
        ts = [self.router, self.w13, self.w2] + ([self.down_s] if self.Fs else [])
        return sum(t.numel() * t.element_size() for t in ts)

    def forward(self, h: torch.Tensor, proj: Optional[torch.Tensor]) -> torch.Tensor:
        T, W = h.shape
        E, top, Fe = self.E, self.top, self.F
        shared = None
        if self.Fs:
            shared = F.linear(mx.glu_clamp(proj[:, :self.Fs], proj[:, self.Fs:2 * self.Fs], self.limit_s, self.alpha),
                              self.down_s)
        wts, idx = mx.route_biased(F.linear(h.float(), self.router), self.correction, top)
        if T * top <= DENSE_MAX_PAIRS or _capturing(h):
            gu = torch.bmm(h.unsqueeze(0).expand(E, T, W), self.w13.transpose(1, 2)).view(E * T, 2 * Fe)
            act = mx.glu_clamp(gu[:, :Fe], gu[:, Fe:], self.limit, self.alpha)
            ys = torch.bmm(act.view(E, T, Fe), self.w2.transpose(1, 2)).view(E * T, W)
            rows = torch.arange(T, dtype=torch.int32, device=h.device)[:, None]
            pos = (idx.clamp(max=E - 1) * T + rows).to(torch.int32)
            return mx.moe_combine(ys, pos, idx, wts, h, shared, E)
        flat = idx.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        offs = [0] + torch.bincount(flat, minlength=E + self.I).cumsum(0).tolist()     # host read of the buckets
        xs = h.index_select(0, order // top)
        ys = torch.empty((T * top, W), dtype=h.dtype, device=h.device)
        for e in range(E):
            a, b = offs[e], offs[e + 1]
            if b > a:
                gu = F.linear(xs[a:b], self.w13[e])
                torch.mm(mx.glu_clamp(gu[:, :Fe], gu[:, Fe:], self.limit, self.alpha), self.w2[e].t(), out=ys[a:b])
        pos = torch.empty_like(order)
        pos[order] = torch.arange(order.numel(), device=order.device)
        return mx.moe_combine(ys, pos.view(T, top).to(torch.int32), idx, wts, h, shared, E)


class InputScaledRoutedFF:
    """Mixture of ``experts`` gated feed-forwards without biases, ``top`` per token.

    Router logits z = W_r h in f32, scores s = sigmoid(z) (``score``; each expert on its own); the
    ``top`` largest are chosen and their scores are the weights, not renormalised.  The weight
    multiplies the expert's INPUT: out = sum_e expert_e(s_e h), expert(x) = W_d (act(W_g x) * (W_u x)).
    Since W (s h) = s (W h), the experts' first projections run on h itself and the activation
    kernel applies s to both halves."""

    def __init__(self, spec: Dict, width: int, act: str = "silu", score: str = "sigmoid"):
        r = spec["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        self.F = int(spec["expert"]["ff"])
        self.act, self.score, self.width = act, score, width
        self.in_rows = 0
        if not 1 <= self.top <= self.E:
            raise ValueError("routed feed-forward: 1 <= top <= experts")

    def shapes(self) -> Dict[str, tuple]:
        s = {"router": (self.E, self.width)}
        for e in range(self.E):
            s.update({f"e{e}.gate": (self.F, self.width), f"e{e}.up": (self.F, self.width),
                      f"e{e}.down": (self.width, self.F)})
        return s

    def load(self, get: Getter, dtype) -> Optional[torch.Tensor]:
        self.router = get("router").float().contiguous()
        self.w13 = torch.stack([torch.cat([get(f"e{e}.gate"), get(f"e{e}.up")], 0) for e in range(self.E)]).to(dtype)
        self.w2 = torch.stack([get(f"e{e}.down") for e in range(self.E)]).to(dtype).contiguous()
        return None

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.router, self.w13, self.w2))

    def forward(self, h: torch.Tensor, proj: Optional[torch.Tensor] = None, x32: Optional[torch.Tensor] = None) -> torch.Tensor:
        """``x32``: the f32 input ``h`` was rounded from, when the caller has it: the router then reads the
        unrounded values (fewer swapped near-ties against an exact evaluation)."""
        T, W = h.shape
        E, top, Fe = self.E, self.top, self.F
        wts, idx = mx.route_scores(F.linear(x32 if x32 is not None else h.float(), self.router), top, self.score)
        ones = torch.ones_like(wts)
        if T * top <= DENSE_MAX_PAIRS or _capturing(h):
            # every expert over every row; rows an expert was not chosen for get scale 0 and are not read
            rows = torch.arange(T, device=h.device)[:, None]
            pos = idx.long() * T + rows
            scale = torch.zeros(E * T, dtype=torch.float32, device=h.device).scatter_(0, pos.reshape(-1), wts.reshape(-1))
            gu = torch.bmm(h.unsqueeze(0).expand(E, T, W), self.w13.transpose(1, 2)).view(E * T, 2 * Fe)
            act = mx.glu_act(gu[:, :Fe], gu[:, Fe:], self.act, scale)
            ys = torch.bmm(act.view(E, T, Fe), self.w2.transpose(1, 2)).view(E * T, W)
            return mx.moe_combine(ys, pos.to(torch.int32), idx, ones, h, None, E)
        flat = idx.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        offs = [0] + torch.bincount(flat, minlength=E).cumsum(0).tolist()              # host read of the buckets
        xs = h.index_select(0, order // top)
        sc = wts.reshape(-1)[order].contiguous()
        # one GEMM pair per expert with rows; the activation runs once over all buckets
        gu = torch.empty((T * top, 2 * Fe), dtype=h.dtype, device=h.device)
        live = [(e, offs[e], offs[e + 1]) for e in range(E) if offs[e + 1] > offs[e]]
        for e, a, b in live:
            torch.mm(xs[a:b], self.w13[e].t(), out=gu[a:b])
        act = mx.glu_act(gu[:, :Fe], gu[:, Fe:], self.act, sc)
        ys = torch.empty((T * top, W), dtype=h.dtype, device=h.device)
        for e, a, b in live:
            torch.mm(act[a:b], self.w2[e].t(), out=ys[a:b])
        pos = torch.empty_like(order)
        pos[order] = torch.arange(order.numel(), device=order.device)
        return mx.moe_combine(ys, pos.view(T, top).to(torch.int32), idx, ones, h, None, E)


class TopSoftmaxRoutedFF:
    """Mixture of ``experts`` plain feed-forwards W_down act(W_up h) (``act``: the square of relu, no
    biases), ``top`` per token: router logits z = W_r h in f32, the ``top`` largest chosen (ties: the
    lower index), weights = softmax over the chosen logits only; the output is the weighted sum of
    the chosen experts' outputs plus, with a ``shared`` entry, an always-on expert of the same form."""

    def __init__(self, spec: Dict, width: int, act: str = "relu2"):
        r = spec["router"]
        self.E, self.top = int(r["experts"]), int(r["top"])
        self.F = int(spec["expert"]["ff"])
        sh = spec.get("shared")
        self.Fs = int(sh["ff"]) if sh else 0
        self.act, self.width = act, width
        self.in_rows = self.Fs                                            # the shared expert's up rows
        if not 1 <= self.top <= self.E or act != "relu2":
            raise ValueError("routed feed-forward: 1 <= top <= experts, activation relu2")

    def shapes(self) -> Dict[str, tuple]:
        s = {"router": (self.E, self.width)}
        for e in range(self.E):
            s.update({f"e{e}.up": (self.F, self.width), f"e{e}.down": (self.width, self.F)})
        if self.Fs:
            s.update({"shared.up": (self.Fs, self.width), "shared.down": (self.width, self.Fs)})
        return s

    def load(self, get: Getter, dtype) -> Optional[torch.Tensor]:
        self.router = get("router").float().contiguous()
        self.w1 = torch.stack([get(f"e{e}.up") for e in range(self.E)]).to(dtype).contiguous()        # [E, F, W]
        self.w2 = torch.stack([get(f"e{e}.down") for e in range(self.E)]).to(dtype).contiguous()      # [E, W, F]
        if not self.Fs:
            return None
        self.down_s = get("shared.down").to(dtype).contiguous()
        return get("shared.up").to(dtype)

    def num_bytes(self) -> int:
        ts = [self.router, self.w1, self.w2] + ([self.down_s] if self.Fs else [])
        return sum(t.numel() * t.element_size() for t in ts)

    def forward(self, h: torch.Tensor, proj: Optional[torch.Tensor] = None, x32: Optional[torch.Tensor] = None) -> torch.Tensor:
        T, W = h.shape
        E, top, Fe = self.E, self.top, self.F
        shared = F.linear(mx.relu2(proj[:, :self.Fs]), self.down_s) if self.Fs else None
        wts, idx = mx.route_scores(F.linear(x32 if x32 is not None else h.float(), self.router), top, "softmax_top")
        if T * top <= DENSE_MAX_PAIRS or _capturing(h):
            up = torch.bmm(h.unsqueeze(0).expand(E, T, W), self.w1.transpose(1, 2)).view(E * T, Fe)
            ys = torch.bmm(mx.relu2(up).view(E, T, Fe), self.w2.transpose(1, 2)).view(E * T, W)
            rows = torch.arange(T, dtype=torch.int32, device=h.device)[:, None]
            return mx.moe_combine(ys, (idx * T + rows).to(torch.int32), idx, wts, h, shared, E)
        flat = idx.reshape(-1).long()
        order = torch.argsort(flat, stable=True)
        offs = [0] + torch.bincount(flat, minlength=E).cumsum(0).tolist()              # host read of the buckets
        xs = h.index_select(0, order // top)
        up = torch.empty((T * top, Fe), dtype=h.dtype, device=h.device)
        live = [(e, offs[e], offs[e + 1]) for e in range(E) if offs[e + 1] > offs[e]]
        for e, a, b in live:
            torch.mm(xs[a:b], self.w1[e].t(), out=up[a:b])
        act = mx.relu2(up)                                   # one activation launch over all buckets
        ys = torch.empty((T * top, W), dtype=h.dtype, device=h.device)
        for e, a, b in live:
            torch.mm(act[a:b], self.w2[e].t(), out=ys[a:b])
        pos = torch.empty_like(order)
        pos[order] = torch.arange(order.numel(), device=order.device)
        return mx.moe_combine(ys, pos.view(T, top).to(torch.int32), idx, wts, h, shared, E)


def _f32(get: Getter, name: str) -> torch.Tensor:
    return get(name).float().contiguous()


class ChannelDeltaMixer:
    """Gated delta rule with a decay per head and key channel.

    q = W_q h, k = W_k h ([kv_heads, dim]), v = W_v h ([heads, vdim]); each through a causal
    per-channel convolution (no bias) and SiLU; q and k become unit vectors per head (q also times
    dim^-1/2); b = sigmoid(W_b h) per head; g = exp(-exp(A_log_h) softplus(W_a2 W_a1 h + dt_bias)) per
    head and key channel.  Per head, on the f32 state S [dim, vdim]:
    S <- g S;  u = b (v - S^T k);  S <- S + k u^T;  o = S^T q.
    Output: o / rms(o) * w_norm * sigmoid(W_g2 W_g1 h), then W_o.  Slot state: S and the last
    taps - 1 inputs of the three convolutions."""
    kind = "channel_delta"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.G = int(spec["heads"]), int(spec.get("kv_heads", spec["heads"]))
        self.D, self.P, self.K = int(spec["dim"]), int(spec["vdim"]), int(spec["conv"])
        self.ra, self.rg = spec.get("decay_rank"), spec.get("gate_rank")      # set by the checkpoint's shapes
        self.width, self.eps = width, eps
        if self.H % self.G or not 1 <= self.K <= 8 or self.D > 512:
            raise ValueError("channel_delta: heads must split into kv_heads, 1 <= conv taps <= 8, dim <= 512")
        self.nq, self.nv = self.G * self.D, self.H * self.P
        self.C = 2 * self.nq + self.nv

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "q.conv": (self.nq, self.K), "k": (self.nq, W), "k.conv": (self.nq, self.K),
                "v": (self.nv, W), "v.conv": (self.nv, self.K), "b": (self.H, W), "A_log": (self.H,), "norm": (self.P,),
                "a1": (self.ra, W), "a2": (self.H * self.D, self.ra), "dt_bias": (self.H * self.D,),
                "g1": (self.rg, W), "g2": (self.nv, self.rg), "o": (W, self.nv)}

    def cache_spec(self):
        return ("slots", {"conv": (max(self.K - 1, 1), self.C), "S": (self.H, self.D, self.P)})

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.conv_w = torch.cat([_f32(get, "q.conv"), _f32(get, "k.conv"), _f32(get, "v.conv")], 0).contiguous()
        self.A_log, self.dt_bias, self.norm_w = _f32(get, "A_log"), _f32(get, "dt_bias"), _f32(get, "norm")
        self.a2 = _f32(get, "a2")                 # the decay's pre-activation is computed in f32
        self.g2 = get("g2").to(dtype).contiguous()
        self.o = get("o").to(dtype).contiguous()
        self.ra, self.rg = self.a2.shape[1], self.g2.shape[1]
        self.in_rows = self.C + self.H + self.ra + self.rg
        return torch.cat([get("q"), get("k"), get("v"), get("b"), get("a1"), get("g1")], 0).to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.conv_w, self.a2, self.g2, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        st = cache[1]
        C, H, nq = self.C, self.H, self.nq
        u = mx.conv_act(proj[:, :C], self.conv_w, None, st["conv"], meta.seg_cu, meta.seg_state, positions,
                        meta.seg_max_len, "silu")
        beta = proj[:, C:C + H]
        a = F.linear(proj[:, C + H:C + H + self.ra].float(), self.a2)
        o = mx.matrix_scan(u[:, :nq], u[:, nq:2 * nq], u[:, 2 * nq:], a, self.dt_bias, st["S"], meta.seg_cu,
                           meta.seg_state, positions, H, self.G, self.D, self.P, "delta", A_log=self.A_log, beta=beta,
                           max_len=meta.seg_max_len)
        gate = F.linear(proj[:, C + H + self.ra:C + H + self.ra + self.rg], self.g2)
        return F.linear(mx.head_norm_gate(o, self.norm_w, self.eps, gate, H, "sigmoid", proj.dtype), self.o)


class GLAMixer:
    """Gated linear attention: q = W_q h dim^-1/2, k = W_k h ([heads, dim]), v = W_v h ([heads, vdim]);
    decay per head and key channel alpha = sigmoid(W_a2 W_a1 h + b_a2)^(1/tau); on the f32 state
    S [dim, vdim]: S <- diag(alpha) S + k v^T, o = S^T q.  Output: RMS norm of each head's o times
    w_norm, times silu(W_g h), then W_o."""
    kind = "gla"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.D, self.P = int(spec["heads"]), int(spec["dim"]), int(spec["vdim"])
        self.tau = float(spec.get("tau", 1.0))
        self.ra = spec.get("decay_rank")
        self.width, self.eps = width, eps
        if self.D > 512 or self.tau <= 0:
            raise ValueError("gla: dim <= 512 and tau > 0")
        self.nq, self.nv = self.H * self.D, self.H * self.P

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "k": (self.nq, W), "v": (self.nv, W), "g": (self.nv, W), "o": (W, self.nv),
                "norm": (self.P,), "a1": (self.ra, W), "a2": (self.nq, self.ra), "a2.b": (self.nq,)}

    def cache_spec(self):
        return ("slots", {"S": (self.H, self.D, self.P)})

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.a2, self.a2_b, self.norm_w = _f32(get, "a2"), _f32(get, "a2.b"), _f32(get, "norm")
        self.o = get("o").to(dtype).contiguous()
        self.ra = self.a2.shape[1]
        self.in_rows = 2 * self.nq + 2 * self.nv + self.ra
        return torch.cat([get("q"), get("k"), get("v"), get("g"), get("a1")], 0).to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.a2, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        st = cache[1]
        nq, nv = self.nq, self.nv
        a = F.linear(proj[:, 2 * nq + 2 * nv:2 * nq + 2 * nv + self.ra].float(), self.a2)
        o = mx.matrix_scan(proj[:, :nq], proj[:, nq:2 * nq], proj[:, 2 * nq:2 * nq + nv], a, self.a2_b, st["S"],
                           meta.seg_cu, meta.seg_state, positions, self.H, self.H, self.D, self.P, "gla", tau=self.tau,
                           max_len=meta.seg_max_len)
        gate = proj[:, 2 * nq + nv:2 * nq + 2 * nv]
        return F.linear(mx.head_norm_gate(o, self.norm_w, self.eps, gate, self.H, "silu", proj.dtype), self.o)


class WindowAttentionMixer:
    """Softmax attention with ``kv_heads`` key/value heads (query head h reads head h // (H/G)), key
    size ``dim`` and value size ``vdim``; RMS norm over the WHOLE query and key projections (before the
    split into heads) with plain weights; no rotation; score = q . k * scale; sliding window
    0 <= i - j < mask.size (no ``mask`` entry: plain causal); head h's output times
    sigmoid(W_g h)_h; then W_o.  The cache holds one row [k | v] per token."""
    kind = "window_attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.G = int(spec["heads"]), int(spec.get("kv_heads", spec["heads"]))
        self.D, self.P = int(spec["dim"]), int(spec["vdim"])
        mask = spec.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 1 << 30
        self.scale = float(spec["scale"]) if "scale" in spec else self.D ** -0.5
        self.width, self.eps = width, eps
        if self.H % self.G or self.D > 512 or self.P > 512:
            raise ValueError("window_attention: heads must split into kv_heads; dim, vdim <= 512")
        self.nq, self.nk, self.nv = self.H * self.D, self.G * self.D, self.G * self.P
        self.in_rows = self.nq + self.nk + self.nv + self.H

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "k": (self.nk, W), "v": (self.nv, W), "q.norm": (self.nq,), "k.norm": (self.nk,),
                "g": (self.H, W), "o": (W, self.H * self.P)}

    def cache_spec(self):
        return ("rows", self.nk + self.nv)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.q_norm, self.k_norm = _f32(get, "q.norm"), _f32(get, "k.norm")
        self.o = get("o").to(dtype).contiguous()
        return torch.cat([get("q"), get("k"), get("v"), get("g")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        rows = cache[1]
        nq, nk, nv = self.nq, self.nk, self.nv
        q = mx.qk_norm_write(proj[:, :nq], proj[:, nq:nq + nk], proj[:, nq + nk:nq + nk + nv], self.q_norm, self.k_norm,
                             self.eps, meta.slots, rows)
        gate = proj[:, nq + nk + nv:nq + nk + nv + self.H]
        o = mx.window_attend(q, rows, meta.seg_cu, positions, meta.seg_bt, self.window, self.scale, meta.seg_max_len,
                             self.H, self.G, self.D, self.P, gate=gate)
        return F.linear(o, self.o)


class GatedLRUMixer:
    """Recurrent block around a real-gated linear recurrent unit of ``width`` channels:
    y = gelu_tanh(W_y h + b_y);  u = conv(W_x h + b_x) (causal per channel, bias, no activation);
    u in ``blocks`` equal parts, in part b: r = sigmoid(R_b u_b + c_b), i = sigmoid(I_b u_b + d_b);
    a = exp(-8 r softplus(lam));  S <- a S + sqrt(1 - a^2) i u (from S = 0, no special first token);
    output W_o (S * y).  Slot state: S (f32) and the last taps - 1 biased convolution inputs."""
    kind = "gated_lru"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.R, self.B, self.K = int(spec["width"]), int(spec["blocks"]), int(spec["conv"])
        self.width, self.eps = width, eps
        if self.R % self.B or not 1 <= self.K <= 8:
            raise ValueError("gated_lru: width must split into blocks, 1 <= conv taps <= 8")
        self.bs = self.R // self.B
        self.in_rows = 2 * self.R

    def shapes(self) -> Dict[str, tuple]:
        R, B, bs, W = self.R, self.B, self.bs, self.width
        return {"y": (R, W), "y.b": (R,), "x": (R, W), "x.b": (R,), "conv": (R, self.K), "conv.b": (R,),
                "ra": (B, bs, bs), "ra.b": (B, bs), "ri": (B, bs, bs), "ri.b": (B, bs), "lam": (R,), "o": (W, R)}

    def cache_spec(self):
        return ("slots", {"conv": (max(self.K - 1, 1), self.R), "S": (self.R,)})

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.y_b, self.x_b = _f32(get, "y.b"), _f32(get, "x.b")
        self.conv_w, self.conv_b, self.lam = _f32(get, "conv"), _f32(get, "conv.b"), _f32(get, "lam")
        # both gates' block matrices as one batched operand [B, in, 2 * out], f32 (they enter the recurrence)
        self.w_ri = torch.cat([_f32(get, "ra").transpose(1, 2), _f32(get, "ri").transpose(1, 2)], 2).contiguous()
        self.r_b, self.i_b = _f32(get, "ra.b").reshape(-1), _f32(get, "ri.b").reshape(-1)
        self.o = get("o").to(dtype).contiguous()
        return torch.cat([get("y"), get("x")], 0).to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.conv_w, self.w_ri, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        st = cache[1]
        T, R, B, bs = proj.shape[0], self.R, self.B, self.bs
        u = mx.conv_act(proj[:, R:2 * R], self.conv_w, self.conv_b, st["conv"], meta.seg_cu, meta.seg_state, positions,
                        meta.seg_max_len, "none", in_bias=self.x_b)
        z = torch.bmm(u.view(T, B, bs).transpose(0, 1), self.w_ri)             # [B, T, 2 bs]: r | i pre-activations
        s = mx.lru_scan(u, z, B, self.r_b, self.i_b, self.lam, proj[:, :R], self.y_b, st["S"], meta.seg_cu,
                        meta.seg_state, positions, proj.dtype, max_len=meta.seg_max_len)
        return F.linear(s, self.o)


def _decays(spec: Dict, heads: int) -> torch.Tensor:
    d = [float(v) for v in spec["decay"]]
    if len(d) != heads or any(not 0.0 <= v <= 1.0 for v in d):
        raise ValueError("decay: one value in [0, 1] per head")
    return torch.tensor(d, dtype=torch.float32)


class LightningMixer:
    """Linear attention with one fixed decay per head: q = silu(W_q h), k = silu(W_k h) ([heads, dim]),
    v = silu(W_v h) ([heads, vdim]); on the f32 state S [dim, vdim]: S <- decay_h S + k v^T, o = S^T q (no
    other scale).  The concatenated heads are RMS-normed together with the weight ``norm``
    [heads * vdim], multiplied by sigmoid(W_g h) and projected by W_o."""
    kind = "lightning"
    in_bias = None             # no bias on the stacked input projection

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.D, self.P = int(spec["heads"]), int(spec["dim"]), int(spec["vdim"])
        self.decay = _decays(spec, self.H)
        self.width, self.eps = width, eps
        if self.D > 512:
            raise ValueError("lightning: dim <= 512")
        self.nq, self.nv = self.H * self.D, self.H * self.P
        self.in_rows = 2 * self.nq + 2 * self.nv

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "k": (self.nq, W), "v": (self.nv, W), "g": (self.nv, W), "o": (W, self.nv),
                "norm": (self.nv,)}

    def cache_spec(self):
        return ("slots", {"S": (self.H, self.D, self.P)})

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.norm_w = _f32(get, "norm")
        self.o = get("o").to(dtype).contiguous()
        self.decay = self.decay.to(self.o.device)
        return torch.cat([get("q"), get("k"), get("v"), get("g")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        st = cache[1]
        nq, nv = self.nq, self.nv
        o = mx.decay_scan(proj[:, :nq], proj[:, nq:2 * nq], proj[:, 2 * nq:2 * nq + nv], self.decay, st["S"], meta.seg_cu,
                          meta.seg_state, positions, self.H, self.D, self.P, act="silu", max_len=meta.seg_max_len)
        gate = proj[:, 2 * nq + nv:2 * nq + 2 * nv]
        return F.linear(mx.head_norm_gate(o, self.norm_w, self.eps, gate, 1, "sigmoid", proj.dtype), self.o)


class _Rotary:
    """The ``rot`` entry of a mixer spec: {dims, base, scaling?} -> frequencies (f32, on the device at load)
    and the factor on cos and sin.  No entry: no rotation."""

    def __init__(self, rot: Optional[Dict], dim: int):
        self.dims = int(rot["dims"]) if rot else 0
        if self.dims % 2 or self.dims > dim:
            raise ValueError("rot.dims must be even and at most the head size")
        self.freq, self.mscale = (mx.rope_freqs(self.dims, float(rot["base"]), rot.get("scaling"))
                                  if self.dims else (None, 1.0))

    def to(self, device):
        if self.freq is not None:
            self.freq = self.freq.to(device)


class RetentionMixer:
    """Linear attention with one fixed decay per head, no softmax and no denominator: q = W_q h,
    k = W_k h ([heads, dim]), v = W_v h ([heads, vdim]); q and k rotated on their first rot.dims entries
    (pair i is entries (i, i + dims/2), angle position * base^(-2i/dims)), then k times dim^-1/2;
    S <- decay_h S + k v^T, o = S^T q on the f32 state.  Each head's o is divided by its root mean square
    (no weight); the heads are multiplied by silu(W_g h) and projected by W_o."""
    kind = "retention"
    in_bias = None

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.D, self.P = int(spec["heads"]), int(spec["dim"]), int(spec["vdim"])
        self.decay = _decays(spec, self.H)
        self.rot = _Rotary(spec.get("rot"), self.D)
        self.width, self.eps = width, eps
        if self.D > 512:
            raise ValueError("retention: dim <= 512")
        self.nq, self.nv = self.H * self.D, self.H * self.P
        self.in_rows = 2 * self.nq + 2 * self.nv

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "k": (self.nq, W), "v": (self.nv, W), "g": (self.nv, W), "o": (W, self.nv)}

    def cache_spec(self):
        return ("slots", {"S": (self.H, self.D, self.P)})

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.o = get("o").to(dtype).contiguous()
        self.decay = self.decay.to(self.o.device)
        self.rot.to(self.o.device)
        return torch.cat([get("q"), get("k"), get("v"), get("g")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        st = cache[1]
        nq, nv = self.nq, self.nv
        # rotated q and k enter the recurrence: they stay f32
        q, k = mx.rope_heads(proj[:, :nq], proj[:, nq:2 * nq], self.H, self.H, self.D, self.rot.freq, positions, "half",
                             self.rot.mscale, k_scale=self.D ** -0.5, q_dtype=torch.float32, k_dtype=torch.float32)
        o = mx.decay_scan(q, k, proj[:, 2 * nq:2 * nq + nv], self.decay, st["S"], meta.seg_cu, meta.seg_state, positions,
                          self.H, self.D, self.P, max_len=meta.seg_max_len)
        gate = proj[:, 2 * nq + nv:2 * nq + 2 * nv]
        return F.linear(mx.head_norm_gate(o, None, self.eps, gate, self.H, "silu", proj.dtype), self.o)


class ChunkAttentionMixer:
    """Softmax attention with ``kv_heads`` key/value heads (query head h reads head h // (H/G)) whose
    VALUES ARE THE KEYS as projected: q = W_q h + b_q, k = W_k h + b_k, v = k before norm and rotation.
    q and k are rotated on their first rot.dims entries (pair i is entries (2i, 2i+1); frequencies
    optionally scaled, see :func:`..ops.mixers.rope_freqs`), then each head is divided by its root mean
    square over dim (no weight).  score = q . k * scale; the query at position i sees keys j <= i of
    its own block, floor(j / mask.size) == floor(i / mask.size), blocks counted from position 0 (no
    ``mask`` entry: plain causal); softmax; W_o on the concatenated heads.  The cache holds one row
    [finished k | raw k] per token."""
    kind = "attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.G = int(spec["heads"]), int(spec.get("kv_heads", spec["heads"]))
        self.D, self.P = int(spec["dim"]), int(spec.get("vdim", spec["dim"]))
        if self.P != self.D:
            raise ValueError("attention: the values are the keys, so vdim must equal dim")
        self.rot = _Rotary(spec.get("rot"), self.D)
        mask = spec.get("mask") or {}
        self.chunk = int(mask["size"]) if mask.get("size") else 0
        self.scale = float(spec["scale"]) if "scale" in spec else self.D ** -0.5
        self.width, self.eps = width, eps
        if self.H % self.G or self.D > 512:
            raise ValueError("attention: heads must split into kv_heads; dim <= 512")
        self.nq, self.nk = self.H * self.D, self.G * self.D
        self.in_rows = self.nq + self.nk

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "q.b": (self.nq,), "k": (self.nk, W), "k.b": (self.nk,), "o": (W, self.H * self.P)}

    def cache_spec(self):
        return ("rows", 2 * self.nk)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.o = get("o").to(dtype).contiguous()
        self.rot.to(self.o.device)
        self.in_bias = torch.cat([get("q.b"), get("k.b")], 0).to(dtype).contiguous()
        return torch.cat([get("q"), get("k")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        rows = cache[1]
        nq, nk = self.nq, self.nk
        kraw = proj[:, nq:nq + nk]
        q, _ = mx.rope_heads(proj[:, :nq], kraw, self.H, self.G, self.D, self.rot.freq, positions, "pairs",
                             self.rot.mscale, norm_eps=self.eps, k_out=rows, slots=meta.slots, v=kraw)
        o = mx.window_attend(q, rows, meta.seg_cu, positions, meta.seg_bt, self.chunk or (1 << 30), self.scale,
                             meta.seg_max_len, self.H, self.G, self.D, self.P, chunked=bool(self.chunk))
        return F.linear(o, self.o)


class ParallelMixer:
    """Two mixers side by side reading the same input (``left``: windowed attention, ``right``: gated
    LRU block).  ``forward`` returns both outputs; the layer takes half the sum of their RMS norms
    over the model width, with the plain weights ``left.out`` / ``right.out``.  Subclasses choose other
    pairs (``left_cls`` / ``right_cls``) and may do without the output norm weights."""
    kind = "parallel"
    left_cls: type = None        # set below the class definitions
    right_cls: type = None
    out_norms = True

    def __init__(self, spec: Dict, width: int, eps: float):
        self.left = self.left_cls(spec["left"], width, eps)
        self.right = self.right_cls(spec["right"], width, eps)
        self.width = width
        self.in_rows = self.left.in_rows + self.right.in_rows

    def shapes(self) -> Dict[str, tuple]:
        s = {f"left.{k}": v for k, v in self.left.shapes().items()}
        s.update({f"right.{k}": v for k, v in self.right.shapes().items()})
        if self.out_norms:
            s.update({"left.out": (self.width,), "right.out": (self.width,)})
        return s

    def cache_spec(self):
        return ("pair", self.left.cache_spec(), self.right.cache_spec())

    def load(self, get: Getter, dtype) -> torch.Tensor:
        if self.out_norms:
            self.out_w = (_f32(get, "left.out"), _f32(get, "right.out"))
        wl = self.left.load(lambda k: get("left." + k), dtype)
        wr = self.right.load(lambda k: get("right." + k), dtype)
        return torch.cat([wl, wr], 0)

    def num_bytes(self) -> int:
        return self.left.num_bytes() + self.right.num_bytes()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache):
        n = self.left.in_rows
        return (self.left.forward(proj[:, :n], positions, meta, cache[1]),
                self.right.forward(proj[:, n:], positions, meta, cache[2]))


ParallelMixer.left_cls, ParallelMixer.right_cls = WindowAttentionMixer, GatedLRUMixer


class SigmoidAttentionMixer:
    """Causal attention without positions and without softmax.  ``kv_heads`` key/value heads (query head h
    reads head h // (H/G)), key size ``dim``, value size ``vdim``, no biases on the projections, no
    rotation; score = q . k * scale; every key j <= i is visible (a ``mask`` entry {size} narrows this to
    a sliding window) and weighs sigmoid(score + pb[h]) with one bias per query head -- the weights of a
    query are independent and are not normalised.  W_o on the concatenated heads.  The cache holds one
    row [k | v] per token."""
    kind = "sigmoid_attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.G = int(spec["heads"]), int(spec.get("kv_heads", spec["heads"]))
        self.D, self.P = int(spec["dim"]), int(spec["vdim"])
        mask = spec.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 1 << 30
        self.scale = float(spec["scale"]) if "scale" in spec else self.D ** -0.5
        self.width, self.eps = width, eps
        if self.H % self.G or self.D > 512 or self.P > 512:
            raise ValueError("sigmoid attention: heads must split into kv_heads; dim, vdim <= 512")
        self.nq, self.nk, self.nv = self.H * self.D, self.G * self.D, self.G * self.P
        self.in_rows = self.nq + self.nk + self.nv

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        return {"q": (self.nq, W), "k": (self.nk, W), "v": (self.nv, W), "pb": (self.H,), "o": (W, self.H * self.P)}

    def cache_spec(self):
        return ("rows", self.nk + self.nv)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.pb = _f32(get, "pb")
        self.o = get("o").to(dtype).contiguous()
        return torch.cat([get("q"), get("k"), get("v")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        rows = cache[1]
        nq, nk, nv = self.nq, self.nk, self.nv
        q = mx.qk_norm_write(proj[:, :nq], proj[:, nq:nq + nk], proj[:, nq + nk:nq + nk + nv], None, None, self.eps,
                             meta.slots, rows)
        o = mx.window_attend(q, rows, meta.seg_cu, positions, meta.seg_bt, self.window, self.scale, meta.seg_max_len,
                             self.H, self.G, self.D, self.P, head_bias=self.pb)
        return F.linear(o, self.o)


class MinGRUMixer:
    """Minimal gated recurrent unit of ``width`` channels: z = sigmoid(W_z h + b_z), u = W_x h + b_x, candidate
    c = u + 1/2 where u >= 0 and sigmoid(u) below; element by element S <- (1 - z) S + z c on an f32 state
    per sequence that starts at zero (the gates read only the current token); output W_o (S * silu(W_g h))."""
    kind = "mingru"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.R = int(spec["width"])
        self.width, self.eps = width, eps
        self.in_rows = 3 * self.R

    def shapes(self) -> Dict[str, tuple]:
        R, W = self.R, self.width
        return {"z": (R, W), "z.b": (R,), "x": (R, W), "x.b": (R,), "g": (R, W), "o": (W, R)}

    def cache_spec(self):
        return ("slots", {"S": (self.R,)})

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.z_b, self.x_b = _f32(get, "z.b"), _f32(get, "x.b")      # added in f32: they enter the recurrence
        self.o = get("o").to(dtype).contiguous()
        return torch.cat([get("z"), get("x"), get("g")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        R = self.R
        s = mx.mingru_scan(proj[:, :R], proj[:, R:2 * R], proj[:, 2 * R:3 * R], self.z_b, self.x_b, cache[1]["S"],
                           meta.seg_cu, meta.seg_state, positions, proj.dtype, max_len=meta.seg_max_len)
        return F.linear(s, self.o)


class WeightedParallelMixer(ParallelMixer):
    """Sigmoid attention (``left``) beside a minimal GRU (``right``) on the same input; the layer adds
    left_scale * left + right_scale * right (``forward`` returns both, ``scales`` the two weights)."""
    left_cls, right_cls = SigmoidAttentionMixer, MinGRUMixer
    out_norms = False

    def __init__(self, spec: Dict, width: int, eps: float):
        super().__init__(spec, width, eps)
        self.scales = (float(spec.get("left_scale", 1.0)), float(spec.get("right_scale", 1.0)))


class SinkWindowAttentionMixer:
    """Softmax attention with ``kv_heads`` key/value heads (query head h reads head h // (H/G)), no biases.
    q and k are rotated on the first rot.dims entries of each head (entry i with entry i + dims/2, angle
    position * base^(-2i/dims), every frequency divided by rot.scaling.factor when given), then each head
    is divided by its root mean square over dim (no weight); score = q . k * scale; position i sees j <= i
    with i - j < mask.size or j < mask.keep_first (the kept first tokens stay at their true positions; no
    ``mask`` entry: plain causal); softmax; W_o.  With ``v_mix`` the values of every such layer but the
    model's first are blended with the first one's values of the same token,
    v <- (1 - vmix) v + vmix v_first (``forward``'s ``v_first``), before they are cached.  The cache
    holds one row [finished k | v] per token."""
    kind = "sink_window_attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.G = int(spec["heads"]), int(spec.get("kv_heads", spec["heads"]))
        self.D, self.P = int(spec["dim"]), int(spec["vdim"])
        self.rot = _Rotary(spec.get("rot"), self.D)
        mask = spec.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 1 << 30
        self.keep = int(mask.get("keep_first") or 0) if mask.get("size") else 0
        self.scale = float(spec["scale"]) if "scale" in spec else self.D ** -0.5
        self.v_mix = bool(spec.get("v_mix"))
        self.lam = 0.0
        self.width, self.eps = width, eps
        if self.H % self.G or self.D > 512 or self.P > 512:
            raise ValueError("attention: heads must split into kv_heads; dim, vdim <= 512")
        self.nq, self.nk, self.nv = self.H * self.D, self.G * self.D, self.G * self.P
        self.in_rows = self.nq + self.nk + self.nv

    def shapes(self) -> Dict[str, tuple]:
        W = self.width
        s = {"q": (self.nq, W), "k": (self.nk, W), "v": (self.nv, W), "o": (W, self.H * self.P)}
        if self.v_mix:
            s["vmix"] = ()
        return s

    def cache_spec(self):
        return ("rows", self.nk + self.nv)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.o = get("o").to(dtype).contiguous()
        self.rot.to(self.o.device)
        if self.v_mix:
            self.lam = float(get("vmix").float().item())
        return torch.cat([get("q"), get("k"), get("v")], 0).to(dtype)

    def num_bytes(self) -> int:
        return self.o.numel() * self.o.element_size()

    def values(self, proj: torch.Tensor) -> torch.Tensor:
        """This layer's values as projected (what later layers blend theirs with)."""
        return proj[:, self.nq + self.nk:self.nq + self.nk + self.nv]

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache,
                v_first: Optional[torch.Tensor] = None) -> torch.Tensor:
        rows = cache[1]
        nq, nk = self.nq, self.nk
        q, _ = mx.rope_heads(proj[:, :nq], proj[:, nq:nq + nk], self.H, self.G, self.D, self.rot.freq, positions, "half",
                             self.rot.mscale, norm_eps=self.eps, k_out=rows, slots=meta.slots, v=self.values(proj),
                             v_mix=v_first, v_lam=self.lam)
        o = mx.window_attend(q, rows, meta.seg_cu, positions, meta.seg_bt, self.window, self.scale, meta.seg_max_len,
                             self.H, self.G, self.D, self.P, keep_first=self.keep)
        return F.linear(o, self.o)


class PlainLatentAttentionMixer:
    """Latent attention without positions: q = W_q h ([heads, dim]); c = RMSnorm(W_dkv h) * w (``kv_rank``
    entries, plain weight); per head k = W_uk c, v = W_uv c; score = q . k * scale; plain causal softmax;
    W_o.  Only c is cached; the kernels run in the latent space (each head's W_uk folded into its query,
    W_uv applied to the attention output), so all heads read the same cache rows."""
    kind = "plain_latent_attention"

    def __init__(self, spec: Dict, width: int, eps: float):
        self.H, self.D, self.P, self.R = int(spec["heads"]), int(spec["dim"]), int(spec["vdim"]), int(spec["kv_rank"])
        mask = spec.get("mask") or {}
        self.window = int(mask["size"]) if mask.get("size") else 1 << 30
        self.scale = float(spec["scale"]) if "scale" in spec else self.D ** -0.5
        self.width, self.eps = width, eps
        if self.R > 512:
            raise ValueError("latent attention: kv_rank <= 512")
        self.nq = self.H * self.D
        self.in_rows = self.nq + self.R

    def shapes(self) -> Dict[str, tuple]:
        W, H = self.width, self.H
        return {"q": (self.nq, W), "dkv": (self.R, W), "dkv.norm": (self.R,), "uk": (H * self.D, self.R),
                "uv": (H * self.P, self.R), "o": (W, H * self.P)}

    def cache_spec(self):
        return ("latent", self.R)

    def load(self, get: Getter, dtype) -> torch.Tensor:
        self.dkv_norm = _f32(get, "dkv.norm")
        self.uk = get("uk").to(dtype).view(self.H, self.D, self.R).contiguous()                       # [H, D, R]
        self.uv_t = get("uv").to(dtype).view(self.H, self.P, self.R).transpose(1, 2).contiguous()     # [H, R, P]
        self.o = get("o").to(dtype).contiguous()
        self.no_freq = torch.zeros(0, dtype=torch.float32, device=self.o.device)
        return torch.cat([get("q"), get("dkv")], 0).to(dtype)

    def num_bytes(self) -> int:
        return sum(t.numel() * t.element_size() for t in (self.uk, self.uv_t, self.o))

    def forward(self, proj: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, cache) -> torch.Tensor:
        rows = cache[1]
        T = proj.shape[0]
        H, D, R = self.H, self.D, self.R
        q = proj[:, :self.nq]
        # the normed latent into the cache (no rotated part: the returned rotated query part is empty)
        q_rot = mx.latent_prep(proj[:, self.nq:self.nq + R], self.dkv_norm, self.eps, self.no_freq, 0, positions,
                               meta.slots, rows, q, H, D, D, R, 0)
        q_lat = torch.bmm(q.reshape(T, H, D).transpose(0, 1), self.uk).transpose(0, 1).contiguous()     # [T, H, R]
        o_lat = mx.latent_attend(q_lat, q_rot, rows, meta.seg_cu, positions, meta.seg_bt, self.window, self.scale,
                                 meta.seg_max_len)
        o = torch.bmm(o_lat.transpose(0, 1), self.uv_t).transpose(0, 1).reshape(T, H * self.P)
        return F.linear(o, self.o)


MIXERS = {"mamba2": Mamba2Mixer, "latent_attention": LatentAttentionMixer, "channel_delta": ChannelDeltaMixer,
          "gla": GLAMixer, "window_attention": WindowAttentionMixer, "gated_lru": GatedLRUMixer,
          "parallel": ParallelMixer, "lightning": LightningMixer, "retention": RetentionMixer,
          "attention": ChunkAttentionMixer, "sigmoid_attention": SigmoidAttentionMixer, "mingru": MinGRUMixer,
          "weighted_parallel": WeightedParallelMixer, "sink_window_attention": SinkWindowAttentionMixer,
          "plain_latent_attention": PlainLatentAttentionMixer}
