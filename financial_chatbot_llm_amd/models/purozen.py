"""Purozen: a layered pre-norm decoder with sigmoid-gated residual updates and a tied vocabulary projection.

``config.json`` lists the layers; each has one sequence mixer and optionally one dense feed-forward
(W_down gelu_tanh(W_up h)).  With n(x) = x / sqrt(mean(x^2) + eps) * (1 + w) -- the norm weights are stored
around zero -- a layer is

    h = n1(x);   x <- x + sigmoid(R1 h + b1) * mixer(h)
    h = n2(x);   x <- x + sigmoid(R2 h + b2) * ff(h)

(``rg1`` / ``rg1.b`` and ``rg2`` / ``rg2.b``: a gate per element on each sublayer's result, read from the same
normed input as the sublayer).  The model ends with the same kind of norm (``final.norm``) and
logits = ``embed`` x: the embedding table is the vocabulary projection.

Mixer types (see :mod:`.mixers`): ``parallel`` -- sigmoid attention beside a minimal GRU, summed with the
config's two weights; ``attention`` -- rotated, unit-RMS q and k, a sliding window that keeps the first
tokens, values blended with those of the model's first ``v_mix`` layer; ``latent_attention`` -- keys and
values from one cached latent per token, no positions.

The residual stream is f32 whatever the activation dtype; one kernel applies a sublayer's gated update
and norms the next sublayer's input (:func:`..ops.mixers.residual_norm`); the gate's projection is
stacked under the sublayer's own input projection, so each sublayer reads ``h`` with ONE GEMM.

Checkpoint tensors: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.rg1``, ``l<i>.rg1.b``, ``l<i>.rg2``,
``l<i>.rg2.b``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``, ``final.norm``.
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn.functional as F

from ..ops import mixers as mx
from .common import AttentionMetadata, HybridCache
from .configs import ModelConfig
from .layered import Layer, LayeredDecoder
from .mixers import DenseFF


def example_config(width: int = 160, vocab: int = 768, pattern: str = "paAl", scale_up: bool = False,
                   heads: int = 0) -> Dict:
    """A config.json-shaped dict for random-weight models (tests, benchmarks).  ``pattern``: one letter per
    layer -- p parallel (sigmoid attention + minimal GRU), a attention (rotation, window, kept first
    tokens, blended values), l latent attention; lower case with a dense feed-forward, upper case without.
    ``scale_up``: sizes in the range of a real model's layers."""
    if scale_up:
        H = heads or width // 128
        G = max(H // 4, 1)
        par = {"left": {"dim": 128, "heads": H, "kv_heads": G, "scale": 128 ** -0.5, "vdim": 128}, "left_scale": 0.7,
               "right": {"width": width}, "right_scale": 1.2}
        att = {"dim": 128, "heads": H, "kv_heads": G, "mask": {"keep_first": 4, "size": 1024},
               "rot": {"base": 10000.0, "dims": 64, "scaling": {"factor": 2.0}}, "scale": 1.0, "v_mix": True, "vdim": 128}
        lat = {"dim": 128, "heads": H, "kv_rank": 256, "scale": 128 ** -0.5, "vdim": 128}
        dense = {"ff": 4 * width, "kind": "dense"}
    else:
        par = {"left": {"dim": 24, "heads": 6, "kv_heads": 2, "scale": 0.3, "vdim": 20}, "left_scale": 0.7,
               "right": {"width": 72}, "right_scale": 1.2}
        att = {"dim": 24, "heads": 6, "kv_heads": 3, "mask": {"keep_first": 3, "size": 37},
               "rot": {"base": 3000.0, "dims": 12, "scaling": {"factor": 2.0}}, "scale": 1.5, "v_mix": True, "vdim": 28}
        lat = {"dim": 20, "heads": 5, "kv_rank": 40, "scale": 0.25, "vdim": 12}
        dense = {"ff": 224, "kind": "dense"}
    kinds = {"p": ("parallel", par), "a": ("attention", att), "l": ("latent_attention", lat)}
    layers = []
    for ch in pattern:
        t, m = kinds[ch.lower()]
        layers.append({"type": t, "mixer": {k: (dict(v) if isinstance(v, dict) else v) for k, v in m.items()},
                       "mlp": dict(dense) if ch.islower() else None})
    return {"architecture": "Purozen", "layers": layers, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}


class _Layer(Layer):
    def __init__(self, i: int, spec: Dict, width: int, eps: float):
        super().__init__(i, spec, width, eps, PurozenModel.mixer_types)
        mlp = spec.get("mlp")
        if mlp is None:
            self.ff = None
        elif mlp["kind"] == "dense":
            self.ff = DenseFF(mlp, width, act="gelu_tanh")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        self.width = width
        self.w_ff = None
        self.norm2 = None
        self.rg_b = {}           # sublayer (1 | 2) -> gate bias f32 [W]

    def norms(self):
        return ("norm1", "norm2") if self.ff is not None else ("norm1",)

    def extra_shapes(self) -> Dict[str, tuple]:
        W, s = self.width, {}
        for q in (1, 2) if self.ff is not None else (1,):
            s.update({f"rg{q}": (W, W), f"rg{q}.b": (W,)})
        return s


class PurozenModel(LayeredDecoder):
    arch = "purozen"
    # the design's layer types -> mixer classes of the registry
    mixer_types = {"parallel": "weighted_parallel", "attention": "sink_window_attention",
                   "latent_attention": "plain_latent_attention"}
    tied_head = True

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16):
        super().__init__(cfg, device, dtype)
        self.has_state = any(l.mixer.kind == "parallel" for l in self.layers)
        # the values every later v_mix layer blends with: those of the first such layer
        mixing = [i for i, l in enumerate(self.layers) if getattr(l.mixer, "v_mix", False)]
        self.v_source = mixing[0] if mixing else -1
        sizes = {self.layers[i].mixer.nv for i in mixing}
        if len(sizes) > 1:
            raise ValueError(f"{cfg.name}: layers that blend values must agree on kv_heads * vdim, got {sorted(sizes)}")

    def make_layer(self, i: int, spec: Dict) -> Layer:
        return _Layer(i, spec, self.cfg.hidden_size, self.cfg.norm_eps)

    @staticmethod
    def _random(name: str, shape, seed: int, device="cpu") -> torch.Tensor:
        leaf = name.rsplit(".", 1)[-1]
        t = LayeredDecoder._random(name, shape, seed, device)
        if leaf in ("norm1", "norm2") or name == "final.norm":     # stored around zero: the norm multiplies by 1 + w
            t = t - 1.0
        return t

    def load_layer(self, l: Layer, get) -> None:
        dt = self.dtype
        f32 = lambda n: get(f"{l.prefix}.{n}").float().contiguous()  # noqa: E731
        l.norm1 = f32("norm1") + 1.0
        w = l.mixer.load(lambda k, p=l.prefix: get(f"{p}.mix.{k}"), dt)
        l.w_in = torch.cat([w, get(f"{l.prefix}.rg1").to(dt)], 0).contiguous()
        l.rg_b[1] = f32("rg1.b")
        if l.ff is not None:
            l.norm2 = f32("norm2") + 1.0
            w = l.ff.load(lambda k, p=l.prefix: get(f"{p}.mlp.{k}"), dt)
            l.w_ff = torch.cat([w, get(f"{l.prefix}.rg2").to(dt)], 0).contiguous()
            l.rg_b[2] = f32("rg2.b")

    def load_extra(self, get) -> None:
        self.final_norm = self.final_norm + 1.0

    # -- forward -----------------------------------------------------------------------------------
    def forward(self, ids: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, kv: HybridCache) -> torch.Tensor:
        """Final-normed hidden states [T, width] of every row of the step."""
        eps, dt, W = self.cfg.norm_eps, self.dtype, self.cfg.hidden_size
        if meta.seg_cu is None:
            raise ValueError("this model needs the segment view of the step (AttentionMetadata.seg_*)")
        x = mx.embed_f32(ids, self.embed)                                   # [T, W] f32
        n = len(self.layers)
        h = mx.residual_norm(x, self.layers[0].norm1, eps, out_dtype=dt)
        v_first = None
        for i, l in enumerate(self.layers):
            m = l.mixer
            proj = F.linear(h, l.w_in)                                      # mixer rows | gate rows
            gate = proj[:, m.in_rows:m.in_rows + W]
            mults = (1.0, 1.0)
            if m.kind == "parallel":
                y, y2 = m.forward(proj[:, :m.in_rows], positions, meta, kv.layers[i])
                mults = m.scales
            elif getattr(m, "v_mix", False):
                y, y2 = m.forward(proj[:, :m.in_rows], positions, meta, kv.layers[i],
                                  v_first=v_first if i != self.v_source else None), None
                if i == self.v_source:
                    v_first = m.values(proj)
            else:
                y, y2 = m.forward(proj[:, :m.in_rows], positions, meta, kv.layers[i]), None
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            # the gated update of this sublayer, fused with the norm of what comes next
            h = mx.residual_norm(x, l.norm2 if l.ff is not None else nxt, eps, a=y, b=y2, mult=mults[0], mult_b=mults[1],
                                 gate=gate, gate_bias=l.rg_b[1], out_dtype=dt)
            if l.ff is not None:
                proj = F.linear(h, l.w_ff)                                  # up rows | gate rows
                y = l.ff.forward(h, proj)
                h = mx.residual_norm(x, nxt, eps, a=y, gate=proj[:, l.ff.in_rows:l.ff.in_rows + W], gate_bias=l.rg_b[2],
                                     out_dtype=dt)
            if self.capture is not None:
                self.capture.append(x.clone())
        return h
