"""Tukedra: a layered pre-norm decoder with several residual streams per token (hyper-connections).

``config.json`` lists the layers; each has one sequence mixer -- ``lightning`` (linear attention with a
fixed decay per head on SiLU-activated q, k, v), ``retention`` (the same recurrence on rotated q and k)
or ``attention`` (chunk-masked softmax attention whose values are the keys as projected), see
:mod:`.mixers` -- and optionally one feed-forward (gated SiLU, or a mixture of relu^2 experts with a
softmax over the chosen router logits plus a shared expert).

The embedding is ``embed[token] * embedding.scale``, copied into ``streams`` residual streams
x_1 .. x_S.  For sublayer q of a layer (1: mixer, 2: feed-forward) with the layer's tensors
``hc<q>.in`` [S], ``hc<q>.out`` [S] and ``hc<q>.mix`` [S, S] (indexed [from, to]):

    u = sum_s in[s] x_s;   y = sublayer(RMSnorm(u) * w_norm<q>);   x_t <- sum_s mix[s, t] x_s + out[t] y

for all streams t at once from the old ones.  Without a ``streams`` entry there is one stream and the
plain sum x <- x + sublayer(RMSnorm(x) * w).  The model ends with RMSnorm(sum_s x_s) * ``final.norm``,
logits = ``head`` x * ``logit_scale`` and then ``logit_softcap`` * tanh(logits / ``logit_softcap``).

The streams are f32 whatever the activation dtype; one kernel writes a sublayer's output back into
the streams and reads + norms the next sublayer's input (:func:`..ops.mixers.hyper_mix`), and the
mixer's input projections are one stacked GEMM per layer.

Checkpoint tensors: ``embed``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.hc1.*``, ``l<i>.hc2.*``,
``l<i>.mix.<name>``, ``l<i>.mlp.<name>``, ``final.norm``, ``head``.
"""
from __future__ import annotations

from typing import Dict

import torch
import torch.nn.functional as F

from ..ops import mixers as mx
from .common import AttentionMetadata, HybridCache
from .configs import ModelConfig
from .layered import Layer, LayeredDecoder
from .mixers import DenseFF, TopSoftmaxRoutedFF


def example_config(width: int = 160, vocab: int = 768, pattern: str = "lRaL", scale_up: bool = False, heads: int = 0,
                   streams: int = 2) -> Dict:
    """A config.json-shaped dict for random-weight models (tests, benchmarks).  ``pattern``: one letter
    per layer -- l/L lightning, r/R retention, a/A attention; lower case with a dense feed-forward, upper
    case with a routed one.  ``scale_up``: sizes in the range of a real model's layers."""
    if scale_up:
        H = heads or width // 128
        lig = {"decay": [1.0 - 2.0 ** (-3 - 5 * h / max(H - 1, 1)) for h in range(H)], "dim": 128, "heads": H, "vdim": 128}
        ret = {"decay": [1.0 - 2.0 ** (-5 - 4 * h / max(H - 1, 1)) for h in range(H)], "dim": 64, "heads": H,
               "rot": {"base": 10000.0, "dims": 64}, "vdim": 128}
        att = {"dim": 128, "heads": H, "kv_heads": max(H // 4, 1), "mask": {"size": 2048},
               "rot": {"base": 10000.0, "dims": 64, "scaling": {"factor": 4.0, "fast": 32.0, "original": 4096, "slow": 1.0}},
               "scale": 1.0, "vdim": 128}
        dense = {"ff": 3 * width, "kind": "dense"}
        moe = {"expert": {"ff": 3 * width // 4}, "kind": "moe", "router": {"experts": 32, "top": 4}, "shared": {"ff": width}}
    else:
        lig = {"decay": [0.7, 0.95, 0.995], "dim": 24, "heads": 3, "vdim": 20}
        ret = {"decay": [0.9, 0.99], "dim": 20, "heads": 2, "rot": {"base": 5000.0, "dims": 12}, "vdim": 28}
        att = {"dim": 24, "heads": 6, "kv_heads": 2, "mask": {"size": 37},
               "rot": {"base": 3000.0, "dims": 16, "scaling": {"factor": 4.0, "fast": 16.0, "original": 256, "slow": 2.0}},
               "scale": 1.5, "vdim": 24}
        dense = {"ff": 224, "kind": "dense"}
        moe = {"expert": {"ff": 56}, "kind": "moe", "router": {"experts": 7, "top": 3}, "shared": {"ff": 40}}
    kinds = {"l": ("lightning", lig), "r": ("retention", ret), "a": ("attention", att)}
    layers = []
    for ch in pattern:
        t, m = kinds[ch.lower()]
        layers.append({"type": t, "mixer": {k: (dict(v) if isinstance(v, dict) else v) for k, v in m.items()},
                       "mlp": dict(moe if ch.isupper() else dense)})
    c = {"architecture": "Tukedra", "embedding": {"scale": 2.0}, "layers": layers, "logit_scale": 0.5,
         "logit_softcap": 20.0, "norm": {"eps": 1e-5}, "vocab": vocab, "width": width}
    if streams:
        c["streams"] = streams
    return c


class _Layer(Layer):
    def __init__(self, i: int, spec: Dict, width: int, eps: float, streams: int):
        super().__init__(i, spec, width, eps, TukedraModel.mixer_types)
        mlp = spec.get("mlp")
        if mlp is None:
            self.ff = None
        elif mlp["kind"] == "dense":
            self.ff = DenseFF(mlp, width, act="silu", gated=True)
        elif mlp["kind"] == "moe":
            self.ff = TopSoftmaxRoutedFF(mlp, width, act="relu2")
        else:
            raise ValueError(f"layer {i}: unknown feed-forward kind {mlp['kind']!r}")
        self.streams = streams
        self.w_ff = None
        self.norm2 = None
        self.hc = {}             # sublayer (1 | 2) -> (in [S], out [S], mix [S, S]) f32

    def norms(self):
        return ("norm1", "norm2") if self.ff is not None else ("norm1",)

    def extra_shapes(self) -> Dict[str, tuple]:
        S = self.streams
        if not S:
            return {}
        s = {}
        for q in (1, 2) if self.ff is not None else (1,):
            s.update({f"hc{q}.in": (S,), f"hc{q}.out": (S,), f"hc{q}.mix": (S, S)})
        return s


class TukedraModel(LayeredDecoder):
    arch = "tukedra"
    mixer_types = ("lightning", "retention", "attention")
    plain_logits = False         # logits are scaled and capped: the fused LM-head sampler does not apply

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16):
        self.streams = int(cfg.streams)
        if self.streams > mx.MAX_STREAMS:
            raise ValueError(f"{cfg.name}: at most {mx.MAX_STREAMS} residual streams are supported")
        super().__init__(cfg, device, dtype)
        self.has_state = any(l.mixer.kind != "attention" for l in self.layers)
        self.embed_scale = float((cfg.embedding or {}).get("scale", 1.0))
        self.logit_scale, self.logit_softcap = float(cfg.logit_scale), float(cfg.logit_softcap)

    def make_layer(self, i: int, spec: Dict) -> Layer:
        return _Layer(i, spec, self.cfg.hidden_size, self.cfg.norm_eps, self.streams)

    def load_layer(self, l: Layer, get) -> None:
        dt, S = self.dtype, max(self.streams, 1)
        f32 = lambda n: get(f"{l.prefix}.{n}").float().contiguous()  # noqa: E731
        l.norm1 = f32("norm1")
        l.w_in = l.mixer.load(lambda k, p=l.prefix: get(f"{p}.mix.{k}"), dt).contiguous()
        if l.ff is not None:
            l.norm2 = f32("norm2")
            w = l.ff.load(lambda k, p=l.prefix: get(f"{p}.mlp.{k}"), dt)
            l.w_ff = w.contiguous() if w is not None else None
        for q in (1, 2) if l.ff is not None else (1,):
            if self.streams:
                l.hc[q] = (f32(f"hc{q}.in"), f32(f"hc{q}.out"), f32(f"hc{q}.mix"))
            else:        # one stream, plain residual sum
                one = torch.ones(1, dtype=torch.float32, device=self.device)
                l.hc[q] = (one, one, one.view(1, 1))
        self._sum_in = torch.ones(S, dtype=torch.float32, device=self.device)

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        # scale and cap in f32: the head product is rounded once, not again after the tanh
        return mx.logit_cap(F.linear(h, self.head).float(), self.logit_scale, self.logit_softcap)

    # -- forward -----------------------------------------------------------------------------------
    def forward(self, ids: torch.Tensor, positions: torch.Tensor, meta: AttentionMetadata, kv: HybridCache) -> torch.Tensor:
        """Final-normed hidden states [T, width] of every row of the step."""
        eps, dt = self.cfg.norm_eps, self.dtype
        if meta.seg_cu is None:
            raise ValueError("this model needs the segment view of the step (AttentionMetadata.seg_*)")
        x = mx.embed_scaled(ids, self.embed, self.embed_scale, max(self.streams, 1))        # [T, S, W] f32
        n = len(self.layers)
        h = mx.hyper_mix(x, None, None, None, self.layers[0].hc[1][0], self.layers[0].norm1, eps, dt)
        for i, l in enumerate(self.layers):
            y = l.mixer.forward(F.linear(h, l.w_in, l.mixer.in_bias), positions, meta, kv.layers[i])
            done = l.hc[1]
            if l.ff is not None:
                h = mx.hyper_mix(x, y, done[2], done[1], l.hc[2][0], l.norm2, eps, dt)
                y = l.ff.forward(h, F.linear(h, l.w_ff) if l.w_ff is not None else None)
                done = l.hc[2]
            nxt = self.layers[i + 1] if i + 1 < n else None
            # the write-back of this layer's last sublayer, fused with the read and norm of what comes next
            h = mx.hyper_mix(x, y, done[2], done[1], nxt.hc[1][0] if nxt else self._sum_in,
                             nxt.norm1 if nxt else self.final_norm, eps, dt)
            if self.capture is not None:
                self.capture.append(x.sum(1))
        return h
