"""Common part of the layered decoders (:mod:`.gezavik`, :mod:`.sigudra`, :mod:`.tukedra`, :mod:`.purozen`): a ``config.json`` lists the
layers, each with one sequence mixer of :mod:`.mixers` and optionally one feed-forward; the residual
stream is f32 whatever the activation dtype; the checkpoint is the model directory itself (tensors
``embed``, ``l<i>.<norm>``, ``l<i>.mix.<name>``, ``l<i>.mlp.<name>``, ``final.norm``, ``head``; linear
weights [out, in]).  A design subclasses :class:`LayeredDecoder` with its block structure: which
feed-forward classes and norms a layer has (``make_layer`` / ``load_layer``) and the step function
(``forward``).  Tensor parallelism is not implemented for these designs (TP = 1); data parallel
replicas work as for every model.
"""
from __future__ import annotations

import math
from typing import Callable, Dict, List, Optional

import torch
import torch.nn.functional as F

from .common import HybridCache, param_seed
from .configs import ModelConfig
from .mixers import MIXERS


class Layer:
    """One layer: its mixer (one of the design's ``mixer_types``), its feed-forward (``ff``, set by the
    design) and its loaded norms."""
    norm_names = ("norm1",)

    def __init__(self, i: int, spec: Dict, width: int, eps: float, mixer_types=None):
        self.prefix = f"l{i}"
        kind = spec["type"]
        # a design names its mixer types: a tuple of registry names, or {the design's own name: registry name}
        names = mixer_types if isinstance(mixer_types, dict) else {k: k for k in (mixer_types or MIXERS)}
        if kind not in names or names[kind] not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}; known: {sorted(names)}")
        self.mixer = MIXERS[names[kind]](spec["mixer"], width, eps)
        self.ff = None
        self.w_in: Optional[torch.Tensor] = None
        self.norm1: Optional[torch.Tensor] = None

    def norms(self):
        return self.norm_names

    def extra_shapes(self) -> Dict[str, tuple]:
        """Further per-layer tensors of the design: {name after the layer prefix: shape}."""
        return {}


class LayeredDecoder:
    arch = ""
    mixer_types: Optional[tuple] = None
    segment_meta = True          # the runner builds the segment view of each step (AttentionMetadata.seg_*)
    has_state = True             # sequences hold a recurrent-state slot; no prefix reuse, no draft rows
    tp_size = 1
    tp_rank = 0
    slot_arrays: Dict = {}       # per-slot records of the model as a whole: {name: (dtype, shape)}
    tied_head = False            # the vocabulary projection is the embedding table (no ``head`` tensor)

    def __init__(self, cfg: ModelConfig, device="cuda", dtype=torch.bfloat16):
        if cfg.arch != self.arch or not cfg.layers:
            raise ValueError(f"{cfg.name} is not a {self.arch} config")
        self.cfg, self.device, self.dtype = cfg, torch.device(device), dtype
        self.layers: List[Layer] = [self.make_layer(i, spec) for i, spec in enumerate(cfg.layers)]
        self.sequence_parallel = False
        self.capture: Optional[list] = None      # debugging: residual stream after every layer
        # head geometry the generic runner asks every decoder for (unused by the segment kernels)
        self.hq = self.hkv = 1
        self.D = 64

    # -- design hooks --------------------------------------------------------------------------------
    def make_layer(self, i: int, spec: Dict) -> Layer:
        raise NotImplementedError

    def load_layer(self, l: Layer, get: Callable[[str], torch.Tensor]) -> None:
        raise NotImplementedError

    def extra_shapes(self) -> Dict[str, tuple]:
        return {}

    def load_extra(self, get: Callable[[str], torch.Tensor]) -> None:
        pass

    # -- weights -----------------------------------------------------------------------------------
    def full_shapes(self) -> Dict[str, tuple]:
        """Checkpoint names and shapes; a ``None`` entry is a size only the tensor itself gives."""
        c = self.cfg
        s = {"embed": (c.vocab_size, c.hidden_size), "final.norm": (c.hidden_size,)}
        if not self.tied_head:
            s["head"] = (c.vocab_size, c.hidden_size)
        s.update(self.extra_shapes())
        for l in self.layers:
            for n in l.norms():
                s[f"{l.prefix}.{n}"] = (c.hidden_size,)
            s.update({f"{l.prefix}.{k}": v for k, v in l.extra_shapes().items()})
            s.update({f"{l.prefix}.mix.{k}": v for k, v in l.mixer.shapes().items()})
            if l.ff is not None:
                s.update({f"{l.prefix}.mlp.{k}": v for k, v in l.ff.shapes().items()})
        return s

    @staticmethod
    def _random(name: str, shape, seed: int, device="cpu") -> torch.Tensor:
        g = torch.Generator(device=device).manual_seed(param_seed(seed, name))
        randn = lambda: torch.randn(shape, generator=g, device=device)  # noqa: E731
        rand = lambda: torch.rand(shape, generator=g, device=device)  # noqa: E731
        leaf = name.rsplit(".", 1)[-1]
        if ".hc" in name and leaf == "in":       # stream read weights: about an average of the streams
            return (1.0 + 0.3 * randn()) / shape[0]
        if ".hc" in name and leaf == "mix":      # stream mixing: near the identity
            return torch.eye(shape[0], device=device) + 0.15 * randn()
        if leaf in ("norm1", "norm2", "norm", "out") and len(shape) == 1:
            return 1.0 + 0.1 * randn()
        if leaf == "A_log":
            return torch.log(1.0 + 7.0 * rand())
        if leaf == "dt_bias":      # softplus^-1 of step sizes in [0.01, 0.2]
            dt = torch.exp(rand() * (math.log(0.2) - math.log(0.01)) + math.log(0.01))
            return dt + torch.log(-torch.expm1(-dt))
        if leaf == "lam":          # softplus(lam) in about [0.01, 0.6]: decays from slow to fast
            return torch.log(torch.expm1(torch.exp(rand() * (math.log(0.6) - math.log(0.01)) + math.log(0.01))))
        if leaf == "D":
            return 1.0 + 0.2 * randn()
        if leaf == "correction":
            return 0.05 * randn()
        if leaf == "vmix":         # blend weight of the first layer's values
            return 0.2 + 0.6 * rand()
        if leaf == "pb":           # sigmoid attention: weights start small
            return -2.0 + 0.5 * randn()
        if name.endswith("a2.b"):  # decay gates biased toward slow decay
            return 2.0 + 0.5 * randn()
        if leaf == "b" and (len(shape) == 1 or name.endswith(("ra.b", "ri.b"))):     # biases
            return 0.1 * randn()
        if leaf == "conv":
            return randn() * shape[1] ** -0.5
        if leaf in ("embed", "bigram"):
            return randn()
        return randn() * shape[-1] ** -0.5

    def init_random(self, seed: int = 0, std: float = 0.02) -> "LayeredDecoder":
        """Deterministic per-name weights, rounded to bf16 as a checkpoint would hold them."""
        shapes = self.full_shapes()
        open_ = [n for n, s in shapes.items() if any(d is None for d in s)]
        if open_:
            raise ValueError(f"random weights need every size in the config; open: {open_[:4]}")
        sd = {n: self._random(n, s, seed, self.device).to(torch.bfloat16) for n, s in shapes.items()}
        return self.load_state(sd)

    def load_state(self, sd: Dict[str, torch.Tensor]) -> "LayeredDecoder":
        shapes = self.full_shapes()
        missing = set(shapes) - set(sd)
        if missing:
            raise KeyError(f"missing weights: {sorted(missing)[:5]}...")
        for n, shape in shapes.items():
            got = tuple(sd[n].shape)
            if len(got) != len(shape) or any(w is not None and w != g for w, g in zip(shape, got)):
                raise ValueError(f"{n}: checkpoint shape {got} != config shape {tuple(shape)}")
        dev, dt = self.device, self.dtype
        get = lambda n: sd[n].to(dev)  # noqa: E731
        self.embed = get("embed").to(dt).contiguous()
        self.head = self.embed if self.tied_head else get("head").to(dt).contiguous()
        self.final_norm = get("final.norm").float().contiguous()
        self.load_extra(get)
        for l in self.layers:
            self.load_layer(l, get)
        return self

    def weight_tensors(self):
        ts = [self.embed] if self.tied_head else [self.embed, self.head]
        for l in self.layers:
            ts += [t for t in (l.w_in, getattr(l, "w_ff", None)) if t is not None]
        return ts

    def num_bytes(self) -> int:
        b = sum(t.numel() * t.element_size() for t in self.weight_tensors())
        for l in self.layers:
            b += l.mixer.num_bytes() + (l.ff.num_bytes() if l.ff else 0)
        return b

    # -- cache -------------------------------------------------------------------------------------
    def cache_specs(self):
        return [l.mixer.cache_spec() for l in self.layers]

    def kv_bytes_per_block(self) -> int:
        return HybridCache.bytes_per_block(self.cache_specs(), 4 if self.dtype == torch.float32 else 2)

    def make_cache(self, num_blocks: int, num_slots: int) -> HybridCache:
        return HybridCache(self.cache_specs(), num_blocks, num_slots, self.dtype, self.device, self.slot_arrays)

    def lm_weight(self) -> torch.Tensor:
        return self.head

    def logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.head)
