"""Model families: Llama-3 (8B/70B), Mixtral-8x7B MoE, BERT/bge encoder, and the layered decoders Gezavik, Sigudra, Tukedra and Purozen."""
from __future__ import annotations

from .configs import LAYERED_ARCHS, REGISTRY, ModelConfig, get_model_config


def build_model(engine_cfg, device, seed: int = 0):
    """Instantiate the decoder named by ``engine_cfg.model`` on ``device`` (random-init unless
    ``engine_cfg.weights`` points at a safetensors checkpoint directory)."""
    from .llama import LlamaModel
    from .mixtral import MixtralModel
    cfg = get_model_config(engine_cfg.model)
    if cfg.arch in LAYERED_ARCHS:
        return _build_layered(cfg, engine_cfg, device, seed)
    if cfg.arch == "mixtral":
        model = MixtralModel(cfg, device=device, fp8=getattr(engine_cfg, "dtype", "bf16") == "fp8",
                             moe_parallel=getattr(engine_cfg, "moe_parallel", "tp"))
    elif cfg.arch == "llama":
        shard = int(getattr(engine_cfg, "shard_of_tp", 0) or 0)
        # estimate mode: rank 0's shard of a TP=shard group, alone on this device (collectives are
        # identity while the process group is TP=1)
        model = LlamaModel(cfg, device=device, tp_rank=0, tp_size=shard) if shard > 1 else LlamaModel(cfg, device=device)
    else:
        raise ValueError(f"{cfg.name} is not a decoder")
    model.sequence_parallel = bool(getattr(engine_cfg, "sequence_parallel", False))
    if engine_cfg.weights:
        from .weights import load_decoder_weights
        load_decoder_weights(model, engine_cfg.weights)
        if cfg.arch == "mixtral" and model.fp8:
            model.quantize_experts()          # checkpoint experts (bf16) -> tiled fp8 + row scales
    else:
        model.init_random(seed=engine_cfg.seed if hasattr(engine_cfg, "seed") else seed)
    return model


def _build_layered(cfg, engine_cfg, device, seed: int):
    """Layered decoders run in bf16 (f32 statistics, state and residual stream) or, with
    ``dtype="fp32"``, in true f32 throughout; their checkpoint is the model directory itself."""
    import os

    import torch

    from .gezavik import GezavikModel
    from .sigudra import SigudraModel
    from .purozen import PurozenModel
    from .tukedra import TukedraModel
    from .weights import read_safetensors
    cls = {"gezavik": GezavikModel, "sigudra": SigudraModel, "tukedra": TukedraModel, "purozen": PurozenModel}[cfg.arch]
    if getattr(engine_cfg, "tp_size", 1) > 1:
        raise ValueError(f"{cfg.name}: tensor parallelism is not implemented for layered decoders")
    dtype = str(getattr(engine_cfg, "dtype", "bf16")).lower()
    if dtype not in ("bf16", "bfloat16", "fp32", "float32"):
        raise ValueError(f"{cfg.name}: dtype must be bf16 or fp32, got {dtype!r}")
    f32 = dtype in ("fp32", "float32")
    if f32:      # no reduced-precision matrix mode for f32 products
        torch.backends.cuda.matmul.allow_tf32 = False
        torch.backends.cudnn.allow_tf32 = False
    model = cls(cfg, device=device, dtype=torch.float32 if f32 else torch.bfloat16)
    src = engine_cfg.weights or (engine_cfg.model if os.path.isdir(engine_cfg.model) else None)
    if src:
        model.load_state(read_safetensors(src))
    else:
        model.init_random(seed=engine_cfg.seed if hasattr(engine_cfg, "seed") else seed)
    return model


__all__ = ["REGISTRY", "ModelConfig", "get_model_config", "build_model"]
