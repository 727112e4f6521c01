"""Op layer: Python entry points for the gfx950 HIP kernels (``csrc/kernels``).

Each op dispatches on the tensor's device: CUDA(HIP) tensors run the native kernel (and fail
loudly if the library is missing), CPU tensors run an fp32 PyTorch reference that is also the
oracle in the numerics tests.
"""
from .activation import gelu_, silu_mul
from .attention import (KV_BS, DecodeWorkspace, decode, default_scale, prefill, rope_cos_sin, rope_kv_write,
                        write_kv_ref)
from .embedding import embedding
from .mixers import (conv_act, conv_silu, decay_scan, embed_f32, embed_pairs, embed_scaled, glu_act, glu_clamp, group_norm,
                     head_norm_gate, hyper_mix, latent_attend, latent_prep, layer_norm_out, logit_cap, lru_scan, matrix_scan,
                     moe_combine, post_norm_add, qk_norm_write, relu2, residual_norm, rope_freqs, rope_heads, route_biased,
                     route_scores, ssm_scan, window_attend)
from .norm import layer_norm, rms_norm
from .retrieval import filtered_topk
from .sampling import (apply_top_k_top_p, fused_lm_head_ok, lm_head_sample, lm_head_sample_shard, lm_head_stream_sample,
                       pick_pairs, sample,
                       sample_shard)

__all__ = ["gelu_", "silu_mul", "KV_BS", "DecodeWorkspace", "decode", "default_scale", "prefill", "rope_cos_sin",
           "rope_kv_write", "write_kv_ref", "embedding", "layer_norm", "rms_norm", "filtered_topk",
           "apply_top_k_top_p", "sample", "conv_silu", "embed_f32", "glu_clamp", "group_norm", "latent_attend",
           "latent_prep", "moe_combine", "relu2", "residual_norm", "route_biased", "ssm_scan", "conv_act", "embed_pairs",
           "glu_act", "head_norm_gate", "layer_norm_out", "lru_scan", "matrix_scan", "post_norm_add", "qk_norm_write",
           "route_scores", "window_attend", "decay_scan", "embed_scaled", "hyper_mix", "logit_cap", "rope_freqs",
           "rope_heads"]
