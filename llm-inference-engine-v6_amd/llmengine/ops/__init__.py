"""The HIP kernels of the engine, as Python functions over device tensors."""
from .lib import KernelError, KernelLibraryError, library, load_kernels
from .choices import KernelChoices
from .kernels import (ATTENTION_MAX_HEAD_DIM, argmax, argmax_into, attention, attention_generic, attention_project, block_weight, can_block, clear, embed_gather, gemm,
                      gemm_generic, is_blocked, policy, rmsnorm, rope_kv_write, rope_q_only, sample, sample_into, sampling_scratch, swiglu,
                      unblock_weight, weight_shape)

from . import mfma                                   # noqa: E402  (installs the MFMA kernels)
from .mfma import (gemm_bf16, gemm_gated, gemm_gated_extra, gemm_qkv_rope, gemm_qkv_rope_supported, gemv_norm, gemv_norm_rope, gemv_norm_rope_supported,
                   gemv_norm_supported, pair_rows_for_rotation)

from . import recurrent                              # noqa: E402
from .recurrent import (GATE_ACTIVATIONS, copy_cols, delta_gates, delta_rule, gated_activation, gated_head_norm, rglru_gates, rglru_scan,
                        rotate_write, short_conv, sigmoid_attention, sigmoid_attention_fits, sigmoid_decay, streams_read_norm, streams_spread,
                        streams_write, streams_write_read_norm, unit_heads)

from . import latent                                 # noqa: E402
from .latent import (head_gemm, latent_attention, latent_attention_fits, latent_prepare, latent_q_rotate, moe_capacity, moe_combine,
                     moe_gemm, moe_plan, moe_route, norm_add, scale_)

from . import window                                 # noqa: E402

__all__ = ["window", "sigmoid_decay", "latent", "head_gemm", "latent_attention", "latent_attention_fits", "latent_prepare", "latent_q_rotate", "moe_capacity",
           "moe_combine", "moe_gemm", "moe_plan", "moe_route", "norm_add", "scale_", "GATE_ACTIVATIONS", "copy_cols", "delta_gates", "delta_rule", "gated_activation", "gated_head_norm", "rglru_gates", "rglru_scan",
           "rotate_write", "short_conv", "sigmoid_attention", "sigmoid_attention_fits", "streams_read_norm", "streams_spread",
           "streams_write", "streams_write_read_norm", "unit_heads", "recurrent", "KernelChoices", "ATTENTION_MAX_HEAD_DIM", "gemm_bf16", "gemm_gated", "gemm_gated_extra", "gemm_qkv_rope", "gemm_qkv_rope_supported", "gemv_norm_rope", "gemv_norm_rope_supported", "pair_rows_for_rotation", "gemv_norm", "gemv_norm_supported", "mfma", "KernelError", "KernelLibraryError", "library", "load_kernels", "argmax", "argmax_into", "attention", "attention_generic", "attention_project", "rope_q_only", "embed_gather", "block_weight", "can_block", "clear",
           "is_blocked", "unblock_weight", "weight_shape",
           "gemm", "gemm_generic", "policy", "rmsnorm", "rope_kv_write", "sample", "sample_into", "sampling_scratch", "swiglu"]
