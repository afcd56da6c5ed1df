"""MI355X-native ring attention hot path.

Exports the names of the reference package (ringattention/__init__.py:26-27 binds ``ringattention``
per backend; here there is one backend, the gfx950 HIP kernels):

    ringattention, ringattention_jax, ringattention_inference, blockwise_feedforward

plus ``ring_axis`` to declare the size of the (virtual) sequence-parallel ring, ``SwiGLU``,
``decode_attention``, the two steps either side of the path, ``rope_kv_append`` and ``rmsnorm_residual``, and
``kernel_family_of_last_call`` (which kernels the automatic choice took).
"""
from .ringattention_hip import (ring_attention, ring_axis, axis_size, below_or_on_diag, run_prefix_keys,
                                kernel_family_of_last_call, _blockwise_attention_fwd, _blockwise_attention_bwd)
from .feedforward import blockwise_feedforward, SwiGLU, gemm_bf16
from .decode import decode_attention, decode_workspace
from .inference import ring_attention_inference
from .steps import rope_kv_append, rmsnorm_residual

ringattention = ring_attention
ringattention_jax = ring_attention
ringattention_inference = ring_attention_inference

__all__ = ["ringattention", "ringattention_jax", "ringattention_inference", "ring_attention",
           "ring_attention_inference", "blockwise_feedforward", "ring_axis",
           "axis_size", "SwiGLU", "decode_attention", "decode_workspace", "below_or_on_diag", "rope_kv_append", "rmsnorm_residual",
           "kernel_family_of_last_call"]
