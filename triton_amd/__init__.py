"""MI355X-native tiled kernels behind the host surface of the Triton tutorials:
`matmul(a, b)`, `attention(q, k, v, causal, sm_scale)` and the block-scaled `mx_matmul`."""
from .ops import attention, chain_dot, dequantize, group_gemm_fn, matmul, matmul_like_input, matmul_persistent, matmul_streamk, mx_matmul  # noqa: F401

__all__ = ["matmul", "chain_dot", "matmul_like_input", "matmul_persistent", "matmul_streamk", "group_gemm_fn", "attention", "mx_matmul", "dequantize"]
