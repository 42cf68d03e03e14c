"""MI355X-native AWQ int4 group-128 batch-1 decode (host-side mirror of the C-ABI in include/awq_hip.h)."""
from ._lib import AwqError, lib, lib_path  # noqa: F401
from .ops import (  # noqa: F401
    Context,
    DeviceBuffer,
    QWeight,
    Sampler,
    MultiHeadAttention,
    MultiHeadAttention_partial,
    RoPERotation,
    argmax_advance,
    copy_embedding,
    dequant,
    ffn_matvec_silu,
    gemm_q,
    gemm_q_static,
    matmul,
    matmul_q,
    matmul_q_parts,
    qkv_matvec,
    rmsnorm,
    rmsnorm_ffn_matvec_silu,
    sample_top_p,
    softmax_logits,
)
from .model import Transformer, SCHEDULE_FUSED, SCHEDULE_PERSISTENT, SCHEDULE_REFERENCE  # noqa: F401
