"""tqhip: the PolarQuant KV-cache hot path on AMD MI355X (gfx950).

Import surface of the reference package (turboquant_mlx/__init__.py:1-22) on torch tensors,
backed by hand-written HIP kernels in libtqhip.so.
"""
from .cache import TurboQuantKVCache
from .v_only_cache import VOnlyTurboQuantCache
from .kvcache import KVCache, create_causal_mask
from .adaptive import make_adaptive_cache
from .quantizer import PolarQuantizer
from .ops import (
    fused_quantize,
    encode_into,
    dequant_into,
    dequant_fp16,
    packed_dequantize,
    packed_fused_qk_scores,
    prerotate_query,
    prerot_fused_qk_scores,
    prerot_packed_dequantize,
    sparse_v_matvec,
    count_active_positions,
    flash_attention_turboquant,
    flash_decode,
    flash_decode_from_q,
    prefill_attention,
    vonly_decode,
    vonly_append_into,
    vonly_decode_step,
    VOnlyStep,
    packed_decode_step,
    PackedStep,
    dense_qk_scores,
    softmax_rows,
    pack_indices,
    unpack_indices,
    packed_dim,
)
from .attention import turboquant_attention, turboquant_prefill_attention, vonly_decode_attention
from .patch import apply_patch, remove_patch, scaled_dot_product_attention
from .rotation import (
    walsh_hadamard_transform,
    randomized_hadamard_transform,
    inverse_randomized_hadamard,
    random_diagonal_sign,
)

__version__ = "0.1.0"
