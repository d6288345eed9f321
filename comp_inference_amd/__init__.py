"""comp_inference_amd: the compressed-weight hot path of comp_inference for MI355X (gfx950).

The public names follow the reference package (comp_inference/__init__.py:13-59); the
implementation is a C-ABI HIP library (libcomp_inference_hip.so) driven through ctypes.
"""
from . import ccore
from .comp_inference import (
    compressed_nbytes,
    extract_exp_and_mantissa,
    get_rans_lut,
    interleave_mantissas,
    interleave_mantissas_ilp2,
    rans_compress_gate_up_fused,
    rans_compress_module_weight,
    rans_compress_qkv_fused,
    rans_decompress_module_weight,
    reconstruct_from_exp_and_mantissa,
    uninterleave_mantissas,
    uninterleave_mantissas_ilp2,
)
from .embedding_hip import (
    fused_rans_embedding,
    fused_rans_embedding_one_stream,
    fused_rans_embedding_triton,
    fused_rans_embedding_triton_uncoalesced,
    fused_rans_embedding_uncoalesced,
)
from .linear_hip import (
    debug_wait_limit,
    dense_matmul,
    device_status,
    fused_rans_linear,
    fused_wide_rows,
    fused_rans_linear_one_stream,
    fused_rans_linear_triton,
    fused_rans_linear_triton_uncoalesced,
    fused_rans_linear_uncoalesced,
    plain_linear_same_order,
    release_scratch,
    splitk_reduce,
    triton_matmul,
)
from .rans_hip import (
    build_checkpoints,
    build_slot_table,
    rans_decomp_flat,
    rans_decomp_tiled,
    rans_decomp_tiled_batch,
    rans_decomp_tiled_one_stream,
    rans_decomp_tiled_uncoalesced,
    rans_decomp_triton,
    rans_decomp_triton_tiled,
    suggest_segments,
)
from .transposed_linear_hip import (
    fused_rans_linear_transposed,
    head_matrix_sums,
    fused_rans_linear_transposed_one_stream,
    fused_rans_linear_transposed_triton,
    fused_rans_linear_transposed_triton_uncoalesced,
    fused_rans_linear_transposed_uncoalesced,
    plain_linear_transposed_same_order,
)
from .pytorch_runtime import (
    RansEmbedding,
    RansLinear,
    RansLMHead,
    RansWorkspace,
    load_compressed_model_with_auto_model,
    swap_in_rans_modules,
)
from .rans_saving import (
    load_compressed_model,
    pack_and_save_tensors,
    parse_rans_info,
    rans_tensors_for_module,
    save_rans_model_package,
)
from .rans_gguf import save_rans_model_gguf
