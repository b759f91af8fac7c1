"""MI355X (gfx950) implementation of ruquant's W4A4 / W4A4H MUL_MAT behind a C ABI.

The product is ``ruquant_amd/lib/librq_w4a4.so`` (hand-written HIP, see ``ruquant_amd/csrc``) and its
header ``include/rq_w4a4.h``. This package is the thin Python host over that ABI: torch is used only to own
device memory and streams.
"""
from .lib import load_library, load_probe_library, build_library, LibraryMissing  # noqa: F401
from .w4a4 import (  # noqa: F401
    TYPE_W4A4, TYPE_W4A4H, TYPE_A4, TYPE_A4H, BLOCK_DTYPE,
    W4A4Weight, supported, hadamard_factor, resolve_clip, tensor_rot,
    mul_mat, mul_mat_fused, fused_workspace_bytes, hadamard, quantize_act, RqError, SharedActivation,
    pack, pack_groups, set_clip, set_rot_len, dequantize_rows, quantize_weights, dequantize,
)
