"""ctypes binding of libvqattn_gfx950.so (the C ABI declared in include/vqattn.h)."""
import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
# VQATTN_LIB points at an alternative build of the same ABI (kernel tuning experiments)
LIB_PATH = os.environ.get("VQATTN_LIB") or os.path.join(_PKG_DIR, "libvqattn_gfx950.so")

_lib = None

_P = c_void_p
_STRIDES = ctypes.POINTER(c_int64)

# name -> (restype, argtypes); one entry per symbol declared in include/vqattn.h
SIGNATURES = {
    "vqa_version": (c_int, []),
    "vqa_strerror": (c_char_p, [c_int]),
    "vqa_decode_default_splits": (c_int, [c_int, c_int, c_int]),
    "vqa_decode_workspace_bytes": (c_size_t, [c_int] * 7),
    "vqa_decode_bf16": (c_int, [_P] * 7 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_float, c_int, _P]),
    "vqa_decode_f16": (c_int, [_P] * 7 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_float, c_int, _P]),
    "vqa_decode_static_bf16": (c_int, [_P] * 6 + [c_int] * 6 + [_STRIDES, c_float, c_int, _P]),
    "vqa_decode_devlen_bf16": (c_int, [_P] * 7 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_float, c_int, _P, _P]),
    "vqa_decode_devlen_f16": (c_int, [_P] * 7 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_float, c_int, _P, _P]),
    "vqa_decode_roped_bf16": (c_int, [_P] * 9 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_float, c_int, _P, _P]),
    "vqa_decode_roped_f16": (c_int, [_P] * 9 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_float, c_int, _P, _P]),
    "vqa_decode_windowed_workspace_bytes": (c_size_t, [c_int] * 6),
    "vqa_decode_windowed_bf16": (c_int, [_P] * 9 + [c_size_t] + [c_int] * 7 + [_STRIDES, c_float, _P]),
    "vqa_decode_windowed_f16": (c_int, [_P] * 9 + [c_size_t] + [c_int] * 7 + [_STRIDES, c_float, _P]),
    "vqa_decode_exact_workspace_bytes": (c_size_t, [c_int] * 5),
    "vqa_decode_exact_bf16": (c_int, [_P] * 6 + [c_size_t] + [c_int] * 4 + [_STRIDES, c_float, c_int, _P]),
    "vqa_decode_exact_f16": (c_int, [_P] * 6 + [c_size_t] + [c_int] * 4 + [_STRIDES, c_float, c_int, _P]),
    "vqa_local_attn_bf16": (c_int, [_P] * 7 + [c_int] * 4 + [_STRIDES, c_int, c_int, c_float, _P]),
    "vqa_local_attn_f16": (c_int, [_P] * 7 + [c_int] * 4 + [_STRIDES, c_int, c_int, c_float, _P]),
    "vqa_rerope_full_bf16": (c_int, [_P] * 7 + [c_int] * 4 + [_STRIDES, c_int, c_int, c_float, _P]),
    "vqa_rerope_full_f16": (c_int, [_P] * 7 + [c_int] * 4 + [_STRIDES, c_int, c_int, c_float, _P]),
    "vqa_prefill_workspace_bytes": (c_size_t, [c_int] * 4),
    "vqa_prefill_bf16": (c_int, [_P] * 10 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_int, c_int, c_int, c_float, _P]),
    "vqa_prefill_f16": (c_int, [_P] * 10 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_int, c_int, c_int, c_float, _P]),
    "vqa_prefill_tiled_bf16": (c_int, [_P] * 10 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_int, c_int, c_int, c_float, _P]),
    "vqa_prefill_tiled_f16": (c_int, [_P] * 10 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_int, c_int, c_int, c_float, _P]),
    "vqa_prefill_pipelined_bf16": (c_int, [_P] * 8 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_int, c_int, c_float, _P]),
    "vqa_prefill_pipelined_f16": (c_int, [_P] * 8 + [c_size_t] + [c_int] * 6 + [_STRIDES, c_int, c_int, c_float, _P]),
    "vqa_prefill_f32": (c_int, [_P] * 6 + [c_int] * 6 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_fwd_bf16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_fwd_f16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_merge_bf16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_merge_f16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_fwd_icnt_bf16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_fwd_icnt_f16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_merge_icnt_bf16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_vqcount_merge_icnt_f16": (c_int, [_P] * 7 + [c_int] * 5 + [_STRIDES, c_int, c_float, _P]),
    "vqa_merge_state_inplace_bf16": (c_int, [_P] * 4 + [c_int] * 4 + [_STRIDES, _P]),
    "vqa_merge_state_inplace_f16": (c_int, [_P] * 4 + [c_int] * 4 + [_STRIDES, _P]),
    "vqa_encode_keys_bf16": (c_int, [_P] * 4 + [c_int] * 6 + [_STRIDES, c_int, c_int, _P]),
    "vqa_encode_keys_f16": (c_int, [_P] * 4 + [c_int] * 6 + [_STRIDES, c_int, c_int, _P]),
    "vqa_rope_bf16": (c_int, [_P] * 6 + [c_int] * 5 + [c_int64, _STRIDES, c_int, _P]),
    "vqa_rope_f16": (c_int, [_P] * 6 + [c_int] * 5 + [c_int64, _STRIDES, c_int, _P]),
    "vqa_count_state_add_bf16": (c_int, [_P] * 4 + [c_int] * 5 + [_STRIDES, _P]),
    "vqa_count_state_add_f16": (c_int, [_P] * 4 + [c_int] * 5 + [_STRIDES, _P]),
    "vqa_count_decode_bf16": (c_int, [_P] * 6 + [c_int] * 4 + [_STRIDES, c_float, _P]),
    "vqa_count_decode_f16": (c_int, [_P] * 6 + [c_int] * 4 + [_STRIDES, c_float, _P]),
    "vqa_count_step_bf16": (c_int, [_P] * 10 + [c_int] * 4 + [_STRIDES, c_float, _P]),
    "vqa_count_step_f16": (c_int, [_P] * 10 + [c_int] * 4 + [_STRIDES, c_float, _P]),
    "vqa_preprocess_workspace_bytes": (c_size_t, [c_int] * 4),
    "vqa_preprocess_bf16": (c_int, [_P] * 7 + [c_size_t] + [c_int] * 5 + [_STRIDES, _P]),
    "vqa_preprocess_f16": (c_int, [_P] * 7 + [c_size_t] + [c_int] * 5 + [_STRIDES, _P]),
    "vqa_preprocess_state_bf16": (c_int, [_P] * 9 + [c_size_t] + [c_int] * 5 + [_STRIDES, _P]),
    "vqa_preprocess_state_f16": (c_int, [_P] * 9 + [c_size_t] + [c_int] * 5 + [_STRIDES, _P]),
}


class VqaError(RuntimeError):
    pass


def load():
    """Load the shared library once.  Raises if it has not been built (python -m vqtree_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise VqaError(
                f"{LIB_PATH} is missing: build it with `python -m vqtree_amd.build` (hipcc, gfx950). "
                "There is no CPU fallback."
            )
        lib = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = lib
    return _lib


def check(status: int):
    if status != 0:
        raise VqaError(f"libvqattn: {load().vqa_strerror(status).decode()} (status {status})")


def strides_array(*values):
    return (c_int64 * len(values))(*values)


def current_stream(device):
    import torch

    return c_void_p(torch.cuda.current_stream(device).cuda_stream)


def require_gpu(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise VqaError("vqtree_amd operators run on the GPU only (tensor on %s)" % t.device)
