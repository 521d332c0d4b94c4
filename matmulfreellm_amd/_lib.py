"""ctypes binding of lib/libmmf_hip.so (the C ABI declared in include/mmf.h).

There is no CPU implementation behind these calls: if the shared library is missing the
first use raises, it never falls back to another code path.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libmmf_hip.so")

MMF_F32, MMF_BF16, MMF_F16 = 0, 1, 2
_DTYPE_IDS = {torch.float32: MMF_F32, torch.bfloat16: MMF_BF16, torch.float16: MMF_F16}
_ERRORS = {-1: "MMF_ERR_ARG (bad shape, null pointer or unsupported dtype combination)",
           -2: "MMF_ERR_WIDE (row wider than the fused kernels support)",
           -3: "MMF_ERR_ALIGN (pointer not 16-byte aligned)"}

_i64, _i32, _f32, _ptr = ctypes.c_int64, ctypes.c_int, ctypes.c_float, ctypes.c_void_p

# name -> (restype, argtypes); must list every symbol include/mmf.h and include/mmf_diag.h declare.
SIGNATURES = {
    "mmf_packed_bytes": (_i64, [_i64, _i64]),
    "mmf_ternarize_workspace_bytes": (_i64, []),
    "mmf_ternarize_pack": (_i32, [_ptr, _i32, _i64, _i64, _ptr, _ptr, _ptr, _ptr]),
    "mmf_ternarize_pack_noalloc_max_elements": (_i64, []),
    "mmf_ternarize_pack_noalloc": (_i32, [_ptr, _i32, _i64, _i64, _ptr, _ptr, _ptr]),
    "mmf_unpack_ternary": (_i32, [_ptr, _i64, _i64, _ptr, _ptr]),
    "mmf_rmsnorm": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32, _i32, _i32, _i32, _ptr]),
    "mmf_rmsnorm_swishgate": (_i32, [_ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32, _i32, _i32, _i32, _ptr]),
    "mmf_swiglu": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _i64, _i64, _i32, _ptr]),
    "mmf_codes_bytes": (_i64, [_i64, _i64, _i32]),
    "mmf_rmsnorm_quant": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32, _i32, _i32, _i32, _i32, _ptr]),
    "mmf_layernorm_quant": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32, _i32, _i32, _i32, _i32, _ptr]),
    "mmf_rmsnorm_quant_fused": (_i32, [_i32, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _f32, _ptr, _f32, _ptr, _ptr, _ptr, _ptr,
                                       _ptr, _i64, _i64, _i32, _i32, _ptr]),
    "mmf_decode_layers_phase_bytes": (_i32, []),
    "mmf_decode_layers_copies": (_i32, []),
    "mmf_decode_layers_words": (_i64, [_i32, _i32, _i32]),
    "mmf_decode_layers": (_i32, [_ptr, _i32, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                 _i32, _i32, _i32, _i32, _i32, _ptr]),
    "mmf_decode_layers_trace_words": (_i32, []),
    "mmf_decode_layers_traced": (_i32, [_ptr, _i32, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr,
                                        _i32, _i32, _i32, _i32, _i32, _i32, _ptr]),
    "mmf_bitlinear_gemv_max_k": (_i64, []),
    "mmf_bitlinear_gemv": (_i32, [_ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _i64, _i64, _f32, _i32, _i32, _ptr]),
    "mmf_bitlinear_gemv_fused": (_i32, [_i32, _i32, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _f32, _ptr, _f32, _ptr, _ptr, _i64, _ptr,
                                        _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _i32, _ptr]),
    "mmf_bitlinear_mfma": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i64, _i32, _i32, _ptr]),
    "mmf_bitlinear_mfma_swiglu": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _i64, _i64, _i64, _i32, _ptr]),
    "mmf_bitlinear_mfma_clock_sink": (_i32, [_ptr, _i64]),
    "mmf_mfma_pipe_probe": (_i32, [_i64, _i64, _i32, _ptr, _ptr]),
    "mmf_diag_check_exact_forms": (_i32, [_ptr, _ptr]),
    "mmf_hgrn_recurrent": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _ptr]),
    "mmf_hgrn_chunk_workspace_bytes": (_i64, [_i64, _i64, _i64, _i32]),
    "mmf_hgrn_chunk": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _i32, _ptr, _ptr]),
    "mmf_hgrn_gate": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _ptr]),
    "mmf_hgrn_step": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _ptr]),
    "mmf_embedding": (_i32, [_ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _ptr]),
    "mmf_argmax": (_i32, [_ptr, _i64, _i64, _i64, _ptr, _i32, _ptr]),
    "mmf_cross_entropy_fwd": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _i64, _i64, _i32, _ptr]),
    "mmf_backward_groups": (_i32, [_i64]),
    "mmf_rmsnorm_bwd": (_i32, [_i32, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _f32,
                               _i32, _i32, _ptr]),
    "mmf_swiglu_bwd": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _ptr, _i64, _i64, _i64, _i32, _ptr]),
    "mmf_hgrn_gate_bwd": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _ptr, _i64, _ptr, _ptr, _i64, _i64, _i32,
                                 _ptr]),
    "mmf_hgrn_recurrent_bwd": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _i32, _ptr]),
    "mmf_cross_entropy_train_fwd": (_i32, [_ptr, _i64, _ptr, _i64, _f32, _f32, _f32, _ptr, _ptr, _ptr, _i64, _i64, _i32, _ptr]),
    "mmf_cross_entropy_train_bwd": (_i32, [_ptr, _i64, _ptr, _i64, _ptr, _ptr, _f32, _f32, _f32, _ptr, _i64, _i64, _i64, _i32, _ptr]),
    "mmf_short_conv_max_kernel_size": (_i32, []),
    "mmf_short_conv_fwd": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _i32, _i32, _ptr]),
    "mmf_short_conv_step": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i32, _i32, _i32, _ptr]),
    "mmf_short_conv_bwd_groups": (_i32, [_i64]),
    "mmf_short_conv_bwd": (_i32, [_ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _ptr, _i64, _i64, _i64, _i32, _i32, _i32, _ptr]),
    "mmf_sample_top_p_max_vocab": (_i64, []),
    "mmf_sample_top_p": (_i32, [_ptr, _i64, _i64, _i64, _f32, _f32, _i64, _ptr, _ptr, _i32, _ptr]),
}

_lib = None


class MMFError(RuntimeError):
    pass


def load():
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise MMFError(f"{LIB_PATH} is missing: build it with `python -m matmulfreellm_amd.build` "
                           "(there is no fallback path)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc, what):
    if rc == 0:
        return
    if rc < 0:
        raise MMFError(f"{what}: {_ERRORS.get(rc, rc)}")
    raise MMFError(f"{what}: HIP error {rc}")


def dtype_id(dtype):
    try:
        return _DTYPE_IDS[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; expected float32, bfloat16 or float16") from None


def require_gpu(*tensors):
    """All given tensors must live on one ROCm device; returns that device."""
    dev = None
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise MMFError("matmulfreellm_amd runs on a ROCm device only: got a tensor on "
                           f"'{t.device}'; move the module and its inputs to 'cuda' (there is no CPU path)")
        if dev is None:
            dev = t.device
        elif t.device != dev:
            raise MMFError(f"tensors on different devices: {dev} and {t.device}")
    return dev


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream
