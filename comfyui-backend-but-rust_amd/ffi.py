"""Python view of the C ABI in include/gpu_api.h, mirroring the reference's Rust declarations (src/ffi.rs:11-40,74-75,
121,246-252) and its checked-call helpers `ok` / `k!` (src/ffi.rs:336-351).

Pointers are raw device addresses (ints); `s` is a hipStream_t handle (int, 0 = default stream).  The library is the
in-tree libgpu_kernels.so; importing this module fails loudly if it has not been built -- there is no fallback path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libgpu_kernels.so")

DT_F32, DT_F16, DT_BF16 = 0, 1, 2
(PRO_PLAIN, PRO_RMS, PRO_GATE, PRO_SWIGLU, PRO_LAYERNORM, PRO_SILU, PRO_GELU, PRO_ADALN, PRO_SITU, PRO_LN_MOD,
 PRO_LN_AFFINE, PRO_GELU_TANH, PRO_LN_AFFINE_SILU, PRO_SITU_FAST) = range(14)

_P, _I64, _I32, _F32, _U64 = C.c_void_p, C.c_int64, C.c_int, C.c_float, C.c_uint64

# name -> argtypes, in the order of include/gpu_api.h
SIGNATURES = {
    "gpu_quant_rows": [_I32, _I32, _P, _I64, _P, _I64, _I64, _P, _F32, _P, _P, _P, _P, _I32, _I32, _I32, _P],
    "gpu_quant_rows_b": [_I32, _I32, _P, _I64, _P, _P, _F32, _P, _P, _P, _P, _I32, _I32, _I32, _P],
    "gpu_rotate_rows_f32": [_I32, _P, _I64, _I64, _P, _F32, _P, _I32, _I32, _P],
    "gpu_sd_quant_rows": [_P, _I64, _P, _P, _I32, _I32, _I32, _P],
    "gpu_sd_ln_quant_rows": [_P, _I64, _P, _P, _F32, _P, _P, _I32, _I32, _I32, _P],
    "gpu_sd_geglu_quant_rows": [_P, _P, _P, _I32, _I32, _I32, _P],
    "gpu_sd_unpad_quant_rows": [_P, _P, _P, _I32, _I32, _I32, _I32, _I32, _P],
    "gpu_sd_group_norm_quant_rows": [_P, _P, _P, _P, _I32, _I64, _I32, _I32, _F32, _P, _P, _I32, _P],
    "gpu_dequant_i8": [_P, _P, _P, _I64, _I64, _P],
    "gpu_embed_dequant": [_P, _P, _P, _I32, _I32, _I32, _P],
    "gpu_convrot_dequant": [_I32, _P, _P, _P, _I64, _I32, _P],
    "gpu_convrot_requant": [_I32, _P, _P, _P, _I64, _I32, _U64, _P],
    "gpu_w6_requant": [_P, _P, _P, _P, _I64, _I32, _U64, _P],
    "gpu_prologue_rows": [_I32, _I32, _P, _I64, _P, _I64, _I64, _P, _F32, _P, _P, _P, _I64, _I32, _I32, _P],
    "gpu_prologue_rows_b": [_I32, _I32, _P, _I64, _P, _P, _F32, _P, _P, _P, _I64, _I32, _I32, _P],
    "gpu_int8_gemm": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P],
    "gpu_int8_gemm_residual": [_P, _P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P],
    "gpu_w6_decode": [_P, _P, _P, _I64, _I32, _I32, _P],
    "gpu_int8_gemm_acc": [_P, _P, _P, _I64, _I64, _I64, _P],
    "gpu_int8_gemm_static": [_P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P],
    "gpu_w6a8_gemm": [_P, _P, _P, _I32, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P],
    "gpu_w6a8_group_gemm": [_P, _P, _P, _P, _P, _P, _P, _I64, _I64, _I64, _I32, _P],
    "gpu_int8_attn_d": [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _I32] + [_I64] * 12 + [_F32, _P],
    "gpu_int8_attn_f16": [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32, _I32] + [_I64] * 12 + [_F32, _P],
    "gpu_int8_attn": [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32] + [_I64] * 12 + [_F32, _P],
    "gpu_int8_attn_sink": [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32] + [_I64] * 12 + [_F32, _F32, _P, _F32, _P],
    "gpu_int8_attn_norm_rope": [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32] + [_I64] * 12 + [_F32, _P, _P, _F32, _P, _I32, _P],
    "gpu_int8_attn_key_bias": [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _I32] + [_I64] * 12 + [_F32, _P, _P],
    "gpu_internal_cvt_pk_u8_probe": [_P, _P, _I32, _P],
    "gpu_internal_attn_sumsq_probe": [_P, _P, _I32, _I32, _P],
    "gpu_internal_w6a8_group_gemm_ablate": [_I32, _P, _P, _P, _P, _P, _I64, _I64, _I64, _P],
    "gpu_internal_w6a8_group_gemm_mode": [_I32],
    "gpu_internal_attn_layout": [_I32, _I32, _I32, _I32, _I32, _P],
    "gpu_internal_attn_layout_d": [_I32, _I32, _I32, _I32, _I32, _I32, _P],
    "gpu_int8_gemm_force_config": [_I32],
    "gpu_act_tables_init": [],
    "gpu_mfma_layout_probe": [_P, _P],
    "gpu_mfma_ceiling_probe": [_I32, _I32, _P, _P, _P],
}


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libgpu_kernels.so is not built (%s); run `python __graft_entry__.py` or the package's build.py" % LIB_PATH)
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = _I32
    lib.gpu_int8_attn_workspace_d.argtypes = [_I32] * 6
    lib.gpu_int8_attn_workspace_d.restype = _I64
    lib.gpu_int8_attn_workspace.argtypes = [_I32] * 5
    lib.gpu_int8_attn_workspace.restype = _I64
    lib.gpu_int8_attn_key_bias_workspace.argtypes = [_I32] * 5
    lib.gpu_int8_attn_key_bias_workspace.restype = _I64
    lib.gpu_int8_gemm_static_limit.argtypes = []
    lib.gpu_int8_gemm_static_limit.restype = _I64
    lib.gpu_kernels_build_info.restype = C.c_char_p
    lib.gpu_kernels_build_info.argtypes = []
    return lib


lib = _load()

_hip = None


def err_str(code):
    """Name of a positive return code: a hipError_t (the reference's cuda::err_str, src/cuda.rs:63-72)."""
    global _hip
    try:
        if _hip is None:
            _hip = C.CDLL("libamdhip64.so")
            _hip.hipGetErrorString.restype = C.c_char_p
            _hip.hipGetErrorString.argtypes = [C.c_int]
        return _hip.hipGetErrorString(int(code)).decode()
    except OSError:
        return "hip error %d" % code


class KernelError(RuntimeError):
    def __init__(self, what, code):
        self.code = code
        if code > 0:
            super().__init__("%s failed: %s" % (what, err_str(code)))
        else:
            super().__init__("%s failed with code %d" % (what, code))


def ok(code, what):
    """Turn a launcher return code into an error naming the call (src/ffi.rs:336-344)."""
    if code != 0:
        raise KernelError(what, code)


def k(name, *args):
    """Checked call, the `k!` macro of src/ffi.rs:346-351."""
    ok(getattr(lib, name)(*args), name)


def raw(name, *args):
    """Unchecked call: returns the launcher's code."""
    return getattr(lib, name)(*args)


# The dense GEMM beside the path lives in a library of its own (include/gpu_blas_api.h), loaded on first use so that the
# int8 path does not depend on hipBLASLt.
BLAS_LIB_PATH = os.path.join(_HERE, "libgpu_blas.so")
_SZ = C.c_size_t
BLAS_SIGNATURES = {
    "gpu_blas_init": [_SZ],
    "gpu_gemm": [_P, _I64, _P, _I64, _P, _I64, _P, _I64, _I64, _I64, _I32, _I32, _I32, _F32, _F32, _P],
}
_blas = None


def blas():
    global _blas
    if _blas is None:
        if not os.path.exists(BLAS_LIB_PATH):
            raise ImportError("libgpu_blas.so is not built (%s); run the package's build.py" % BLAS_LIB_PATH)
        L = C.CDLL(BLAS_LIB_PATH)
        for name, args in BLAS_SIGNATURES.items():
            fn = getattr(L, name)
            fn.argtypes = args
            fn.restype = _I32
        _blas = L
    return _blas


def kb(name, *args):
    """Checked call into the dense-GEMM library."""
    ok(getattr(blas(), name)(*args), name)


def build_info():
    return lib.gpu_kernels_build_info().decode()
