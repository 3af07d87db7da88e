"""ctypes view of the CPU oracle (oracle/qlinear_oracle.c).  TEST INFRASTRUCTURE ONLY.

Only tests/, the smoke check and the bench's CPU-baseline leg may import this module; the product path never does.
Arrays are numpy; bf16 and f16 tensors travel as uint16 bit patterns.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libqlinear_oracle.so")
F32, F16, BF16 = 0, 1, 2
_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            from . import build as _b
            _b.build()
        L = C.CDLL(_LIB_PATH)
        vp, i64, i32, f32 = C.c_void_p, C.c_int64, C.c_int, C.c_float
        L.orc_f32_to_bf16.restype = C.c_uint16; L.orc_f32_to_bf16.argtypes = [f32]
        L.orc_f32_to_f16.restype = C.c_uint16; L.orc_f32_to_f16.argtypes = [f32]
        L.orc_bf16_to_f32.restype = f32; L.orc_bf16_to_f32.argtypes = [C.c_uint16]
        L.orc_f16_to_f32.restype = f32; L.orc_f16_to_f32.argtypes = [C.c_uint16]
        L.orc_e4m3_to_f32.restype = f32; L.orc_e4m3_to_f32.argtypes = [C.c_uint8]
        L.orc_fht.restype = i32; L.orc_fht.argtypes = [vp, i32, i32]
        L.orc_quant_rows.restype = i32; L.orc_quant_rows.argtypes = [i32, vp, i64, vp, vp, i32, i32, i32]
        L.orc_rotate_rows_f32.restype = i32; L.orc_rotate_rows_f32.argtypes = [vp, i64, vp, i32, i32]
        L.orc_quant_rows_wide.restype = i32; L.orc_quant_rows_wide.argtypes = [i32, vp, i64, vp, vp, i32, i32, i32]
        L.orc_situ_rows_wide.restype = i32; L.orc_situ_rows_wide.argtypes = [i32, vp, i64, i64, vp, i32, i32]
        L.orc_sd_source_rows.restype = i32
        L.orc_sd_source_rows.argtypes = [i32, vp, i64, vp, vp, f32, i32, i32, i32, i32, i64, vp, i32, i32]
        L.orc_convrot_requant.restype = i32; L.orc_convrot_requant.argtypes = [i32, vp, vp, vp, i32, i32, C.c_uint64]
        L.orc_convrot_dequant.restype = i32; L.orc_convrot_dequant.argtypes = [i32, vp, vp, vp, i64, i32]
        L.orc_dequant_i8.restype = i32; L.orc_dequant_i8.argtypes = [vp, vp, vp, i64, i64]
        L.orc_f32_to_e4m3.restype = C.c_uint8; L.orc_f32_to_e4m3.argtypes = [f32]
        L.orc_w6_requant.restype = i32; L.orc_w6_requant.argtypes = [vp, vp, vp, vp, i64, i32, C.c_uint64]
        L.orc_prologue_rows.restype = i32
        L.orc_prologue_rows.argtypes = [i32, i32, vp, i64, vp, i64, i64, vp, vp, f32, vp, vp, vp, i64, i32, i32]
        L.orc_sd_quant_rows.restype = i32; L.orc_sd_quant_rows.argtypes = [vp, i64, vp, vp, i32, i32, i32]
        L.orc_int8_gemm_acc.restype = None; L.orc_int8_gemm_acc.argtypes = [vp, vp, vp, i64, i64, i64]
        L.orc_epilogue.restype = None; L.orc_epilogue.argtypes = [vp, vp, vp, vp, vp, i64, i64, i32, i32]
        L.orc_epilogue_residual.restype = None
        L.orc_epilogue_residual.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i32, i32]
        L.orc_int8_gemm.restype = i32; L.orc_int8_gemm.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i32, i32]
        L.orc_int8_gemm_residual.restype = i32
        L.orc_int8_gemm_residual.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i32, i32]
        L.orc_w6_decode.restype = i32; L.orc_w6_decode.argtypes = [vp, vp, vp, i64, i32, i32]
        L.orc_w6_pack_planes.restype = None; L.orc_w6_pack_planes.argtypes = [vp, vp, i64, i32]
        L.orc_w6_pack_words.restype = None; L.orc_w6_pack_words.argtypes = [vp, vp, i64, i32]
        L.orc_w6_unpack_words.restype = None; L.orc_w6_unpack_words.argtypes = [vp, vp, i64, i32]
        L.orc_w6a8_group_gemm.restype = i32
        L.orc_w6a8_group_gemm.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i32]
        L.orc_linear_w8a8.restype = i32
        L.orc_linear_w8a8.argtypes = [i32, vp, i64, i32, vp, vp, vp, vp, i32, i32, i32, i32, i32, vp]
        L.orc_set_threads.restype = None; L.orc_set_threads.argtypes = [i32]
        L.orc_attn_rot128.restype = None; L.orc_attn_rot128.argtypes = [vp]
        L.orc_attn_quant_qk.restype = i32
        L.orc_attn_quant_qk_norm.restype = i32
        L.orc_attn_quant_qk_norm.argtypes = [i32, vp, vp, i32, i32, i32, i32, i32, i64, i64, i64, i64, i64, i64, i32, i32, vp, vp,
                                             vp, vp, vp, i32, vp, vp, vp, C.c_float, i32]
        L.orc_attn_int8_bias.restype = i32
        L.orc_attn_int8_bias.argtypes = [i32, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, C.c_float, vp, vp, i64, i64, i64]
        L.orc_attn_quant_qk_d.restype = i32
        L.orc_attn_quant_qk_d.argtypes = [i32, vp, vp, i32, i32, i32, i32, i32, i32, i64, i64, i64, i64, i64, i64, i32, i32, vp, vp,
                                          vp, vp, vp, i32, vp, vp, vp, C.c_float, i32]
        L.orc_attn_quant_v_d.restype = i32
        L.orc_attn_quant_v_d.argtypes = [i32, vp, i32, i32, i32, i32, i64, i64, i64, vp, vp]
        L.orc_attn_int8_d.restype = i32
        L.orc_attn_int8_d.argtypes = [i32, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, i32, f32, f32, vp, i64, i64, i64, i32]
        L.orc_attn_rotate_d.restype = None
        L.orc_attn_rotate_d.argtypes = [vp, i32, i32]
        L.orc_attn_rotate.restype = None
        L.orc_attn_rotate.argtypes = [vp, i32]
        L.orc_attn_sumsq128.restype = C.c_float
        L.orc_attn_sumsq128.argtypes = [vp, i32]
        L.orc_attn_norm_rope_row.restype = None
        L.orc_attn_norm_rope_row.argtypes = [vp, vp, vp, C.c_float, i32]
        L.orc_attn_quant_qk.argtypes = [i32, vp, vp, i32, i32, i32, i32, i32, i64, i64, i64, i64, i64, i64, i32, i32, vp, vp, vp, vp, vp]
        L.orc_attn_quant_v.restype = i32; L.orc_attn_quant_v.argtypes = [i32, vp, i32, i32, i32, i64, i64, i64, vp, vp]
        L.orc_attn_int8.restype = i32
        L.orc_attn_int8.argtypes = [i32, vp, vp, vp, vp, vp, vp, i32, i32, i32, i32, i32, i32, f32, f32, vp, i64, i64, i64, i32]
        L.orc_attn_cta_k.restype = i32; L.orc_attn_cta_k.argtypes = [i32, i32]
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dt=None):
    a = np.ascontiguousarray(a)
    if dt is not None:
        assert a.dtype == dt, (a.dtype, dt)
    return a


_OUT_NP = {F32: np.float32, F16: np.uint16, BF16: np.uint16}
_IN_NP = {F32: np.float32, F16: np.uint16, BF16: np.uint16}


def bf16_bits(x):
    """float32 array -> bf16 bit patterns (RNE), elementwise through the oracle's scalar routine semantics."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & 0x7fffffff) > 0x7f800000
    r = ((u + (0x7fff + ((u >> 16) & 1))) >> 16).astype(np.uint16)
    r[nan] = ((u[nan] >> 16) | 0x40).astype(np.uint16)
    return r


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_to_f32(b):
    return np.ascontiguousarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def to_f32(a, dt):
    return a.astype(np.float32) if dt == F32 else bf16_to_f32(a) if dt == BF16 else f16_to_f32(a)


def fht(row, g):
    r = np.array(row, dtype=np.float32, copy=True).reshape(-1)
    rc = lib().orc_fht(_p(r), r.size, g)
    assert rc == 0, rc
    return r.reshape(np.shape(row))


def quant_rows(dtype, x, K, rotate, x_stride=None):
    """x: [M, x_stride] array (uint16 bits for bf16, float32 for f32). Returns (rc, q int8 [M,K], scales f32 [M])."""
    x = _c(x, _IN_NP[dtype])
    M = x.shape[0]
    x_stride = x.shape[1] if x_stride is None else x_stride
    q = np.zeros((M, K), np.int8)
    s = np.zeros((M,), np.float32)
    rc = lib().orc_quant_rows(dtype, _p(x), x_stride, _p(q), _p(s), M, K, rotate)
    return rc, q, s


def prologue_rows(dtype, prologue, x, K, g=None, up_offset=0, norm_w=None, norm_b=None, eps=0.0, mod_scale=None,
                  mod_shift=None):
    """Row prologue (RMS / LayerNorm variants, gate, SwiGLU, activations) -> the T row the quantizer consumes.
    x, g: [M, stride] arrays in the dtype's storage (uint16 bits or float32); norm_w/norm_b float32 [K];
    mod_scale/mod_shift [K] in the dtype's storage.  Returns (rc, out [M, K])."""
    x = _c(x, _IN_NP[dtype])
    M = x.shape[0]
    g = None if g is None else _c(g, _IN_NP[dtype])
    norm_w = None if norm_w is None else _c(norm_w, np.float32)
    norm_b = None if norm_b is None else _c(norm_b, np.float32)
    mod_scale = None if mod_scale is None else _c(mod_scale, _IN_NP[dtype])
    mod_shift = None if mod_shift is None else _c(mod_shift, _IN_NP[dtype])
    out = np.zeros((M, K), _IN_NP[dtype])
    rc = lib().orc_prologue_rows(dtype, prologue, _p(x), x.shape[1], _p(g), 0 if g is None else g.shape[1], up_offset,
                                 _p(norm_w), _p(norm_b), float(eps), _p(mod_scale), _p(mod_shift), _p(out), K, M, K)
    return rc, out


def quant_rows_wide(rd, x, K, rotate):
    """fp32 rows [M, K] quantized with the rounding of type rd -> (rc, q, scales)."""
    x = _c(x, np.float32)
    M = x.shape[0]
    q = np.zeros((M, K), np.int8)
    s = np.zeros(M, np.float32)
    rc = lib().orc_quant_rows_wide(rd, _p(x), x.shape[1], _p(q), _p(s), M, K, rotate)
    return rc, q, s


def situ_rows_wide(dtype, x, K, up_offset):
    """situ_f(x[:, :K], x[:, up_offset:up_offset+K]) as unrounded fp32 -> (rc, out [M, K])."""
    x = _c(x, _IN_NP[dtype])
    out = np.zeros((x.shape[0], K), np.float32)
    rc = lib().orc_situ_rows_wide(dtype, _p(x), x.shape[1], up_offset, _p(out), x.shape[0], K)
    return rc, out


def convrot_requant(dtype, x, seed=0):
    """Weight rows [N, K] (float32, or bf16 bits) -> (rc, rotated int8 codes, row scales); seed 0 rounds to nearest."""
    x = _c(x, _IN_NP[dtype])
    N, K = x.shape
    q = np.zeros((N, K), np.int8)
    s = np.zeros(N, np.float32)
    rc = lib().orc_convrot_requant(dtype, _p(x), _p(q), _p(s), N, K, seed)
    return rc, q, s


def convrot_dequant(mode, q, s):
    """H256(q * s[row]); mode 0 float32, 1 bf16 bits, 2 float32 holding bf16 values (the embedding form)."""
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    N, K = q.shape
    out = np.zeros((N, K), np.uint16 if mode == 1 else np.float32)
    rc = lib().orc_convrot_dequant(mode, _p(q), _p(s), _p(out), N, K)
    return rc, out


def dequant_i8(q, s):
    q = _c(q, np.int8)
    s = _c(s, np.float32)
    out = np.zeros(q.shape, np.float32)
    rc = lib().orc_dequant_i8(_p(q), _p(s), _p(out), q.shape[0], q.shape[1])
    return rc, out


def w6_requant(w_bits, seed):
    """bf16 weight bits [N, K] in the original basis -> (rc, packed [N, 3K/4], s_rel e4m3 bits [N, K/32], s_channel [N])."""
    w = _c(w_bits, np.uint16)
    N, K = w.shape
    packed = np.zeros((N, K * 3 // 4), np.uint8)
    s_rel = np.zeros((N, K // 32), np.uint8)
    s_ch = np.zeros(N, np.float32)
    rc = lib().orc_w6_requant(_p(w), _p(packed), _p(s_rel), _p(s_ch), N, K, seed)
    return rc, packed, s_rel, s_ch


SD_LN, SD_GEGLU, SD_UNPAD, SD_GN = 1, 2, 3, 4


def sd_source_rows(mode, x, M, K, x_stride=0, w=None, b=None, eps=0.0, heads=0, d=0, dp=0, groups=0, P=0):
    """The half row of the SD fused quantizer sources (LayerNorm, GEGLU, head un-padding, GroupNorm) -> (rc, [M, K] bits)."""
    x = _c(x, np.uint16)
    w = None if w is None else _c(w, np.float32)
    b = None if b is None else _c(b, np.float32)
    out = np.zeros((M, K), np.uint16)
    rc = lib().orc_sd_source_rows(mode, _p(x), x_stride, _p(w), _p(b), float(eps), heads, d, dp, groups, P, _p(out), M, K)
    return rc, out


def rotate_rows_f32(x, K, x_stride=None):
    x = _c(x, np.float32)
    M = x.shape[0]
    x_stride = x.shape[1] if x_stride is None else x_stride
    out = np.zeros((M, K), np.float32)
    rc = lib().orc_rotate_rows_f32(_p(x), x_stride, _p(out), M, K)
    return rc, out


def sd_quant_rows(x, K, rotate, x_stride=None):
    x = _c(x, np.uint16)
    M = x.shape[0]
    x_stride = x.shape[1] if x_stride is None else x_stride
    q = np.zeros((M, K), np.int8)
    s = np.zeros((M,), np.float32)
    rc = lib().orc_sd_quant_rows(_p(x), x_stride, _p(q), _p(s), M, K, rotate)
    return rc, q, s


def int8_gemm_acc(A, W):
    A = _c(A, np.int8); W = _c(W, np.int8)
    M, K = A.shape
    N = W.shape[0]
    acc = np.zeros((M, N), np.int32)
    lib().orc_int8_gemm_acc(_p(A), _p(W), _p(acc), M, N, K)
    return acc


def epilogue(acc, xs, ws, bias, out_dt, fma):
    acc = _c(acc, np.int32); xs = _c(xs, np.float32); ws = _c(ws, np.float32)
    bias = None if bias is None else _c(bias, _OUT_NP[out_dt])
    M, N = acc.shape
    D = np.zeros((M, N), _OUT_NP[out_dt])
    lib().orc_epilogue(_p(acc), _p(xs), _p(ws), _p(bias), _p(D), M, N, out_dt, int(fma))
    return D


def epilogue_residual(acc, xs, ws, bias, rscale, resid, out_dt, fma):
    acc = _c(acc, np.int32); xs = _c(xs, np.float32); ws = _c(ws, np.float32)
    bias = None if bias is None else _c(bias, _OUT_NP[out_dt])
    rscale = _c(rscale, _OUT_NP[out_dt]); resid = _c(resid, _OUT_NP[out_dt])
    M, N = acc.shape
    D = np.zeros((M, N), _OUT_NP[out_dt])
    lib().orc_epilogue_residual(_p(acc), _p(xs), _p(ws), _p(bias), _p(rscale), _p(resid), _p(D), M, N, out_dt,
                                int(fma))
    return D


def int8_gemm(A, W, xs, ws, bias, out_dt, fma=1):
    acc = int8_gemm_acc(A, W)
    return epilogue(acc, xs, ws, bias, out_dt, fma)


def int8_gemm_residual(A, W, xs, ws, bias, rscale, resid, out_dt, fma=1):
    acc = int8_gemm_acc(A, W)
    return epilogue_residual(acc, xs, ws, bias, rscale, resid, out_dt, fma)


def e4m3_table():
    L = lib()
    return np.array([L.orc_e4m3_to_f32(i) for i in range(256)], np.float32)


def w6_decode(q, s_rel, N, K, G):
    q = _c(q, np.uint8); s_rel = _c(s_rel, np.uint8)
    out = np.zeros((N, K), np.int8)
    rc = lib().orc_w6_decode(_p(q), _p(s_rel), _p(out), N, K, G)
    return rc, out


def w6_pack_planes(codes):
    codes = _c(codes, np.uint8)
    N, K = codes.shape
    q = np.zeros((N, K * 3 // 4), np.uint8)
    lib().orc_w6_pack_planes(_p(codes), _p(q), N, K)
    return q


def w6_pack_words(qv):
    qv = _c(qv, np.int8)
    N, K = qv.shape
    p = np.zeros((N, K * 3 // 4), np.uint8)
    lib().orc_w6_pack_words(_p(qv), _p(p), N, K)
    return p


def w6_unpack_words(p, K):
    p = _c(p, np.uint8)
    N = p.shape[0]
    qv = np.zeros((N, K), np.int8)
    lib().orc_w6_unpack_words(_p(p), _p(qv), N, K)
    return qv


def w6a8_group_gemm(A, packed, xs, sw, bias, out_dt, want_partials=False):
    A = _c(A, np.int8); packed = _c(packed, np.uint8); xs = _c(xs, np.float32); sw = _c(sw, np.float32)
    bias = None if bias is None else _c(bias, _OUT_NP[out_dt])
    M, K = A.shape
    N = packed.shape[0]
    D = np.zeros((M, N), _OUT_NP[out_dt])
    part = np.zeros((M, N, K // 128), np.int32) if want_partials else None
    rc = lib().orc_w6a8_group_gemm(_p(A), _p(packed), _p(xs), _p(sw), _p(bias), _p(D), _p(part), M, N, K, out_dt)
    return rc, D, part


def linear_w8a8(dtype, x, rotate, W, ws, bias, out_dt, fma=1, threads=None):
    """Whole linear on the CPU; returns (rc, D, threads_used)."""
    x = _c(x, _IN_NP[dtype]); W = _c(W, np.int8); ws = _c(ws, np.float32)
    bias = None if bias is None else _c(bias, _OUT_NP[out_dt])
    M, K = x.shape
    N = W.shape[0]
    if threads is not None:
        lib().orc_set_threads(threads)
    D = np.zeros((M, N), _OUT_NP[out_dt])
    t = C.c_int(0)
    rc = lib().orc_linear_w8a8(dtype, _p(x), K, rotate, _p(W), _p(ws), _p(bias), _p(D), M, N, K, out_dt, int(fma),
                               C.byref(t))
    return rc, D, t.value


def attn_rot128(row):
    """Sign diagonal + normalized Walsh-Hadamard over 128 channels, in place on a copy."""
    r = np.ascontiguousarray(row, dtype=np.float32).copy()
    assert r.shape == (128,)
    lib().orc_attn_rot128(_p(r))
    return r


def attn_sumsq128(row, split):
    """Sum of squares of a 128-channel float32 row in the reference's warp order (split: rope_mode 2's lane layout)."""
    r = np.ascontiguousarray(row, dtype=np.float32)
    assert r.shape == (128,)
    return float(lib().orc_attn_sumsq128(_p(r), 1 if split else 0))


def attn_norm_rope_row(row, w, rope_row, eps, rope_mode):
    """RMSNorm, weight and RoPE of one 128-channel row of bf16 values given as float32; returns the new row."""
    r = np.ascontiguousarray(row, dtype=np.float32).copy()
    assert r.shape == (128,)
    w = None if w is None else np.ascontiguousarray(w, dtype=np.float32)
    rope_row = None if rope_row is None else np.ascontiguousarray(rope_row, dtype=np.float32)
    lib().orc_attn_norm_rope_row(_p(r), None if w is None else _p(w), None if rope_row is None else _p(rope_row), float(eps),
                                 int(rope_mode))
    return r


def attn_rotate(row, lk):
    """The rotation the Q/K quantizers apply to a row of 64, 128 or 256 channels for a sequence of lk keys: H4 on runs of
    four channels up to 256 keys; beyond, H64 (head dim 64), the sign diagonal and H128 (128), H128 on each half (256)."""
    r = np.ascontiguousarray(row, dtype=np.float32).copy()
    assert r.shape in ((64,), (128,), (256,))
    lib().orc_attn_rotate_d(_p(r), r.shape[0], int(lk))
    return r


def attn_quant(dt, q, k, v, use_anchor=True, norm=None):
    """q [b,lq,h,128], k/v [b,lk,hk,128] contiguous (uint16 bits for bf16/f16).  Returns a dict with the int8 tensors
    in [b,heads,len,128] order, the scales, the anchors and the key tile length.  norm = dict(qw, kw, rope, eps,
    rope_mode): per-head RMSNorm (+ weight, + RoPE from rope [max(lq,lk), 64, 2] float32) of q, and of k when kw is
    given, ahead of the quantizers."""
    b, lq, h, D = q.shape
    _, lk, hk, _ = k.shape
    assert D in (64, 128, 256) and v.shape == k.shape
    q, k, v = np.ascontiguousarray(q), np.ascontiguousarray(k), np.ascontiguousarray(v)
    ck = lib().orc_attn_cta_k(lk, D)
    qg, kb = (lq + 127) // 128 * (128 // (16 if D == 256 else 32)), (lk + ck - 1) // ck
    out = dict(ck=ck, qi=np.zeros((b, h, lq, D), np.int8), qs=np.zeros((b, h, qg * 8), np.float32),
               ki=np.zeros((b, hk, lk, D), np.int8), ks=np.zeros((b, hk, kb * 4), np.float32),
               anchors=np.zeros((b, hk), np.int32), vi=np.zeros((b, hk, lk, D), np.int8),
               vs=np.zeros((b, hk, D), np.float32))
    if norm is None:
        rc = lib().orc_attn_quant_qk_d(dt, _p(q), _p(k), b, lq, lk, h, hk, D, lq * h * D, h * D, D, lk * hk * D, hk * D, D, ck,
                                       1 if use_anchor else 0, _p(out["qi"]), _p(out["qs"]), _p(out["ki"]), _p(out["ks"]),
                                       _p(out["anchors"]), 0, None, None, None, 0.0, 0)
    else:
        assert D == 128
        f = {n: (None if norm.get(n) is None else np.ascontiguousarray(norm[n], dtype=np.float32)) for n in ("qw", "kw", "rope")}
        if f["rope"] is not None:
            assert f["rope"].size >= max(lq, lk) * D
        pp = {n: (None if a is None else _p(a)) for n, a in f.items()}
        rc = lib().orc_attn_quant_qk_norm(dt, _p(q), _p(k), b, lq, lk, h, hk, lq * h * D, h * D, D, lk * hk * D, hk * D, D, ck,
                                          1 if use_anchor else 0, _p(out["qi"]), _p(out["qs"]), _p(out["ki"]), _p(out["ks"]),
                                          _p(out["anchors"]), 1, pp["qw"], pp["kw"], pp["rope"], float(norm["eps"]),
                                          int(norm["rope_mode"]))
    assert rc == 0, rc
    rc = lib().orc_attn_quant_v_d(dt, _p(v), b, lk, hk, D, lk * hk * D, hk * D, D, _p(out["vi"]), _p(out["vs"]))
    assert rc == 0
    return out


def attn_int8_bias(dt, q, k, v, scale, bias, quant=None):
    """attn_int8 with bias (float32 [lk]) added to each key's logits; a bias that is not finite masks its key."""
    b, lq, h, D = q.shape
    lk, hk = k.shape[1], k.shape[2]
    z = quant if quant is not None else attn_quant(dt, q, k, v, True)
    bias = np.ascontiguousarray(bias, dtype=np.float32)
    assert bias.shape == (lk,)
    o = np.zeros((b, lq, h, D), np.float32 if dt == F32 else np.uint16)
    rc = lib().orc_attn_int8_bias(dt, _p(z["qi"]), _p(z["ki"]), _p(z["vi"]), _p(z["qs"]), _p(z["ks"]), _p(z["vs"]), b, lq, lk,
                                  h, hk, z["ck"], float(scale), _p(bias), _p(o), lq * h * D, h * D, D)
    assert rc == 0
    return o


def attn_int8(dt, q, k, v, scale, use_anchor=True, quant=None, sink=0.0, norm=None):
    """The whole int8 attention: o [b,lq,h,128] in dtype dt (uint16 bits for bf16/f16).  sink: that many more keys of
    score zero and value zero in the denominator (callers pass use_anchor=False with it, as the reference does)."""
    b, lq, h, D = q.shape
    lk, hk = k.shape[1], k.shape[2]
    z = quant if quant is not None else attn_quant(dt, q, k, v, use_anchor, norm)
    o = np.zeros((b, lq, h, D), np.float32 if dt == F32 else np.uint16)
    rc = lib().orc_attn_int8_d(dt, _p(z["qi"]), _p(z["ki"]), _p(z["vi"]), _p(z["qs"]), _p(z["ks"]), _p(z["vs"]), b, lq, lk,
                               h, hk, D, z["ck"], float(scale), float(sink), _p(o), lq * h * D, h * D, D,
                               1 if (dt == F16 and lk <= 512 and z["ck"] == 64) else 0)
    assert rc == 0
    return o
