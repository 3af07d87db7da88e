"""Host-side call pattern of one quantized linear, as the reference's model code issues it (src/dit.rs:550-555,
src/unet.rs:436-456, src/h3.rs:1208-1251): quantize rows, then the fused int8 GEMM.  torch supplies device memory and
the stream; all arithmetic happens in libgpu_kernels.so.
"""
import torch

from . import ffi

_TORCH_DT = {torch.float32: ffi.DT_F32, torch.float16: ffi.DT_F16, torch.bfloat16: ffi.DT_BF16}
_DT_TORCH = {v: k for k, v in _TORCH_DT.items()}


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _dense(*ts):
    """The kernels read these operands as dense row-major device arrays: a view with other strides would be read as if
    it were dense and give wrong results without an error, so it is refused here."""
    for t in ts:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("expected a CUDA tensor")
        if not t.is_contiguous():
            raise ValueError("expected a contiguous tensor, got strides %s for shape %s" % (t.stride(), tuple(t.shape)))


def _rows(t):
    """Row operands may have a row stride; their last axis must be dense."""
    if not t.is_cuda or t.dim() != 2 or t.stride(1) != 1:
        raise ValueError("expected a 2-D CUDA tensor with a dense last axis, got strides %s" % (t.stride(),))


def _want(t, dtype, what):
    if t is not None and t.dtype != dtype:
        raise ValueError("%s must be %s, got %s" % (what, dtype, t.dtype))


def quant_rows(x, rotate=0, K=None, q=None, scales=None):
    """x: [M, x_stride] bf16 or f32 CUDA tensor -> (q int8 [M,K], scales f32 [M])."""
    _rows(x)
    M, x_stride = x.shape
    K = x_stride if K is None else K
    q = torch.empty((M, K), dtype=torch.int8, device=x.device) if q is None else q
    scales = torch.empty((M,), dtype=torch.float32, device=x.device) if scales is None else scales
    _dense(q, scales)
    _want(q, torch.int8, "q"); _want(scales, torch.float32, "scales")
    ffi.k("gpu_quant_rows", _TORCH_DT[x.dtype], ffi.PRO_PLAIN, _ptr(x), x.stride(0), 0, 0, 0, 0, 0.0, 0, 0, _ptr(q),
          _ptr(scales), M, K, rotate, _stream())
    return q, scales


def quant_rows_pro(x, prologue, K, rotate=0, g=None, up_offset=0, norm_w=None, eps=0.0, mod_scale=None, mod_shift=None):
    """gpu_quant_rows with a row prologue (src/dit.rs:510-611 call patterns): x [M, x_stride], optional gate logits g."""
    M = x.shape[0]
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scales = torch.empty((M,), dtype=torch.float32, device=x.device)
    ffi.k("gpu_quant_rows", _TORCH_DT[x.dtype], prologue, _ptr(x), x.stride(0), _ptr(g), 0 if g is None else g.stride(0),
          up_offset, _ptr(norm_w), float(eps), _ptr(mod_scale), _ptr(mod_shift), _ptr(q), _ptr(scales), M, K, rotate, _stream())
    return q, scales


def quant_rows_b(x, prologue, K, norm_w, norm_b, eps, rotate=0, mod_scale=None, mod_shift=None):
    M = x.shape[0]
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scales = torch.empty((M,), dtype=torch.float32, device=x.device)
    ffi.k("gpu_quant_rows_b", _TORCH_DT[x.dtype], prologue, _ptr(x), x.stride(0), _ptr(norm_w), _ptr(norm_b), float(eps),
          _ptr(mod_scale), _ptr(mod_shift), _ptr(q), _ptr(scales), M, K, rotate, _stream())
    return q, scales


def prologue_rows(x, prologue, K, g=None, up_offset=0, norm_w=None, norm_b=None, eps=0.0, mod_scale=None, mod_shift=None,
                  b_variant=False):
    """gpu_prologue_rows / gpu_prologue_rows_b: the prologue's output row in x's dtype, [M, K]."""
    M = x.shape[0]
    out = torch.empty((M, K), dtype=x.dtype, device=x.device)
    if b_variant:
        ffi.k("gpu_prologue_rows_b", _TORCH_DT[x.dtype], prologue, _ptr(x), x.stride(0), _ptr(norm_w), _ptr(norm_b), float(eps),
              _ptr(mod_scale), _ptr(mod_shift), _ptr(out), K, M, K, _stream())
    else:
        ffi.k("gpu_prologue_rows", _TORCH_DT[x.dtype], prologue, _ptr(x), x.stride(0), _ptr(g), 0 if g is None else g.stride(0),
              up_offset, _ptr(norm_w), float(eps), _ptr(mod_scale), _ptr(mod_shift), _ptr(out), K, M, K, _stream())
    return out


def sd_quant_rows(x, rotate=0, K=None):
    M, x_stride = x.shape
    K = x_stride if K is None else K
    q = torch.empty((M, K), dtype=torch.int8, device=x.device)
    scales = torch.empty((M,), dtype=torch.float32, device=x.device)
    ffi.k("gpu_sd_quant_rows", _ptr(x), x.stride(0), _ptr(q), _ptr(scales), M, K, rotate, _stream())
    return q, scales


def gemm(A, B, bias=None, transb=True, out_dtype=None, alpha=1.0, beta=0.0, D=None):
    """gpu_gemm (src/ffi.rs, csrc/gemm.cu:55): D = alpha * A . B^T (transb) or A . B, + bias, + beta * D."""
    ffi.kb("gpu_blas_init", 32 << 20)
    M, K = A.shape
    N = B.shape[0] if transb else B.shape[1]
    out_dtype = A.dtype if out_dtype is None else out_dtype
    D = torch.empty((M, N), dtype=out_dtype, device=A.device) if D is None else D
    ffi.kb("gpu_gemm", _ptr(A), A.stride(0), _ptr(B), B.stride(0), _ptr(D), D.stride(0), _ptr(bias), M, N, K, 1 if transb else 0,
           _TORCH_DT[A.dtype], _TORCH_DT[out_dtype], float(alpha), float(beta), _stream())
    return D


def dequant_i8(q, s):
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    ffi.k("gpu_dequant_i8", _ptr(q), _ptr(s), _ptr(out), q.shape[0], q.shape[1], _stream())
    return out


def embed_dequant(q, s):
    """Rows of an int8 ConvRot embedding table -> fp32 rows of bf16 values (src/te.rs:441)."""
    out = torch.empty(q.shape, dtype=torch.float32, device=q.device)
    ffi.k("gpu_embed_dequant", _ptr(q), _ptr(s), _ptr(out), q.shape[0], q.shape[1], 1, _stream())
    return out


def convrot_dequant(q, s, dtype=torch.bfloat16):
    """Rotated int8 weight + row scales -> the weight in its original basis (src/lora.rs:589)."""
    out = torch.empty(q.shape, dtype=dtype, device=q.device)
    ffi.k("gpu_convrot_dequant", _TORCH_DT[dtype], _ptr(q), _ptr(s), _ptr(out), q.shape[0], q.shape[1], _stream())
    return out


def convrot_requant(w, seed=0):
    """Weight in its original basis -> rotated int8 + row scales (src/lora.rs:592, src/moss.rs:91)."""
    N, K = w.shape
    q = torch.empty((N, K), dtype=torch.int8, device=w.device)
    s = torch.empty((N,), dtype=torch.float32, device=w.device)
    ffi.k("gpu_convrot_requant", _TORCH_DT[w.dtype], _ptr(w), _ptr(q), _ptr(s), N, K, seed, _stream())
    return q, s


def w6_requant(w, seed):
    """bf16 weight [N, K] -> (packed uint8 [N, 3K/4], s_rel e4m3 bits uint8 [N, K/32], s_channel f32 [N]), src/lora.rs:630."""
    N, K = w.shape
    packed = torch.empty((N, K * 3 // 4), dtype=torch.uint8, device=w.device)
    s_rel = torch.empty((N, K // 32), dtype=torch.uint8, device=w.device)
    s_ch = torch.empty((N,), dtype=torch.float32, device=w.device)
    ffi.k("gpu_w6_requant", _ptr(w), _ptr(packed), _ptr(s_rel), _ptr(s_ch), N, K, seed, _stream())
    return packed, s_rel, s_ch


def _sd_out(M, K, dev):
    return torch.empty((M, K), dtype=torch.int8, device=dev), torch.empty((M,), dtype=torch.float32, device=dev)


def sd_ln_quant_rows(x, w, b, eps, rotate=0, K=None):
    """LayerNorm (half) then the fp16 quantizer, src/unet.rs call pattern of gpu_sd_ln_quant_rows."""
    M = x.shape[0]
    K = x.shape[1] if K is None else K
    q, s = _sd_out(M, K, x.device)
    ffi.k("gpu_sd_ln_quant_rows", _ptr(x), x.stride(0), _ptr(w), _ptr(b), float(eps), _ptr(q), _ptr(s), M, K, rotate, _stream())
    return q, s


def sd_geglu_quant_rows(x, rotate=0):
    M, I = x.shape[0], x.shape[1] // 2
    q, s = _sd_out(M, I, x.device)
    ffi.k("gpu_sd_geglu_quant_rows", _ptr(x), _ptr(q), _ptr(s), M, I, rotate, _stream())
    return q, s


def sd_unpad_quant_rows(x, d, rotate=0):
    M, H, dp = x.shape
    q, s = _sd_out(M, H * d, x.device)
    ffi.k("gpu_sd_unpad_quant_rows", _ptr(x), _ptr(q), _ptr(s), M, H, d, dp, rotate, _stream())
    return q, s


def sd_group_norm_quant_rows(x, w, b, groups, eps, rotate=0):
    N, P, C = x.shape
    q, s = _sd_out(N * P, C, x.device)
    sums = torch.empty(16 * N * groups + 16, dtype=torch.uint8, device=x.device)
    ffi.k("gpu_sd_group_norm_quant_rows", _ptr(x), _ptr(w), _ptr(b), _ptr(sums), N, P, C, groups, float(eps), _ptr(q), _ptr(s),
          rotate, _stream())
    return q, s, sums


def rotate_rows_f32(x, K=None, prologue=ffi.PRO_PLAIN, up_offset=0, norm_w=None, eps=0.0):
    M, x_stride = x.shape
    K = x_stride if K is None else K
    out = torch.empty((M, K), dtype=torch.float32, device=x.device)
    ffi.k("gpu_rotate_rows_f32", prologue, _ptr(x), x.stride(0), up_offset, _ptr(norm_w), float(eps), _ptr(out), M, K,
          _stream())
    return out


def _gemm_operands(A, W, xs, ws):
    _dense(A, W, xs, ws)
    _want(A, torch.int8, "A"); _want(W, torch.int8, "W"); _want(xs, torch.float32, "xs"); _want(ws, torch.float32, "ws")
    if A.dim() != 2 or W.dim() != 2 or A.shape[1] != W.shape[1]:
        raise ValueError("A [M,K] and W [N,K] must share K, got %s and %s" % (tuple(A.shape), tuple(W.shape)))


def int8_gemm(A, W, xs, ws, bias=None, out_dtype=torch.bfloat16, D=None):
    _gemm_operands(A, W, xs, ws)
    M, K = A.shape
    N = W.shape[0]
    D = torch.empty((M, N), dtype=out_dtype, device=A.device) if D is None else D
    _dense(bias, D)
    _want(bias, out_dtype, "bias"); _want(D, out_dtype, "D")
    ffi.k("gpu_int8_gemm", _ptr(A), _ptr(W), _ptr(xs), _ptr(ws), _ptr(bias), _ptr(D), M, N, K, _TORCH_DT[out_dtype],
          _stream())
    return D


def int8_gemm_residual(A, W, xs, ws, bias, rscale, resid, D=None):
    """D = resid + rscale * (...); pass D=resid for the in-place form the DiT block uses."""
    _gemm_operands(A, W, xs, ws)
    M, K = A.shape
    N = W.shape[0]
    D = torch.empty_like(resid) if D is None else D
    _dense(bias, rscale, resid, D)
    for t_, what in ((bias, "bias"), (rscale, "rscale"), (D, "D")):
        _want(t_, resid.dtype, what)
    ffi.k("gpu_int8_gemm_residual", _ptr(A), _ptr(W), _ptr(xs), _ptr(ws), _ptr(bias), _ptr(rscale), _ptr(resid), _ptr(D),
          M, N, K, _TORCH_DT[resid.dtype], _stream())
    return D


def int8_gemm_acc(A, W):
    _dense(A, W)
    _want(A, torch.int8, "A"); _want(W, torch.int8, "W")
    M, K = A.shape
    N = W.shape[0]
    acc = torch.empty((M, N), dtype=torch.int32, device=A.device)
    ffi.k("gpu_int8_gemm_acc", _ptr(A), _ptr(W), _ptr(acc), M, N, K, _stream())
    return acc


def w6_decode(wq, s_rel, N, K, G):
    _dense(wq, s_rel)
    out = torch.empty((N, K), dtype=torch.int8, device=wq.device)
    ffi.k("gpu_w6_decode", _ptr(wq), _ptr(s_rel), _ptr(out), N, K, G, _stream())
    return out


def w6a8_gemm(A, wq, s_rel, G, xs, s_channel, bias=None, out_dtype=torch.bfloat16):
    """W6A8 linear on already-quantized rows: packed two-plane weights wq [N, 3K/4], e4m3 s_rel [N, K/G], f32 s_channel."""
    _dense(A, wq, s_rel, xs, s_channel, bias)
    _want(A, torch.int8, "A"); _want(xs, torch.float32, "xs"); _want(s_channel, torch.float32, "s_channel")
    M, K = A.shape
    N = wq.shape[0]
    D = torch.empty((M, N), dtype=out_dtype, device=A.device)
    ffi.k("gpu_w6a8_gemm", _ptr(A), _ptr(wq), _ptr(s_rel), G, _ptr(xs), _ptr(s_channel), _ptr(bias), _ptr(D), M, N, K,
          _TORCH_DT[out_dtype], _stream())
    return D


def w6a8_group_gemm(A, packed, xs, sw, bias=None, out_dtype=torch.bfloat16, want_partials=False):
    """W6A8 linear on already-quantized rows with the library's own weight format: 24-bit words of four 6-bit codes,
    packed [N, 3K/4], and f32 group scales sw [N, K/128].  Returns D, or (D, partials [M, N, K/128]) on request."""
    _dense(A, packed, xs, sw, bias)
    _want(A, torch.int8, "A"); _want(xs, torch.float32, "xs"); _want(sw, torch.float32, "sw")
    M, K = A.shape
    N = packed.shape[0]
    D = torch.empty((M, N), dtype=out_dtype, device=A.device)
    part = torch.empty((M, N, K // 128), dtype=torch.int32, device=A.device) if want_partials else None
    ffi.k("gpu_w6a8_group_gemm", _ptr(A), _ptr(packed), _ptr(xs), _ptr(sw), _ptr(bias), _ptr(D), _ptr(part), M, N, K,
          _TORCH_DT[out_dtype], _stream())
    return (D, part) if want_partials else D


def linear_w8a8(x, W, ws, bias=None, rotate=0, out_dtype=None):
    """One W8A8 linear: y = dequant(quant(x) . W^T)."""
    q, xs = quant_rows(x, rotate)
    return int8_gemm(q, W, xs, ws, bias, x.dtype if out_dtype is None else out_dtype)


def _f32_vec(t, n, what):
    if t is None:
        return None
    if t.dtype != torch.float32 or not t.is_contiguous() or t.numel() < n:
        raise ValueError("%s must be contiguous float32 with at least %d elements" % (what, n))
    return _ptr(t)


def int8_attn_norm_rope(q, k, v, scale, qw, kw, eps, rope, rope_mode, ws=None):
    """int8_attn with per-head RMSNorm (weight qw / kw, float32 [128]) and RoPE (rope float32 [max(lq, lk), 64, 2] of
    (cos, sin), rope_mode 1 interleaved pairs, 2 split halves, 0 none) applied to q, and to k when kw is given, inside the
    quantizers; q and k are not written (csrc/attn_int8.cu:163-174, the DiT's call at src/dit.rs:575).  bf16."""
    b, lq, h, D = q.shape
    lk, hk = k.shape[1], k.shape[2]
    assert q.dtype == torch.bfloat16 and D == 128
    assert q.stride(3) == 1 and k.stride(3) == 1 and v.stride(3) == 1
    if ws is None:
        ws = torch.empty((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device=q.device)
    o = torch.empty((b, lq, h, D), dtype=q.dtype, device=q.device)
    ffi.k("gpu_int8_attn_norm_rope", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(ws), b, lq, lk, h, hk, q.stride(0), q.stride(1),
          q.stride(2), k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1),
          o.stride(2), float(scale), _f32_vec(qw, D, "qw"), _f32_vec(kw, D, "kw"), float(eps),
          _f32_vec(rope, max(lq, lk) * D, "rope"), int(rope_mode), _stream())
    return o


def int8_attn_key_bias(q, k, v, scale, bias, ws=None):
    """int8_attn with bias (float32 [lk], one row for every batch item, head and query) added to the logits of each key
    (csrc/attn_int8.cu:184-223, the DiT's call at src/dit.rs:573).  bf16."""
    b, lq, h, D = q.shape
    lk, hk = k.shape[1], k.shape[2]
    assert q.dtype == torch.bfloat16 and D == 128
    assert q.stride(3) == 1 and k.stride(3) == 1 and v.stride(3) == 1
    if ws is None:
        ws = torch.empty((ffi.lib.gpu_int8_attn_key_bias_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device=q.device)
    o = torch.empty((b, lq, h, D), dtype=q.dtype, device=q.device)
    ffi.k("gpu_int8_attn_key_bias", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(ws), b, lq, lk, h, hk, q.stride(0), q.stride(1),
          q.stride(2), k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1),
          o.stride(2), float(scale), _f32_vec(bias, lk, "bias"), _stream())
    return o


def int8_attn_sink(q, k, v, scale, sink, ws=None, qw=None, eps=0.0):
    """int8_attn over the keys given plus `sink` zero keys with zero values (bf16), csrc/attn_int8.cu:193-202.  qw
    (float32 [128]): q is RMS-normalized with that weight first, k taken as it is."""
    b, lq, h, D = q.shape
    lk, hk = k.shape[1], k.shape[2]
    assert q.dtype == torch.bfloat16 and D == 128
    if ws is None:
        ws = torch.empty((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device=q.device)
    o = torch.empty((b, lq, h, D), dtype=q.dtype, device=q.device)
    ffi.k("gpu_int8_attn_sink", _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(ws), b, lq, lk, h, hk, q.stride(0), q.stride(1),
          q.stride(2), k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1),
          o.stride(2), float(scale), float(sink), _f32_vec(qw, D, "qw"), float(eps), _stream())
    return o


def int8_attn(q, k, v, scale, ws=None):
    """INT8 attention over q [b, lq, h, 128], k/v [b, lk, hk, 128] (bf16 or f16, any strides with a contiguous last
    axis): the reference's attention_int8 call pattern (csrc/attn_int8.cu:101-118).  Returns o [b, lq, h, 128]."""
    b, lq, h, D = q.shape
    lk, hk = k.shape[1], k.shape[2]
    assert q.stride(3) == 1 and k.stride(3) == 1 and v.stride(3) == 1
    if ws is None:
        ws = torch.empty((ffi.lib.gpu_int8_attn_workspace_d(b, h, hk, lq, lk, D),), dtype=torch.uint8, device=q.device)
    o = torch.empty((b, lq, h, D), dtype=q.dtype, device=q.device)
    name = "gpu_int8_attn_f16" if q.dtype == torch.float16 else "gpu_int8_attn_d"
    ffi.k(name, _ptr(q), _ptr(k), _ptr(v), _ptr(o), _ptr(ws), b, lq, lk, h, hk, D, q.stride(0), q.stride(1), q.stride(2),
          k.stride(0), k.stride(1), k.stride(2), v.stride(0), v.stride(1), v.stride(2), o.stride(0), o.stride(1),
          o.stride(2), float(scale), _stream())
    return o
