"""Parity of the HIP kernels with the CPU oracle, through the C ABI, on a real MI355X.

Bars: int8 codes, per-row scales and int32 accumulators bit-exact; bf16/f16/f32 outputs bit-exact against the oracle's
fused-multiply-add epilogue and within one unit in the last place of the output type of its unfused form.
"""
import hashlib
import json
import os

import numpy as np
import pytest
import torch

import oracle
from oracle import BF16, F16, F32
from conftest import ROOT, pkg

pytestmark = pytest.mark.gpu

ffi = pkg("ffi")
ql = pkg("qlinear")
synth = pkg("synth")
DEV = "cuda:0"
TDT = {BF16: torch.bfloat16, F16: torch.float16, F32: torch.float32}


def say(*a):
    print(*a, flush=True)


def dev_bits(bits, dt):
    """numpy array (uint16 bits for bf16/f16, float32 for f32) -> CUDA tensor of that dtype."""
    if dt == F32:
        return torch.from_numpy(np.ascontiguousarray(bits, dtype=np.float32)).to(DEV)
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).to(DEV).view(TDT[dt])


def host_bits(t):
    if t.dtype == torch.float32:
        return t.cpu().numpy()
    return t.view(torch.int16).cpu().numpy().view(np.uint16)


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def ulp_close(a_bits, b_bits, dt, addend=0.0):
    """Within one unit in the last place of the output type.  The fused and unfused epilogues differ by the rounding of
    the product t1 = t0*ws, half an ulp of |t1| <= |result| + |addend| (addend = the bias), which under cancellation is
    more than an ulp of the result itself."""
    a = oracle.to_f32(a_bits, dt).astype(np.float64)
    b = oracle.to_f32(b_bits, dt).astype(np.float64)
    ulp = {BF16: 2.0 ** -7, F16: 2.0 ** -10, F32: 2.0 ** -23}[dt]
    return (np.abs(a - b) <= ulp * (np.maximum(np.abs(a), np.abs(b)) + np.abs(addend)) + 1e-30).all()


# ------------------------------------------------------------------------------------------------ MFMA layout
def test_mfma_operand_layout_is_what_the_gemm_assumes():
    out = torch.zeros(1024, dtype=torch.int32, device=DEV)
    ffi.k("gpu_mfma_layout_probe", out.data_ptr(), 0)
    torch.cuda.synchronize()
    got = out.cpu().numpy().reshape(64, 16)
    lane = np.arange(64)[:, None]
    r = np.arange(16)[None, :]
    i = 8 * (r // 4) + 4 * (lane // 32) + (r % 4)
    j = lane % 32 + 0 * r
    want = i * 32 + j
    if not np.array_equal(got, want):
        say("probe (i,j) for lane 0:", [(int(v) // 32, int(v) % 32) for v in got[0]])
        say("probe (i,j) for lane 1:", [(int(v) // 32, int(v) % 32) for v in got[1]])
        say("probe (i,j) for lane 32:", [(int(v) // 32, int(v) % 32) for v in got[32]])
    assert np.array_equal(got, want)


# ------------------------------------------------------------------------------------------------ quantizers
QUANT_CASES = [
    # (M, K, rotate, kind)
    (256, 1024, 0, "normal"), (7, 256, 1, "normal"), (5, 256, 0, "t3"), (33, 1024, 256, "t3"), (3, 640, 0, "normal"),
    (9, 640, 64, "normal"), (4, 384, 128, "t3"), (130, 3072, 1, "t3"), (66, 3072, 128, "t3"), (5, 4096, 1, "normal"),
    (3, 5120, 1, "t3"), (2, 12288, 1, "t3"), (2, 12288, 128, "t3"), (1, 13824, 0, "normal"), (1, 32768, 1, "normal"),
    (2, 16384, 64, "normal"), (1, 6144, 1, "t3"),
]


@pytest.mark.parametrize("M,K,rotate,kind", QUANT_CASES)
def test_quant_rows_bf16_bit_exact(M, K, rotate, kind):
    say("quant_rows bf16", M, K, rotate, kind)
    xb = synth.bf16_bits(synth.activations(100 + K + rotate, M, K, kind, (3, K - 1)))
    rc, q, s = oracle.quant_rows(BF16, xb, K, rotate)
    assert rc == 0
    qd, sd = ql.quant_rows(dev_bits(xb, BF16), rotate)
    torch.cuda.synchronize()
    assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32))
    assert np.array_equal(qd.cpu().numpy(), q)


@pytest.mark.parametrize("M,K,rotate", [(5, 256, 0), (4, 1024, 1), (3, 2304, 64), (2, 8192, 1), (3, 512, 128)])
def test_quant_rows_f32_bit_exact(M, K, rotate):
    say("quant_rows f32", M, K, rotate)
    x = synth.activations(200 + K, M, K, "t3")
    rc, q, s = oracle.quant_rows(F32, x, K, rotate)
    assert rc == 0
    qd, sd = ql.quant_rows(dev(x), rotate)
    torch.cuda.synchronize()
    assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32))
    assert np.array_equal(qd.cpu().numpy(), q)


def test_quant_rows_special_rows_and_stride():
    K = 512
    rows = np.zeros((8, K), np.float32)
    rows[1, 7] = 20.0; rows[1, 9] = -20.0; rows[1, 11] = 10.0
    rows[2, 0] = np.inf; rows[2, 1] = -np.inf; rows[2, 2] = 1.0
    rows[3, 0] = np.nan; rows[3, 1] = 2.0; rows[3, 2] = -1.0
    rows[4, :] = 1e-35
    rows[5, 0] = 131.0; rows[5, 1] = -131.0                      # a +-127.5 tie row if one exists for this amax
    for A in range(128, 256):                                    # find an amax whose quotient rounds to 127.5
        a = np.float32(A)
        st = oracle.bf16_to_f32(oracle.bf16_bits(np.array([a * np.float32(1 / 127)])))[0]
        if oracle.bf16_to_f32(oracle.bf16_bits(np.array([a / st], np.float32)))[0] == np.float32(127.5):
            rows[5, 0] = a; rows[5, 1] = -a
            break
    rows[6] = synth.normal(9, 1, K) * np.float32(3e37)           # near the top of the range
    rows[7] = synth.normal(9, 2, K) * np.float32(1e-30)
    xb = oracle.bf16_bits(rows)
    for rotate in (0, 1):
        rc, q, s = oracle.quant_rows(BF16, xb, K, rotate)
        qd, sd = ql.quant_rows(dev_bits(xb, BF16), rotate)
        torch.cuda.synchronize()
        assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32)), rotate
        assert np.array_equal(qd.cpu().numpy(), q), rotate
        if rotate == 0:
            assert q[5, 0] == 127 and q[5, 1] == -128
    # rows that are a window of a wider buffer (x_stride > K), as the SwiGLU call sites read them (src/dit.rs:605)
    wide = synth.bf16_bits(synth.activations(10, 6, 3 * K, "normal"))
    rc, q, s = oracle.quant_rows(BF16, wide, K, 1, x_stride=3 * K)
    xd = dev_bits(wide, BF16)
    qd, sd = ql.quant_rows(xd, 1, K=K)
    torch.cuda.synchronize()
    assert np.array_equal(qd.cpu().numpy(), q) and np.array_equal(sd.cpu().numpy(), s)


@pytest.mark.parametrize("M,K,rotate", [(8, 640, 0), (70, 640, 64), (9, 1280, 256), (5, 2560, 256), (3, 5120, 64), (2, 320, 64)])
def test_sd_quant_rows_bit_exact(M, K, rotate):
    say("sd_quant_rows", M, K, rotate)
    xb = synth.f16_bits(synth.activations(300 + K, M, K, "normal", (5,)))
    xb[0, :] = 0
    rc, q, s = oracle.sd_quant_rows(xb, K, rotate)
    assert rc == 0
    qd, sd = ql.sd_quant_rows(dev_bits(xb, F16), rotate)
    torch.cuda.synchronize()
    assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32))
    assert np.array_equal(qd.cpu().numpy(), q)


def test_rotate_rows_f32_bit_exact():
    x = synth.activations(400, 6, 3 * 1024, "t3")
    rc, out = oracle.rotate_rows_f32(x, 1024, x_stride=3 * 1024)
    got = ql.rotate_rows_f32(dev(x), K=1024)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint32), out.view(np.uint32))


# ------------------------------------------------------------------------------------------------ row prologues
def pro_case(dt, seed, M, K, cols):
    """Inputs of every prologue for one shape, in the oracle's storage form: x rows [M, cols] (a gate/up half at
    column K + 64), gate logits, norm weight/bias, modulation vectors."""
    rnd = lambda stream, *shape: synth.normal(seed, stream, int(np.prod(shape))).reshape(shape)
    conv = {BF16: synth.bf16_bits, F16: synth.f16_bits, F32: lambda a: np.ascontiguousarray(a, dtype=np.float32)}[dt]
    x = rnd(1, M, cols) * np.float32(1.5)
    x[0, :6] = [0.0, -0.0, 30.0, -30.0, 6.0, -6.0]
    if M > 1:
        x[1, :] = 0
    return dict(x=conv(x), g=conv(rnd(2, M, K + 8) * np.float32(2)), w=(1 + 0.2 * rnd(3, K)).astype(np.float32),
                b=(0.1 * rnd(4, K)).astype(np.float32), ms=conv(0.3 * rnd(5, K)), sh=conv(0.3 * rnd(6, K)))


def pro_args(name, c, K):
    """Keyword arguments of one prologue (host arrays)."""
    a = dict(eps=1e-6)
    if name == "GATE":
        a["g"] = c["g"]
    if name in ("SWIGLU", "SITU"):
        a["up_offset"] = K + 64
    if name in ("RMS_W", "LAYERNORM_W", "LN_AFFINE", "LN_AFFINE_SILU", "RMS_W_MOD", "LAYERNORM_B"):
        a["norm_w"] = c["w"]
    if name in ("LN_AFFINE", "LN_AFFINE_SILU"):
        a["norm_b"] = c["b"]
    if name in ("ADALN", "LN_MOD", "RMS_W_MOD", "LAYERNORM_MOD"):
        a["mod_scale"], a["mod_shift"] = c["ms"], c["sh"]
    return a


PRO_ID = dict(PLAIN=0, RMS=1, RMS_W=1, RMS_W_MOD=1, GATE=2, SWIGLU=3, LAYERNORM=4, LAYERNORM_W=4, LAYERNORM_MOD=4,
              LAYERNORM_B=4, SILU=5, GELU=6, ADALN=7, SITU=8, LN_MOD=9, LN_AFFINE=10, GELU_TANH=11, LN_AFFINE_SILU=12)
A_NAMES = ["PLAIN", "RMS", "RMS_W", "RMS_W_MOD", "GATE", "SWIGLU", "LAYERNORM", "LAYERNORM_W", "LAYERNORM_MOD", "SILU", "GELU",
           "ADALN", "SITU"]
B_NAMES = ["PLAIN", "LAYERNORM_B", "LN_MOD", "LN_AFFINE", "LN_AFFINE_SILU", "SILU", "GELU", "GELU_TANH"]


def to_dev_args(a, dt):
    d = dict(a)
    for k in ("g", "mod_scale", "mod_shift"):
        if k in d:
            d[k] = dev_bits(d[k], dt)
    for k in ("norm_w", "norm_b"):
        if k in d:
            d[k] = dev(d[k])
    return d


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("M,K", [(5, 256), (3, 3072), (2, 200), (3, 5120)])
def test_prologue_rows_bit_exact(M, K, dt):
    cols = 2 * K + 64
    c = pro_case(dt, 500 + K, M, K, cols)
    xd = dev_bits(c["x"], dt)
    for name in A_NAMES:
        say("prologue_rows", name, M, K, dt)
        a = pro_args(name, c, K)
        rc, want = oracle.prologue_rows(dt, PRO_ID[name], c["x"], K, **a)
        assert rc == 0
        got = ql.prologue_rows(xd, PRO_ID[name], K, **to_dev_args(a, dt))
        torch.cuda.synchronize()
        gb, wb = host_bits(got), want
        assert np.array_equal(gb.view(np.uint32 if dt == F32 else np.uint16), wb.view(np.uint32 if dt == F32 else np.uint16)), name


@pytest.mark.parametrize("dt", [BF16, F16, F32])
@pytest.mark.parametrize("M,K", [(4, 64), (5, 1152), (2, 4096)])
def test_prologue_rows_b_bit_exact(M, K, dt):
    c = pro_case(dt, 600 + K, M, K, K + 16)
    xd = dev_bits(c["x"], dt)
    for name in B_NAMES:
        say("prologue_rows_b", name, M, K, dt)
        a = pro_args(name, c, K)
        rc, want = oracle.prologue_rows(dt, PRO_ID[name], c["x"], K, **a)
        assert rc == 0
        got = ql.prologue_rows(xd, PRO_ID[name], K, b_variant=True, **to_dev_args(a, dt))
        torch.cuda.synchronize()
        view = np.uint32 if dt == F32 else np.uint16
        assert np.array_equal(host_bits(got).view(view), want.view(view)), name


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("M,K,rotate", [(6, 256, 0), (4, 3072, 1), (3, 3072, 128), (2, 1024, 64), (3, 12288, 1)])
def test_quant_rows_with_prologue_equals_prologue_then_quantizer(M, K, rotate, dt):
    """gpu_quant_rows(prologue) == quantizer(oracle prologue row): every prologue ends on a rounding to T
    (csrc/kernels.cu:100-179), so the two-step form has the fused kernel's codes and scales."""
    cols = 2 * K + 64
    c = pro_case(dt, 700 + K + rotate, M, K, cols)
    xd = dev_bits(c["x"], dt)
    for name in ["RMS_W", "RMS_W_MOD", "GATE", "SWIGLU", "LAYERNORM", "LAYERNORM_MOD", "SILU", "GELU", "ADALN", "LN_MOD", "GELU_TANH"]:
        say("quant_rows prologue", name, M, K, rotate, dt)
        a = pro_args(name, c, K)
        rc, row = oracle.prologue_rows(dt, PRO_ID[name], c["x"], K, **a)
        rc2, q, s = oracle.quant_rows(dt, row, K, rotate)
        assert rc == 0 and rc2 == 0
        qd, sd = ql.quant_rows_pro(xd, PRO_ID[name], K, rotate, **to_dev_args(a, dt))
        torch.cuda.synchronize()
        assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32)), name
        assert np.array_equal(qd.cpu().numpy(), q), name
    # the fused SiTU hands unrounded fp32 values to the quantizer (csrc/kernels.cu:107-112); the lossy id runs the same code
    rc, wide = oracle.situ_rows_wide(dt, c["x"], K, K + 64)
    rc2, q, s = oracle.quant_rows_wide(dt, wide, K, rotate)
    assert rc == 0 and rc2 == 0
    for pro in (ffi.PRO_SITU, ffi.PRO_SITU_FAST):
        say("quant_rows prologue SITU", pro, M, K, rotate, dt)
        qd, sd = ql.quant_rows_pro(xd, pro, K, rotate, up_offset=K + 64)
        torch.cuda.synchronize()
        assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32)), pro
        assert np.array_equal(qd.cpu().numpy(), q), pro


def test_quant_rows_b_and_rotate_rows_f32_with_prologues():
    M, K = 5, 1536
    c = pro_case(BF16, 801, M, K, K + 16)
    xd = dev_bits(c["x"], BF16)
    for name in ("LN_MOD", "LN_AFFINE"):
        a = pro_args(name, c, K)
        rc, row = oracle.prologue_rows(BF16, PRO_ID[name], c["x"], K, **a)
        for rotate in (0, 1):
            rc2, q, s = oracle.quant_rows(BF16, row, K, rotate)
            d = to_dev_args(a, BF16)
            qd, sd = ql.quant_rows_b(xd, PRO_ID[name], K, d.get("norm_w"), d.get("norm_b"), 1e-6, rotate,
                                     d.get("mod_scale"), d.get("mod_shift"))
            torch.cuda.synchronize()
            assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32)), (name, rotate)
            assert np.array_equal(qd.cpu().numpy(), q), (name, rotate)
    K = 1024
    cf = pro_case(F32, 802, 4, K, 2 * K + 64)
    xf = dev(cf["x"])
    for name in ("RMS_W", "SWIGLU"):
        a = pro_args(name, cf, K)
        rc, row = oracle.prologue_rows(F32, PRO_ID[name], cf["x"], K, **a)
        rc2, want = oracle.rotate_rows_f32(row, K)
        d = to_dev_args(a, F32)
        got = ql.rotate_rows_f32(xf, K, PRO_ID[name], d.get("up_offset", 0), d.get("norm_w"), 1e-6)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32)), name


@pytest.mark.parametrize("rotate", [0, 64, 256])
def test_sd_fused_quantizers_equal_source_then_quantizer(rotate):
    """gpu_sd_{ln,geglu,unpad,group_norm}_quant_rows == fp16 quantizer of the oracle's half row (csrc/sd.cu:608-724)."""
    def check(tag, got, row, K):
        rc, q, s = oracle.sd_quant_rows(row, K, rotate)
        torch.cuda.synchronize()
        assert rc == 0
        assert np.array_equal(got[1].cpu().numpy().view(np.uint32), s.view(np.uint32)), tag
        assert np.array_equal(got[0].cpu().numpy(), q), tag
    M, K = 37, 1280
    rnd = lambda stream, *shape: synth.normal(900 + rotate, stream, int(np.prod(shape))).reshape(shape)
    w = (1 + 0.2 * rnd(1, K)).astype(np.float32)
    b = (0.1 * rnd(2, K)).astype(np.float32)
    x = synth.f16_bits(rnd(3, M, K + 64) * np.float32(1.5))
    x[1, :] = 0
    say("sd ln", rotate)
    rc, row = oracle.sd_source_rows(oracle.SD_LN, x, M, K, x_stride=K + 64, w=w, b=b, eps=1e-5)
    check("ln", ql.sd_ln_quant_rows(dev_bits(x, F16), dev(w), dev(b), 1e-5, rotate, K=K), row, K)
    say("sd geglu", rotate)
    xg = synth.f16_bits(rnd(4, M, 2 * K) * np.float32(2))
    rc, row = oracle.sd_source_rows(oracle.SD_GEGLU, xg, M, K)
    check("geglu", ql.sd_geglu_quant_rows(dev_bits(xg, F16), rotate), row, K)
    say("sd unpad", rotate)
    H, d, dp = 16, 80, 96                                                # K = 1280
    xu = synth.f16_bits(rnd(5, M, H * dp))
    rc, row = oracle.sd_source_rows(oracle.SD_UNPAD, xu, M, H * d, heads=H, d=d, dp=dp)
    check("unpad", ql.sd_unpad_quant_rows(dev_bits(xu, F16).view(M, H, dp), d, rotate), row, H * d)
    say("sd gn", rotate)
    N, P, C, G = 2, 40, 512, 32
    xn = synth.f16_bits(rnd(6, N * P, C) * np.float32(1.5) + np.float32(0.3))
    rc, row = oracle.sd_source_rows(oracle.SD_GN, xn, N * P, C, w=w[:C], b=b[:C], eps=1e-5, groups=G, P=P)
    qd, sd, sums = ql.sd_group_norm_quant_rows(dev_bits(xn, F16).view(N, P, C), dev(w[:C].copy()), dev(b[:C].copy()), G, 1e-5, rotate)
    check("gn", (qd, sd), row, C)
    # the statistics are left where the reference leaves them: (mean, rstd) floats at byte 16 * (n * G + g)
    st = sums.cpu().numpy()[:16 * N * G].view(np.float32).reshape(N * G, 4)[:, :2]
    xf = oracle.to_f32(xn, F16).astype(np.float64).reshape(N, P, G, C // G)
    mean = xf.mean(axis=(1, 3)).reshape(-1)
    var = xf.var(axis=(1, 3)).reshape(-1)
    assert np.allclose(st[:, 0], mean, rtol=1e-6, atol=1e-7) and np.allclose(st[:, 1], 1 / np.sqrt(var + 1e-5), rtol=1e-6)


def test_sd_fused_quantizer_argument_checks():
    z = torch.zeros(64, dtype=torch.float16, device=DEV)
    p = z.data_ptr()
    assert ffi.raw("gpu_sd_ln_quant_rows", p, 640, p, p, 0.0, p, p, 1, 640, 128, 0) == -1
    assert ffi.raw("gpu_sd_geglu_quant_rows", p, p, p, 1, 320, 256, 0) == -1
    assert ffi.raw("gpu_sd_unpad_quant_rows", p, p, p, 1, 8, 40, 32, 0, 0) == -1      # dp < d
    assert ffi.raw("gpu_sd_group_norm_quant_rows", p, p, p, p, 1, 4, 30, 4, 0.0, p, p, 0, 0) == -1
    assert ffi.raw("gpu_sd_geglu_quant_rows", p, p, p, 0, 320, 0, 0) == 0


# ------------------------------------------------------------------------------------------------ weight-side formats
@pytest.mark.parametrize("N,K", [(7, 256), (33, 3072), (5, 1280), (2, 12288), (1030, 512)])
def test_convrot_dequant_and_embed_bit_exact(N, K):
    say("convrot_dequant", N, K)
    q = synth.randint(40 + K, 1, N * K, -128, 127).astype(np.int8).reshape(N, K)
    s = synth.uniform(40 + K, 2, N, 1e-3, 1e-2)
    qd, sd = dev(q), dev(s)
    for mode, dt in ((0, torch.float32), (1, torch.bfloat16)):
        rc, want = oracle.convrot_dequant(mode, q, s)
        got = ql.convrot_dequant(qd, sd, dt)
        torch.cuda.synchronize()
        assert rc == 0 and np.array_equal(host_bits(got).view(want.dtype if mode else np.uint32), want.view(np.uint32) if not mode else want)
    rc, want = oracle.convrot_dequant(2, q, s)
    got = ql.embed_dequant(qd, sd)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert ffi.raw("gpu_embed_dequant", qd.data_ptr(), sd.data_ptr(), got.data_ptr(), N, K, 0, 0) == -1
    assert ffi.raw("gpu_convrot_dequant", 0, qd.data_ptr(), sd.data_ptr(), got.data_ptr(), N, 200, 0) == -1


@pytest.mark.parametrize("N,K", [(9, 64), (5, 100), (3, 4096), (1025, 48)])
def test_dequant_i8_bit_exact(N, K):
    q = synth.randint(50 + K, 1, N * K, -128, 127).astype(np.int8).reshape(N, K)
    s = synth.uniform(50 + K, 2, N, 1e-3, 1e-2)
    rc, want = oracle.dequant_i8(q, s)
    got = ql.dequant_i8(dev(q), dev(s))
    torch.cuda.synchronize()
    assert rc == 0 and np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))
    assert ffi.raw("gpu_dequant_i8", 0, 0, 0, 4, 6, 0) == -1


@pytest.mark.parametrize("dt", [BF16, F32])
@pytest.mark.parametrize("N,K", [(6, 256), (40, 3072), (3, 12288)])
def test_convrot_requant_bit_exact(N, K, dt):
    say("convrot_requant", N, K, dt)
    w = synth.normal(60 + K, 1, N * K).reshape(N, K) * np.float32(0.05)
    w[0, :] = 0
    x = synth.bf16_bits(w) if dt == BF16 else w
    xd = dev_bits(x, dt)
    for seed in (0, 1, 0x1234_5678_9abc, 2 ** 63 + 12345):
        rc, q, s = oracle.convrot_requant(dt, x, seed)
        qd, sd = ql.convrot_requant(xd, seed)
        torch.cuda.synchronize()
        assert rc == 0
        assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32)), seed
        assert np.array_equal(qd.cpu().numpy(), q), seed
    # the round trip of the LoRA baker (src/lora.rs:589-592): dequant to the original basis, requant with rounding to
    # nearest, gives the codes back when the weight was exactly representable (bf16 storage costs at most one code)
    rc, q0, s0 = oracle.convrot_requant(dt, x, 0)
    back = ql.convrot_dequant(dev(q0), dev(s0), torch.float32)
    q1, s1 = ql.convrot_requant(back, 0)
    torch.cuda.synchronize()
    assert np.abs(q1.cpu().numpy().astype(np.int32) - q0).max() <= 1
    assert ffi.raw("gpu_convrot_requant", 0, xd.data_ptr(), qd.data_ptr(), sd.data_ptr(), N, 300, 0, 0) == -1


@pytest.mark.parametrize("N,K", [(5, 256), (33, 3072), (3, 13824), (300, 512)])
def test_w6_requant_bit_exact(N, K):
    say("w6_requant", N, K)
    w = synth.normal(70 + K, 1, N * K).reshape(N, K) * np.float32(0.04)
    w[0, :32] = 0
    if N > 2:
        w[2, :] = 0
    wb = synth.bf16_bits(w)
    wd = dev_bits(wb, BF16)
    for seed in (0, 99, 2 ** 40 + 5):
        rc, packed, s_rel, s_ch = oracle.w6_requant(wb, seed)
        pd, rd, cd = ql.w6_requant(wd, seed)
        torch.cuda.synchronize()
        assert rc == 0
        assert np.array_equal(cd.cpu().numpy().view(np.uint32), s_ch.view(np.uint32)), seed
        assert np.array_equal(rd.cpu().numpy(), s_rel), seed
        assert np.array_equal(pd.cpu().numpy(), packed), seed
    # what it writes is what gpu_w6_decode reads
    rc, grid = oracle.w6_decode(packed, s_rel, N, K, 32)
    got = ql.w6_decode(pd, rd, N, K, 32)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), grid)
    assert ffi.raw("gpu_w6_requant", wd.data_ptr(), pd.data_ptr(), rd.data_ptr(), cd.data_ptr(), N, 300, 1, 0) == -1


def test_checkpoint_linears_run_like_the_reference_sequence(tmp_path):
    """Weights as the reference's checkpoints store them (safetensors: int8 ConvRot with row scales, W6 triplet, dense),
    loaded and run through quantize -> GEMM; int8 and W6 outputs bit-exact against the oracle's sequence."""
    from safetensors import safe_open
    from safetensors.torch import save_file
    wts = pkg("weights")
    N, K, M = 96, 512, 40
    W = synth.randint(81, 1, N * K, -127, 127).astype(np.int8).reshape(N, K)
    ws = synth.uniform(81, 2, N, 1e-3, 1e-2)
    bias = oracle.bf16_bits(synth.normal(81, 3, N) * np.float32(0.02))
    codes = (synth.w6_codes(81, N, K).astype(np.int16) + 32).astype(np.uint8)
    packed = oracle.w6_pack_planes(codes)
    s_rel = synth.randint(81, 4, N * (K // 32), 0x38, 0x48).astype(np.uint8).reshape(N, K // 32)
    s_ch = synth.uniform(81, 5, N, 1e-3, 1e-2)
    dense = synth.normal(81, 6, N * K).reshape(N, K) * np.float32(0.05)
    path = str(tmp_path / "m.safetensors")
    save_file({
        "a.weight": torch.from_numpy(W), "a.weight_scale": torch.from_numpy(ws),
        "a.bias": torch.from_numpy(bias.view(np.int16)).view(torch.bfloat16),
        "a.comfy_quant": torch.tensor(list(json.dumps({"format": "int8_tensorwise", "convrot": True, "convrot_groupsize": 256}).encode()), dtype=torch.uint8),
        "b.weight": torch.from_numpy(packed), "b.weight_s_rel": torch.from_numpy(s_rel).view(torch.float8_e4m3fn),
        "b.weight_s_channel": torch.from_numpy(s_ch),
        "c.weight": torch.from_numpy(oracle.bf16_bits(dense).view(np.int16)).view(torch.bfloat16),
    }, path)
    xb = synth.bf16_bits(synth.activations(82, M, K, "t3"))
    x = dev_bits(xb, BF16)
    rc, q, xs = oracle.quant_rows(BF16, xb, K, 1)
    with safe_open(path, framework="pt") as st:
        a = wts.load_linear(st, "a", DEV)
        b = wts.load_linear(st, "b", DEV)
        c = wts.load_linear(st, "c", DEV)
    ya = wts.forward(a, x)
    yb = wts.forward(b, x)
    yc = wts.forward(c, x)
    torch.cuda.synchronize()
    want_a = oracle.epilogue(oracle.int8_gemm_acc(q, W), xs, ws, bias, BF16, fma=1)
    assert np.array_equal(host_bits(ya), want_a)
    rc, grid = oracle.w6_decode(packed, s_rel, N, K, 32)
    want_b = oracle.epilogue(oracle.int8_gemm_acc(q, grid), xs, s_ch, None, BF16, fma=1)
    assert np.array_equal(host_bits(yb), want_b)
    ref = oracle.bf16_to_f32(xb).astype(np.float64) @ oracle.bf16_to_f32(oracle.bf16_bits(dense)).astype(np.float64).T
    assert np.allclose(yc.float().cpu().numpy(), ref, rtol=2.0 ** -7, atol=1e-3)


def test_dit_block_linear_chain_matches_oracle_composition():
    """The linear launches of one DiT block in the order and with the argument patterns of src/dit.rs:545-611: RMS +
    modulation prologue -> fused QKV+gate GEMM; gate prologue reading the gate columns inside the QKV buffer -> output
    projection with the residual added in place; RMS + modulation -> MLP gate|up GEMM; SwiGLU prologue on the two halves of
    that buffer -> down projection with the residual in place.  (Attention itself is outside this path: the q columns
    stand in for its output.)  The final hidden state must equal the oracle's composition bit for bit."""
    rows, F, QKV, MLP, eps = 70, 512, 1024, 1024, 1e-6
    QKVG = QKV + F
    rnd = lambda st, *shape: synth.normal(91, st, int(np.prod(shape))).reshape(shape)
    wq = lambda st, n, k: synth.randint(91, st, n * k, -127, 127).astype(np.int8).reshape(n, k)
    x0 = synth.bf16_bits(rnd(1, rows, F))
    pre, post = (1 + 0.1 * rnd(2, F)).astype(np.float32), (1 + 0.1 * rnd(3, F)).astype(np.float32)
    mv = [synth.bf16_bits(0.2 * rnd(10 + i, F)) for i in range(6)]
    Wqkvg, Wo, Wgu, Wd = wq(20, QKVG, F), wq(21, F, F), wq(22, 2 * MLP, F), wq(23, F, MLP)
    sc = lambda st, n: synth.uniform(91, st, n, 2e-4, 1e-3)
    sqkvg, so, sgu, sd = sc(30, QKVG), sc(31, F), sc(32, 2 * MLP), sc(33, F)

    # oracle composition
    def o_quant(pro, xb, K, **kw):
        rc, row = oracle.prologue_rows(BF16, pro, xb, K, **kw)
        rc2, q, s = oracle.quant_rows(BF16, row, K, 1)
        assert rc == 0 and rc2 == 0
        return q, s
    x = x0.copy()
    q, s = o_quant(1, x, F, norm_w=pre, eps=eps, mod_scale=mv[0], mod_shift=mv[1])
    qkvg = oracle.epilogue(oracle.int8_gemm_acc(q, Wqkvg), s, sqkvg, None, BF16, fma=1)
    attn = np.ascontiguousarray(qkvg[:, :F])
    q, s = o_quant(2, attn, F, g=np.ascontiguousarray(qkvg[:, QKV:]))
    x = oracle.epilogue_residual(oracle.int8_gemm_acc(q, Wo), s, so, None, mv[2], x, BF16, fma=1)
    q, s = o_quant(1, x, F, norm_w=post, eps=eps, mod_scale=mv[3], mod_shift=mv[4])
    gu = oracle.epilogue(oracle.int8_gemm_acc(q, Wgu), s, sgu, None, BF16, fma=1)
    q, s = o_quant(3, gu, MLP, up_offset=MLP)
    x = oracle.epilogue_residual(oracle.int8_gemm_acc(q, Wd), s, sd, None, mv[5], x, BF16, fma=1)

    # the same launches through the C ABI
    xd = dev_bits(x0, BF16)
    mvd = [dev_bits(m, BF16) for m in mv]
    a8, asc = ql.quant_rows_pro(xd, ffi.PRO_RMS, F, 1, norm_w=dev(pre), eps=eps, mod_scale=mvd[0], mod_shift=mvd[1])
    qkvg_d = ql.int8_gemm(a8, dev(Wqkvg), asc, dev(sqkvg), None, torch.bfloat16)
    attn_d = qkvg_d[:, :F].contiguous()
    gate_view = qkvg_d[:, QKV:]                               # the gate columns where they lie: row stride QKVG
    a8, asc = ql.quant_rows_pro(attn_d, ffi.PRO_GATE, F, 1, g=gate_view)
    ql.int8_gemm_residual(a8, dev(Wo), asc, dev(so), None, mvd[2], xd, D=xd)
    a8, asc = ql.quant_rows_pro(xd, ffi.PRO_RMS, F, 1, norm_w=dev(post), eps=eps, mod_scale=mvd[3], mod_shift=mvd[4])
    gu_d = ql.int8_gemm(a8, dev(Wgu), asc, dev(sgu), None, torch.bfloat16)
    a8, asc = ql.quant_rows_pro(gu_d, ffi.PRO_SWIGLU, MLP, 1, up_offset=MLP)
    ql.int8_gemm_residual(a8, dev(Wd), asc, dev(sd), None, mvd[5], xd, D=xd)
    torch.cuda.synchronize()
    assert np.array_equal(host_bits(qkvg_d), qkvg) and np.array_equal(host_bits(gu_d), gu)
    assert np.array_equal(host_bits(xd), x)


def test_unet_feed_forward_chain_matches_oracle_composition():
    """The feed-forward of an SD/SDXL transformer block as src/unet.rs:429-456 launches it, fp16 throughout: LayerNorm
    fused into the quantizer -> GEGLU up-projection with bias; GEGLU fused into the quantizer -> down-projection added to
    the hidden state in place (residual scale of ones)."""
    M, C, I, rot = 130, 640, 2560, 64
    rnd = lambda st, *shape: synth.normal(95, st, int(np.prod(shape))).reshape(shape)
    wq = lambda st, n, k: synth.randint(95, st, n * k, -127, 127).astype(np.int8).reshape(n, k)
    x0 = synth.f16_bits(rnd(1, M, C))
    lw, lb = (1 + 0.1 * rnd(2, C)).astype(np.float32), (0.05 * rnd(3, C)).astype(np.float32)
    Wup, Wdn = wq(4, 2 * I, C), wq(5, C, I)
    sup, sdn = synth.uniform(95, 6, 2 * I, 2e-4, 1e-3), synth.uniform(95, 7, C, 1e-4, 5e-4)
    bup, bdn = synth.f16_bits(0.02 * rnd(8, 2 * I)), synth.f16_bits(0.02 * rnd(9, C))
    ones = synth.f16_bits(np.ones(C, np.float32))
    # oracle
    rc, row = oracle.sd_source_rows(oracle.SD_LN, x0, M, C, x_stride=C, w=lw, b=lb, eps=1e-5)
    rc, q, s = oracle.sd_quant_rows(row, C, rot)
    h = oracle.epilogue(oracle.int8_gemm_acc(q, Wup), s, sup, bup, F16, fma=1)
    rc, row = oracle.sd_source_rows(oracle.SD_GEGLU, h, M, I)
    rc, q, s = oracle.sd_quant_rows(row, I, rot)
    want = oracle.epilogue_residual(oracle.int8_gemm_acc(q, Wdn), s, sdn, bdn, ones, x0, F16, fma=1)
    # C ABI
    xd = dev_bits(x0, F16)
    a8, asc = ql.sd_ln_quant_rows(xd, dev(lw), dev(lb), 1e-5, rot)
    hd = ql.int8_gemm(a8, dev(Wup), asc, dev(sup), dev_bits(bup, F16), torch.float16)
    a8, asc = ql.sd_geglu_quant_rows(hd, rot)
    ql.int8_gemm_residual(a8, dev(Wdn), asc, dev(sdn), dev_bits(bdn, F16), dev_bits(ones, F16), xd, D=xd)
    torch.cuda.synchronize()
    assert np.array_equal(host_bits(hd), h)
    assert np.array_equal(host_bits(xd), want)


def test_text_encoder_mlp_chain_weight_only_int8():
    """A text-encoder MLP as src/te.rs:490-513 runs it: weight-only int8 ConvRot weights, fp32 activations rotated
    instead of the weights (x @ ((q s) H)^T == (x H) @ (q s)^T), fp32 GEMMs, the residual through beta = 1.  The rotated
    rows are bit-exact against the oracle; the GEMM results are checked against float64."""
    M, D, FF, eps = 24, 512, 1024, 1e-6
    rnd = lambda st, *shape: synth.normal(97, st, int(np.prod(shape))).reshape(shape)
    wq = lambda st, n, k: synth.randint(97, st, n * k, -127, 127).astype(np.int8).reshape(n, k)
    x0 = rnd(1, M, D).astype(np.float32)
    ln = (1 + 0.1 * rnd(2, D)).astype(np.float32)
    Wgu, Wd = wq(3, 2 * FF, D), wq(4, D, FF)
    sgu, sd = synth.uniform(97, 5, 2 * FF, 2e-4, 1e-3), synth.uniform(97, 6, D, 2e-4, 1e-3)
    # oracle for the rotated rows, float64 for the products
    rc, row = oracle.prologue_rows(F32, 1, x0, D, norm_w=ln, eps=eps)
    rc, xr = oracle.rotate_rows_f32(row, D)
    gu64 = xr.astype(np.float64) @ (Wgu.astype(np.float64) * sgu[:, None].astype(np.float64)).T
    xd = dev(x0)
    xr_d = ql.rotate_rows_f32(xd, D, ffi.PRO_RMS, 0, dev(ln), eps)
    gu_d = ql.gemm(xr_d, ql.dequant_i8(dev(Wgu), dev(sgu)), None, True, torch.float32)
    torch.cuda.synchronize()
    assert np.array_equal(xr_d.cpu().numpy().view(np.uint32), xr.view(np.uint32))
    assert np.allclose(gu_d.cpu().numpy(), gu64, rtol=1e-4, atol=1e-4)
    gu = gu_d.cpu().numpy()
    rc, row2 = oracle.prologue_rows(F32, 3, gu, FF, up_offset=FF)
    rc, xr2 = oracle.rotate_rows_f32(row2, FF)
    xr2_d = ql.rotate_rows_f32(gu_d, FF, ffi.PRO_SWIGLU, FF)
    out = ql.gemm(xr2_d, ql.dequant_i8(dev(Wd), dev(sd)), None, True, torch.float32, beta=1.0, D=xd)   # x += mlp(x)
    torch.cuda.synchronize()
    assert np.array_equal(xr2_d.cpu().numpy().view(np.uint32), xr2.view(np.uint32))
    want = x0.astype(np.float64) + xr2.astype(np.float64) @ (Wd.astype(np.float64) * sd[:, None].astype(np.float64)).T
    assert np.allclose(out.cpu().numpy(), want, rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------------------------------------ dense GEMM
@pytest.mark.parametrize("in_dt,out_dt", [(torch.bfloat16, torch.bfloat16), (torch.float16, torch.float16),
                                          (torch.float32, torch.float32), (torch.bfloat16, torch.float32)])
@pytest.mark.parametrize("M,N,K,transb,with_bias", [(64, 256, 512, True, True), (130, 96, 320, True, False),
                                                     (48, 128, 256, False, True), (1, 3072, 256, True, True)])
def test_gpu_gemm_against_float64(M, N, K, transb, with_bias, in_dt, out_dt):
    """gpu_gemm over hipBLASLt: fp32 accumulation of the inputs' products, checked against a float64 product of the same
    rounded inputs.  Tolerance: two units of the output type plus the fp32 accumulation error over K."""
    say("gpu_gemm", M, N, K, transb, with_bias, in_dt, out_dt)
    g = torch.Generator().manual_seed(M + N + K)
    A = torch.randn(M, K, generator=g).to(in_dt)
    B = (torch.randn(N, K, generator=g) if transb else torch.randn(K, N, generator=g)).to(in_dt) * 0.1
    bias = torch.randn(N, generator=g).to(out_dt) if with_bias else None
    want = A.double() @ (B.double().T if transb else B.double())
    if with_bias:
        want = want + bias.double()
    got = ql.gemm(A.to(DEV), B.to(DEV), None if bias is None else bias.to(DEV), transb, out_dt)
    torch.cuda.synchronize()
    unit = {torch.bfloat16: 2.0 ** -8, torch.float16: 2.0 ** -11, torch.float32: 2.0 ** -24}[out_dt]
    mag = A.double().abs() @ (B.double().abs().T if transb else B.double().abs())
    assert ((got.cpu().double() - want).abs() <= 2 * unit * want.abs() + K * 2.0 ** -24 * mag + 1e-30).all()
    # alpha and beta
    D = torch.ones((M, N), dtype=out_dt, device=DEV)
    ql.gemm(A.to(DEV), B.to(DEV), None, transb, out_dt, alpha=0.5, beta=2.0, D=D)
    torch.cuda.synchronize()
    want2 = 0.5 * (want - (bias.double() if with_bias else 0)) + 2.0
    assert ((D.cpu().double() - want2).abs() <= 2 * unit * (want2.abs() + 2) + K * 2.0 ** -24 * mag + 1e-30).all()


def test_rotated_quant_golden_fixture():
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "rotated_quant.json")))
    xb = synth.bf16_bits(synth.activations(11, 8, 1024, "t3"))
    assert hashlib.sha256(xb.tobytes()).hexdigest() == g["x_sha256"]
    for grp in (64, 128, 256):
        qd, sd = ql.quant_rows(dev_bits(xb, BF16), grp)
        torch.cuda.synchronize()
        q = qd.cpu().numpy()
        s = sd.cpu().numpy().view(np.uint32)
        assert hashlib.sha256(q.tobytes()).hexdigest() == g["q_g%d_sha256" % grp]
        assert hashlib.sha256(s.tobytes()).hexdigest() == g["xs_bits_g%d_sha256" % grp]
        assert q.reshape(-1)[::g["stride"]].tolist() == g["q_g%d_sample" % grp]


# ------------------------------------------------------------------------------------------------ GEMM
def rand_i8(seed, stream, M, K, lo=-128, hi=127):
    return synth.randint(seed, stream, M * K, lo, hi).astype(np.int8).reshape(M, K)


ACC_CASES = [(1, 96, 256), (3, 32, 16), (64, 64, 64), (65, 72, 48), (100, 104, 320), (130, 260, 80), (257, 96, 3072),
             (300, 520, 192), (33, 8, 1024), (260, 300, 64), (512, 256, 128), (777, 1000, 448), (300, 260, 384), (1100, 1500, 256), (200, 1056, 256), (256, 2048, 1536), (1, 1024, 512),
             (77, 4096, 1280), (250, 25000, 128)]


@pytest.mark.parametrize("cfg", [2, 1, 6, 7, 9])
@pytest.mark.parametrize("M,N,K", ACC_CASES)
def test_int8_gemm_acc_bit_exact(M, N, K, cfg):
    say("gemm_acc", M, N, K, "cfg", cfg)
    A = rand_i8(1, 500 + M, M, K)
    W = rand_i8(1, 600 + N, N, K)
    A[0, :] = -128
    W[0, :] = -128                                           # the extreme product, K * 2^14
    want = oracle.int8_gemm_acc(A, W)
    ffi.raw("gpu_int8_gemm_force_config", cfg)
    try:
        got = ql.int8_gemm_acc(dev(A), dev(W))
        torch.cuda.synchronize()
    finally:
        ffi.raw("gpu_int8_gemm_force_config", -1)
    assert np.array_equal(got.cpu().numpy(), want)


# K % 16 == 8: the reference's alignment-8 configurations (csrc/vendor/cutlass_gemm_int8.cu:191,237-247)
@pytest.mark.parametrize("M,N,K", [(5, 40, 8), (130, 264, 136), (300, 1030, 1000), (64, 2048, 4104)])
def test_int8_gemm_k_multiple_of_8_only(M, N, K):
    say("gemm_k8", M, N, K)
    A = rand_i8(6, 1, M, K)
    W = rand_i8(6, 2, N, K)
    xs = synth.uniform(6, 3, M, 0.005, 0.2)
    ws = synth.uniform(6, 4, N, 1e-3, 1e-2)
    bias = oracle.bf16_bits(synth.normal(6, 5, N) * np.float32(0.02))
    rscale = oracle.bf16_bits(synth.normal(6, 6, N))
    resid = oracle.bf16_bits(synth.normal(6, 7, M * N).reshape(M, N))
    want = oracle.int8_gemm_acc(A, W)
    Ad, Wd = dev(A), dev(W)
    got = ql.int8_gemm_acc(Ad, Wd)
    d = ql.int8_gemm(Ad, Wd, dev(xs), dev(ws), dev_bits(bias, BF16), torch.bfloat16)
    r = ql.int8_gemm_residual(Ad, Wd, dev(xs), dev(ws), dev_bits(bias, BF16), dev_bits(rscale, BF16), dev_bits(resid, BF16))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    assert np.array_equal(host_bits(d), oracle.epilogue(want, xs, ws, bias, BF16, fma=1))
    assert np.array_equal(host_bits(r), oracle.epilogue_residual(want, xs, ws, bias, rscale, resid, BF16, fma=1))
    # no tile configuration of the reference takes K % 8 != 0
    assert ffi.raw("gpu_int8_gemm", Ad.data_ptr(), Wd.data_ptr(), 0, 0, 0, 0, M, N, K - 4, 2, 0) == -200


# More 256x256 tiles than CUs, and not a multiple of the CU count: the persistent kernel's workgroups then own unequal
# numbers of tiles, and every output form runs through its coalesced epilogue.
MANY_TILE_CASES = [(4352, 4096, 256), (4100, 4400, 384), (2304, 8200, 640),
                   # either side of the dispatcher's thresholds: two row tiles of the weight-streaming kernel with K split
                   # (planes beyond the per-stream buffer), ring tiles for few tiles and long K, short K at M <= 256 on
                   # the register-staged and ring tiles, M <= 128 with K = 1536 on the weight-streaming kernel, and a
                   # shape where the two-group tiles cover half of the CUs
                   (384, 1056, 8192), (512, 4096, 2048), (256, 1024, 1024), (256, 12288, 1024), (200, 2048, 2048),
                   (100, 3008, 1536), (2048, 2048, 512)]


@pytest.mark.parametrize("M,N,K", MANY_TILE_CASES)
def test_int8_gemm_many_tiles_bit_exact(M, N, K):
    say("gemm_many_tiles", M, N, K)
    A = rand_i8(4, 500 + M, M, K)
    W = rand_i8(4, 600 + N, N, K)
    want = oracle.int8_gemm_acc(A, W)
    xs = synth.uniform(4, 3, M, 0.005, 0.2)
    ws = synth.uniform(4, 4, N, 1e-3, 1e-2)
    bias = oracle.bf16_bits(synth.normal(4, 5, N) * np.float32(0.02))
    rscale = oracle.bf16_bits(synth.normal(4, 6, N))
    resid = oracle.bf16_bits(synth.normal(4, 7, M * N).reshape(M, N))
    want_d = oracle.epilogue(want, xs, ws, bias, BF16, fma=1)
    want_r = oracle.epilogue_residual(want, xs, ws, bias, rscale, resid, BF16, fma=1)
    Ad, Wd = dev(A), dev(W)
    got = ql.int8_gemm_acc(Ad, Wd)
    d = ql.int8_gemm(Ad, Wd, dev(xs), dev(ws), dev_bits(bias, BF16), torch.bfloat16)
    r = ql.int8_gemm_residual(Ad, Wd, dev(xs), dev(ws), dev_bits(bias, BF16), dev_bits(rscale, BF16), dev_bits(resid, BF16))
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    assert np.array_equal(host_bits(d), want_d)
    assert np.array_equal(host_bits(r), want_r)
    if M == 4352:   # the other output types through the same split into 256x256 rounds and a 128x192 remainder
        for dt, tdt, tob in ((F32, torch.float32, lambda a: a.astype(np.float32)), (F16, torch.float16, oracle.f16_bits)):
            b2 = tob(synth.normal(4, 5, N) * np.float32(0.02))
            w2 = oracle.epilogue(want, xs, ws, b2, dt, fma=1)
            d2 = ql.int8_gemm(Ad, Wd, dev(xs), dev(ws), dev_bits(b2, dt), tdt)
            torch.cuda.synchronize()
            view = np.uint32 if dt == F32 else np.uint16
            assert np.array_equal(host_bits(d2).view(view), w2.view(view)), dt


@pytest.mark.parametrize("out_dt", [BF16, F16, F32])
@pytest.mark.parametrize("M,N,K,with_bias", [(37, 96, 256, True), (130, 264, 192, False), (256, 1024, 1024, True), (100, 2048, 1024, True),
                                                     (4100, 648, 384, True)])
def test_int8_gemm_epilogue(M, N, K, with_bias, out_dt):
    say("gemm", M, N, K, with_bias, out_dt)
    A = rand_i8(2, 1, M, K, -127, 127)
    W = rand_i8(2, 2, N, K, -127, 127)
    xs = synth.uniform(2, 3, M, 0.005, 0.2)
    ws = synth.uniform(2, 4, N, 1e-3, 1e-2)
    tob = {BF16: oracle.bf16_bits, F16: oracle.f16_bits, F32: lambda a: a.astype(np.float32)}[out_dt]
    bias = tob(synth.normal(2, 5, N) * np.float32(0.02)) if with_bias else None
    want = oracle.int8_gemm(A, W, xs, ws, bias, out_dt, fma=1)
    loose = oracle.int8_gemm(A, W, xs, ws, bias, out_dt, fma=0)
    for cfg in (-1, 1, 2, 6, 7, 9):
        ffi.raw("gpu_int8_gemm_force_config", cfg)
        try:
            got = ql.int8_gemm(dev(A), dev(W), dev(xs), dev(ws), None if bias is None else dev_bits(bias, out_dt), TDT[out_dt])
            torch.cuda.synchronize()
        finally:
            ffi.raw("gpu_int8_gemm_force_config", -1)
        gb = host_bits(got)
        assert np.array_equal(gb.view(np.uint32 if out_dt == F32 else np.uint16), want.view(np.uint32 if out_dt == F32 else np.uint16)), cfg
        assert ulp_close(gb, loose, out_dt, 0.0 if bias is None else np.abs(oracle.to_f32(bias, out_dt))[None, :])


@pytest.mark.parametrize("out_dt", [BF16, F16, F32])
def test_int8_gemm_residual_in_place(out_dt):
    M, N, K = 150, 136, 256
    A = rand_i8(3, 1, M, K, -127, 127)
    W = rand_i8(3, 2, N, K, -127, 127)
    xs = synth.uniform(3, 3, M, 0.005, 0.2)
    ws = synth.uniform(3, 4, N, 1e-3, 1e-2)
    tob = {BF16: oracle.bf16_bits, F16: oracle.f16_bits, F32: lambda a: a.astype(np.float32)}[out_dt]
    bias = tob(synth.normal(3, 5, N) * np.float32(0.02))
    rscale = tob(synth.normal(3, 6, N))
    resid = tob(synth.normal(3, 7, M * N).reshape(M, N))
    want = oracle.int8_gemm_residual(A, W, xs, ws, bias, rscale, resid, out_dt, fma=1)
    loose = oracle.int8_gemm_residual(A, W, xs, ws, bias, rscale, resid, out_dt, fma=0)
    x = dev_bits(resid, out_dt)                      # D aliases resid, as in src/dit.rs:592
    ql.int8_gemm_residual(dev(A), dev(W), dev(xs), dev(ws), dev_bits(bias, out_dt), dev_bits(rscale, out_dt), x, D=x)
    torch.cuda.synchronize()
    gb = host_bits(x)
    view = np.uint32 if out_dt == F32 else np.uint16
    assert np.array_equal(gb.view(view), want.view(view))
    # two roundings: the unfused form can differ by one ulp of z scaled by rscale, plus one ulp of the result
    a = oracle.to_f32(gb, out_dt).astype(np.float64)
    b = oracle.to_f32(loose, out_dt).astype(np.float64)
    ulp = {BF16: 2.0 ** -7, F16: 2.0 ** -10, F32: 2.0 ** -23}[out_dt]
    assert (np.abs(a - b) <= 4 * ulp * (np.abs(a) + np.abs(b) + 1.0)).all()
    # without bias, out of place
    want2 = oracle.int8_gemm_residual(A, W, xs, ws, None, rscale, resid, out_dt, fma=1)
    got2 = ql.int8_gemm_residual(dev(A), dev(W), dev(xs), dev(ws), None, dev_bits(rscale, out_dt), dev_bits(resid, out_dt))
    torch.cuda.synchronize()
    assert np.array_equal(host_bits(got2).view(view), want2.view(view))


RESID_CASES = [  # (M, N, K, kernel families that can run the shape)
    (200, 1024, 4096, (-1, 6, 1, 2)),          # skinny: split K, planes summed by the reduce kernel
    (256, 2400, 1024, (-1, 6, 1)),             # skinny: one K slice, the streaming kernel's own epilogue
    (600, 768, 512, (-1, 1, 2, 7, 9)),         # tile kernels and the persistent kernels
]


@pytest.mark.parametrize("out_dt", [BF16, F16, F32])
@pytest.mark.parametrize("M,N,K,cfgs", RESID_CASES)
def test_int8_gemm_residual_in_place_every_kernel_family(M, N, K, cfgs, out_dt):
    """gpu_int8_gemm_residual with D aliasing resid (the down-projection pattern of src/dit.rs:592) through every kernel
    family: the streaming kernel's residual epilogue, the split-K reduce kernel's, the persistent kernels' and the
    tile kernels', bit-exact against the oracle."""
    say("gemm_residual", M, N, K, out_dt)
    A = rand_i8(13, 1, M, K, -127, 127)
    W = rand_i8(13, 2, N, K, -127, 127)
    xs = synth.uniform(13, 3, M, 0.005, 0.2)
    ws = synth.uniform(13, 4, N, 1e-3, 1e-2)
    tob = {BF16: oracle.bf16_bits, F16: oracle.f16_bits, F32: lambda a: a.astype(np.float32)}[out_dt]
    bias = tob(synth.normal(13, 5, N) * np.float32(0.02))
    rscale = tob(synth.normal(13, 6, N))
    resid = tob(synth.normal(13, 7, M * N).reshape(M, N))
    want = oracle.int8_gemm_residual(A, W, xs, ws, bias, rscale, resid, out_dt, fma=1)
    view = np.uint32 if out_dt == F32 else np.uint16
    Ad, Wd, xsd, wsd = dev(A), dev(W), dev(xs), dev(ws)
    bd, rsd = dev_bits(bias, out_dt), dev_bits(rscale, out_dt)
    for cfg in cfgs:
        x = dev_bits(resid, out_dt)
        ffi.raw("gpu_int8_gemm_force_config", cfg)
        try:
            ql.int8_gemm_residual(Ad, Wd, xsd, wsd, bd, rsd, x, D=x)
            torch.cuda.synchronize()
        finally:
            ffi.raw("gpu_int8_gemm_force_config", -1)
        assert np.array_equal(host_bits(x).view(view), want.view(view)), cfg


def test_config0_end_to_end_matches_golden_fixture():
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "config0_w8a8.json")))
    c = synth.config0(0)
    dig = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
    assert dig(c["x"]) == g["x_sha256"] and dig(c["W"]) == g["W_sha256"]
    x = dev_bits(c["x"], BF16)
    W, ws, bias = dev(c["W"]), dev(c["ws"]), dev_bits(c["bias"], BF16)
    q, xs = ql.quant_rows(x, 0)
    acc = ql.int8_gemm_acc(q, W)
    d = ql.int8_gemm(q, W, xs, ws, bias, torch.bfloat16)
    d2 = ql.linear_w8a8(x, W, ws, bias, rotate=0)
    torch.cuda.synchronize()
    s = g["stride"]
    assert dig(q.cpu().numpy()) == g["q_sha256"] and q.cpu().numpy().reshape(-1)[::s].tolist() == g["q_sample"]
    assert dig(xs.cpu().numpy().view(np.uint32)) == g["xs_bits_sha256"]
    assert dig(acc.cpu().numpy()) == g["acc_sha256"] and acc.cpu().numpy().reshape(-1)[::s].tolist() == g["acc_sample"]
    db = host_bits(d)
    assert dig(db) == g["d_fma_bits_sha256"] and db.reshape(-1)[::s].tolist() == g["d_fma_bits_sample"]
    assert np.array_equal(host_bits(d2), db)
    nofma = np.array(g["d_nofma_bits_sample"], np.uint16)
    assert ulp_close(db.reshape(-1)[::s], nofma, BF16)


# ------------------------------------------------------------------------------------------------ W6
def test_w6_decode_exhaustive_and_random():
    K, G = 64, 16
    codes = np.arange(64, dtype=np.uint8)[None, :].repeat(256, axis=0)
    wq = oracle.w6_pack_planes(codes)
    s_rel = np.arange(256, dtype=np.uint8)[:, None].repeat(K // G, axis=1)
    rc, want = oracle.w6_decode(wq, s_rel, 256, K, G)
    got = ql.w6_decode(dev(wq), dev(s_rel), 256, K, G)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)
    N, K, G = 77, 5376, 32
    codes = (synth.w6_codes(6, N, K).astype(np.int16) + 32).astype(np.uint8)
    wq = oracle.w6_pack_planes(codes)
    s_rel = synth.w6_srel_bytes(6, N, K, G)
    rc, want = oracle.w6_decode(wq, s_rel, N, K, G)
    got = ql.w6_decode(dev(wq), dev(s_rel), N, K, G)
    torch.cuda.synchronize()
    assert np.array_equal(got.cpu().numpy(), want)


def test_w6a8_linear_matches_decode_then_gemm():
    """The H3-style W6A8 linear (src/h3.rs:1208-1251): rows quantized with the 256-wide rotation, weights decoded from
    the packed planes, per-row s_channel as the weight scale."""
    M, K, N, G = 300, 1536, 640, 32
    xb = synth.bf16_bits(synth.activations(8, M, K, "t3"))
    codes = (synth.w6_codes(8, N, K).astype(np.int16) + 32).astype(np.uint8)
    wq = oracle.w6_pack_planes(codes)
    s_rel = synth.w6_srel_bytes(8, N, K, G)
    s_ch = synth.uniform(8, 30, N, 1e-3, 1e-2)
    bias = synth.bf16_bits(synth.normal(8, 31, N) * np.float32(0.02))
    rc, q, xs = oracle.quant_rows(BF16, xb, K, 1)
    rc2, w8 = oracle.w6_decode(wq, s_rel, N, K, G)
    assert rc == 0 and rc2 == 0
    want = oracle.int8_gemm(q, w8, xs, s_ch, bias, BF16, fma=1)
    qd, xsd = ql.quant_rows(dev_bits(xb, BF16), 1)
    got = ql.w6a8_gemm(qd, dev(wq), dev(s_rel), G, xsd, dev(s_ch), dev_bits(bias, BF16))
    torch.cuda.synchronize()
    assert np.array_equal(host_bits(got), want)
    assert ffi.raw("gpu_w6a8_gemm", 0, 0, 0, 32, 0, 0, 0, 0, 4, 8, 48, 2, 0) == -1


# A beyond 4 GiB: byte offsets into A no longer fit 32 bits, which the DMA kernels' lane offsets assume; the dispatcher has
# to take the register-staged tiles with 64-bit addressing.  Checked on sampled rows against the oracle.
def test_int8_gemm_with_operand_beyond_4_gib():
    M, N, K = 66000, 96, 65536
    say("gemm_4gib", M, N, K)
    g = torch.Generator(device="cuda").manual_seed(77)
    A = torch.randint(-128, 128, (M, K), dtype=torch.int8, device="cuda", generator=g)
    W = torch.randint(-128, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    assert A.numel() > 1 << 32
    acc = ql.int8_gemm_acc(A, W)
    xs = dev(synth.uniform(8, 3, M, 0.005, 0.2))
    ws = dev(synth.uniform(8, 4, N, 1e-3, 1e-2))
    d = ql.int8_gemm(A, W, xs, ws, None, torch.float32)
    torch.cuda.synchronize()
    rows = sorted({0, 1, 255, 256, 32767, 32768, 65535, 65536, 65537, M - 2, M - 1} | {int(r) for r in synth.randint(8, 9, 24, 0, M - 1)})
    idx = torch.tensor(rows, device="cuda")
    Ah, Wh = A[idx].cpu().numpy(), W.cpu().numpy()
    want = oracle.int8_gemm_acc(Ah, Wh)
    assert np.array_equal(acc[idx].cpu().numpy(), want)
    want_d = oracle.epilogue(want, xs[idx].cpu().numpy(), ws.cpu().numpy(), None, F32, fma=1)
    assert np.array_equal(d[idx].cpu().numpy().view(np.uint32), want_d.view(np.uint32))
    # every row: the checksum identity sum_n acc[m, n] = A[m, :] . sum_n W[n, :]
    wsum = W.to(torch.int32).sum(0).to(torch.float64)
    lhs = acc.to(torch.float64).sum(1)
    rhs = torch.empty(M, dtype=torch.float64, device="cuda")
    for r0 in range(0, M, 6000):
        rhs[r0:r0 + 6000] = A[r0:r0 + 6000].to(torch.float64) @ wsum
    assert torch.equal(lhs, rhs)


@pytest.mark.parametrize("rotate", [128, 256])
def test_quant_rows_with_more_than_2_to_the_31_elements(rotate):
    """Element offsets past 2^31 and byte offsets past 2^32 (the longest row the reference takes, K = 32768, reduced over
    eight waves): sampled rows against the oracle, and every row's scale against the maximum of |codes * scale|."""
    M, K = 66000, 32768
    say("quant_big", M, K, rotate)
    g = torch.Generator(device="cuda").manual_seed(78)
    x = torch.empty((M, K), dtype=torch.bfloat16, device="cuda")
    for r0 in range(0, M, 6000):   # in slices: randn makes an fp32 temporary
        x[r0:r0 + 6000] = (torch.randn((min(6000, M - r0), K), device="cuda", generator=g) * (1 + (r0 % 7))).to(torch.bfloat16)
    assert x.numel() > 1 << 31
    q, sc = ql.quant_rows(x, rotate)
    torch.cuda.synchronize()
    rows = sorted({0, 1, 32767, 32768, 65535, 65536, 65537, M - 1} | {int(r) for r in synth.randint(8, 19, 8, 0, M - 1)})
    idx = torch.tensor(rows, device="cuda")
    xb = x[idx].view(torch.int16).cpu().numpy().view(np.uint16)
    rc, wq, wsc = oracle.quant_rows(BF16, xb, K, rotate)
    assert rc == 0
    assert np.array_equal(q[idx].cpu().numpy(), wq)
    assert np.array_equal(sc[idx].cpu().numpy().view(np.uint32), wsc.view(np.uint32))
    # every row was written: a code of magnitude 127 (the row maximum) in each, and a positive finite scale
    amax = torch.empty(M, dtype=torch.int16, device="cuda")
    for r0 in range(0, M, 6000):
        amax[r0:r0 + 6000] = q[r0:r0 + 6000].to(torch.int16).abs().amax(1)
    assert bool((amax >= 126).all()) and bool(torch.isfinite(sc).all()) and bool((sc > 0).all())


# ------------------------------------------------------------------------------------------------ graph capture
@pytest.mark.parametrize("M,N,K,entry", [(4096, 4096, 256, "gpu_int8_gemm"),          # two-group kernel
                                           (1024, 2304, 256, "gpu_int8_gemm"),          # ring kernel on 128x192 tiles
                                           (256, 24576, 3072, "gpu_int8_gemm"),         # weight-streaming kernel, whole K
                                           (640, 1536, 512, "gpu_int8_gemm"),           # register-staged tiles
                                           (256, 2048, 4096, "gpu_int8_gemm_static")])  # weight-streaming kernel, split K, static planes
def test_linear_replays_from_a_captured_graph(M, N, K, entry):
    """The quantizer and the GEMM allocate nothing on these routes (the split-K shape through the entry point with the
    static planes), so one linear can be captured.  Three replays with new activations and eager work between them,
    each against the oracle's linear on the same inputs."""
    say("graph", M, N, K, entry)
    W, ws, bias = synth.w8_weights(21, N, K)
    bias = oracle.bf16_bits(bias)
    Wd, wsd, bd = dev(W), dev(ws), dev_bits(bias, BF16)
    x = torch.zeros((M, K), dtype=torch.bfloat16, device="cuda")
    q = torch.empty((M, K), dtype=torch.int8, device="cuda")
    xs = torch.empty((M,), dtype=torch.float32, device="cuda")
    D = torch.empty((M, N), dtype=torch.bfloat16, device="cuda")

    def call():
        s = torch.cuda.current_stream().cuda_stream
        ffi.k("gpu_quant_rows", ffi.DT_BF16, ffi.PRO_PLAIN, x.data_ptr(), K, 0, 0, 0, 0, 0.0, 0, 0, q.data_ptr(), xs.data_ptr(), M, K, 128, s)
        ffi.k(entry, q.data_ptr(), Wd.data_ptr(), xs.data_ptr(), wsd.data_ptr(), bd.data_ptr(), D.data_ptr(), M, N, K, ffi.DT_BF16, s)

    call()                       # sets the kernels' LDS limits and, for the static entry point, finds its array
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(3):
        xb = synth.bf16_bits(synth.activations(30 + rep, M, K, "t3"))
        x.copy_(dev_bits(xb, BF16))
        D.zero_()
        graph.replay()
        torch.cuda.synchronize()
        rc, want, _ = oracle.linear_w8a8(BF16, xb, 128, W, ws, bias, BF16, threads=8)
        assert rc == 0
        assert np.array_equal(host_bits(D), want.view(np.uint16)), "replay %d" % rep
        _ = (torch.randn(1024, device="cuda") * 2).sum().item()   # eager work between the replays


# ------------------------------------------------------------------------- W6A8, packed words + fp32 group scales
W6G_CASES = [  # (M, N, K, out_dt, with_bias)
    (256, 128, 128, BF16, True), (100, 200, 256, BF16, False), (300, 136, 640, F32, True), (513, 260, 384, F16, True),
    (1, 8, 128, BF16, True), (777, 1000, 1280, BF16, True),
    (2200, 4000, 256, BF16, True),     # 288 tiles: workgroups walk more than one tile, two groups each
    (1500, 5300, 128, F16, False),     # 252 tiles of one group: the DMA stream is always a tile ahead
    (2304, 4224, 384, F32, True),      # 297 tiles, whole tiles only
]


@pytest.mark.parametrize("mode", [0, 1, -1])
@pytest.mark.parametrize("M,N,K,out_dt,with_bias", W6G_CASES)
def test_w6a8_group_gemm_matches_oracle(M, N, K, out_dt, with_bias, mode):
    """Both forms of the kernel (weights expanded inside it, mode 0; expanded once beforehand, mode 1; the library's own
    choice by M, -1) against the oracle: every int32 group partial and every output bit."""
    say("w6a8_group", M, N, K, out_dt, with_bias, "mode", mode)
    ffi.raw("gpu_internal_w6a8_group_gemm_mode", mode)
    try:
        _w6a8_group_case(M, N, K, out_dt, with_bias)
    finally:
        ffi.raw("gpu_internal_w6a8_group_gemm_mode", -1)


def _w6a8_group_case(M, N, K, out_dt, with_bias):
    A = rand_i8(9, 1, M, K, -127, 127)
    A[0, :] = -128
    qv = synth.w6_codes(9, N, K)
    qv[0, :] = -32                                           # extreme partial: 128 * 128 * 32
    qv[N - 1, :] = 31
    packed = oracle.w6_pack_words(qv)
    xs = synth.uniform(9, 3, M, 0.005, 0.2)
    sw = synth.w6_group_scales(9, N, K)
    tob = {BF16: oracle.bf16_bits, F16: oracle.f16_bits, F32: lambda a: a.astype(np.float32)}[out_dt]
    bias = tob(synth.normal(9, 5, N) * np.float32(0.02)) if with_bias else None
    rc, want, want_part = oracle.w6a8_group_gemm(A, packed, xs, sw, bias, out_dt, want_partials=True)
    assert rc == 0
    bd = None if bias is None else dev_bits(bias, out_dt)
    got, part = ql.w6a8_group_gemm(dev(A), dev(packed), dev(xs), dev(sw), bd, TDT[out_dt], want_partials=True)
    got2 = ql.w6a8_group_gemm(dev(A), dev(packed), dev(xs), dev(sw), bd, TDT[out_dt])
    torch.cuda.synchronize()
    assert np.array_equal(part.cpu().numpy(), want_part)
    view = np.uint32 if out_dt == F32 else np.uint16
    assert np.array_equal(host_bits(got).view(view), want.view(view))
    assert np.array_equal(host_bits(got2).view(view), want.view(view))


def test_w6a8_group_gemm_argument_checks():
    assert ffi.raw("gpu_w6a8_group_gemm", 0, 0, 0, 0, 0, 0, 0, 4, 8, 64, 2, 0) == -1      # K % 128
    assert ffi.raw("gpu_w6a8_group_gemm", 0, 0, 0, 0, 0, 0, 0, 4, 8, 128, 7, 0) == -200   # out_dt
    assert ffi.raw("gpu_w6a8_group_gemm", 0, 0, 0, 0, 0, 0, 0, 0, 8, 128, 2, 0) == 0      # empty


# ------------------------------------------------------------------------------------------------ full-size shapes
FULL = [  # (name, M, K, N, rotate, kind)
    ("dit mlp up", 4608, 3072, 12288, 128, "t3"),
    ("dit mlp down", 4608, 12288, 3072, 1, "t3"),
    ("dit mlp down, block 128", 4608, 12288, 3072, 128, "t3"),
    ("skinny gate+up", 256, 4096, 24576, 128, "normal"),
    ("skinny down", 256, 12288, 4096, 1, "normal"),
    ("skinny down, block 128", 256, 12288, 4096, 128, "normal"),
    ("sdxl geglu", 8192, 640, 5120, 0, "normal"),
    ("dit qkv", 4608, 3072, 9216, 128, "t3"),
    ("dit out-proj", 4608, 3072, 3072, 128, "t3"),
    ("sdxl attn proj", 8192, 640, 640, 0, "normal"),
    ("sdxl down", 8192, 2560, 640, 0, "normal"),
]


@pytest.mark.parametrize("name,M,K,N,rotate,kind", FULL)
def test_full_size_linear_rows_against_oracle(name, M, K, N, rotate, kind):
    """At the benchmark sizes the oracle is too slow for the whole output: check the quantizer on every row, the GEMM on
    a spread of rows (bit-exact), and a checksum identity over the whole int32 result: sum_n acc[m,n] = A[m,:] . sum_n W[n,:]."""
    say("full size", name, M, K, N, rotate)
    xb = synth.bf16_bits(synth.activations(7, M, K, kind, synth.outlier_columns(7, K, 0.001)))
    W, ws, bias32 = synth.w8_weights(7, N, K)
    bias = synth.bf16_bits(bias32)
    rc, q, xs = oracle.quant_rows(BF16, xb, K, rotate)
    assert rc == 0
    x = dev_bits(xb, BF16)
    Wd, wsd, bd = dev(W), dev(ws), dev_bits(bias, BF16)
    qd, xsd = ql.quant_rows(x, rotate)
    d = ql.int8_gemm(qd, Wd, xsd, wsd, bd, torch.bfloat16)
    acc = ql.int8_gemm_acc(qd, Wd)
    torch.cuda.synchronize()
    assert np.array_equal(qd.cpu().numpy(), q) and np.array_equal(xsd.cpu().numpy(), xs)
    rows = sorted(set([0, 1, 31, 32, 127, 128, 255, M // 2, M - 129, M - 2, M - 1] + list(range(5, M, 256))))   # every tile row
    want = oracle.int8_gemm(q[rows], W, xs[rows], ws, bias, BF16, fma=1)
    got = host_bits(d[torch.tensor(rows, device=DEV)])
    assert np.array_equal(got, want)
    colsum = W.astype(np.int64).sum(axis=0)
    want_rowsum = q.astype(np.int64) @ colsum
    got_rowsum = acc.to(torch.int64).sum(dim=1).cpu().numpy()
    assert np.array_equal(got_rowsum, want_rowsum)
    # every kernel family that can run the shape gives the same bits
    for cfg in (1, 7, 9) if M > 256 and M * N < 8192 * 5120 else (1,) if M > 256 else (6, 1):
        ffi.raw("gpu_int8_gemm_force_config", cfg)
        try:
            d2 = ql.int8_gemm(qd, Wd, xsd, wsd, bd, torch.bfloat16)
            torch.cuda.synchronize()
        finally:
            ffi.raw("gpu_int8_gemm_force_config", -1)
        assert torch.equal(d2.view(torch.int16), d.view(torch.int16)), cfg


SD_FULL = [("sdxl attn proj", 8192, 640, 640, 64), ("sdxl geglu", 8192, 640, 5120, 64), ("sdxl down", 8192, 2560, 640, 256)]


@pytest.mark.parametrize("name,M,K,N,rotate", SD_FULL)
def test_full_size_sd_linear_rows_against_oracle(name, M, K, N, rotate):
    """The SD UNet reading of the SDXL-level shapes (src/unet.rs:367-456): fp16 activations through gpu_sd_quant_rows with
    the widest rotation that divides K, fp16 bias and output.  Quantizer on every row, GEMM on a spread of rows,
    checksum identity over the whole int32 result."""
    say("full size sd", name, M, K, N, rotate)
    xh = oracle.f16_bits(synth.activations(17, M, K, "normal", synth.outlier_columns(17, K, 0.001)))
    W, ws, bias32 = synth.w8_weights(17, N, K)
    bias = oracle.f16_bits(bias32)
    rc, q, xs = oracle.sd_quant_rows(xh, K, rotate)
    assert rc == 0
    qd, xsd = ql.sd_quant_rows(dev_bits(xh, F16), rotate)
    Wd = dev(W)
    d = ql.int8_gemm(qd, Wd, xsd, dev(ws), dev_bits(bias, F16), torch.float16)
    acc = ql.int8_gemm_acc(qd, Wd)
    torch.cuda.synchronize()
    assert np.array_equal(qd.cpu().numpy(), q) and np.array_equal(xsd.cpu().numpy(), xs)
    rows = sorted(set([0, 1, 127, 128, 255, M // 2, M - 2, M - 1] + list(range(5, M, 256))))
    want = oracle.int8_gemm(q[rows], W, xs[rows], ws, bias, F16, fma=1)
    assert np.array_equal(host_bits(d[torch.tensor(rows, device=DEV)]), want.view(np.uint16))
    want_rowsum = q.astype(np.int64) @ W.astype(np.int64).sum(axis=0)
    assert np.array_equal(acc.to(torch.int64).sum(dim=1).cpu().numpy(), want_rowsum)


W6G_FULL = [("video-dit ffn up", 8192, 5120, 13824), ("video-dit ffn down", 8192, 13824, 5120)]


@pytest.mark.parametrize("name,M,K,N", W6G_FULL)
def test_full_size_w6a8_group_gemm(name, M, K, N):
    """The fused-unpack W6A8 kernel at the video-DiT sizes (40 and 108 scale groups, 3456 and 1280 tiles): a spread of
    rows (one per tile row and the edges) bit-exact against the oracle; every int32 group partial of a 160-row band
    bit-exact and equal, summed over n, to A[m, group] . sum_n codes[n, group]; outputs of that band equal the full run's."""
    say("full size w6a8", name, M, K, N)
    g = torch.Generator().manual_seed(K)
    A = torch.randint(-127, 128, (M, K), dtype=torch.int8, generator=g).numpy()
    A[0, :] = -128
    qv = synth.w6_codes(21, N, K)
    qv[0, :] = -32
    packed = oracle.w6_pack_words(qv)
    xs = synth.uniform(21, 3, M, 0.005, 0.2)
    sw = synth.w6_group_scales(21, N, K)
    bias = oracle.bf16_bits(synth.normal(21, 5, N) * np.float32(0.02))
    Ad, pd, xsd, swd, bd = dev(A), dev(packed), dev(xs), dev(sw), dev_bits(bias, BF16)
    got = ql.w6a8_group_gemm(Ad, pd, xsd, swd, bd, torch.bfloat16)
    torch.cuda.synchronize()
    rows = sorted(set([0, 1, 255, 256, M // 2, M - 1] + list(range(7, M, 256))))
    rc, want, _ = oracle.w6a8_group_gemm(A[rows], packed, xs[rows], sw, bias, BF16)
    assert rc == 0
    assert np.array_equal(host_bits(got[torch.tensor(rows, device=DEV)]), want.view(np.uint16))
    # both forms of the kernel at this size: 0 unpacks inside the GEMM in every workgroup, 1 expands the weights once first
    # (what the call picks by itself from 4096 rows on)
    for mode in (0, 1):
        ffi.raw("gpu_internal_w6a8_group_gemm_mode", mode)
        try:
            forced = ql.w6a8_group_gemm(Ad, pd, xsd, swd, bd, torch.bfloat16)
            torch.cuda.synchronize()
        finally:
            ffi.raw("gpu_internal_w6a8_group_gemm_mode", -1)
        assert torch.equal(forced.view(torch.int16), got.view(torch.int16)), mode
        assert np.array_equal(host_bits(forced[torch.tensor(rows, device=DEV)]), want.view(np.uint16)), mode
    # a band of rows that straddles a tile boundary, with the partials dumped
    r0, nr = 3 * 256 - 80, 160
    band, part = ql.w6a8_group_gemm(Ad[r0:r0 + nr].contiguous(), pd, xsd[r0:r0 + nr].contiguous(), swd, bd, torch.bfloat16, want_partials=True)
    torch.cuda.synchronize()
    assert torch.equal(band.view(torch.int16), got[r0:r0 + nr].view(torch.int16))
    part = part.cpu().numpy().astype(np.int64).reshape(nr, N, K // 128)
    colsum = qv.astype(np.int64).reshape(N, K // 128, 128).sum(axis=0)             # [group, 128]
    want_sum = np.einsum("mgk,gk->mg", A[r0:r0 + nr].astype(np.int64).reshape(nr, K // 128, 128), colsum)
    assert np.array_equal(part.sum(axis=1), want_sum)
    rc, _, want_part = oracle.w6a8_group_gemm(A[r0:r0 + 4], packed, xs[r0:r0 + 4], sw, bias, BF16, want_partials=True)
    assert np.array_equal(part[:4].reshape(want_part.shape), want_part)


# ------------------------------------------------------------------------------------------------ random shapes
def _bits_of(x, dt):
    return x.astype(np.float32) if dt == F32 else (oracle.bf16_bits(x) if dt == BF16 else oracle.f16_bits(x))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_int8_gemm_random_shapes_bit_exact(seed):
    """Forty shapes per seed drawn over the ranges that select every kernel family and every alignment class (skinny,
    split K, K % 16 == 8, odd N, tails of every tile size), all three entry points, all output types."""
    rng = np.random.default_rng(seed)
    for it in range(40):
        kind = int(rng.integers(0, 6))
        if kind == 0:   M, N, K = int(rng.integers(1, 257)), int(rng.integers(1, 700)) * 8, int(rng.integers(1, 40)) * 128
        elif kind == 1: M, N, K = int(rng.integers(257, 3000)), int(rng.integers(64, 500)) * 8, int(rng.integers(1, 12)) * 128
        elif kind == 2: M, N, K = int(rng.integers(1, 1200)), int(rng.integers(1, 1500)), int(rng.integers(1, 80)) * 8
        elif kind == 3: M, N, K = int(rng.integers(1500, 5200)), int(rng.integers(64, 640)) * 8, int(rng.integers(1, 5)) * 128
        elif kind == 4: M, N, K = int(rng.integers(1, 600)), int(rng.integers(1, 300)) * 4, int(rng.integers(1, 60)) * 16
        else:           M, N, K = int(rng.integers(200, 2600)), int(rng.integers(512, 3000)), int(rng.integers(2, 20)) * 64
        while M * N * K > 2e9:
            M = max(1, M // 2)
        dt = [BF16, F16, F32][int(rng.integers(0, 3))]
        with_bias = bool(rng.integers(0, 4))
        say("gemm_random", seed, it, M, N, K, dt, with_bias)
        A = rng.integers(-128, 128, (M, K), dtype=np.int8)
        W = rng.integers(-128, 128, (N, K), dtype=np.int8)
        xs = rng.uniform(0.005, 0.2, M).astype(np.float32)
        ws = rng.uniform(1e-3, 1e-2, N).astype(np.float32)
        bias = _bits_of(rng.normal(size=N).astype(np.float32) * np.float32(0.02), dt) if with_bias else None
        rscale = _bits_of(rng.normal(size=N).astype(np.float32), dt)
        resid = _bits_of(rng.normal(size=(M, N)).astype(np.float32), dt)
        want = oracle.int8_gemm_acc(A, W)
        Ad, Wd = dev(A), dev(W)
        bd = dev_bits(bias, dt) if with_bias else None
        got = ql.int8_gemm_acc(Ad, Wd)
        d = ql.int8_gemm(Ad, Wd, dev(xs), dev(ws), bd, TDT[dt])
        r = ql.int8_gemm_residual(Ad, Wd, dev(xs), dev(ws), bd, dev_bits(rscale, dt), dev_bits(resid, dt))
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy(), want), (M, N, K)
        assert np.array_equal(host_bits(d), oracle.epilogue(want, xs, ws, bias, dt, fma=1)), (M, N, K, dt)
        assert np.array_equal(host_bits(r), oracle.epilogue_residual(want, xs, ws, bias, rscale, resid, dt, fma=1)), (M, N, K, dt)


@pytest.mark.parametrize("seed", [21, 22])
def test_quant_rows_random_shapes_and_data_bit_exact(seed):
    """150 draws per seed over dtype (bf16, f32, the SD fp16 quantizer), row length up to 32768, every rotation width, row
    strides wider than K, and data that is Gaussian, heavy-tailed, scaled by 1e-30 .. 1e30, mostly zero, or carries an
    infinity, a NaN, 3e38 or 1e-38."""
    rng = np.random.default_rng(seed)

    def data(M, width):
        k = int(rng.integers(0, 5))
        if k == 0:
            x = rng.normal(size=(M, width)).astype(np.float32)
        elif k == 1:
            x = (rng.standard_t(3, size=(M, width)) * 4).astype(np.float32)
        elif k == 2:
            x = (rng.normal(size=(M, width)) * 10.0 ** int(rng.integers(-30, 30))).astype(np.float32)
        elif k == 3:
            x = rng.normal(size=(M, width)).astype(np.float32)
            x[rng.random((M, width)) < 0.7] = 0
        else:
            x = rng.normal(size=(M, width)).astype(np.float32)
            x[int(rng.integers(0, M)), int(rng.integers(0, width))] = [np.inf, -np.inf, np.nan, 3e38, 1e-38][int(rng.integers(0, 5))]
        if M > 1 and rng.random() < 0.3:
            x[int(rng.integers(0, M))] = 0
        return x

    for it in range(150):
        which = int(rng.integers(0, 3))
        rotate = int([0, 1, 64, 128, 256][int(rng.integers(0, 5))])
        if which == 2:   # gpu_sd_quant_rows takes 0, 64 or 256
            rotate = {128: 64, 1: 256}.get(rotate, rotate)
        gran = 256 if rotate in (1, 256) else 128 if rotate == 128 else 64
        K = int(rng.integers(1, 32768 // gran + 1)) * gran
        if rng.random() < 0.7:
            K = int(rng.integers(1, max(2, 6144 // gran))) * gran
        M = int(rng.integers(1, 70))
        stride = K if (which == 2 or rng.random() < 0.6) else K + 8 * int(rng.integers(1, 40))
        say("quant_random", seed, it, which, M, K, stride, rotate)
        x = data(M, stride)
        if which == 0:
            xb = oracle.bf16_bits(x)
            rc, q, s = oracle.quant_rows(BF16, xb, K, rotate, x_stride=stride)
            qd, sd = ql.quant_rows(dev_bits(xb, BF16), rotate, K=K)
        elif which == 1:
            rc, q, s = oracle.quant_rows(F32, x, K, rotate, x_stride=stride)
            qd, sd = ql.quant_rows(dev(x), rotate, K=K)
        else:
            xb = oracle.f16_bits(np.clip(x, -6e4, 6e4))
            rc, q, s = oracle.sd_quant_rows(xb, K, rotate)
            qd, sd = ql.sd_quant_rows(dev_bits(xb, F16), rotate)
        torch.cuda.synchronize()
        assert rc == 0
        assert np.array_equal(sd.cpu().numpy().view(np.uint32), s.view(np.uint32)), (which, M, K, stride, rotate)
        assert np.array_equal(qd.cpu().numpy(), q), (which, M, K, stride, rotate)
