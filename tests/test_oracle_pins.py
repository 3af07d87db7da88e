"""Pins for the CPU oracle: every function is checked against something that does not share its code --
library casts and arithmetic (torch bf16/f16/float8 tensors, numpy int64 matmul), closed forms (the Kronecker
Hadamard matrix), exact rational arithmetic, and hand-worked special cases."""
from fractions import Fraction

import numpy as np
import pytest
import torch

import oracle
from oracle import BF16, F16, F32

H4 = np.array([[1, 1, 1, -1], [1, 1, -1, 1], [1, -1, 1, 1], [-1, 1, 1, 1]], dtype=np.float64)


def kron_h(n):
    h = np.ones((1, 1))
    for _ in range(n):
        h = np.kron(h, H4)
    return h / (2.0 ** n)


def rand_bits(seed, n):
    return np.random.default_rng(seed).integers(0, 2 ** 32, size=n, dtype=np.uint32)


# ----------------------------------------------------------------------------------------------- rounding helpers
def test_bf16_round_matches_torch_cast():
    bits = np.concatenate([rand_bits(1, 400000),
                           np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x7f7fffff, 0x3f808000, 0x3f818000,
                                     0x3f807fff, 0x3f808001, 0x00000001, 0x00008000, 0x7f7f8000], np.uint32)])
    f = bits.view(np.float32)
    keep = ~np.isnan(f)
    f = f[keep]
    want = torch.from_numpy(f.copy()).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = oracle.bf16_bits(f)
    assert np.array_equal(got, want)
    L = oracle.lib()
    for v in f[:2000]:
        assert L.orc_f32_to_bf16(float(v)) == int(oracle.bf16_bits(np.array([v]))[0])
    assert np.isnan(oracle.bf16_to_f32(np.array([L.orc_f32_to_bf16(float("nan"))], np.uint16))[0])


def test_f16_round_matches_numpy_cast():
    L = oracle.lib()
    rng = np.random.default_rng(2)
    vals = np.concatenate([
        rand_bits(3, 20000).view(np.float32),
        rng.normal(0, 1, 20000).astype(np.float32),
        (rng.normal(0, 1, 5000) * 1e-6).astype(np.float32),      # half subnormal range
        (rng.normal(0, 1, 5000) * 6e4).astype(np.float32),        # near half max
        np.array([65504, 65519.99, 65520, 65536, 5.96e-8, 2.98e-8, 2.9802322e-8, 2.9802326e-8, 6.1e-5, 0, -0.0,
                  float("inf"), -float("inf"), 1.00048828125, 1.0009765625, 1.00146484375], np.float32)])
    vals = vals[~np.isnan(vals)]
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.orc_f32_to_f16(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, want)
    allh = np.arange(65536, dtype=np.uint16)
    back = np.array([L.orc_f16_to_f32(int(h)) for h in allh], np.float32)
    ref = allh.view(np.float16).astype(np.float32)
    ok = np.isnan(ref) | (back.view(np.uint32) == ref.view(np.uint32))
    assert ok.all()


# ----------------------------------------------------------------------------------------------- Hadamard
@pytest.mark.parametrize("g,n", [(64, 3), (256, 4)])
def test_fht_equals_kronecker_matrix(g, n):
    H = kron_h(n)
    assert np.array_equal(H, H.T)
    assert np.allclose(H @ H, np.eye(g))
    rng = np.random.default_rng(g)
    # small integers: every partial sum is exactly representable, so any association order gives the same bits
    x = rng.integers(-8, 9, size=(3, 2 * g)).astype(np.float32)
    y = oracle.fht(x.reshape(-1), g).reshape(3, 2, g)
    want = np.einsum("ij,rbj->rbi", H, x.reshape(3, 2, g).astype(np.float64))
    assert np.array_equal(y.astype(np.float64), want)
    # basis vectors give the columns of H exactly (entries are +-2^-n)
    for j in (0, 1, 5, g // 2 + 3, g - 1):
        e = np.zeros(g, np.float32)
        e[j] = 1
        assert np.array_equal(oracle.fht(e, g).astype(np.float64), H[:, j])
    # general floats: close to the float64 product, and the transform is its own inverse up to rounding
    xf = rng.normal(0, 1, size=g).astype(np.float32)
    yf = oracle.fht(xf, g)
    assert np.allclose(yf, H @ xf.astype(np.float64), rtol=0, atol=1e-5)
    assert np.allclose(oracle.fht(yf, g), xf, atol=1e-5)
    assert abs(np.linalg.norm(yf) - np.linalg.norm(xf)) < 1e-4


def test_fht_association_order_is_left_to_right():
    # One stage-0 butterfly with inputs chosen so that the order of the float adds changes the result:
    # x0 + x1 rounds 2^24 + 1 back to 2^24 (tie to even), then + x2 cancels, then -/+ x3.
    x0, x1, x2, x3 = np.float32(2 ** 24), np.float32(1), np.float32(-2 ** 24), np.float32(1)
    r = [((x0 + x1) + x2) - x3, ((x0 + x1) - x2) + x3, ((x0 - x1) + x2) + x3, ((-x0 + x1) + x2) + x3]
    # worked by hand: row 0 is ((2^24+1 -> 2^24) - 2^24) - 1 = -1, where pairing (x0+x2)+(x1-x3) would give 0
    assert [float(v) for v in r] == [-1.0, 33554432.0, 0.0, -33554432.0]
    for g, n in ((64, 3), (256, 4)):
        x = np.zeros(g, np.float32)
        x[:4] = [x0, x1, x2, x3]
        y = oracle.fht(x, g)
        # later stages see (v,0,0,0) butterflies: outputs 0.5*(v, v, v, -v), all exact
        Hrest = kron_h(n - 1)[:, 0] * (2.0 ** (n - 1))              # signs of the first column of the remaining factor
        want = np.concatenate([0.5 * np.array(r, np.float64) * s for s in Hrest]) / (2.0 ** (n - 1))
        assert np.array_equal(y.astype(np.float64), want)


def test_fht128_is_orthonormal_h2_kron_h64():
    H2 = np.array([[1, 1], [1, -1]], np.float64) / np.sqrt(2.0)
    H = np.kron(H2, kron_h(3))
    assert np.allclose(H @ H.T, np.eye(128))
    rng = np.random.default_rng(5)
    x = rng.normal(0, 1, 256).astype(np.float32)
    y = oracle.fht(x, 128)
    want = np.concatenate([H @ x[:128].astype(np.float64), H @ x[128:].astype(np.float64)])
    assert np.allclose(y, want, atol=2e-6)
    assert np.allclose(oracle.fht(y, 128), x, atol=2e-6)


# ----------------------------------------------------------------------------------------------- quantizer
def torch_quant_bf16(xbits):
    """The quantizer as PyTorch tensor arithmetic in bf16 (what the reference says it emulates, csrc/kernels.cu:3-4)."""
    x = torch.from_numpy(xbits.view(np.int16).copy()).view(torch.bfloat16)
    amax = x.float().abs().amax(dim=1)
    scale = torch.clamp(torch.clamp(amax, max=3.38953139e38) * torch.tensor(1.0 / 127.0, dtype=torch.float32), min=1e-30)
    st = scale.to(torch.bfloat16)
    q = torch.clamp(torch.round(x / st[:, None]), -128, 127).to(torch.int8)
    return q.numpy(), scale.numpy()


def test_quant_rows_plain_matches_torch_bf16(synth):
    x = synth.bf16_bits(synth.activations(3, 64, 1024, "normal", (3, 700)))
    rc, q, s = oracle.quant_rows(BF16, x, 1024, 0)
    assert rc == 0
    qt, st = torch_quant_bf16(x)
    assert np.array_equal(s.view(np.uint32), st.view(np.uint32))
    assert np.array_equal(q, qt)
    assert q.max() == 127 and q.min() <= -120


@pytest.mark.parametrize("g", [64, 128, 256])
def test_quant_rows_rotated_matches_torch_on_rotated_rows(synth, g):
    K = 512
    xb = synth.bf16_bits(synth.activations(4, 16, K, "t3"))
    rc, q, s = oracle.quant_rows(BF16, xb, K, g)
    assert rc == 0
    rot = np.stack([oracle.fht(r, g) for r in synth.bf16_to_f32(xb)])
    # scale comes from the unrounded rotated row, codes from its bf16 rounding (csrc/kernels.cu:224,241,254)
    amax = np.abs(rot).max(axis=1).astype(np.float32)
    scale = np.maximum(amax * np.float32(1.0 / 127.0), np.float32(1e-30)).astype(np.float32)
    assert np.array_equal(s, scale)
    xr = torch.from_numpy(rot).to(torch.bfloat16)
    stt = torch.from_numpy(scale).to(torch.bfloat16)
    qt = torch.clamp(torch.round(xr / stt[:, None]), -128, 127).to(torch.int8).numpy()
    assert np.array_equal(q, qt)


def test_quant_rows_f32_is_true_division(synth):
    x = synth.activations(5, 8, 256, "normal")
    rc, q, s = oracle.quant_rows(F32, x, 256, 0)
    assert rc == 0
    amax = np.abs(x).max(axis=1)
    scale = amax * np.float32(1.0 / 127.0)
    assert np.array_equal(s, scale)
    qt = np.clip(np.rint(x / scale[:, None]), -128, 127).astype(np.int8)     # numpy float32 divide is IEEE
    assert np.array_equal(q, qt)


def test_quant_rows_special_rows():
    K = 256
    rows = np.zeros((6, K), np.float32)
    rows[1, 7] = 20.0; rows[1, 9] = -20.0; rows[1, 11] = 10.0            # single outlier pair -> +-127, half -> 64 (tie even)
    rows[2, 0] = np.inf; rows[2, 1] = -np.inf; rows[2, 2] = 1.0            # inf: amax clamps to the bf16 maximum
    rows[3, 0] = np.nan; rows[3, 1] = 2.0; rows[3, 2] = -1.0               # NaN is dropped from amax and encodes as -128
    rows[4, :] = 1e-35                                                     # below the scale floor
    rc, q, s = oracle.quant_rows(BF16, oracle.bf16_bits(rows), K, 0)
    assert rc == 0
    assert s[0] == np.float32(1e-30) and not q[0].any()                    # zero row: max(0*(1/127), 1e-30)
    assert q[1, 7] == 127 and q[1, 9] == -127 and q[1, 11] in (63, 64) and s[1] == np.float32(20.0) * np.float32(1 / 127)
    assert s[2] == np.float32(3.38953139e38) * np.float32(1 / 127)
    assert q[2, 0] == 127 and q[2, 1] == -128 and q[2, 2] == 0
    assert s[3] == np.float32(2.0) * np.float32(1 / 127) and q[3, 0] == -128 and q[3, 1] == 127
    assert s[4] == np.float32(1e-30) and (q[4] == 0).all()
    # finite but NaN-free rows agree with torch as well
    qt, st = torch_quant_bf16(oracle.bf16_bits(rows[[0, 1, 4]]))
    assert np.array_equal(q[[0, 1, 4]], qt)


def test_quant_rows_minus_128_is_reachable():
    # amax = A*2^e with an 8-bit significand; when bf16(scale) rounds down far enough, A/bf16(scale) rounds to 127.5
    # in bf16 and rint(127.5) = 128 clamps to 127 while rint(-127.5) = -128 is kept.
    found = 0
    for A in range(128, 256):
        a = np.float32(A)
        scale = a * np.float32(1.0 / 127.0)
        st = oracle.bf16_to_f32(oracle.bf16_bits(np.array([scale])))[0]
        t = oracle.bf16_to_f32(oracle.bf16_bits(np.array([a / st], np.float32)))[0]
        row = np.zeros((1, 256), np.float32)
        row[0, 0] = a; row[0, 1] = -a
        rc, q, s = oracle.quant_rows(BF16, oracle.bf16_bits(row), 256, 0)
        if t == np.float32(127.5):
            found += 1
            assert q[0, 0] == 127 and q[0, 1] == -128
        else:
            assert t in (np.float32(127.0), np.float32(126.5), np.float32(126.0)) and q[0, 0] == -q[0, 1]
    assert found > 0


def test_quant_rows_argument_codes():
    x = np.zeros((2, 512), np.uint16)
    assert oracle.quant_rows(BF16, x, 200, 0)[0] == -1          # K not a multiple of 64
    assert oracle.quant_rows(BF16, x, 320, 1)[0] == -1          # 256-wide rotation needs K % 256 == 0
    assert oracle.quant_rows(F16, x, 256, 0)[0] == -4           # dtype must be bf16 or f32 (csrc/kernels.cu:294-297)
    big = np.zeros((1, 32768 + 256), np.uint16)
    assert oracle.quant_rows(BF16, big, 32768 + 256, 0)[0] == -2
    assert oracle.quant_rows(BF16, big, 32768, 1)[0] == 0


def test_quant_rows_stride(synth):
    x = synth.bf16_bits(synth.activations(6, 4, 768, "normal"))
    rc, q, s = oracle.quant_rows(BF16, x, 256, 1, x_stride=768)
    rc2, q2, s2 = oracle.quant_rows(BF16, np.ascontiguousarray(x[:, :256]), 256, 1)
    assert rc == rc2 == 0 and np.array_equal(q, q2) and np.array_equal(s, s2)


def test_rotate_rows_f32(synth):
    x = synth.activations(7, 3, 512, "normal")
    rc, out = oracle.rotate_rows_f32(x, 512)
    assert rc == 0
    H = kron_h(4)
    want = np.einsum("ij,rbj->rbi", H, x.reshape(3, 2, 256).astype(np.float64)).reshape(3, 512)
    assert np.allclose(out, want, atol=1e-5)
    assert oracle.rotate_rows_f32(x, 320)[0] == -1


def torch_sd_quant(xbits, rot_rows=None):
    x = torch.from_numpy(xbits.view(np.int16).copy()).view(torch.float16)
    if rot_rows is not None:
        x = torch.from_numpy(rot_rows).to(torch.float16)
    mx = x.float().abs().amax(dim=1)
    scale = torch.clamp(mx, min=1e-30) / torch.tensor(127.0)
    sh = scale.to(torch.float16)
    q = torch.where(sh[:, None].float() > 0, (x / sh[:, None]).float(), (x.float() / scale[:, None]).to(torch.float16).float())
    q = torch.clamp(torch.round(q), -128, 127).to(torch.int8)
    return q.numpy(), scale.numpy()


@pytest.mark.parametrize("rotate", [0, 64, 256])
def test_sd_quant_rows_matches_torch_f16(synth, rotate):
    K = 768 if rotate != 256 else 512
    xb = synth.f16_bits(synth.activations(8, 24, K, "normal", (5,)))
    xb[3, :] = 0                                                  # zero row: scale 1e-30/127, divides in float
    rc, q, s = oracle.sd_quant_rows(xb, K, rotate)
    assert rc == 0
    rot = None
    if rotate:
        rot = np.stack([oracle.fht(r, rotate) for r in oracle.f16_to_f32(xb)])
    qt, st = torch_sd_quant(xb, rot)
    assert np.array_equal(s.view(np.uint32), st.view(np.uint32))
    assert np.array_equal(q, qt)
    assert s[3] == np.float32(1e-30) / np.float32(127.0) and not q[3].any()
    assert oracle.sd_quant_rows(xb, K, 128)[0] == -1
    assert oracle.sd_quant_rows(xb, 640, 256)[0] == -1


# ----------------------------------------------------------------------------------------------- GEMM + epilogue
def test_int8_gemm_acc_exact(synth):
    A = synth.randint(1, 31, 37 * 192, -128, 127).astype(np.int8).reshape(37, 192)
    W = synth.randint(1, 32, 50 * 192, -128, 127).astype(np.int8).reshape(50, 192)
    acc = oracle.int8_gemm_acc(A, W)
    assert np.array_equal(acc.astype(np.int64), A.astype(np.int64) @ W.astype(np.int64).T)
    A2 = np.full((32, 256), -128, np.int8); W2 = np.full((16, 256), -128, np.int8)   # torch._int_mm needs M>16, K%8
    t = torch._int_mm(torch.from_numpy(A2), torch.from_numpy(W2).t().contiguous()).numpy()
    assert np.array_equal(oracle.int8_gemm_acc(A2, W2), t) and t[0, 0] == 256 * 128 * 128


def _round_to(x64_exact_fraction, out_dt):
    """Round an exact rational to float32 (RNE), then to the output type through library casts."""
    f = x64_exact_fraction
    # RNE to float32 from an exact Fraction: go through float64 only if exact, else use integer arithmetic
    if f == 0:
        return np.float32(0)
    sign = -1 if f < 0 else 1
    f = abs(f)
    e = 0
    while f >= 2: f /= 2; e += 1
    while f < 1: f *= 2; e -= 1
    m = f * (1 << 23)
    lo = m.numerator // m.denominator
    rem = m - lo
    if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and (lo & 1)):
        lo += 1
    return np.float32(sign * float(lo) * 2.0 ** (e - 23))


def test_epilogue_forms(synth):
    M, N = 9, 40
    acc = synth.randint(2, 41, M * N, -3000000, 3000000).astype(np.int32).reshape(M, N)
    xs = synth.uniform(2, 42, M, 0.01, 0.2)
    ws = synth.uniform(2, 43, N, 1e-3, 1e-2)
    bias32 = synth.normal(2, 44, N) * np.float32(0.02)
    for out_dt, tobits, tof in ((BF16, oracle.bf16_bits, oracle.bf16_to_f32), (F16, oracle.f16_bits, oracle.f16_to_f32),
                                (F32, lambda a: a.astype(np.float32), lambda a: a)):
        bias = tobits(bias32)
        bf = tof(bias).astype(np.float32)
        # separate multiply and add: numpy float32 arithmetic is IEEE and never fuses
        t = (acc.astype(np.float32) * xs[:, None]) * ws[None, :] + bf[None, :]
        assert np.array_equal(oracle.epilogue(acc, xs, ws, bias, out_dt, fma=0), tobits(t))
        t_nb = (acc.astype(np.float32) * xs[:, None]) * ws[None, :] + np.float32(0)
        assert np.array_equal(oracle.epilogue(acc, xs, ws, None, out_dt, fma=0), tobits(t_nb))
        # fused multiply-add: exact rational t0*ws + bias rounded once
        t0 = acc.astype(np.float32) * xs[:, None]
        want = np.array([[_round_to(Fraction(float(t0[m, n])) * Fraction(float(ws[n])) + Fraction(float(bf[n])), out_dt)
                          for n in range(N)] for m in range(M)], np.float32)
        got = oracle.epilogue(acc, xs, ws, bias, out_dt, fma=1)
        assert np.array_equal(got, tobits(want))
        # the two forms are within one unit in the last place of the output type
        a = tof(oracle.epilogue(acc, xs, ws, bias, out_dt, fma=0)).astype(np.float64)
        b = tof(got).astype(np.float64)
        ulp = {BF16: 2.0 ** -7, F16: 2.0 ** -10, F32: 2.0 ** -23}[out_dt]
        assert (np.abs(a - b) <= ulp * (np.maximum(np.abs(a), np.abs(b)) + np.abs(bf)[None, :]) + 1e-30).all()


def test_epilogue_residual(synth):
    M, N = 5, 24
    acc = synth.randint(3, 51, M * N, -2000000, 2000000).astype(np.int32).reshape(M, N)
    xs = synth.uniform(3, 52, M, 0.01, 0.2)
    ws = synth.uniform(3, 53, N, 1e-3, 1e-2)
    bias = oracle.bf16_bits(synth.normal(3, 54, N) * np.float32(0.02))
    rscale = oracle.bf16_bits(synth.normal(3, 55, N))
    resid = oracle.bf16_bits(synth.normal(3, 56, M * N).reshape(M, N))
    z = oracle.bf16_to_f32(oracle.epilogue(acc, xs, ws, bias, BF16, fma=0))     # first rounding, as the plain kernel
    want = oracle.bf16_bits(z * oracle.bf16_to_f32(rscale)[None, :] + oracle.bf16_to_f32(resid))
    assert np.array_equal(oracle.epilogue_residual(acc, xs, ws, bias, rscale, resid, BF16, fma=0), want)
    L = oracle.lib()
    D = np.zeros((M, N), np.uint16)
    A = np.zeros((M, 16), np.int8); W = np.zeros((N, 16), np.int8)
    vp = lambda a: a.ctypes.data
    assert L.orc_int8_gemm_residual(vp(A), vp(W), vp(xs), vp(ws), None, None, vp(resid), vp(D), M, N, 16, BF16, 1) == -201
    assert L.orc_int8_gemm_residual(vp(A), vp(W), vp(xs), vp(ws), None, vp(rscale), vp(resid), vp(D), M, N, 0, BF16, 1) == -201
    assert L.orc_int8_gemm_residual(vp(A), vp(W), vp(xs), vp(ws), None, vp(rscale), vp(resid), vp(D), 0, N, 16, BF16, 1) == 0
    assert L.orc_int8_gemm(vp(A), vp(W), vp(xs), vp(ws), None, vp(D), M, N, 0, BF16, 1) == 0
    assert L.orc_int8_gemm(vp(A), vp(W), vp(xs), vp(ws), None, vp(D), M, N, 16, 7, 1) == -200


# ----------------------------------------------------------------------------------------------- W6
def test_e4m3_table_matches_torch_float8():
    t = oracle.e4m3_table()
    ref = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    both_nan = np.isnan(t) & np.isnan(ref)
    assert ((t.view(np.uint32) == ref.view(np.uint32)) | both_nan).all()
    assert np.isnan(t[0x7f]) and np.isnan(t[0xff]) and t[0x7e] == 448.0 and t[0x01] == 2.0 ** -9 and t[0x38] == 1.0


def test_w6_plane_layout_known_answer():
    # K = 32: element e has its low nibble in byte e/2 (bits 4*(e&1)) and its top two bits in byte 16 + e/4 (bits 2*(e&3))
    K = 32
    row = np.zeros((1, 24), np.uint8)
    row[0, 0] = 0x21          # e0 nib 1, e1 nib 2
    row[0, 16] = 0b00_00_11_10  # e0 top 2, e1 top 3
    row[0, 15] = 0xF0         # e31 nib 15
    row[0, 23] = 0b01_00_00_00  # e31 top 1
    s = np.full((1, 1), 0x38, np.uint8)   # e4m3 1.0
    rc, out = oracle.w6_decode(row, s, 1, K, 32)
    assert rc == 0
    assert out[0, 0] == (1 | 2 << 4) - 32 and out[0, 1] == (2 | 3 << 4) - 32 and out[0, 31] == (15 | 1 << 4) - 32
    assert out[0, 2] == -32
    assert oracle.w6_decode(row, s, 1, 48, 32)[0] == -1 and oracle.w6_decode(row, s, 1, 32, 8)[0] == -1


def test_w6_decode_exhaustive_codes_times_scales():
    tbl = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    K, G = 64, 16
    codes = np.arange(64, dtype=np.uint8)[None, :].repeat(256 * 1, axis=0)          # row n uses scale byte n
    q = oracle.w6_pack_planes(codes)
    s_rel = np.arange(256, dtype=np.uint8)[:, None].repeat(K // G, axis=1)
    rc, out = oracle.w6_decode(q, s_rel, 256, K, G)
    assert rc == 0
    with np.errstate(invalid="ignore"):
        v = (codes.astype(np.float32) - np.float32(32)) * tbl[:, None]
        want = np.clip(np.rint(v), -127, 127)
    finite = ~np.isnan(want)
    assert np.array_equal(out[finite], want[finite].astype(np.int8))
    assert (out[~finite] == -127).all()      # NaN scale: fmaxf(-127, NaN) = -127 on the device


def test_w6_word_packing_roundtrip(synth):
    qv = synth.w6_codes(4, 7, 256)
    p = oracle.w6_pack_words(qv)
    assert p.shape == (7, 192)
    assert np.array_equal(oracle.w6_unpack_words(p, 256), qv)
    u = (qv[0, :4].astype(np.int32) + 32)
    w = int(u[0]) | int(u[1]) << 6 | int(u[2]) << 12 | int(u[3]) << 18
    assert [int(b) for b in p[0, :3]] == [w & 255, (w >> 8) & 255, (w >> 16) & 255]


def test_w6a8_group_gemm_partials_and_output(synth):
    M, N, K = 6, 10, 256
    A = synth.randint(5, 61, M * K, -127, 127).astype(np.int8).reshape(M, K)
    qv = synth.w6_codes(5, N, K)
    sw = synth.w6_group_scales(5, N, K)
    xs = synth.uniform(5, 62, M, 0.01, 0.1)
    bias = oracle.bf16_bits(synth.normal(5, 63, N) * np.float32(0.02))
    rc, D, part = oracle.w6a8_group_gemm(A, oracle.w6_pack_words(qv), xs, sw, bias, BF16, want_partials=True)
    assert rc == 0
    want_p = np.einsum("mgk,ngk->mng", A.reshape(M, 2, 128).astype(np.int64), qv.reshape(N, 2, 128).astype(np.int64))
    assert np.array_equal(part.astype(np.int64), want_p)
    ref = (want_p * sw[None].astype(np.float64)).sum(-1) * xs[:, None] + oracle.bf16_to_f32(bias)[None]
    got = oracle.bf16_to_f32(D).astype(np.float64)
    assert np.allclose(got, ref, rtol=2.0 ** -7, atol=1e-6)
