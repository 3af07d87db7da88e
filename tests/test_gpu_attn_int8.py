"""INT8 attention on the GPU against the CPU oracle (quantizer stages bit-exact, outputs within a stated tolerance) and
against exact softmax attention.

The quantizer stages are integer/rounding work and must match the oracle bit for bit.  The attention output is floating
point: the kernel's exp2 is the hardware instruction (1 ulp) where the oracle's is correctly rounded, so a u8
probability can land one step away when the exponent sits on a rounding boundary, and the denominators are summed in a
different order; the tolerance below is what one such step per row can move an output.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle
from conftest import pkg

pytestmark = pytest.mark.gpu


def _pkg():
    return pkg("qlinear"), pkg("ffi")


def _bits(t):
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def _to_f32(bits, dt):
    return oracle.bf16_to_f32(bits) if dt == oracle.BF16 else oracle.f16_to_f32(bits)


def _inputs(b, lq, lk, h, hk, dtype, seed, k_offset=0.0, v_scale=1.0, D=128):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(b, lq, h, D, generator=g)
    k = torch.randn(b, lk, hk, D, generator=g) + k_offset
    v = torch.randn(b, lk, hk, D, generator=g) * v_scale
    return q.to(dtype), k.to(dtype), v.to(dtype)


def _exact(q, k, v, scale):
    h, hk = q.shape[2], k.shape[2]
    qq = q.double().permute(0, 2, 1, 3)
    kk = k.double().permute(0, 2, 1, 3).repeat_interleave(h // hk, 1)
    vv = v.double().permute(0, 2, 1, 3).repeat_interleave(h // hk, 1)
    return (torch.softmax(qq @ kk.transpose(-1, -2) * scale, -1) @ vv).permute(0, 2, 1, 3).numpy()


def _row_mass(q, k, scale):
    """sum_k exp(logit_k - max logit) per (b, lq, h): the softmax denominator in units of the row's largest weight."""
    h, hk = q.shape[2], k.shape[2]
    qq = q.double().permute(0, 2, 1, 3)
    kk = k.double().permute(0, 2, 1, 3).repeat_interleave(h // hk, 1)
    s = qq @ kk.transpose(-1, -2) * scale
    return torch.exp(s - s.amax(-1, keepdim=True)).sum(-1).permute(0, 2, 1).numpy()


def _layout(ffi, b, h, hk, lq, lk):
    out = (C.c_int64 * 10)()
    assert ffi.raw("gpu_internal_attn_layout", b, h, hk, lq, lk, C.cast(out, C.c_void_p)) == 0
    return list(out)


CASES = [
    # b, lq, lk, h, hk, dtype, k_offset
    (1, 200, 300, 4, 2, torch.bfloat16, 0.0),
    (2, 77, 64, 2, 2, torch.bfloat16, 0.0),
    (1, 1, 1, 1, 1, torch.bfloat16, 0.0),
    (1, 129, 65, 2, 1, torch.float16, 0.0),
    (1, 257, 63, 3, 3, torch.bfloat16, 4.0),      # a K offset large enough for the anchor to switch on
    (1, 96, 1025, 2, 2, torch.bfloat16, 0.0),     # 128-key tiles with a ragged last tile of one key
    (1, 130, 1500, 4, 1, torch.float16, 2.0),
    (1, 33, 1152, 1, 1, torch.bfloat16, 0.0),     # 128-key tiles, no ragged tail
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: "b%d_lq%d_lk%d_h%d_hk%d_%s_off%g" % (c[0], c[1], c[2], c[3], c[4], str(c[5])[6:], c[6]))
def test_attention_against_oracle(case):
    ql, ffi = _pkg()
    b, lq, lk, h, hk, dtype, off = case
    dt = oracle.BF16 if dtype == torch.bfloat16 else oracle.F16
    q, k, v = _inputs(b, lq, lk, h, hk, dtype, seed=lq * 7 + lk, k_offset=off)
    scale = 128 ** -0.5
    ref_q = oracle.attn_quant(dt, _bits(q), _bits(k), _bits(v))
    ref = _to_f32(oracle.attn_int8(dt, _bits(q), _bits(k), _bits(v), scale, quant=ref_q), dt)

    ws_bytes = ffi.lib.gpu_int8_attn_workspace_d(b, h, hk, lq, lk, 128)
    ws = torch.zeros((ws_bytes,), dtype=torch.uint8, device="cuda")
    o = ql.int8_attn(q.cuda(), k.cuda(), v.cuda(), scale, ws=ws)
    torch.cuda.synchronize()
    w = ws.cpu().numpy()
    qi_o, ki_o, qs_o, ks_o, vt_o, vs_o, an_o, vsum_o, ck, kb = _layout(ffi, b, h, hk, lq, lk)
    assert ck == ref_q["ck"]

    def take(at, n, dtp):
        return w[at:at + n * np.dtype(dtp).itemsize].view(dtp)

    # quantizer stages: bit-exact
    assert np.array_equal(take(an_o, b * hk, np.int32).reshape(b, hk), ref_q["anchors"])
    if off >= 2.0:
        assert (ref_q["anchors"] >= 0).all(), "this case is meant to exercise the anchor"
    assert np.array_equal(take(qi_o, b * h * lq * 128, np.int8).reshape(b, h, lq, 128), ref_q["qi"])
    nblk = kb * (ck // 32)
    # K lies in fragment order: [32-key block][channel step of 32][half of 16 channels][key][16 bytes]
    ki = take(ki_o, b * hk * nblk * 32 * 128, np.int8).reshape(b, hk, nblk, 4, 2, 32, 16)
    ki = ki.transpose(0, 1, 2, 5, 3, 4, 6).reshape(b, hk, nblk * 32, 128)[:, :, :lk]
    assert np.array_equal(ki, ref_q["ki"])
    qs = take(qs_o, ref_q["qs"].size, np.float32).reshape(ref_q["qs"].shape)
    # groups with no row below lq are never read; compare the groups that own a row
    own = np.zeros(ref_q["qs"].shape[-1], bool)
    for r in range(lq):
        own[(r // 32) * 8 + r % 8] = True
    assert np.array_equal(qs[..., own].view(np.uint32), ref_q["qs"][..., own].view(np.uint32))
    assert np.array_equal(take(ks_o, ref_q["ks"].size, np.float32).view(np.uint32), ref_q["ks"].reshape(-1).view(np.uint32))
    assert np.array_equal(take(vs_o, b * hk * 128, np.float32).view(np.uint32), ref_q["vs"].reshape(-1).view(np.uint32))
    vt = take(vt_o, b * hk * nblk * 128 * 32, np.int8).reshape(b, hk, nblk, 128, 32)
    pos = np.arange(32)
    key_of_pos = ((pos % 16) // 4) * 8 + (pos // 16) * 4 + pos % 4
    vi_pad = np.zeros((b, hk, nblk * 32, 128), np.int8)
    vi_pad[:, :, :lk] = ref_q["vi"]
    want_vt = vi_pad.reshape(b, hk, nblk, 32, 128)[:, :, :, key_of_pos, :].transpose(0, 1, 2, 4, 3)
    assert np.array_equal(vt, want_vt)
    vsum = take(vsum_o, b * hk * kb * 128, np.int32).reshape(b, hk, kb, 128)
    want_sum = 128 * vi_pad.reshape(b, hk, kb, ck, 128).astype(np.int64).sum(3)
    assert np.array_equal(vsum, want_sum)

    # outputs
    got = _to_f32(_bits(o), dt)
    vmax = float(v.float().abs().max())
    ulp = 2.0 ** (-8 if dt == oracle.BF16 else -11)
    # What can differ from the oracle beyond output rounding is a probability that lands one u8 step away at a rounding
    # boundary (hardware exp2 against a correctly rounded one).  The row's largest probability is 255 and its
    # denominator 255 * mass, so one step of one key moves an output by at most max|v| / (255 * mass): room for four.
    mass = _row_mass(q, k, scale)[..., None]
    tol = 4 * vmax / (255.0 * mass) + 2 * ulp * np.abs(ref)
    err = np.abs(got - ref)
    assert (err <= tol).all(), "max excess %g" % float((err - tol).max())
    assert (err <= ulp * np.abs(ref) + 1e-30).mean() > 0.97, "more than 3 % of outputs differ from the oracle by over one ulp"

    # and the whole thing is attention: close to exact softmax attention of the same rounded inputs
    ex = _exact(q, k, v, scale)
    cos = float((got * ex).sum() / np.sqrt((got * got).sum() * (ex * ex).sum()))
    assert cos > 0.9995, cos


def test_attention_strided_views_match_contiguous():
    """q, k, v as slices of one packed [b, l, 3, h, 128] tensor and o written into a wider buffer."""
    ql, ffi = _pkg()
    b, l, h = 2, 150, 3
    g = torch.Generator().manual_seed(5)
    qkv = torch.randn(b, l, 3, h, 128, generator=g).bfloat16().cuda()
    q, k, v = qkv[:, :, 0], qkv[:, :, 1], qkv[:, :, 2]
    scale = 0.11
    a = ql.int8_attn(q, k, v, scale)
    c = ql.int8_attn(q.contiguous(), k.contiguous(), v.contiguous(), scale)
    assert torch.equal(a, c)


@pytest.mark.parametrize("shape", [(1, 70, 200, 2, 2, 56.0), (1, 40, 1100, 2, 1, 180.0)])
def test_attention_with_sink_keys(shape):
    """gpu_int8_attn_sink: against the oracle (anchor off, denominator + sink * exp2(-m)) and against exact attention over
    the keys plus that many zero keys with zero values."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk, sink = shape
    q, k, v = _inputs(b, lq, lk, h, hk, torch.bfloat16, seed=17, k_offset=3.0)
    scale = 128 ** -0.5
    ref = _to_f32(oracle.attn_int8(oracle.BF16, _bits(q), _bits(k), _bits(v), scale, use_anchor=False, sink=sink), oracle.BF16)
    ws = torch.zeros((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device="cuda")
    o = ql.int8_attn_sink(q.cuda(), k.cuda(), v.cuda(), scale, sink, ws=ws)
    torch.cuda.synchronize()
    an_o = _layout(ffi, b, h, hk, lq, lk)[6]
    assert (ws.cpu().numpy()[an_o:an_o + 4 * b * hk].view(np.int32) == -1).all(), "the anchor must be off with a sink"
    got = _to_f32(_bits(o), oracle.BF16)
    vmax = float(v.float().abs().max())
    tol = 2 * vmax / 255.0 + 2 * 2.0 ** -8 * np.abs(ref)
    assert (np.abs(got - ref) <= tol).all()
    n = int(sink)
    kz = torch.cat([k, torch.zeros(b, n, hk, 128, dtype=k.dtype)], 1)
    vz = torch.cat([v, torch.zeros(b, n, hk, 128, dtype=v.dtype)], 1)
    ex = _exact(q, kz, vz, scale)
    cos = float((got * ex).sum() / np.sqrt((got * got).sum() * (ex * ex).sum()))
    assert cos > 0.9995, cos
    assert np.abs(got - ex).max() < 0.03


def _rope_table(n, seed):
    """[n, 64, 2] of (cos, sin) at angles that grow with position, as a rotary table does."""
    g = torch.Generator().manual_seed(seed)
    freq = torch.exp(-torch.rand(64, generator=g) * 6.0)
    ang = torch.arange(n, dtype=torch.float32)[:, None] * freq[None, :]
    return torch.stack([torch.cos(ang), torch.sin(ang)], -1).contiguous()


def _norm_rope_f64(x, w, rope, eps, mode):
    """The transform in float64 with one rounding to bf16 at the end: what the fused stage approximates."""
    x = x.double()
    y = x * torch.rsqrt((x * x).mean(-1, keepdim=True) + eps)
    if w is not None:
        y = y * w.double()
    if rope is None or mode == 0:
        return y
    r = rope[: x.shape[1]].double()[None, :, None]          # [1, l, 1, 64, 2]
    c, s = r[..., 0], r[..., 1]
    if mode == 1:
        a, b2 = y[..., 0::2], y[..., 1::2]
        return torch.stack([c * a - s * b2, s * a + c * b2], -1).reshape(y.shape)
    a, b2 = y[..., :64], y[..., 64:]
    return torch.cat([a * c - b2 * s, b2 * c + a * s], -1)


NORM_CASES = [
    # b, lq, lk, h, hk, rope_mode, rope table, qw, kw, k_offset
    (1, 150, 210, 2, 1, 1, True, True, True, 0.0),
    (1, 150, 210, 2, 1, 2, True, True, True, 0.0),
    (2, 77, 64, 2, 2, 0, False, True, True, 0.0),
    (1, 65, 100, 2, 2, 2, False, True, True, 0.0),        # rope_mode 2 without a table: its lane order for the sum only
    (1, 90, 130, 2, 2, 1, True, True, False, 3.0),         # kw null: k untouched (not even rotated), anchor on raw k
    (1, 64, 1100, 2, 1, 2, True, False, True, 0.0),        # 128-key tiles, qw null (ones)
    (1, 257, 95, 1, 1, 1, True, True, True, 0.0),
]


@pytest.mark.parametrize("case", NORM_CASES, ids=lambda c: "b%d_lq%d_lk%d_h%d_hk%d_mode%d_rope%d_qw%d_kw%d_off%g" % c)
def test_attention_with_fused_norm_and_rope(case):
    """gpu_int8_attn_norm_rope: Q/K codes, scales and anchors bit-exact against the oracle's restatement of the fused
    stage, outputs within the attention tolerance, and the whole thing close to exact attention over q and k transformed
    in float64."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk, mode, has_rope, has_qw, has_kw, off = case
    q, k, v = _inputs(b, lq, lk, h, hk, torch.bfloat16, seed=31 + lq + mode, k_offset=off)
    q = q * 3.0                                             # a norm that has something to do
    g = torch.Generator().manual_seed(lq)
    qw = (1.0 + 0.3 * torch.randn(128, generator=g)) if has_qw else None
    kw = (1.0 + 0.3 * torch.randn(128, generator=g)) if has_kw else None
    rope = _rope_table(max(lq, lk), 3) if has_rope else None
    eps, scale = 1e-6, 128 ** -0.5
    norm = dict(qw=None if qw is None else qw.numpy(), kw=None if kw is None else kw.numpy(),
                rope=None if rope is None else rope.numpy(), eps=eps, rope_mode=mode)
    ref_q = oracle.attn_quant(oracle.BF16, _bits(q), _bits(k), _bits(v), norm=norm)
    ref = _to_f32(oracle.attn_int8(oracle.BF16, _bits(q), _bits(k), _bits(v), scale, quant=ref_q), oracle.BF16)

    ws = torch.zeros((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device="cuda")
    dev = lambda t: None if t is None else t.cuda()
    qd, kd = q.cuda(), k.cuda()
    q0, k0 = qd.clone(), kd.clone()
    o = ql.int8_attn_norm_rope(qd, kd, v.cuda(), scale, dev(qw), dev(kw), eps, dev(rope), mode, ws=ws)
    torch.cuda.synchronize()
    assert torch.equal(qd, q0) and torch.equal(kd, k0), "q and k in memory are left as they were"
    w = ws.cpu().numpy()
    qi_o, ki_o, qs_o, ks_o, vt_o, vs_o, an_o, vsum_o, ck, kb = _layout(ffi, b, h, hk, lq, lk)

    def take(at, n, dtp):
        return w[at:at + n * np.dtype(dtp).itemsize].view(dtp)

    assert np.array_equal(take(an_o, b * hk, np.int32).reshape(b, hk), ref_q["anchors"])
    if off >= 2.0:
        assert (ref_q["anchors"] >= 0).all()
    assert np.array_equal(take(qi_o, b * h * lq * 128, np.int8).reshape(b, h, lq, 128), ref_q["qi"])
    nblk = kb * (ck // 32)
    ki = take(ki_o, b * hk * nblk * 32 * 128, np.int8).reshape(b, hk, nblk, 4, 2, 32, 16)
    ki = ki.transpose(0, 1, 2, 5, 3, 4, 6).reshape(b, hk, nblk * 32, 128)[:, :, :lk]
    assert np.array_equal(ki, ref_q["ki"])
    own = np.zeros(ref_q["qs"].shape[-1], bool)
    for r in range(lq):
        own[(r // 32) * 8 + r % 8] = True
    qs = take(qs_o, ref_q["qs"].size, np.float32).reshape(ref_q["qs"].shape)
    assert np.array_equal(qs[..., own].view(np.uint32), ref_q["qs"][..., own].view(np.uint32))
    assert np.array_equal(take(ks_o, ref_q["ks"].size, np.float32).view(np.uint32), ref_q["ks"].reshape(-1).view(np.uint32))

    got = _to_f32(_bits(o), oracle.BF16)
    vmax = float(v.float().abs().max())
    tol = 2 * vmax / 255.0 + 2 * 2.0 ** -8 * np.abs(ref)
    assert (np.abs(got - ref) <= tol).all()

    qn = _norm_rope_f64(q, qw, rope, eps, mode).bfloat16()
    kn = _norm_rope_f64(k, kw, rope, eps, mode).bfloat16() if has_kw else k
    ex = _exact(qn, kn, v, scale)
    cos = float((got * ex).sum() / np.sqrt((got * got).sum() * (ex * ex).sum()))
    assert cos > 0.999, cos



def test_fused_norm_sums_squares_in_the_reference_lane_order():
    """Rows where the order of the fp32 additions shows (values of very different size, and random ones): both device
    forms of the sum against the oracle's, whose order is pinned by hand-derived cases on the CPU."""
    ql, ffi = _pkg()
    g = torch.Generator().manual_seed(2)
    rows = [torch.ones(128), torch.ones(128)]
    rows[0][0] = 4096.0
    rows[1][64] = 4096.0
    x = torch.stack(rows + [torch.randn(128, generator=g) * (10.0 ** float(torch.randint(-3, 4, (1,), generator=g))) for _ in range(62)])
    x[5] *= torch.exp(torch.randn(128, generator=g) * 4)
    for split in (0, 1):
        out = torch.zeros(2 * x.shape[0], device="cuda")
        assert ffi.raw("gpu_internal_attn_sumsq_probe", C.c_void_p(x.cuda().data_ptr()), C.c_void_p(out.data_ptr()), x.shape[0], split, None) == 0
        got = out.cpu().numpy().reshape(-1, 2)
        want = np.array([oracle.attn_sumsq128(r.numpy(), split) for r in x], np.float32)
        assert np.array_equal(got[:, 0].view(np.uint32), want.view(np.uint32))
        assert np.array_equal(got[:, 1].view(np.uint32), want.view(np.uint32))


def test_attention_norm_rope_equals_two_passes():
    """The fused stage sees exactly the bf16 values a separate norm + rope pass would have stored: running the plain
    entry point on q and k transformed row by row by the oracle gives the same workspace and the same output."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk = 1, 70, 90, 2, 2
    q, k, v = _inputs(b, lq, lk, h, hk, torch.bfloat16, seed=77)
    g = torch.Generator().manual_seed(1)
    qw, kw = 1.0 + 0.2 * torch.randn(128, generator=g), 1.0 + 0.2 * torch.randn(128, generator=g)
    rope = _rope_table(max(lq, lk), 9)
    scale, eps = 0.09, 1e-5
    for mode in (1, 2):
        def apply(x, w):
            out = torch.empty_like(x)
            xf = x.float().numpy()
            for bi in range(x.shape[0]):
                for r in range(x.shape[1]):
                    for hh in range(x.shape[2]):
                        out[bi, r, hh] = torch.from_numpy(oracle.attn_norm_rope_row(xf[bi, r, hh], w.numpy(), rope[r].numpy(), eps, mode)).bfloat16()
            return out
        q2, k2 = apply(q, qw), apply(k, kw)
        ws1 = torch.zeros((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device="cuda")
        ws2 = torch.zeros_like(ws1)
        o1 = ql.int8_attn_norm_rope(q.cuda(), k.cuda(), v.cuda(), scale, qw.cuda(), kw.cuda(), eps, rope.cuda(), mode, ws=ws1)
        o2 = ql.int8_attn(q2.cuda(), k2.cuda(), v.cuda(), scale, ws=ws2)
        assert torch.equal(ws1, ws2)
        assert torch.equal(o1, o2)


def test_attention_sink_with_q_norm():
    """gpu_int8_attn_sink with qw: q normalized (weight, no rotation), k as it is, anchor off."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk, sink = 1, 50, 180, 2, 1, 76.0
    q, k, v = _inputs(b, lq, lk, h, hk, torch.bfloat16, seed=23)
    qw = 1.0 + 0.25 * torch.randn(128, generator=torch.Generator().manual_seed(4))
    scale, eps = 128 ** -0.5, 1e-6
    norm = dict(qw=qw.numpy(), kw=None, rope=None, eps=eps, rope_mode=0)
    ref_q = oracle.attn_quant(oracle.BF16, _bits(q), _bits(k), _bits(v), use_anchor=False, norm=norm)
    ref = _to_f32(oracle.attn_int8(oracle.BF16, _bits(q), _bits(k), _bits(v), scale, quant=ref_q, sink=sink), oracle.BF16)
    ws = torch.zeros((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device="cuda")
    o = ql.int8_attn_sink(q.cuda(), k.cuda(), v.cuda(), scale, sink, ws=ws, qw=qw.cuda(), eps=eps)
    torch.cuda.synchronize()
    lay = _layout(ffi, b, h, hk, lq, lk)
    w = ws.cpu().numpy()
    assert np.array_equal(w[lay[0]:lay[0] + b * h * lq * 128].view(np.int8).reshape(b, h, lq, 128), ref_q["qi"])
    assert (w[lay[6]:lay[6] + 4 * b * hk].view(np.int32) == -1).all()
    got = _to_f32(_bits(o), oracle.BF16)
    tol = 2 * float(v.float().abs().max()) / 255.0 + 2 * 2.0 ** -8 * np.abs(ref)
    assert (np.abs(got - ref) <= tol).all()


def test_attention_unaligned_views_take_the_scalar_paths():
    """Rows that start on odd element offsets with strides that are not multiples of four: the 8-byte vector accesses
    are off for inputs and output, and the result is the same bits as for contiguous tensors."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk = 1, 45, 130, 2, 1
    q, k, v = (t.cuda() for t in _inputs(b, lq, lk, h, hk, torch.float16, seed=23))
    scale = 0.09
    want = ql.int8_attn(q, k, v, scale)

    def odd_view(t):
        bb, l, hh, d = t.shape
        row = hh * d + 2
        base = torch.zeros(bb * l * row + 1, dtype=t.dtype, device=t.device)
        view = base.as_strided((bb, l, hh, d), (l * row, row, d, 1), 1)
        view.copy_(t)
        return view

    qo, ko, vo = odd_view(q), odd_view(k), odd_view(v)
    oo = odd_view(torch.zeros_like(q))
    ws = torch.zeros((ffi.lib.gpu_int8_attn_workspace_d(b, h, hk, lq, lk, 128),), dtype=torch.uint8, device="cuda")
    P = lambda t: C.c_void_p(t.data_ptr())
    assert qo.data_ptr() % 4 == 2 and qo.stride(1) % 4 == 2
    ffi.k("gpu_int8_attn_f16", P(qo), P(ko), P(vo), P(oo), P(ws), b, lq, lk, h, hk, 128, *qo.stride()[:3], *ko.stride()[:3],
          *vo.stride()[:3], *oo.stride()[:3], scale, None)
    torch.cuda.synchronize()
    assert torch.equal(oo, want)


def test_u8_pack_conversion_rounds_to_nearest_even_and_saturates():
    """The probabilities are rounded by the hardware's float -> u8 pack conversion; the reference rounds with
    cvt.rni.sat.u8 and the oracle with clamp + rint.  Every integer 0..255 with fractions either side of one half, the
    exact halves, and values outside the range."""
    ql, ffi = _pkg()
    fr = np.array([0.0, 0.25, 0.4999, 0.5, 0.5001, 0.75, 0.999, np.float32(0.49999997)], np.float32)
    x = (np.arange(256, dtype=np.float32)[:, None] + fr[None, :]).reshape(-1)
    x = np.concatenate([x, np.array([255.4, 255.5, 255.6, 256.0, 300.0, 1e9, -0.4, -0.5, -1.0, -1e9, np.nan], np.float32)])
    xd = torch.from_numpy(x).cuda()
    yd = torch.zeros(x.size, dtype=torch.int32, device="cuda")
    ffi.k("gpu_internal_cvt_pk_u8_probe", C.c_void_p(xd.data_ptr()), C.c_void_p(yd.data_ptr()), x.size, None)
    torch.cuda.synchronize()
    want = np.rint(np.clip(np.nan_to_num(x, nan=0.0), 0.0, 255.0)).astype(np.int32)
    assert np.array_equal(yd.cpu().numpy(), want)


def test_attention_replays_from_a_captured_graph():
    """The call allocates nothing and clears its accumulators with kernels, so it can be captured (after one eager call
    on the device, which sets the kernel's LDS limit).  Three replays with eager work and new inputs between them, each
    against the eager result for the same inputs."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk = 1, 200, 1300, 2, 2
    q, k, v = (t.cuda() for t in _inputs(b, lq, lk, h, hk, torch.bfloat16, seed=31))
    ws = torch.zeros((ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk),), dtype=torch.uint8, device="cuda")
    o = torch.empty_like(q)
    P = lambda t: C.c_void_p(t.data_ptr())

    def call():
        ffi.k("gpu_int8_attn", P(q), P(k), P(v), P(o), P(ws), b, lq, lk, h, hk, *q.stride()[:3], *k.stride()[:3],
              *v.stride()[:3], *o.stride()[:3], 0.088, C.c_void_p(torch.cuda.current_stream().cuda_stream))

    call()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    g = torch.Generator(device="cuda").manual_seed(5)
    for rep in range(3):
        q.copy_(torch.randn(q.shape, device="cuda", generator=g).to(q.dtype))
        k.copy_((torch.randn(k.shape, device="cuda", generator=g) + rep).to(k.dtype))
        v.copy_(torch.randn(v.shape, device="cuda", generator=g).to(v.dtype))
        o.zero_()
        graph.replay()
        torch.cuda.synchronize()
        got = o.clone()
        want = ql.int8_attn(q, k, v, 0.088)      # eager, its own workspace
        torch.cuda.synchronize()
        assert torch.equal(got, want), "replay %d differs from the eager call" % rep


def test_attention_refuses_what_it_does_not_build():
    ql, ffi = _pkg()
    x = torch.zeros(1, 4, 1, 128, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    p = lambda t: C.c_void_p(t.data_ptr())
    args = lambda D, h, hk: (p(x), p(x), p(x), p(x), p(ws), 1, 4, 4, h, hk, D, 512, 128, 128, 512, 128, 128, 512, 128, 128, 512, 128, 128, 0.1, None)
    assert ffi.raw("gpu_int8_attn_d", *args(96, 1, 1)) == -400
    assert ffi.lib.gpu_int8_attn_workspace_d(1, 1, 1, 4, 4, 96) == 0 and ffi.lib.gpu_int8_attn_workspace_d(1, 1, 1, 4, 4, 512) == 0
    assert ffi.lib.gpu_int8_attn_workspace_d(1, 1, 1, 4, 4, 128) > 0 and ffi.lib.gpu_int8_attn_workspace_d(1, 1, 1, 4, 4, 64) > 0
    assert ffi.raw("gpu_int8_attn_d", *args(128, 3, 2)) == -400
    assert ffi.raw("gpu_int8_attn_d", *args(128, 1, 1)) == 0
    torch.cuda.synchronize()


def test_attention_dit_size_against_exact_attention():
    """The DiT joint-attention shape (4608 tokens, 24 heads): no oracle at this size, so the check is against fp32 softmax
    attention on the GPU, and row-stochasticity: attention over constant V returns that constant."""
    ql, ffi = _pkg()
    b, l, h = 1, 4608, 24
    g = torch.Generator(device="cuda").manual_seed(3)
    q = torch.randn(b, l, h, 128, generator=g, device="cuda").bfloat16()
    k = (torch.randn(b, l, h, 128, generator=g, device="cuda") + 0.3).bfloat16()
    v = torch.randn(b, l, h, 128, generator=g, device="cuda").bfloat16()
    scale = 128 ** -0.5
    o = ql.int8_attn(q, k, v, scale).float()
    ex = torch.nn.functional.scaled_dot_product_attention(q.float().transpose(1, 2), k.float().transpose(1, 2),
                                                          v.float().transpose(1, 2), scale=scale).transpose(1, 2)
    cos = float((o * ex).sum() / torch.sqrt((o * o).sum() * (ex * ex).sum()))
    assert cos > 0.999, cos
    vc = torch.full_like(v, 0.75)
    oc = ql.int8_attn(q, k, vc, scale).float()
    assert float((oc - 0.75).abs().max()) <= 0.75 * 2 ** -7


BIAS_CASES = [
    # b, lq, lk, h, hk, kind
    (1, 100, 150, 2, 1, "sparse"),        # 64-key tiles, ragged last tile
    (2, 64, 64, 2, 2, "sparse"),
    (1, 70, 1024, 2, 2, "sparse"),        # the longest sequence of the per-key route
    (1, 90, 1100, 2, 1, "tiles"),         # 128-key tiles: constant tiles (zero and non-zero), varying tiles, ragged last
    (1, 130, 1536, 4, 2, "tiles"),        # no ragged tail: the last tile still takes the float route
    (1, 50, 1300, 1, 1, "masked"),        # -inf keys, one whole tile of them
    (1, 60, 200, 2, 2, "masked"),
    (1, 40, 300, 2, 1, "all_masked"),
]


def _bias_for(kind, lk, seed):
    rng = np.random.default_rng(seed)
    bias = np.zeros(lk, np.float32)
    hot = rng.choice(lk, max(1, lk // 7), replace=False)
    bias[hot] = rng.choice(np.array([0.6, 1.2, -1.5], np.float32), hot.size)
    if kind == "tiles" or kind == "masked":
        if lk > 1024:
            bias[128:384] = 0.0
            bias[512:640] = 0.75
    if kind == "masked":
        bias[rng.choice(lk, lk // 4, replace=False)] = -np.inf
        if lk > 1024:
            bias[640:768] = -np.inf
    if kind == "all_masked":
        bias[:] = -np.inf
    return bias


@pytest.mark.parametrize("case", BIAS_CASES, ids=lambda c: "b%d_lq%d_lk%d_h%d_hk%d_%s" % c)
def test_attention_with_key_bias(case):
    """gpu_int8_attn_key_bias against the oracle's restatement of the reference's two masked routes (quantizer stages
    bit-exact as in the plain call, outputs within the attention tolerance) and against exact attention with the bias on
    the logits."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk, kind = case
    q, k, v = _inputs(b, lq, lk, h, hk, torch.bfloat16, seed=lq + lk)
    bias = _bias_for(kind, lk, lk)
    scale = 128 ** -0.5
    ref_q = oracle.attn_quant(oracle.BF16, _bits(q), _bits(k), _bits(v))
    ref = _to_f32(oracle.attn_int8_bias(oracle.BF16, _bits(q), _bits(k), _bits(v), scale, bias, quant=ref_q), oracle.BF16)
    n = ffi.lib.gpu_int8_attn_key_bias_workspace(b, h, hk, lq, lk)
    assert n > ffi.lib.gpu_int8_attn_workspace(b, h, hk, lq, lk)
    ws = torch.zeros((n,), dtype=torch.uint8, device="cuda")
    o = ql.int8_attn_key_bias(q.cuda(), k.cuda(), v.cuda(), scale, torch.from_numpy(bias).cuda(), ws=ws)
    torch.cuda.synchronize()
    lay = _layout(ffi, b, h, hk, lq, lk)
    w = ws.cpu().numpy()
    assert np.array_equal(w[lay[0]:lay[0] + b * h * lq * 128].view(np.int8).reshape(b, h, lq, 128), ref_q["qi"])
    assert np.array_equal(w[lay[6]:lay[6] + 4 * b * hk].view(np.int32).reshape(b, hk), ref_q["anchors"])
    got = _to_f32(_bits(o), oracle.BF16)
    assert np.isfinite(got).all()
    if kind == "all_masked":
        if lk <= 1024:
            assert (got == 0).all()
        return
    vmax = float(v.float().abs().max())
    tol = 2 * vmax / 255.0 + 2 * 2.0 ** -8 * np.abs(ref)
    err = np.abs(got - ref)
    assert (err <= tol).all(), "max excess %g" % float((err - tol).max())
    assert (err <= 2.0 ** -8 * np.abs(ref) + 1e-30).mean() > 0.97

    keep = np.isfinite(bias)
    kk, vv = k[:, keep], v[:, keep]
    hh, hkk = q.shape[2], k.shape[2]
    qq = q.double().permute(0, 2, 1, 3)
    kd = kk.double().permute(0, 2, 1, 3).repeat_interleave(hh // hkk, 1)
    vd = vv.double().permute(0, 2, 1, 3).repeat_interleave(hh // hkk, 1)
    logits = qq @ kd.transpose(-1, -2) * scale + torch.from_numpy(bias[keep]).double()
    ex = (torch.softmax(logits, -1) @ vd).permute(0, 2, 1, 3).numpy()
    cos = float((got * ex).sum() / np.sqrt((got * got).sum() * (ex * ex).sum()))
    assert cos > 0.9995, cos


def test_attention_key_bias_moves_weight_to_the_biased_keys():
    """A large bias on one key makes every query attend to it: the output is that key's value row (to quantization)."""
    ql, ffi = _pkg()
    for lk in (200, 1200):
        q, k, v = _inputs(1, 32, lk, 1, 1, torch.bfloat16, seed=3)
        bias = torch.zeros(lk)
        bias[lk // 2] = 60.0
        o = ql.int8_attn_key_bias(q.cuda(), k.cuda(), v.cuda(), 128 ** -0.5, bias.cuda())
        want = v[0, lk // 2, 0].float()
        assert (o[0, :, 0].float().cpu() - want).abs().max() < 2 * float(v.float().abs().max()) / 127 + 0.02


@pytest.mark.parametrize("amp", [1.0, 1e-3])
def test_attention_f16_short_sequences_take_the_unfused_path(amp):
    """f16 with at most 512 keys: float denominators in every tile.  Against the oracle, which pins that path on the
    CPU, and against exact attention (keys past lk weigh nothing, also with tiny q and k)."""
    ql, ffi = _pkg()
    b, lq, lk, h, hk = 1, 70, 100, 2, 1
    q, k, v = _inputs(b, lq, lk, h, hk, torch.float32, seed=8)
    q, k, v = (q * amp).half(), (k * amp).half(), v.half()
    ref = _to_f32(oracle.attn_int8(oracle.F16, _bits(q), _bits(k), _bits(v), 0.088), oracle.F16)
    got = _to_f32(_bits(ql.int8_attn(q.cuda(), k.cuda(), v.cuda(), 0.088)), oracle.F16)
    vmax = float(v.float().abs().max())
    tol = 2 * vmax / 255.0 + 2 * 2.0 ** -11 * np.abs(ref)
    assert (np.abs(got - ref) <= tol).all()
    ex = _exact(q, k, v, 0.088)
    cos = float((got * ex).sum() / np.sqrt((got * got).sum() * (ex * ex).sum()))
    assert cos > 0.9995, cos


HD_CASES = [
    # D, b, lq, lk, h, hk, dtype, k_offset
    (64, 1, 200, 300, 4, 2, torch.bfloat16, 0.0),
    (64, 2, 77, 64, 2, 2, torch.float16, 0.0),        # f16, short: unfused path, H4 rotation
    (64, 1, 129, 1500, 2, 1, torch.float16, 3.0),      # head dim 64 keeps 64-key tiles at any length; anchor on
    (64, 1, 1, 1, 1, 1, torch.bfloat16, 0.0),
    (256, 1, 100, 150, 2, 1, torch.bfloat16, 0.0),     # 16-row Q blocks, H4 rotation
    (256, 1, 70, 400, 2, 2, torch.float16, 2.5),       # plain H128 per half, anchor on, unfused path
    (256, 1, 150, 1100, 2, 1, torch.bfloat16, 0.0),    # 128-key tiles
    (256, 1, 33, 1025, 1, 1, torch.float16, 0.0),
]


@pytest.mark.parametrize("case", HD_CASES, ids=lambda c: "D%d_b%d_lq%d_lk%d_h%d_hk%d_%s_off%g" % (c[:6] + (str(c[6])[6:], c[7])))
def test_attention_head_dims_64_and_256(case):
    """gpu_int8_attn_d / gpu_int8_attn_f16 at head dims 64 and 256: anchors, Q and K codes and scales, V scales bit-exact
    against the oracle; outputs within the attention tolerance; close to exact attention."""
    ql, ffi = _pkg()
    D, b, lq, lk, h, hk, dtype, off = case
    dt = oracle.BF16 if dtype == torch.bfloat16 else oracle.F16
    q, k, v = _inputs(b, lq, lk, h, hk, dtype, seed=D + lq + lk, k_offset=off, D=D)
    scale = D ** -0.5
    ref_q = oracle.attn_quant(dt, _bits(q), _bits(k), _bits(v))
    ref = _to_f32(oracle.attn_int8(dt, _bits(q), _bits(k), _bits(v), scale, quant=ref_q), dt)
    ws_bytes = ffi.lib.gpu_int8_attn_workspace_d(b, h, hk, lq, lk, D)
    assert ws_bytes > 0
    ws = torch.zeros((ws_bytes,), dtype=torch.uint8, device="cuda")
    o = ql.int8_attn(q.cuda(), k.cuda(), v.cuda(), scale, ws=ws)
    torch.cuda.synchronize()
    w = ws.cpu().numpy()
    out = (C.c_int64 * 10)()
    assert ffi.raw("gpu_internal_attn_layout_d", b, h, hk, lq, lk, D, C.cast(out, C.c_void_p)) == 0
    qi_o, ki_o, qs_o, ks_o, vt_o, vs_o, an_o, vsum_o, ck, kb = list(out)
    assert ck == ref_q["ck"]

    def take(at, n, dtp):
        return w[at:at + n * np.dtype(dtp).itemsize].view(dtp)

    assert np.array_equal(take(an_o, b * hk, np.int32).reshape(b, hk), ref_q["anchors"])
    if off >= 2.0:
        assert (ref_q["anchors"] >= 0).all()
    assert np.array_equal(take(qi_o, b * h * lq * D, np.int8).reshape(b, h, lq, D), ref_q["qi"])
    nblk = kb * (ck // 32)
    ki = take(ki_o, b * hk * nblk * 32 * D, np.int8).reshape(b, hk, nblk, D // 32, 2, 32, 16)
    ki = ki.transpose(0, 1, 2, 5, 3, 4, 6).reshape(b, hk, nblk * 32, D)[:, :, :lk]
    assert np.array_equal(ki, ref_q["ki"])
    wq = 16 if D == 256 else 32
    own = np.zeros(ref_q["qs"].shape[-1], bool)
    for r in range(lq):
        own[(r // wq) * 8 + r % 8] = True
    qs = take(qs_o, ref_q["qs"].size, np.float32).reshape(ref_q["qs"].shape)
    assert np.array_equal(qs[..., own].view(np.uint32), ref_q["qs"][..., own].view(np.uint32))
    assert np.array_equal(take(ks_o, ref_q["ks"].size, np.float32).view(np.uint32), ref_q["ks"].reshape(-1).view(np.uint32))
    assert np.array_equal(take(vs_o, b * hk * D, np.float32).view(np.uint32), ref_q["vs"].reshape(-1).view(np.uint32))
    vt = take(vt_o, b * hk * nblk * D * 32, np.int8).reshape(b, hk, nblk, D, 32)
    pos = np.arange(32)
    key_of_pos = ((pos % 16) // 4) * 8 + (pos // 16) * 4 + pos % 4
    vi_pad = np.zeros((b, hk, nblk * 32, D), np.int8)
    vi_pad[:, :, :lk] = ref_q["vi"]
    want_vt = vi_pad.reshape(b, hk, nblk, 32, D)[:, :, :, key_of_pos, :].transpose(0, 1, 2, 4, 3)
    assert np.array_equal(vt, want_vt)

    got = _to_f32(_bits(o), dt)
    vmax = float(v.float().abs().max())
    ulp = 2.0 ** (-8 if dt == oracle.BF16 else -11)
    tol = 2 * vmax / 255.0 + 2 * ulp * np.abs(ref)
    err = np.abs(got - ref)
    assert (err <= tol).all(), "max excess %g" % float((err - tol).max())
    assert (err <= ulp * np.abs(ref) + 1e-30).mean() > 0.97
    ex = _exact(q, k, v, scale)
    cos = float((got * ex).sum() / np.sqrt((got * got).sum() * (ex * ex).sum()))
    assert cos > 0.9995, cos
