"""Synthetic workloads for the quantized-linear path: counter-hashed, so every consumer regenerates identical bytes.

Inputs are a pure function of (seed, stream, index): a 64-bit mixing hash feeds uniforms, Box-Muller normals and
Student-t draws.  The same idea as the reference's GPU golden test, which regenerates its inputs from an integer
hash instead of storing them (tests/sparse_attn_match_comfy.rs:10-18).  bf16/f16 tensors are returned as uint16 bit
patterns.
"""
import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def _mix(z):
    z = (z + np.uint64(0x9E3779B97F4A7C15)) & _M64
    z = ((z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)) & _M64
    z = ((z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)) & _M64
    return z ^ (z >> np.uint64(31))


def hash_u64(seed, stream, n, offset=0):
    with np.errstate(over="ignore"):
        base = _mix(np.uint64(seed) * np.uint64(0x632BE59BD9B4E019) + np.uint64(stream))
        idx = np.arange(offset, offset + n, dtype=np.uint64)
        return _mix(idx ^ base)


def u01(seed, stream, n):
    """Uniform in (0, 1), 53 random bits."""
    h = hash_u64(seed, stream, n)
    return ((h >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, stream, n):
    u1 = u01(seed, 2 * stream, n)
    u2 = u01(seed, 2 * stream + 1, n)
    return (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def uniform(seed, stream, n, lo, hi):
    return (lo + (hi - lo) * u01(seed, stream, n)).astype(np.float32)


def randint(seed, stream, n, lo, hi):
    """Integers uniform in [lo, hi]."""
    h = hash_u64(seed, stream, n)
    return (np.int64(lo) + (h % np.uint64(hi - lo + 1)).astype(np.int64))


def student_t3(seed, stream, n):
    z = normal(seed, 4 * stream + 1000, n).astype(np.float64)
    c = sum(normal(seed, 4 * stream + 1001 + j, n).astype(np.float64) ** 2 for j in range(3))
    return (z / np.sqrt(c / 3.0)).astype(np.float32)


def bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    return ((u + (np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1)))) >> np.uint32(16)).astype(np.uint16)


def bf16_to_f32(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f16_bits(x):
    return np.ascontiguousarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


C0_OUTLIER_COLS = (3, 127, 256, 389, 512, 700, 901, 1023)


def activations(seed, M, K, kind="normal", outlier_cols=(), outlier_gain=20.0):
    """float32 [M, K] activations before rounding to the activation dtype.

    kind "normal": N(0,1).  kind "t3": N(0,1) rows times a per-channel Student-t(3) scale (heavy-tailed channels).
    """
    x = normal(seed, 1, M * K).reshape(M, K)
    if kind == "t3":
        x = x * student_t3(seed, 2, K)[None, :]
    for c in outlier_cols:
        x[:, c] *= np.float32(outlier_gain)
    return x


def outlier_columns(seed, K, frac):
    n = int(np.ceil(frac * K))
    cols = randint(seed, 7, 4 * n + 8, 0, K - 1)
    out = []
    for c in cols:
        if int(c) not in out:
            out.append(int(c))
        if len(out) == n:
            break
    return tuple(out)


def w8_weights(seed, N, K):
    """int8 [N,K] uniform in [-127,127], f32 per-channel scales U[1e-3,1e-2], f32 bias N(0,0.02) (round it yourself)."""
    W = randint(seed, 11, N * K, -127, 127).astype(np.int8).reshape(N, K)
    ws = uniform(seed, 12, N, 1e-3, 1e-2)
    bias = normal(seed, 13, N) * np.float32(0.02)
    return W, ws, bias


def w6_codes(seed, N, K):
    """Symmetric 6-bit values uniform in [-31, 31] as int8 [N,K]."""
    return randint(seed, 21, N * K, -31, 31).astype(np.int8).reshape(N, K)


def w6_group_scales(seed, N, K, group=128):
    return uniform(seed, 22, N * (K // group), 1e-3, 1e-2).reshape(N, K // group)


def w6_srel_bytes(seed, N, K, G=32):
    """fp8-e4m3 relative scales as bytes: positive, finite, spread over [0.5, 4] so decoded values stay in int8."""
    # exponent field 6..8 (2^-1 .. 2^1), mantissa 0..7 -> values in [0.5, 3.75]
    e = randint(seed, 23, N * (K // G), 6, 8).astype(np.uint8)
    m = randint(seed, 24, N * (K // G), 0, 7).astype(np.uint8)
    return ((e << np.uint8(3)) | m).reshape(N, K // G)


def config0(seed=0):
    """The CPU-runnable anchor case: X bf16 [256,1024] with 8 outlier columns x20; W int8 [1024,1024]; per-channel scales; bias."""
    M, K, N = 256, 1024, 1024
    x = activations(seed, M, K, "normal", C0_OUTLIER_COLS)
    W, ws, bias = w8_weights(seed, N, K)
    return dict(M=M, K=K, N=N, x=bf16_bits(x), W=W, ws=ws, bias=bf16_bits(bias))
