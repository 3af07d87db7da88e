"""gpu_int8_gemm_static, the entry point that allocates nothing, against gpu_int8_gemm: bit-equal outputs through the C ABI
on two calls in a row, the second with a smaller input (the static split-K planes keep the first call's contents)."""
import importlib
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, ROOT)

pytestmark = pytest.mark.gpu

torch = pytest.importorskip("torch")
if not torch.cuda.is_available():
    pytest.skip("needs a GPU", allow_module_level=True)

import oracle  # noqa: E402

ffi = importlib.import_module("comfyui-backend-but-rust_amd.ffi")
synth = importlib.import_module("comfyui-backend-but-rust_amd.synth")
DEV = "cuda:0"


def _inputs(seed, M, N, K):
    A = synth.randint(seed, 1, M * K, -127, 127).astype(np.int8).reshape(M, K)
    W = synth.randint(seed, 2, N * K, -127, 127).astype(np.int8).reshape(N, K)
    xs = synth.uniform(seed, 3, M, 0.005, 0.2)
    ws = synth.uniform(seed, 4, N, 1e-3, 1e-2)
    bias = oracle.bf16_bits(synth.normal(seed, 5, N) * np.float32(0.02))
    return A, W, xs, ws, bias


def _run(name, A, W, xs, ws, bias):
    M, K = A.shape
    N = W.shape[0]
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    Ad, Wd, xsd, wsd = t(A), t(W), t(xs), t(ws)
    bd = t(bias.view(np.int16))
    D = torch.full((M, N), -1, dtype=torch.int16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    ffi.k(name, Ad.data_ptr(), Wd.data_ptr(), xsd.data_ptr(), wsd.data_ptr(), bd.data_ptr(), D.data_ptr(), M, N, K, ffi.DT_BF16, s)
    torch.cuda.synchronize()
    return D.cpu().numpy().view(np.uint16)


# split-K shapes of the skinny path (M <= 256, N too narrow to give every CU a column slab), larger first
SHAPES = [(256, 4096, 4096), (100, 1024, 2048)]


def test_static_entry_point_matches_allocating_one_twice_in_a_row():
    assert ffi.lib.gpu_int8_gemm_static_limit() == 24 << 20
    for i, (M, N, K) in enumerate(SHAPES):
        print("no-alloc case", i, M, N, K, flush=True)
        A, W, xs, ws, bias = _inputs(40 + i, M, N, K)
        want = _run("gpu_int8_gemm", A, W, xs, ws, bias)
        got = _run("gpu_int8_gemm_static", A, W, xs, ws, bias)
        assert np.array_equal(got, want), (M, N, K)
        if i == 1:   # and against the oracle, so that both being wrong the same way cannot pass
            ref = oracle.int8_gemm(A, W, xs, ws, bias, oracle.BF16, fma=1)
            assert np.array_equal(got, ref.view(np.uint16))


def test_static_entry_point_on_shapes_without_scratch():
    """Shapes that take other kernel families need no scratch and give the same bits too."""
    for (M, N, K) in [(300, 520, 256), (64, 64, 64)]:
        A, W, xs, ws, bias = _inputs(50, M, N, K)
        assert np.array_equal(_run("gpu_int8_gemm_static", A, W, xs, ws, bias), _run("gpu_int8_gemm", A, W, xs, ws, bias))


def test_static_entry_point_refuses_what_would_need_an_allocation():
    """K % 16 == 8 runs on padded copies that gpu_int8_gemm allocates; the entry point that may not allocate refuses it.
    (The split-K planes of every M <= 256 shape fit the static array on a 256-CU device: slices * N <= 256 * 96.)"""
    M, N, K = 64, 128, 136
    A, W, xs, ws, bias = _inputs(60, M, N, K)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(DEV)
    Ad, Wd, xsd, wsd, bd = t(A), t(W), t(xs), t(ws), t(bias.view(np.int16))
    D = torch.zeros((M, N), dtype=torch.int16, device=DEV)
    s = torch.cuda.current_stream().cuda_stream
    args = (Ad.data_ptr(), Wd.data_ptr(), xsd.data_ptr(), wsd.data_ptr(), bd.data_ptr(), D.data_ptr(), M, N, K, ffi.DT_BF16, s)
    assert ffi.raw("gpu_int8_gemm_static", *args) == -200
    assert ffi.raw("gpu_int8_gemm", *args) == 0
    torch.cuda.synchronize()
    assert np.array_equal(D.cpu().numpy().view(np.uint16), oracle.int8_gemm(A, W, xs, ws, bias, oracle.BF16, fma=1).view(np.uint16))
