"""CPU-only checks of the drop-in boundary: the library loads, exports every symbol the header declares, and refuses bad
arguments with the reference's return codes before touching the GPU."""
import ctypes
import json
import os
import re

import numpy as np
import pytest

import oracle
from conftest import ROOT, pkg

ffi = pkg("ffi")


def header_functions(name="gpu_api.h"):
    text = open(os.path.join(ROOT, "include", name)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"\b(gpu_[a-z0-9_]+)\s*\(", text)


def test_library_exports_every_declared_symbol():
    names = header_functions()
    assert {"gpu_quant_rows", "gpu_quant_rows_b", "gpu_rotate_rows_f32", "gpu_sd_quant_rows", "gpu_int8_gemm",
            "gpu_int8_gemm_residual", "gpu_w6_decode"} <= set(names)
    lib = ctypes.CDLL(ffi.LIB_PATH)
    for n in names:
        assert hasattr(lib, n), n
    for n in ffi.SIGNATURES:
        assert n in names, "ffi.py binds %s, which the header does not declare" % n
    assert "gfx950" in ffi.build_info()
    # the dense-GEMM library: loads (hipBLASLt resolves) and exports what its header declares
    blas_names = header_functions("gpu_blas_api.h")
    assert set(blas_names) == {"gpu_blas_init", "gpu_gemm"} == set(ffi.BLAS_SIGNATURES)
    blas = ctypes.CDLL(ffi.BLAS_LIB_PATH)
    for n in blas_names:
        assert hasattr(blas, n), n
    assert ffi.blas().gpu_gemm(0, 0, 0, 0, 0, 0, 0, 4, 4, 4, 1, 2, 2, 1.0, 0.0, 0) == -100    # before gpu_blas_init


def test_header_constants_match_reference_codes():
    text = open(os.path.join(ROOT, "include", "gpu_api.h")).read()
    assert re.search(r"DT_F32 = 0, DT_F16 = 1, DT_BF16 = 2", text)
    assert (ffi.PRO_PLAIN, ffi.PRO_RMS, ffi.PRO_GATE, ffi.PRO_SWIGLU, ffi.PRO_ADALN, ffi.PRO_SITU_FAST) == (0, 1, 2, 3, 7, 13)
    for name, val in (("PRO_LN_MOD", 9), ("PRO_LN_AFFINE", 10), ("PRO_GELU_TANH", 11), ("PRO_LN_AFFINE_SILU", 12)):
        assert re.search(r"%s = %d\b" % (name, val), text)


def q(dtype=2, pro=0, K=256, rotate=0, M=4):
    return ffi.raw("gpu_quant_rows", dtype, pro, 0, K, 0, 0, 0, 0, 0.0, 0, 0, 0, 0, M, K, rotate, 0)


def test_quant_rows_refusals_match_reference_order():
    assert q(K=200) == -1                       # csrc/kernels.cu:275
    assert q(K=320, rotate=1) == -1
    assert q(K=192, rotate=128) == -1
    assert q(dtype=1) == -4                     # :297
    assert q(dtype=1, pro=99) == -4             # dtype is looked at before the prologue id
    assert q(pro=99) == -3 and q(pro=12) == -3  # :292 (LN_AFFINE_SILU is not in the quantizer's list)
    assert q(K=32768 + 256) == -2               # :265
    assert q(pro=ffi.PRO_SITU, M=0) == 0 and q(pro=ffi.PRO_SITU_FAST, M=0) == 0
    assert q(pro=ffi.PRO_RMS, M=0) == 0
    assert q(M=0) == 0
    # the oracle agrees on the shared codes
    x = np.zeros((1, 512), np.uint16)
    assert oracle.quant_rows(oracle.BF16, x, 200, 0)[0] == -1
    assert oracle.quant_rows(oracle.F16, x, 256, 0)[0] == -4


def test_other_entry_point_refusals():
    assert ffi.raw("gpu_quant_rows_b", 2, ffi.PRO_LN_MOD, 0, 300, 0, 0, 0.0, 0, 0, 0, 0, 1, 300, 0, 0) == -1
    assert ffi.raw("gpu_quant_rows_b", 0, ffi.PRO_LN_MOD, 0, 256, 0, 0, 0.0, 0, 0, 0, 0, 1, 256, 0, 0) == -4
    assert ffi.raw("gpu_quant_rows_b", 2, ffi.PRO_RMS, 0, 256, 0, 0, 0.0, 0, 0, 0, 0, 1, 256, 0, 0) == -3
    assert ffi.raw("gpu_rotate_rows_f32", ffi.PRO_PLAIN, 0, 320, 0, 0, 0.0, 0, 1, 320, 0) == -1
    assert ffi.raw("gpu_rotate_rows_f32", ffi.PRO_GATE, 0, 256, 0, 0, 0.0, 0, 1, 256, 0) == -3
    pr = lambda dt, pro: ffi.raw("gpu_prologue_rows", dt, pro, 0, 256, 0, 0, 0, 0, 0.0, 0, 0, 0, 256, 0, 256, 0)
    assert pr(1, ffi.PRO_RMS) == -4 and pr(2, ffi.PRO_LN_MOD) == -3 and pr(2, 99) == -3 and pr(2, ffi.PRO_RMS) == 0
    pb = lambda dt, pro: ffi.raw("gpu_prologue_rows_b", dt, pro, 0, 256, 0, 0, 0.0, 0, 0, 0, 256, 0, 256, 0)
    assert pb(7, ffi.PRO_LN_MOD) == -4 and pb(1, ffi.PRO_RMS) == -3 and pb(1, ffi.PRO_GELU_TANH) == 0
    assert ffi.raw("gpu_sd_quant_rows", 0, 640, 0, 0, 1, 640, 128, 0) == -1     # csrc/sd.cu:600
    assert ffi.raw("gpu_sd_quant_rows", 0, 640, 0, 0, 1, 640, 256, 0) == -1
    assert ffi.raw("gpu_w6_decode", 0, 0, 0, 4, 48, 32, 0) == -1                # csrc/h3.cu:41
    assert ffi.raw("gpu_w6_decode", 0, 0, 0, 4, 64, 8, 0) == -1
    assert ffi.raw("gpu_w6_decode", 0, 0, 0, 0, 64, 32, 0) == 0


def test_gemm_refusals_and_empty_shapes():
    g = lambda M, N, K, dt=2: ffi.raw("gpu_int8_gemm", 0, 0, 0, 0, 0, 0, M, N, K, dt, 0)
    assert g(0, 8, 16) == 0 and g(8, 0, 16) == 0 and g(8, 8, 0) == 0       # csrc/vendor/cutlass_gemm_int8.cu:377
    assert g(8, 8, 16, dt=5) == -200                                         # csrc/gemm.cu:126
    assert g(8, 8, 20) == -200                                               # K % 8: no tile configuration takes it (:191, :237-247)
    r = lambda M, N, K, rs=1, res=1, dt=2: ffi.raw("gpu_int8_gemm_residual", 0, 0, 0, 0, 0, rs, res, 0, M, N, K, dt, 0)
    assert r(0, 8, 16) == 0 and r(8, 0, 16) == 0                             # :353
    assert r(8, 8, 0) == -201                                                # :355, csrc/gemm.cu:137
    assert r(8, 8, 16, rs=0) == -201 and r(8, 8, 16, res=0) == -201          # :357
    assert r(8, 8, 16, dt=9) == -201


def test_ok_and_k_raise_like_the_reference():
    ffi.ok(0, "anything")
    with pytest.raises(ffi.KernelError, match="gpu_quant_rows failed with code -1"):
        ffi.k("gpu_quant_rows", 2, 0, 0, 200, 0, 0, 0, 0, 0.0, 0, 0, 0, 0, 4, 200, 0, 0)
    with pytest.raises(ffi.KernelError, match="x failed: "):
        ffi.ok(1, "x")


def test_oracle_reproduces_golden_fixtures(synth):
    import hashlib
    dig = lambda a: hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()
    g = json.load(open(os.path.join(ROOT, "tests", "golden", "config0_w8a8.json")))
    c = synth.config0(0)
    assert dig(c["x"]) == g["x_sha256"] and dig(c["W"]) == g["W_sha256"] and dig(c["ws"]) == g["ws_sha256"]
    rc, qq, xs = oracle.quant_rows(oracle.BF16, c["x"], c["K"], 0)
    acc = oracle.int8_gemm_acc(qq, c["W"])
    assert dig(qq) == g["q_sha256"] and dig(xs.view(np.uint32)) == g["xs_bits_sha256"] and dig(acc) == g["acc_sha256"]
    assert qq.reshape(-1)[::g["stride"]].tolist() == g["q_sample"]
    d = oracle.epilogue(acc, xs, c["ws"], c["bias"], oracle.BF16, fma=1)
    assert dig(d) == g["d_fma_bits_sha256"] and d.reshape(-1)[::g["stride"]].tolist() == g["d_fma_bits_sample"]
    # the plain formula of the config text (scale = absmax/127, RNE, float product) lands within 1 code of the bf16 path
    x = synth.bf16_to_f32(c["x"])
    plain = np.clip(np.rint(x / (np.abs(x).max(1, keepdims=True) / np.float32(127))), -127, 127)
    assert np.abs(plain - qq).max() <= 1
    r = json.load(open(os.path.join(ROOT, "tests", "golden", "rotated_quant.json")))
    xr = synth.bf16_bits(synth.activations(11, 8, 1024, "t3"))
    assert dig(xr) == r["x_sha256"]
    for grp in (64, 128, 256):
        rc, q2, s2 = oracle.quant_rows(oracle.BF16, xr, 1024, grp)
        assert dig(q2) == r["q_g%d_sha256" % grp] and dig(s2.view(np.uint32)) == r["xs_bits_g%d_sha256" % grp]


def _write_checkpoint(path, extra=None, groupsize=256, scalar_scale=False):
    import torch
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(3)
    N, K = 64, 512
    t = {
        "blk.fc.weight": torch.randint(-127, 128, (N, K), dtype=torch.int8, generator=g),
        "blk.fc.weight_scale": torch.tensor([0.01]) if scalar_scale else torch.rand(N, generator=g) * 0.01 + 0.001,
        "blk.fc.bias": (torch.randn(N, generator=g) * 0.02).to(torch.bfloat16),
        "blk.fc.comfy_quant": torch.tensor(list(json.dumps({"format": "int8_tensorwise", "convrot": True,
                                                            "convrot_groupsize": groupsize}).encode()), dtype=torch.uint8),
        "blk.w6.weight": torch.randint(0, 256, (N, K * 3 // 4), dtype=torch.uint8, generator=g),
        "blk.w6.weight_s_rel": torch.randint(0x30, 0x50, (N, K // 32), dtype=torch.uint8, generator=g).view(torch.float8_e4m3fn),
        "blk.w6.weight_s_channel": torch.rand(N, generator=g) * 0.01,
        "blk.dense.weight": torch.randn(N, K, generator=g).to(torch.bfloat16),
    }
    t.update(extra or {})
    save_file(t, path)
    return t


def test_checkpoint_layouts_are_read_like_the_reference(tmp_path):
    import torch
    from safetensors import safe_open
    wts = pkg("weights")
    p = str(tmp_path / "a.safetensors")
    t = _write_checkpoint(p)
    with safe_open(p, framework="pt") as st:
        fc = wts.load_linear(st, "blk.fc", device="cpu")
        assert fc.kind == "int8_convrot" and (fc.n, fc.k) == (64, 512) and fc.scale.shape == (64,)
        assert torch.equal(fc.weight, t["blk.fc.weight"]) and fc.bias.dtype == torch.bfloat16
        w6 = wts.load_linear(st, "blk.w6", device="cpu")
        assert w6.kind == "w6" and (w6.n, w6.k) == (64, 512) and w6.s_rel.dtype == torch.uint8 and w6.s_rel.shape == (64, 16)
        assert wts.load_linear(st, "blk.dense", device="cpu").kind == "dense"
    # one scale for all rows is expanded on the host (src/relayvsr.rs:141-149)
    p2 = str(tmp_path / "b.safetensors")
    _write_checkpoint(p2, scalar_scale=True)
    with safe_open(p2, framework="pt") as st:
        s = wts.load_linear(st, "blk.fc", device="cpu").scale
        assert s.shape == (64,) and (s == s[0]).all()
    # other group sizes and scale counts are refused
    p3 = str(tmp_path / "c.safetensors")
    _write_checkpoint(p3, groupsize=64)
    with safe_open(p3, framework="pt") as st:
        with pytest.raises(wts.CheckpointError, match="groups of 256"):
            wts.load_linear(st, "blk.fc", device="cpu")
    p4 = str(tmp_path / "d.safetensors")
    _write_checkpoint(p4, extra={"blk.fc.weight_scale": torch.ones(7)})
    with safe_open(p4, framework="pt") as st:
        with pytest.raises(wts.CheckpointError, match="7 weight scales for 64 rows"):
            wts.load_linear(st, "blk.fc", device="cpu")


def test_makefile_and_build_script_list_the_same_units_and_flags():
    """The Makefile (native hosts) and build.py (this repository's Python side) must compile the same units with the
    same arithmetic flags, or the two libraries would differ in bits."""
    import importlib
    pkg_dir = os.path.join(ROOT, "comfyui-backend-but-rust_amd")
    mk = open(os.path.join(pkg_dir, "Makefile")).read()
    units = re.search(r"^UNITS\s*:=\s*(.+)$", mk, re.M).group(1).split()
    build = importlib.import_module("comfyui-backend-but-rust_amd.build")
    assert sorted(u + ".hip" for u in units) == sorted(build.SOURCES)
    flags = re.search(r"^FLAGS\s*:=\s*((?:.*\\\n)*.*)$", mk, re.M).group(1).replace("\\\n", " ").split()
    flags = [f.replace("$(ARCH)", build.ARCH) for f in flags]
    assert sorted(flags) == sorted(build.FLAGS)
    for src, extra in build.EXTRA.items():
        line = re.search(r"^csrc/%s\.o: FLAGS \+= (.+)$" % re.escape(src[:-4]), mk, re.M)
        assert line and line.group(1).split() == extra


def test_rust_host_crate_follows_the_headers_and_the_build_script():
    """rust/src/sys.rs is generated from the headers (same names, arity and scalar types as the ctypes table), and
    rust/build.rs compiles the units and flags that build.py does.  No Rust toolchain is needed for either check."""
    import importlib
    import subprocess
    import sys
    r = subprocess.run([sys.executable, os.path.join(ROOT, "rust", "gen_sys.py"), "--check"], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr
    text = open(os.path.join(ROOT, "rust", "src", "sys.rs")).read()
    decls = {m.group(1): m.group(2) for m in re.finditer(r"pub fn (gpu_\w+)\(([^)]*)\)", text)}
    assert set(decls) == set(header_functions()) | set(header_functions("gpu_blas_api.h"))
    # c_uint64 and c_size_t are one ctypes class on this platform
    kinds = {ffi._P: {"P", "PM"}, ffi._I64: {"i64"}, ffi._I32: {"i32"}, ffi._F32: {"f32"}, ffi._U64: {"u64", "usize"}}
    for table in (ffi.SIGNATURES, ffi.BLAS_SIGNATURES):
        for name, argtypes in table.items():
            rust = [a.split(":")[1].strip() for a in " ".join(decls[name].split()).split(",") if a.strip()]
            assert len(rust) == len(argtypes), name
            for rt, ct in zip(rust, argtypes):
                assert rt in kinds[ct], (name, rt, ct)
    build = importlib.import_module("comfyui-backend-but-rust_amd.build")
    rs = open(os.path.join(ROOT, "rust", "build.rs")).read()
    units = re.findall(r'"(\w+\.hip)"', rs[rs.index("const UNITS"):rs.index("];")])
    assert sorted(units) == sorted(build.SOURCES)
    for flag in build.FLAGS:
        if not flag.startswith("--offload-arch"):
            assert '"%s"' % flag in rs, flag
    for src, extra in build.EXTRA.items():
        assert src in rs and all('"%s"' % e in rs for e in extra)
