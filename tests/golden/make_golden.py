"""Regenerates tests/golden/*.json from the CPU oracle and the counter-hashed synthetic inputs.

The reference holds no golden vector for this path and cannot be built or imported offline, so nothing here comes from
running reference code: expected values are the oracle's, whose functions are pinned independently in
tests/test_oracle_pins.py.  Inputs are not stored (they are a pure function of the seed); outputs are stored as every
61st value plus a SHA-256 of the whole tensor, the layout the reference's own GPU golden test uses
(tests/sparse_attn_match_comfy.rs:10-43, tools/sparse_attn_ref.py:18).

Run from the repository root:  python tests/golden/make_golden.py
"""
import hashlib
import importlib
import json
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle  # noqa: E402

synth = importlib.import_module("comfyui-backend-but-rust_amd.synth")
STRIDE = 61


def digest(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def sample(a):
    return np.ascontiguousarray(a).reshape(-1)[::STRIDE].tolist()


def pack(name, a):
    return {name + "_sha256": digest(a), name + "_sample": sample(a)}


def config0():
    c = synth.config0(0)
    rc, q, xs = oracle.quant_rows(oracle.BF16, c["x"], c["K"], 0)
    assert rc == 0
    acc = oracle.int8_gemm_acc(q, c["W"])
    d1 = oracle.epilogue(acc, xs, c["ws"], c["bias"], oracle.BF16, fma=1)
    d0 = oracle.epilogue(acc, xs, c["ws"], c["bias"], oracle.BF16, fma=0)
    out = {"config": "config 0: W8A8 linear, M=256 K=1024 N=1024, seed 0, no rotation", "stride": STRIDE,
           "x_sha256": digest(c["x"]), "W_sha256": digest(c["W"]), "ws_sha256": digest(c["ws"]),
           "bias_sha256": digest(c["bias"])}
    out.update(pack("q", q))
    out.update(pack("xs_bits", xs.view(np.uint32)))
    out.update(pack("acc", acc))
    out.update(pack("d_fma_bits", d1))
    out.update(pack("d_nofma_bits", d0))
    return out


def rotated():
    """A small rotated case per group width: codes and scales of 8 rows of K = 1024."""
    out = {"stride": STRIDE}
    x = synth.bf16_bits(synth.activations(11, 8, 1024, "t3"))
    out["x_sha256"] = digest(x)
    for g in (64, 128, 256):
        rc, q, xs = oracle.quant_rows(oracle.BF16, x, 1024, g)
        assert rc == 0
        out.update(pack("q_g%d" % g, q))
        out.update(pack("xs_bits_g%d" % g, xs.view(np.uint32)))
    return out


if __name__ == "__main__":
    here = os.path.dirname(os.path.abspath(__file__))
    for name, fn in (("config0_w8a8.json", config0), ("rotated_quant.json", rotated)):
        with open(os.path.join(here, name), "w") as f:
            json.dump(fn(), f)
        print("wrote", name, os.path.getsize(os.path.join(here, name)), "bytes")
