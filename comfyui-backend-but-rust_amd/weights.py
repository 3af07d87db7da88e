"""Quantized linears as the reference's checkpoints store them, and the launch sequence that runs one.

On-disk layout (safetensors), as read by the reference's loaders:
  int8 ConvRot   `<m>.weight` I8 [N, K], already in the rotated basis; `<m>.weight_scale` F32 [N] or a single value for
                 all rows (src/relayvsr.rs:141-149); optional `<m>.comfy_quant`, a byte tensor holding JSON
                 {"format": "int8_tensorwise", "convrot": true, "convrot_groupsize": 256}: anything but int8 ConvRot
                 with groups of 256 is refused (src/relayvsr.rs:123-136, src/h3.rs:289-292)
  W6             `<m>.weight` packed [N, 3K/4] (nibble plane, then 2-bit plane), `<m>.weight_s_rel` F8_E4M3 [N, K/32],
                 `<m>.weight_s_channel` F32 [N] (src/h3.rs:490-497)
  dense          `<m>.weight` in bf16 / f16 / f32
  all            optional `<m>.bias`
"""
import json
from dataclasses import dataclass
from typing import Optional

import torch

from . import ffi, qlinear


class CheckpointError(ValueError):
    pass


@dataclass
class Linear:
    kind: str                       # "int8_convrot", "w6" or "dense"
    n: int
    k: int
    weight: torch.Tensor            # int8 [N,K] | uint8 packed [N,3K/4] | float [N,K]
    scale: Optional[torch.Tensor] = None      # f32 [N]: row scales (int8) or s_channel (w6)
    s_rel: Optional[torch.Tensor] = None      # uint8 e4m3 bits [N, K/32] (w6)
    bias: Optional[torch.Tensor] = None


def _has(st, key):
    return key in st.keys()


def load_linear(st, name, device="cuda:0", bias_dtype=None):
    """`st`: an open safetensors file (safetensors.safe_open(path, framework="pt")).  `name`: the prefix of `.weight`."""
    w = st.get_tensor(name + ".weight")
    bias = st.get_tensor(name + ".bias") if _has(st, name + ".bias") else None
    if bias is not None:
        bias = bias.to(device=device, dtype=bias_dtype or bias.dtype)
    if _has(st, name + ".weight_s_rel"):
        s_rel = st.get_tensor(name + ".weight_s_rel")
        s_ch = st.get_tensor(name + ".weight_s_channel").float()
        n = w.shape[0]
        if w.shape[1] % 3:
            raise CheckpointError("%s: packed W6 rows of %d bytes" % (name, w.shape[1]))
        k = w.shape[1] * 4 // 3
        if tuple(s_rel.shape) != (n, k // 32) or s_ch.numel() != n:
            raise CheckpointError("%s: W6 scales %s / %s for [%d, %d]" % (name, tuple(s_rel.shape), tuple(s_ch.shape), n, k))
        return Linear("w6", n, k, w.view(torch.uint8).to(device), s_ch.reshape(n).to(device), s_rel.view(torch.uint8).to(device), bias)
    if w.dtype == torch.int8:
        q = name + ".comfy_quant"
        if _has(st, q):
            cfg = json.loads(bytes(st.get_tensor(q).view(torch.uint8).tolist()))
            fmt = cfg.get("format")
            if cfg.get("convrot") is not True or cfg.get("convrot_groupsize") != 256 or (isinstance(fmt, str) and not fmt.startswith("int8")):
                raise CheckpointError("%s: only int8 ConvRot (groups of 256) weights run here, not %s" % (name, cfg))
        n, k = w.shape
        s = st.get_tensor(name + ".weight_scale").float().reshape(-1)
        if s.numel() == 1:
            s = s.expand(n).contiguous()
        elif s.numel() != n:
            raise CheckpointError("%s: %d weight scales for %d rows" % (name, s.numel(), n))
        return Linear("int8_convrot", n, k, w.to(device), s.to(device), None, bias)
    return Linear("dense", w.shape[0], w.shape[1], w.to(device), None, None, bias)


def forward(lin, x, out_dtype=torch.bfloat16):
    """y = x W^T + b with the launches the reference issues for this storage form (src/dit.rs:550-555,
    src/h3.rs:1208-1251): quantize rows with the 256-wide rotation, then the int8 GEMM; W6 weights are decoded to the
    int8 grid first; dense weights go to gpu_gemm."""
    if lin.kind == "dense":
        return qlinear.gemm(x, lin.weight, lin.bias, True, out_dtype)
    q, xs = qlinear.quant_rows(x, 1)
    if lin.kind == "w6":
        return qlinear.w6a8_gemm(q, lin.weight, lin.s_rel, 32, xs, lin.scale, lin.bias, out_dtype)
    return qlinear.int8_gemm(q, lin.weight, xs, lin.scale, lin.bias, out_dtype)
