#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

A step is one W8A8 linear over one batch of synthetic activations already resident in HBM: per-token int8
quantization with the ConvRot rotation (gpu_quant_rows), then the int8 GEMM with the fused dequant/bias epilogue
(gpu_int8_gemm).  The default workload is the one the headline metric is quoted on: the image-DiT MLP up-projection,
M=4608 tokens, K=3072, N=12288, bf16 in and out, Hadamard block 128.

Prints ONE JSON line: whole-step throughput in TOPS (2*M*N*K per step), the roofline of the dominant kernel (the int8
GEMM against the dense int8 MFMA peak) from HIP events recorded inside the timed region, the CPU oracle timed on a
bounded row sample, the memory-bound skinny (M=256) linears as HBM GB/s, the other linears of the model configurations
and the W6A8 (packed 6-bit weights, unpack fused into the GEMM) pair.
"""
import argparse
import importlib
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA, 5.0 POP/s
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E, 8 TB/s
SETTLE_MS = 150.0         # untimed load before every timed loop, see settle()
LAST_SPREAD = {}
EVENT_KIND = [None]       # which kind of events the last time_linear() used


class StreamEvents:
    """HIP timing events created with hipEventDisableSystemFence, recorded on the launch stream.  An event with the
    default flags makes the command processor write back and invalidate the caches at system scope when it completes;
    between two kernels that costs 1.5-2 us of the following kernel's interval each time.  The flag is the one the HIP
    headers name for events that only measure time.  torch.cuda.Event has no way to pass it, so the three runtime calls
    are made through ctypes on the HIP runtime the process has already loaded; if that runtime cannot be reached this
    way, torch's default-flag events are used instead and `kind` says so."""
    DISABLE_SYSTEM_FENCE = 0x20000000

    def __init__(self, torch, n, stream):
        self.kind = "hipEventDisableSystemFence"
        self.ev = []
        try:
            import ctypes
            self.c = ctypes
            self.hip = ctypes.CDLL("libamdhip64.so")
            self.hip.hipEventCreateWithFlags.argtypes = [ctypes.POINTER(ctypes.c_void_p), ctypes.c_uint]
            self.hip.hipEventRecord.argtypes = [ctypes.c_void_p, ctypes.c_void_p]
            self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
            self.hip.hipEventDestroy.argtypes = [ctypes.c_void_p]
            self.stream = ctypes.c_void_p(stream.cuda_stream)
            for _ in range(n):
                e = ctypes.c_void_p()
                self._ok(self.hip.hipEventCreateWithFlags(ctypes.byref(e), self.DISABLE_SYSTEM_FENCE), "hipEventCreateWithFlags")
                self.ev.append(e)
            # one recorded pair must read back, or the runtime reached here is not the one torch launches on
            self.record(0); self.record(1)
            torch.cuda.synchronize()
            self.ms(0, 1)
        except (OSError, AttributeError, RuntimeError) as err:
            print("bench.py: timing-only HIP events unavailable (%s); using torch's events" % err, file=sys.stderr)
            self.close()
            self.kind = "torch default flags"
            self.hip = None
            self.tstream = stream
            self.ev = [torch.cuda.Event(enable_timing=True) for _ in range(n)]

    @staticmethod
    def _ok(rc, what):
        if rc != 0:
            raise RuntimeError("%s failed with HIP error %d" % (what, rc))

    def record(self, i):
        if self.hip is None:
            self.ev[i].record(self.tstream)
        else:
            self._ok(self.hip.hipEventRecord(self.ev[i], self.stream), "hipEventRecord")

    def ms(self, i, j):
        if self.hip is None:
            return self.ev[i].elapsed_time(self.ev[j])
        f = self.c.c_float()
        self._ok(self.hip.hipEventElapsedTime(self.c.byref(f), self.ev[i], self.ev[j]), "hipEventElapsedTime")
        return f.value

    def close(self):
        if getattr(self, "hip", None) is not None:
            for e in self.ev:
                self.hip.hipEventDestroy(e)
        self.ev = []


def settle(torch, fn, ms=SETTLE_MS):
    """Runs `fn` untimed for about `ms` milliseconds of GPU time.  After any idle gap (0.2 s is enough: host-side input
    generation between two measurements) the part's power management holds the shader clock down and lets it rise over
    the next 30-40 ms of sustained load: the same step measures 190-210 us in its first 30 calls and 162 us from call
    200 on.  A serving loop runs in the settled state, so every timed loop here starts from it."""
    st = torch.cuda.current_stream()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    fn()
    e0.record(st)
    fn()
    fn()
    e1.record(st)
    torch.cuda.synchronize()
    per = max(e0.elapsed_time(e1) / 2.0, 1e-3)
    for _ in range(min(20000, int(ms / per) + 1)):
        fn()


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--shape", default="4608,3072,12288", help="M,K,N of the timed linear")
    ap.add_argument("--rotate", type=int, default=128, help="Hadamard block (0 = none, 64, 128, 256)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-skinny", action="store_true")
    ap.add_argument("--no-extra", action="store_true", help="skip the other linears of the model configurations and the W6A8 shapes")
    ap.add_argument("--no-graph", action="store_true", help="skip the captured-graph replays of the linears")
    ap.add_argument("--attention-only", action="store_true",
                    help="time only the INT8 attention shapes and print them as one JSON line (for profiling that path alone)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="target CPU time of the baseline sample")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run a plain 256 MiB device copy a few times: under rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE its "
                         "known size calibrates the counters that roofline.traffic is derived from")
    return ap.parse_args()


def make_inputs(torch, synth, M, K, N, seed=0, dev="cuda:0", kind="t3"):
    import numpy as np
    x = synth.bf16_bits(synth.activations(seed, M, K, kind))
    W, ws, bias = synth.w8_weights(seed, N, K)
    bias = synth.bf16_bits(bias)
    host = dict(x=x, W=W, ws=ws, bias=bias)
    t = lambda a: torch.from_numpy(np.ascontiguousarray(a)).to(dev)
    devs = dict(x=t(x.view(np.int16)).view(torch.bfloat16), W=t(W), ws=t(ws),
                bias=t(bias.view(np.int16)).view(torch.bfloat16))
    return host, devs


def time_linear(torch, ffi, d, M, K, N, rotate, steps, warmup, nbuf=1, settled=True):
    """Times `steps` linears; returns (ms_total, ms_quant_avg, ms_gemm_avg).  nbuf > 1 rotates among copies of the
    weights so that a memory-bound shape cannot live in the 256 MB last-level cache."""
    st = torch.cuda.current_stream()
    s = st.cuda_stream
    q = torch.empty((M, K), dtype=torch.int8, device="cuda:0")
    xs = torch.empty((M,), dtype=torch.float32, device="cuda:0")
    D = torch.empty((M, N), dtype=torch.bfloat16, device="cuda:0")
    Ws = [d["W"]] + [d["W"].clone() for _ in range(nbuf - 1)]

    # Two events per step: one in front of the quantizer (event 2i), one between the two launches (2i+1); the event in
    # front of the next step's quantizer (one more after the last step) closes the GEMM's interval.
    def step(i, evs=None):
        W = Ws[i % nbuf]
        if evs: evs.record(2 * i)
        ffi.k("gpu_quant_rows", ffi.DT_BF16, ffi.PRO_PLAIN, d["x"].data_ptr(), K, 0, 0, 0, 0, 0.0, 0, 0, q.data_ptr(),
              xs.data_ptr(), M, K, rotate, s)
        if evs: evs.record(2 * i + 1)
        ffi.k("gpu_int8_gemm", q.data_ptr(), W.data_ptr(), xs.data_ptr(), d["ws"].data_ptr(), d["bias"].data_ptr(),
              D.data_ptr(), M, N, K, ffi.DT_BF16, s)

    if settled:
        settle(torch, lambda: step(0))
    for i in range(warmup):
        step(i)
    evs = StreamEvents(torch, 2 * steps + 1, st)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        step(i, evs)
    evs.record(2 * steps)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    gpu_ms = evs.ms(0, 2 * steps)
    tqs = sorted(evs.ms(2 * i, 2 * i + 1) for i in range(steps))
    tgs = sorted(evs.ms(2 * i + 1, 2 * i + 2) for i in range(steps))
    tq, tg = sum(tqs) / steps, sum(tgs) / steps
    EVENT_KIND[0] = evs.kind
    evs.close()
    LAST_SPREAD.clear()
    LAST_SPREAD.update(quant_rows_us_median=round(tqs[steps // 2] * 1e3, 2), quant_rows_us_min=round(tqs[0] * 1e3, 2),
                       int8_gemm_us_median=round(tgs[steps // 2] * 1e3, 2), int8_gemm_us_min=round(tgs[0] * 1e3, 2))
    return max(gpu_ms, 0.0), wall_ms, tq, tg


def time_linear_graph(torch, ffi, d, M, K, N, rotate, steps, nbuf):
    """The same linear (quantizer + GEMM, rotating among `nbuf` weight copies) captured once into a HIP graph of `nbuf`
    steps and replayed: microseconds per step as a serving loop that replays graphs sees them, without the host's launch
    calls and with whatever the runtime saves between the kernels of a graph."""
    q = torch.empty((M, K), dtype=torch.int8, device="cuda:0")
    xs = torch.empty((M,), dtype=torch.float32, device="cuda:0")
    D = torch.empty((M, N), dtype=torch.bfloat16, device="cuda:0")
    Ws = [d["W"]] + [d["W"].clone() for _ in range(nbuf - 1)]
    side = torch.cuda.Stream()

    def step(i, s):
        ffi.k("gpu_quant_rows", ffi.DT_BF16, ffi.PRO_PLAIN, d["x"].data_ptr(), K, 0, 0, 0, 0, 0.0, 0, 0, q.data_ptr(),
              xs.data_ptr(), M, K, rotate, s)
        ffi.k("gpu_int8_gemm_static", q.data_ptr(), Ws[i % nbuf].data_ptr(), xs.data_ptr(), d["ws"].data_ptr(), d["bias"].data_ptr(),
              D.data_ptr(), M, N, K, ffi.DT_BF16, s)

    with torch.cuda.stream(side):
        step(0, side.cuda_stream)            # first call outside the capture: attributes, the static scratch's address
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            for i in range(nbuf):
                step(i, side.cuda_stream)
        reps = max(1, steps // nbuf)
        for _ in range(max(2, int(0.1 / (nbuf * 40e-6)))):   # about 100 ms of replays: the settled power state
            g.replay()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record(side)
        for _ in range(reps):
            g.replay()
        e1.record(side)
        torch.cuda.synchronize()
    return e0.elapsed_time(e1) / (reps * nbuf) * 1e3


def time_w6a8(torch, ffi, M, K, N, steps, warmup):
    """The group-scaled W6A8 GEMM (24-bit words of four 6-bit codes, fp32 scales per 128 along K) on synthetic weights
    with codes uniform in [-31, 31]; returns the average microseconds of gpu_w6a8_group_gemm as it dispatches by itself
    (at these M the call expands the weights into scratch first, then runs the GEMM kernel on them), with the unpack
    forced inside the GEMM kernel, and with the expansion forced."""
    g = torch.Generator(device="cuda:0").manual_seed(4)
    u = torch.randint(1, 64, (N, K // 4, 4), dtype=torch.int32, device="cuda:0", generator=g)   # u = q + 32
    w = u[..., 0] | (u[..., 1] << 6) | (u[..., 2] << 12) | (u[..., 3] << 18)
    packed = torch.stack((w & 255, (w >> 8) & 255, w >> 16), dim=-1).to(torch.uint8).reshape(N, K // 4 * 3).contiguous()
    del u, w
    A = torch.randint(-127, 128, (M, K), dtype=torch.int8, device="cuda:0", generator=g)
    xs = torch.rand(M, device="cuda:0", generator=g) * 0.1 + 0.01
    sw = torch.rand(N, K // 128, device="cuda:0", generator=g) * 9e-3 + 1e-3
    bias = (torch.randn(N, device="cuda:0", generator=g) * 0.02).to(torch.bfloat16)
    D = torch.empty((M, N), dtype=torch.bfloat16, device="cuda:0")
    st = torch.cuda.current_stream()

    def run():
        ffi.k("gpu_w6a8_group_gemm", A.data_ptr(), packed.data_ptr(), xs.data_ptr(), sw.data_ptr(), bias.data_ptr(), D.data_ptr(),
              0, M, N, K, ffi.DT_BF16, st.cuda_stream)

    settle(torch, run)
    res = []
    for mode in (-1, 0, 1):
        ffi.raw("gpu_internal_w6a8_group_gemm_mode", mode)
        for _ in range(warmup):
            run()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(st)
        for _ in range(steps):
            run()
        e1.record(st)
        torch.cuda.synchronize()
        res.append(e0.elapsed_time(e1) / steps * 1e3)
    ffi.raw("gpu_internal_w6a8_group_gemm_mode", -1)
    return tuple(res)


def time_w6_reference_format(torch, ffi, M, K, N, steps, warmup):
    """The reference's own W6 format (two planes + e4m3 scale per 32 + f32 row scale) at an H3 linear's shape:
    gpu_w6_decode alone, gpu_w6a8_gemm (decode into a stream-ordered buffer, then the int8 GEMM), and gpu_int8_gemm alone on
    the decoded weights, in microseconds.  The last is what a kernel that decoded inside the GEMM could at best reach:
    it would do the GEMM's work plus the decode's arithmetic on the same CUs."""
    dev = "cuda:0"
    g = torch.Generator(device=dev).manual_seed(5)
    wq = torch.randint(0, 256, (N, K // 4 * 3), dtype=torch.uint8, device=dev, generator=g)
    # e4m3 bytes with exponent field 6..8 and any mantissa: scales in [0.5, 3.75]
    s_rel = (torch.randint(6, 9, (N, K // 32), device=dev, generator=g) * 8 + torch.randint(0, 8, (N, K // 32), device=dev, generator=g)).to(torch.uint8)
    s_ch = torch.rand(N, device=dev, generator=g) * 9e-3 + 1e-3
    A = torch.randint(-127, 128, (M, K), dtype=torch.int8, device=dev, generator=g)
    xs = torch.rand(M, device=dev, generator=g) * 0.1 + 0.01
    w8 = torch.empty((N, K), dtype=torch.int8, device=dev)
    D = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    st = torch.cuda.current_stream()
    s = st.cuda_stream

    def timed(fn):
        settle(torch, fn)
        for _ in range(warmup):
            fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(st)
        for _ in range(steps):
            fn()
        e1.record(st)
        torch.cuda.synchronize()
        return e0.elapsed_time(e1) / steps * 1e3

    dec = timed(lambda: ffi.k("gpu_w6_decode", wq.data_ptr(), s_rel.data_ptr(), w8.data_ptr(), N, K, 32, s))
    lin = timed(lambda: ffi.k("gpu_w6a8_gemm", A.data_ptr(), wq.data_ptr(), s_rel.data_ptr(), 32, xs.data_ptr(), s_ch.data_ptr(), 0,
                              D.data_ptr(), M, N, K, ffi.DT_BF16, s))
    bias0 = torch.zeros(N, dtype=torch.bfloat16, device=dev)
    gemm = timed(lambda: ffi.k("gpu_int8_gemm", A.data_ptr(), w8.data_ptr(), xs.data_ptr(), s_ch.data_ptr(), bias0.data_ptr(),
                               D.data_ptr(), M, N, K, ffi.DT_BF16, s))
    return dec, lin, gemm


def time_mfma_ceiling(torch, ffi):
    """The matrix pipes alone: four waves per CU issuing nothing but v_mfma_i32_32x32x32_i8 on register operands, with
    pseudo-random and with all-zero bits, and the same with v_mfma_i32_16x16x64_i8 (the form the large-shape GEMM uses:
    the same operations per cycle, accumulators touched half as often).  The chip's power management sets the clock by
    what the instructions toggle, so this is the ceiling any int8 GEMM on this part runs under; the kernel's own
    shader-clock counts give that clock."""
    dev = "cuda:0"
    cu = torch.cuda.get_device_properties(0).multi_processor_count
    cyc = torch.zeros(cu, dtype=torch.int64, device=dev)
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    st = torch.cuda.current_stream()
    iters, reps = 600, 10
    out = {"kernel": "gpu_mfma_ceiling_probe: %d workgroups x 4 waves x %d x 64 MFMA" % (cu, iters)}
    for name, rnd in (("random_bits", 1), ("zero_bits", 0), ("random_bits_16x16x64", 3), ("zero_bits_16x16x64", 2)):
        run = lambda: ffi.k("gpu_mfma_ceiling_probe", iters, rnd, cyc.data_ptr(), sink.data_ptr(), st.cuda_stream)
        settle(torch, run)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(st)
        for _ in range(reps):
            run()
        e1.record(st)
        torch.cuda.synchronize()
        ms = e0.elapsed_time(e1) / reps
        ops = cu * 4.0 * iters * 64 * 65536
        cycles = float(cyc.double().mean().item())
        out[name] = {"TOPS": round(ops / ms / 1e9, 1), "frac_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4),
                     "shader_clock_GHz": round(cycles / (ms * 1e6), 3), "cycles_per_mfma": round(cycles / (iters * (128.0 if rnd & 2 else 64.0)), 2)}
    return out


def time_row_kernels(torch, ffi, steps):
    """The HBM-bound kernels either side of the GEMM, each timed alone with HIP events on the launch stream: name,
    microseconds and algorithmic GB/s (bytes the call must read and write once)."""
    dev = "cuda:0"
    st = torch.cuda.current_stream()
    s = st.cuda_stream
    g = torch.Generator(device=dev).manual_seed(7)
    P = lambda t: 0 if t is None else t.data_ptr()
    out = []

    def timed(name, nbytes, fn):
        settle(torch, fn)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(st)
        for _ in range(steps):
            fn()
        e1.record(st)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        out.append({"name": name, "us": round(us, 2), "GBs": round(nbytes / us / 1e3, 1),
                    "frac_hbm": round(nbytes / us / 1e3 / PEAK_HBM_GBS, 4)})

    M, K = 4608, 3072
    x = torch.randn(M, 2 * K, device=dev, generator=g).to(torch.bfloat16)
    w = torch.rand(K, device=dev, generator=g) + 0.5
    ms = (torch.randn(K, device=dev, generator=g) * 0.3).to(torch.bfloat16)
    q = torch.empty((M, K), dtype=torch.int8, device=dev)
    xs = torch.empty((M,), dtype=torch.float32, device=dev)
    quant = lambda pro, xs_, up, nw, m_, sh_: ffi.k("gpu_quant_rows", ffi.DT_BF16, pro, x.data_ptr(), xs_, 0, 0, up, P(nw), 1e-6,
                                                    P(m_), P(sh_), q.data_ptr(), xs.data_ptr(), M, K, 1, s)
    timed("gpu_quant_rows PLAIN rotate 256, M=4608 K=3072 bf16", M * K * 3, lambda: quant(ffi.PRO_PLAIN, 2 * K, 0, None, None, None))
    timed("gpu_quant_rows RMS + modulation, rotate 256", M * K * 3,
          lambda: quant(ffi.PRO_RMS, 2 * K, 0, w, ms, ms))
    timed("gpu_quant_rows SWIGLU, rotate 256", M * K * 5, lambda: quant(ffi.PRO_SWIGLU, 2 * K, K, None, None, None))
    Ms, I = 8192, 2560
    xg = torch.randn(Ms, 2 * I, device=dev, generator=g).to(torch.float16)
    qs = torch.empty((Ms, I), dtype=torch.int8, device=dev)
    ss = torch.empty((Ms,), dtype=torch.float32, device=dev)
    timed("gpu_sd_quant_rows rotate 64, M=8192 K=2560 f16", Ms * I * 3,
          lambda: ffi.k("gpu_sd_quant_rows", xg.data_ptr(), 2 * I, qs.data_ptr(), ss.data_ptr(), Ms, I, 64, s))
    timed("gpu_sd_geglu_quant_rows rotate 64, M=8192 I=2560", Ms * I * 5,
          lambda: ffi.k("gpu_sd_geglu_quant_rows", xg.data_ptr(), qs.data_ptr(), ss.data_ptr(), Ms, I, 64, s))
    N = 12288
    wq = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=g)
    wsc = torch.rand(N, device=dev, generator=g) * 0.01 + 0.001
    wf = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    w32 = torch.empty((N, K), dtype=torch.float32, device=dev)
    timed("gpu_convrot_dequant bf16, N=12288 K=3072", N * K * 3,
          lambda: ffi.k("gpu_convrot_dequant", ffi.DT_BF16, wq.data_ptr(), wsc.data_ptr(), wf.data_ptr(), N, K, s))
    timed("gpu_convrot_requant bf16 stochastic, N=12288 K=3072", N * K * 3,
          lambda: ffi.k("gpu_convrot_requant", ffi.DT_BF16, wf.data_ptr(), wq.data_ptr(), wsc.data_ptr(), N, K, 12345, s))
    timed("gpu_dequant_i8, N=12288 K=3072", N * K * 5,
          lambda: ffi.k("gpu_dequant_i8", wq.data_ptr(), wsc.data_ptr(), w32.data_ptr(), N, K, s))
    return out


def time_attention(torch, ffi, steps):
    """INT8 attention (quantizers + attention kernel, one call), HIP events on the launch stream: the image-DiT joint
    attention as the plain call, as the DiT issues it (fused q/k norm + RoPE) and with a per-key bias; a long video
    shape; the SDXL UNet's head dim 64 in fp16.  ops = 4 * b * h * lq * lk * head_dim (the two matrix products)."""
    dev = "cuda:0"
    st = torch.cuda.current_stream()
    g = torch.Generator(device=dev).manual_seed(11)
    out = []
    cases = (("image-dit joint attention", "gpu_int8_attn_d", 1, 4608, 24, 24, 128, torch.bfloat16),
             ("image-dit joint attention, fused q/k norm + rope", "gpu_int8_attn_norm_rope", 1, 4608, 24, 24, 128, torch.bfloat16),
             ("image-dit joint attention, per-key bias", "gpu_int8_attn_key_bias", 1, 4608, 24, 24, 128, torch.bfloat16),
             ("long video attention", "gpu_int8_attn_d", 2, 8192, 16, 16, 128, torch.bfloat16),
             ("sdxl self-attention 64x64 latent, 10 heads of 64", "gpu_int8_attn_f16", 2, 4096, 10, 10, 64, torch.float16))
    for (name, entry, b, l, h, hk, hd, dtype) in cases:
        q, k, v = (torch.randn(b, l, hh, hd, device=dev, generator=g).to(dtype) for hh in (h, hk, hk))
        o = torch.empty_like(q)
        nws = ffi.lib.gpu_int8_attn_key_bias_workspace(b, h, hk, l, l) if entry.endswith("key_bias") else ffi.lib.gpu_int8_attn_workspace_d(b, h, hk, l, l, hd)
        ws = torch.empty((nws,), dtype=torch.uint8, device=dev)
        sq, sk = q.stride(), k.stride()
        head = (q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ws.data_ptr(), b, l, l, h, hk)
        strides = (sq[0], sq[1], sq[2], sk[0], sk[1], sk[2], sk[0], sk[1], sk[2], sq[0], sq[1], sq[2])
        if entry == "gpu_int8_attn_norm_rope":
            qw, kw = (1.0 + 0.1 * torch.randn(hd, device=dev, generator=g) for _ in range(2))
            ang = torch.arange(l, device=dev, dtype=torch.float32)[:, None] * torch.exp(-6.0 * torch.rand(hd // 2, device=dev, generator=g))[None, :]
            rope = torch.stack([torch.cos(ang), torch.sin(ang)], -1).contiguous()
            call = lambda: ffi.k(entry, *head, *strides, hd ** -0.5, qw.data_ptr(), kw.data_ptr(), 1e-6, rope.data_ptr(), 1, st.cuda_stream)
        elif entry == "gpu_int8_attn_key_bias":
            bias = torch.zeros(l, device=dev)
            bias[torch.randint(0, l, (l // 16,), device=dev, generator=g)] = 0.6
            call = lambda: ffi.k(entry, *head, *strides, hd ** -0.5, bias.data_ptr(), st.cuda_stream)
        else:
            call = lambda: ffi.k(entry, *head, hd, *strides, hd ** -0.5, st.cuda_stream)
        settle(torch, call)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        e0.record(st)
        for _ in range(steps):
            call()
        e1.record(st)
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        ops = 4.0 * b * h * l * l * hd
        out.append({"name": name, "b": b, "lq": l, "lk": l, "h": h, "hk": hk, "head_dim": hd, "kernel": entry,
                    "us": round(us, 1), "TOPS": round(ops / us / 1e6, 1), "frac_int8_peak": round(ops / us / 1e6 / PEAK_INT8_TOPS, 4)})
        del q, k, v, o, ws
    return out


def cpu_baseline(host, M, K, N, rotate, target_s):
    """The oracle's whole linear (quantize, int32 GEMM, epilogue) on a row sample sized for about `target_s` seconds."""
    import oracle
    threads = min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16")))
    rows = min(M, 64)
    t0 = time.perf_counter()
    rc, _, used = oracle.linear_w8a8(oracle.BF16, host["x"][:rows], rotate, host["W"], host["ws"], host["bias"], oracle.BF16,
                                     threads=threads)
    dt = time.perf_counter() - t0
    assert rc == 0
    rows2 = int(min(M, max(rows, rows * target_s / max(dt, 1e-3))))
    rows2 -= rows2 % threads if rows2 > threads else 0
    t0 = time.perf_counter()   # one untimed pass at the sample size: the first call's time includes thread start-up and cold caches
    rc, _, used = oracle.linear_w8a8(oracle.BF16, host["x"][:rows2], rotate, host["W"], host["ws"], host["bias"], oracle.BF16,
                                     threads=threads)
    assert rc == 0
    reps = max(1, int(round(target_s / max(time.perf_counter() - t0, 1e-3))))   # whole passes when M rows take under the target
    t0 = time.perf_counter()
    for _ in range(reps):
        rc, _, used = oracle.linear_w8a8(oracle.BF16, host["x"][:rows2], rotate, host["W"], host["ws"], host["bias"],
                                         oracle.BF16, threads=threads)
        assert rc == 0
    dt = (time.perf_counter() - t0) / reps
    return {"value": 2.0 * rows2 * N * K / dt / 1e12, "unit": "TOPS", "cores": used, "kind": "port",
            "sample": "first %d of %d rows, whole linear (quantize + int32 GEMM + epilogue), %d passes of %.2f s" % (rows2, M, reps, dt)}


def cpu_config0(synth, target_s=1.5):
    """BASELINE.json's configuration 0 (M=256, K=1024, N=1024, no rotation) on the host's cores: the oracle's whole
    linear timed in full, with one thread and with all of them."""
    import oracle
    M, K, N = 256, 1024, 1024
    x = synth.bf16_bits(synth.activations(0, M, K, "normal"))
    W, ws, bias = synth.w8_weights(0, N, K)
    bias = synth.bf16_bits(bias)
    out = {"M": M, "K": K, "N": N, "kind": "port", "unit": "TOPS"}
    for label, threads in (("one_thread", 1), ("all_threads", min(os.cpu_count() or 1, int(os.environ.get("OMP_NUM_THREADS", "16"))))):
        t0 = time.perf_counter()
        rc, _, used = oracle.linear_w8a8(oracle.BF16, x, 0, W, ws, bias, oracle.BF16, threads=threads)
        assert rc == 0
        reps = max(1, int(round(target_s / max(time.perf_counter() - t0, 1e-4))))
        t0 = time.perf_counter()
        for _ in range(reps):
            rc, _, used = oracle.linear_w8a8(oracle.BF16, x, 0, W, ws, bias, oracle.BF16, threads=threads)
            assert rc == 0
        dt = (time.perf_counter() - t0) / reps
        out[label] = {"value": round(2.0 * M * N * K / dt / 1e12, 5), "ms": round(dt * 1e3, 3), "cores": used, "passes": reps}
    return out


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (--gpus %d refused)" % a.gpus, file=sys.stderr)
        sys.exit(2)
    import torch
    ffi = importlib.import_module("comfyui-backend-but-rust_amd.ffi")
    synth = importlib.import_module("comfyui-backend-but-rust_amd.synth")
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(1)
    M, K, N = (int(v) for v in a.shape.split(","))
    if a.attention_only:
        print(json.dumps({"attention": time_attention(torch, ffi, max(5, min(40, a.steps // 3)))}))
        return
    if a.copy_probe:
        src = torch.empty(256 << 20, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    host, d = make_inputs(torch, synth, M, K, N)
    # the same loop from an idle GPU first (reported beside the headline, not as it), then from the settled power state
    time.sleep(0.5)
    _, cold_wall, cold_tq, cold_tg = time_linear(torch, ffi, d, M, K, N, a.rotate, min(a.steps, 50), min(a.warmup, 10), settled=False)
    gpu_ms, wall_ms, tq, tg = time_linear(torch, ffi, d, M, K, N, a.rotate, a.steps, a.warmup)
    spread = dict(LAST_SPREAD)
    ops = 2.0 * M * N * K
    ms_per_step = wall_ms / a.steps
    value = ops / (ms_per_step * 1e-3) / 1e12
    gemm_tops = ops / (tg * 1e-3) / 1e12
    quant_bytes = M * K * 2 + M * K + M * 4
    traffic = None   # HBM bytes per GEMM launch, measured off-line with rocprofv3 counters (profiles/hbm_traffic.json)
    try:
        with open(os.path.join(ROOT, "profiles", "hbm_traffic.json")) as f:
            rec = json.load(f).get("int8_gemm M%d K%d N%d bf16" % (M, K, N))
        traffic = rec["bytes"] if rec else None
    except (OSError, ValueError):
        pass
    out = {
        "metric": "W8A8 linear TOPS @M%d K%d N%d (quantize + int8 GEMM + dequant epilogue)" % (M, K, N),
        "value": round(value, 2), "unit": "TOPS", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic", "settle_ms": SETTLE_MS, "events": EVENT_KIND[0],
        "config": {"workload": "image-DiT MLP up-projection W8A8 linear, bf16 activations M=%d K=%d -> N=%d, Hadamard "
                               "block %d, per-channel scales, bf16 bias and output" % (M, K, N, a.rotate),
                   "M": M, "K": K, "N": N, "rotate": a.rotate},
        "roofline": {"bound": "mfma", "kernel": "int8_gemm_pp_kernel (gpu_int8_gemm, one launch: 256x256 tiles for the rows that fill whole rounds, 128x256 tiles for the rest; v_mfma_i32_16x16x64_i8)", "achieved": round(gemm_tops, 2),
                     "peak": PEAK_INT8_TOPS, "unit": "TOP/s", "frac": round(gemm_tops / PEAK_INT8_TOPS, 4),
                     "frac_median": round(ops / (spread["int8_gemm_us_median"] * 1e-6) / 1e12 / PEAK_INT8_TOPS, 4),
                     "frac_best": round(ops / (spread["int8_gemm_us_min"] * 1e-6) / 1e12 / PEAK_INT8_TOPS, 4),
                     "traffic": traffic, "avg_launch_us": round(tg * 1e3, 2),
                     "algorithmic_ops": ops, "algorithmic_bytes": M * K + M * 4 + N * K + N * 4 + N * 2 + M * N * 2},
        "kernels": {"quant_rows_us": round(tq * 1e3, 2), "quant_rows_GBs": round(quant_bytes / (tq * 1e-3) / 1e9, 1),
                    "int8_gemm_us": round(tg * 1e3, 2), "gpu_ms_total": round(gpu_ms, 4), **spread},
        "from_idle": {"steps": min(a.steps, 50), "warmup": min(a.warmup, 10), "ms_per_step": round(cold_wall / min(a.steps, 50), 5),
                      "value": round(ops / (cold_wall / min(a.steps, 50) * 1e-3) / 1e12, 2), "quant_rows_us": round(cold_tq * 1e3, 2),
                      "int8_gemm_us": round(cold_tg * 1e3, 2),
                      "note": "the first steps after 0.5 s of idle, no settling load: the clock is still rising"},
    }
    if not a.no_graph:
        out["graph_replay"] = {"linear_us": round(time_linear_graph(torch, ffi, d, M, K, N, a.rotate, a.steps, 1), 2),
                               "note": "quantizer + GEMM captured once into a HIP graph and replayed (gpu_int8_gemm_static inside the capture)"}
    if not a.no_skinny:
        sk = []
        for (m, k, n) in ((256, 4096, 24576), (256, 12288, 4096)):
            h2, d2 = make_inputs(torch, synth, m, k, n, seed=1, kind="normal")
            nbuf = max(2, int(600e6 // (n * k)) + 1)
            _, wall2, tq2, tg2 = time_linear(torch, ffi, d2, m, k, n, a.rotate, a.steps, a.warmup, nbuf=nbuf)
            gemm_bytes = m * k + m * 4 + n * k + n * 4 + n * 2 + m * n * 2
            sp2 = dict(LAST_SPREAD)
            graph_us = None if a.no_graph else time_linear_graph(torch, ffi, d2, m, k, n, a.rotate, a.steps, nbuf)
            sk.append({"M": m, "K": k, "N": n, "int8_gemm_us": round(tg2 * 1e3, 2),
                       "GBs": round(gemm_bytes / (tg2 * 1e-3) / 1e9, 1),
                       "frac_hbm": round(gemm_bytes / (tg2 * 1e-3) / 1e9 / PEAK_HBM_GBS, 4),
                       "int8_gemm_us_median": sp2["int8_gemm_us_median"], "int8_gemm_us_min": sp2["int8_gemm_us_min"],
                       "frac_hbm_best": round(gemm_bytes / (sp2["int8_gemm_us_min"] * 1e-6) / 1e9 / PEAK_HBM_GBS, 4),
                       "quant_rows_us": round(tq2 * 1e3, 2), "linear_us_by_events": round((tq2 + tg2) * 1e3, 2),
                       "linear_us_graph_replay": None if graph_us is None else round(graph_us, 2), "weight_copies_rotated": nbuf})
            del h2, d2
        out["skinny"] = sk
    if not a.no_extra:
        # the other linears of the image-DiT block and the SDXL-UNet level, then the video-DiT W6A8 pair
        extra = []
        few = max(5, min(40, a.steps // 3))
        for (name, m, k, n, rot) in (("config 0 anchor", 256, 1024, 1024, 0), ("dit qkv", 4608, 3072, 9216, a.rotate), ("dit out-proj", 4608, 3072, 3072, a.rotate),
                                     ("dit mlp down", 4608, 12288, 3072, a.rotate), ("sdxl attn proj", 8192, 640, 640, 0),
                                     ("sdxl geglu up", 8192, 640, 5120, 0), ("sdxl down", 8192, 2560, 640, 0)):
            h2, d2 = make_inputs(torch, synth, m, k, n, seed=2, kind="t3" if rot else "normal")
            _, wall2, tq2, tg2 = time_linear(torch, ffi, d2, m, k, n, rot, few, 3)
            extra.append({"name": name, "M": m, "K": k, "N": n, "rotate": rot, "quant_rows_us": round(tq2 * 1e3, 2),
                          "int8_gemm_us": round(tg2 * 1e3, 2), "gemm_TOPS": round(2.0 * m * n * k / (tg2 * 1e-3) / 1e12, 1)})
            del h2, d2
        out["linears"] = extra
        w6 = []
        for (name, m, k, n) in (("video-dit ffn up", 8192, 5120, 13824), ("video-dit ffn down", 8192, 13824, 5120)):
            us, us_fused, us_expanded = time_w6a8(torch, ffi, m, k, n, few, 2)
            w6.append({"name": name, "M": m, "K": k, "N": n, "kernel": "gpu_w6a8_group_gemm", "us": round(us, 1),
                       "us_unpack_inside_the_gemm": round(us_fused, 1), "us_expanded_once_into_scratch": round(us_expanded, 1),
                       "TOPS": round(2.0 * m * n * k / us / 1e6, 1), "frac_int8_peak": round(2.0 * m * n * k / us / 1e6 / PEAK_INT8_TOPS, 4)})
        out["w6a8"] = w6
        w6r = []
        for (name, m, k, n) in (("h3 ffn gate+up", 8192, 5376, 28672), ("h3 ffn down", 8192, 14336, 5376)):
            dec, lin, gemm = time_w6_reference_format(torch, ffi, m, k, n, few, 2)
            w6r.append({"name": name, "M": m, "K": k, "N": n, "gpu_w6_decode_us": round(dec, 1),
                        "gpu_w6_decode_GBs": round(n * k * 1.78125 / dec / 1e3, 1),
                        "gpu_w6a8_gemm_us": round(lin, 1), "gpu_int8_gemm_alone_us": round(gemm, 1), "TOPS": round(2.0 * m * n * k / lin / 1e6, 1),
                        "frac_int8_peak": round(2.0 * m * n * k / lin / 1e6 / PEAK_INT8_TOPS, 4)})
        out["w6_reference_format"] = w6r
        out["row_kernels"] = time_row_kernels(torch, ffi, few)
        out["attention"] = time_attention(torch, ffi, few)
    out["mfma_ceiling"] = time_mfma_ceiling(torch, ffi)
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(host, M, K, N, a.rotate, a.cpu_seconds)
        out["cpu_baseline_config0"] = cpu_config0(synth)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
