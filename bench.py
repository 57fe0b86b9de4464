#!/usr/bin/env python3
"""Benchmark of the W8A8 quantized-linear hot path on one MI355X.

One step = one pass of the block-FP8 linear path (per-token-group FP8 quantization
of the bf16 activations, then the block-scaled FP8 GEMM) over the five
DeepSeek-V3 linear shapes at a prefill chunk of M = 4096, through the public
operator API.  Inputs are synthetic and resident in HBM before timing starts.

Prints ONE JSON line: whole-step block-FP8 GEMM throughput, the roofline of the
dominant kernel (the GEMM, timed with events on the launch stream; next to the
published peak the MFMA pipe's measured ceiling under a register-only loop and the
shader clock the run saw), the quantization kernel's HBM figure inside the step,
a `configs` block with every configuration of the baseline (graph-timed per shape),
and a CPU baseline (the torch restatement of the same path on the host cores).

    python bench.py [--gpus 1] [--steps K] [--warmup W]
    python bench.py --sweep sweep.jsonl                # every configuration, one line per shape
    python bench.py --ceiling                          # only the MFMA pipe's sustained rate
"""
import argparse
import json
import os
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))

PEAK_HBM_GBS = 8000.0       # MI355X HBM3E, published
PEAK_FP8_TFLOPS = 5000.0    # dense FP8 MFMA, published (no sparsity)
PEAK_INT8_TOPS = 5000.0

TIMED_BLOCKS = 3  # the headline's K timed steps are run this many times; the fastest block is reported
DSV3_NK = [(24576, 1536), (32768, 512), (7168, 16384), (4096, 7168), (2112, 7168)]
LLAMA8B_NK = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
LLAMA70B_NK = [("qkv", 10240, 8192), ("o", 8192, 8192), ("gate_up", 57344, 8192), ("down", 8192, 28672)]


def group_quant_bytes(m, k):
    return 2 * m * k + m * k + 4 * m * (k // 128)


def token_quant_bytes(m, k):
    return 3 * m * k + 4 * m


def block_gemm_bytes(m, n, k):
    kb, nb = (k + 127) // 128, (n + 127) // 128
    return m * k + n * k + 4 * m * kb + 4 * nb * kb + 2 * m * n


def rowcol_gemm_bytes(m, n, k, bias=False):
    return m * k + n * k + 4 * m + 4 * n + 2 * m * n + (2 * n if bias else 0)


def make_block_weight(n, k, seed, dev):
    """N(0, 0.02) weights quantized per 128x128 block on the device (input data, not timed)."""
    import torch

    g = torch.Generator(device=dev).manual_seed(seed)
    w = torch.randn((n, k), generator=g, device=dev, dtype=torch.float32) * 0.02
    nb, kb = (n + 127) // 128, (k + 127) // 128
    wp = torch.zeros((nb * 128, kb * 128), device=dev)
    wp[:n, :k] = w
    t = wp.view(nb, 128, kb, 128).permute(0, 2, 1, 3)
    scale = t.abs().amax(dim=(2, 3)) / 448.0
    scale = torch.where(scale == 0, torch.ones_like(scale), scale)
    q = (t / scale[:, :, None, None]).clamp(-448, 448).permute(0, 2, 1, 3).reshape(nb * 128, kb * 128)[:n, :k]
    return q.contiguous().to(torch.float8_e4m3fn), scale.contiguous()


def make_activation(m, k, seed, dev):
    import torch

    g = torch.Generator(device=dev).manual_seed(seed)
    return torch.randn((m, k), generator=g, device=dev, dtype=torch.float32).to(torch.bfloat16)


class BenchKernels:
    """ctypes binding of sglang_amd/libsglq_bench.so (csrc/bench_kernels.hip): the register-only MFMA
    loop, the clock probe and the streaming passes.  Measurement helpers only; the operators never load it."""

    VARIANTS = {0: "16x16x128 accumulate in place", 1: "16x16x128 from zero + fold FMAs (block-scaled kind)",
                2: "32x32x64 accumulate in place", 3: "32x32x64 pairs from zero + fold FMAs",
                4: "16x16x128 with per-lane exponent bytes for both operands, accumulate in place (power-of-two block scales)"}

    def __init__(self, dev):
        import ctypes

        import torch

        path = ROOT / "sglang_amd" / "libsglq_bench.so"
        if not path.exists():
            raise RuntimeError(f"{path} is missing: build it first (python -m sglang_amd.build)")
        c = ctypes
        self.lib = c.CDLL(str(path))
        self.lib.sglqb_mfma_ceiling.argtypes = [c.c_int, c.c_int, c.c_void_p, c.c_void_p, c.c_void_p, c.c_int, c.c_void_p]
        self.lib.sglqb_clock_probe.argtypes = [c.c_void_p, c.c_int, c.c_void_p]
        self.lib.sglqb_stream.argtypes = [c.c_int, c.c_void_p, c.c_void_p, c.c_int64, c.c_void_p, c.c_int, c.c_void_p]
        self.lib.sglqb_lds_fill.argtypes = [c.c_int, c.c_void_p, c.c_int, c.c_int64, c.c_int, c.c_int64, c.c_int, c.c_int, c.c_void_p, c.c_void_p,
                                            c.c_int, c.c_void_p]
        self.dev = dev
        self.cus = torch.cuda.get_device_properties(dev).multi_processor_count
        self.torch = torch

    def _stream(self):
        return self.torch.cuda.current_stream(self.dev).cuda_stream

    def clock_sample(self):
        """(shader cycles, 100 MHz ticks) per compute unit at this point of the current stream, as a device
        tensor [4096, 2] (slots of CUs that no block of the probe landed on stay zero)."""
        out = self.torch.zeros((4096, 2), dtype=self.torch.int64, device=self.dev)
        rc = self.lib.sglqb_clock_probe(out.data_ptr(), 32 * self.cus, self._stream())
        assert rc == 0, rc
        return out

    @staticmethod
    def clock_mhz(before, after):
        """Average shader clock between two samples: shader cycles per tick of the 100 MHz reference counter,
        the median over the compute units that reported both times."""
        b, a = before.cpu().double(), after.cpu().double()
        ok = (b[:, 1] > 0) & (a[:, 1] > b[:, 1])
        if not bool(ok.any()):
            return 0.0
        return float((((a[:, 0] - b[:, 0]) / (a[:, 1] - b[:, 1]))[ok]).median() * 100.0)

    def operands(self, kind="random"):
        torch = self.torch
        g = torch.Generator(device=self.dev).manual_seed(1)
        if kind == "random":  # N(0,1) rounded to e4m3: what quantized activations and weights look like
            t = torch.randn(96 * 1024, generator=g, device=self.dev).to(torch.float8_e4m3fn)
        else:                 # 0, 1, 2: few bits toggle
            t = torch.randint(0, 3, (96 * 1024,), generator=g, device=self.dev).float().to(torch.float8_e4m3fn)
        return t.view(torch.uint8)

    def mfma_ceiling(self, variant, operands, iters=20000):
        """PFLOP/s and shader clock of the register-only MFMA loop: 8 waves per CU, one block per CU."""
        torch = self.torch
        sink = torch.empty(self.cus * 512, dtype=torch.float32, device=self.dev)
        clocks = torch.zeros(self.cus * 2, dtype=torch.int64, device=self.dev)
        run = lambda: self.lib.sglqb_mfma_ceiling(variant, iters, operands.data_ptr(), sink.data_ptr(), clocks.data_ptr(),
                                                  self.cus, self._stream())
        for _ in range(2):
            assert run() == 0
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        assert run() == 0
        e.record()
        torch.cuda.synchronize()
        ms = s.elapsed_time(e)
        c = clocks.cpu().view(self.cus, 2).double()
        flops = 2097152.0 * 8 * self.cus * iters
        mhz = float((c[:, 0] / c[:, 1]).mean() * 100.0)
        tflops = flops / ms / 1e9
        # MFMA-pipe utilisation at that clock: 4 SIMDs x 65536 flop per 32 cycles = 8192 flop per CU and cycle
        util = tflops * 1e12 / (self.cus * 8192.0 * mhz * 1e6)
        return {"variant": self.VARIANTS[variant], "TFLOPs": round(tflops, 1), "clock_mhz": round(mhz, 0),
                "mfma_pipe_utilisation": round(util, 3), "ms": round(ms, 2)}


def calibrate_copy(dev):
    """One plain copy kernel of known size (stream_kernel<0> of libsglq_bench.so: reads 256 MiB, writes 256 MiB),
    the yardstick for what the profiler's FETCH_SIZE / WRITE_SIZE counters report per byte."""
    import torch

    bk = BenchKernels(dev)
    src = torch.zeros(256 << 20, dtype=torch.uint8, device=dev)
    dst = torch.empty_like(src)
    sink = torch.zeros(8 * bk.cus, dtype=torch.int32, device=dev)
    rc = bk.lib.sglqb_stream(0, src.data_ptr(), dst.data_ptr(), src.numel(), sink.data_ptr(), 8 * bk.cus, bk._stream())
    assert rc == 0, rc
    torch.cuda.synchronize()


def run_launches(args):
    """bench.py --launches "M,N,K;M,N,K;...": each listed block-FP8 linear (group quantization, then the GEMM) as
    plain launches, `--launch-reps` times each after one untimed call, in the order given: the program to put under
    `rocprofv3 --pmc ...`, whose per-dispatch rows then map to the shapes by order.  Prints one JSON line with
    the kernel each shape selected and its event-timed duration."""
    import torch

    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import per_token_group_quant_fp8_pow2, sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    lib = _lib.load()
    dev = torch.device("cuda:0")
    if args.calibrate_copy:
        calibrate_copy(dev)
    # --force-tile CODE: every GEMM on the kernel that sglq_debug_force_tile(CODE) names (include/sglq.h), to put a
    # kernel that the selection rules do not pick for a shape under the profiler next to the one they do pick
    lib.sglq_debug_force_tile(args.force_tile)
    if args.ue8m0:
        quant = lambda x: per_token_group_quant_fp8_pow2(x, 128, column_major_scales=True)
        gemm = fp8_blockwise_scaled_mm_ue8m0
    else:
        quant = lambda x: sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
        gemm = fp8_blockwise_scaled_mm
    rows = []
    if args.kind != "block_fp8":
        # the per-token kinds: per_token_quant_fp8 + fp8_scaled_mm, or per_token_quant_int8 + int8_scaled_mm
        from sglang_amd.quantization.fp8_kernel import sglang_per_token_quant_fp8
        from sglang_amd.quantization.int8_kernel import per_token_quant_int8
        from sglang_amd.sgl_kernel import fp8_scaled_mm, int8_scaled_mm

        quant = sglang_per_token_quant_fp8 if args.kind == "fp8" else per_token_quant_int8
        gemm = lambda xq, w, xs, ws, dt: (fp8_scaled_mm if args.kind == "fp8" else int8_scaled_mm)(xq, w, xs, ws, dt, None)
    for i, spec in enumerate(args.launches.split(";")):
        m, n, k = (int(v) for v in spec.split(","))
        if args.kind == "block_fp8":
            wq, ws = make_block_weight(n, k, 7000 + i, dev)
        else:
            g = torch.Generator(device=dev).manual_seed(7000 + i)
            if args.kind == "fp8":
                wq = (torch.randn((n, k), generator=g, device=dev) * 0.5).to(torch.float8_e4m3fn)
            else:
                wq = torch.randint(-127, 128, (n, k), generator=g, device=dev, dtype=torch.int8)
            ws = (torch.rand((n, 1), generator=g, device=dev) * 9e-3 + 1e-3).t()  # (the call below passes ws.t(): [N, 1])
        if args.ue8m0:
            ws = torch.exp2(torch.ceil(torch.log2(ws)))
        x = make_activation(m, k, 7100 + i, dev)
        xq, xs = quant(x)
        gemm(xq, wq.t(), xs, ws.t(), torch.bfloat16)
        torch.cuda.synchronize()
        # --rotate-weights: every repetition reads another copy of the weight, 320 MB and more in rotation, so that
        # none finds its weight in the 256 MiB last-level cache (as in a model whose layers come by once per step)
        copies = max(2, min(48, -(-320_000_000 // (n * k)))) if args.rotate_weights else 1
        wqs = [wq] + [wq.clone() for _ in range(copies - 1)]
        t = Timer()
        for rep in range(args.launch_reps):
            xq, xs = quant(x)
            wr = wqs[(rep + 1) % copies]
            t.time(lambda: gemm(xq, wr.t(), xs, ws.t(), torch.bfloat16))
        torch.cuda.synchronize()
        del wqs
        us = t.total_ms() / t.count() * 1e3
        nbytes = block_gemm_bytes(m, n, k) if args.kind == "block_fp8" else rowcol_gemm_bytes(m, n, k)
        rows.append({"M": m, "N": n, "K": k, "kernel": lib.sglq_debug_last_gemm_kernel().decode(), "gemm_us": round(us, 2),
                     "TFLOPs": round(2.0 * m * n * k / us / 1e6, 1), "GBs": round(nbytes / us / 1e3, 1),
                     "algorithmic_bytes": nbytes})
        del wq, x, xq
    lib.sglq_debug_force_tile(0)
    print(json.dumps({"launches": rows, "reps": args.launch_reps, "kind": args.kind, "force_tile": args.force_tile}), flush=True)


def run_ab(args):
    """bench.py --ab OTHER.so --launches "M,N,K;...": the block-FP8 GEMM of another build of libsglq.so (for instance
    one compiled from an earlier commit with the flags of sglang_amd/build.py) against the tree's library in ONE
    process: the two alternate, four rounds of 60 back-to-back calls each after 60 untimed ones, the shader clock read
    around every timed block.  One JSON line per (shape, library, round) and whether the outputs are equal bit for bit."""
    import ctypes
    from ctypes import c_int, c_int64, c_void_p

    import torch

    dev = torch.device("cuda:0")
    bk = BenchKernels(dev)
    sig = [c_void_p, c_int64, c_void_p, c_int64, c_void_p, c_int64, c_int64, c_void_p, c_int64, c_int64,
           c_void_p, c_int64, c_int, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p]
    libs = []
    for name, path in (("other", args.ab), ("tree", str(ROOT / "sglang_amd" / "libsglq.so"))):
        lib = ctypes.CDLL(path)
        lib.sglq_fp8_blockwise_scaled_mm.argtypes = sig
        lib.sglq_debug_last_gemm_kernel.restype = ctypes.c_char_p
        libs.append((name, lib))
    ws = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
    for i, spec in enumerate(args.launches.split(";")):
        m, n, k = (int(v) for v in spec.split(","))
        wq, wsc = make_block_weight(n, k, 7000 + i, dev)
        g = torch.Generator(device=dev).manual_seed(7100 + i)
        x = (torch.randn((m, k), generator=g, device=dev) * 2).to(torch.float8_e4m3fn)
        sa = (torch.rand((k // 128, m), generator=g, device=dev) + 0.5).t()
        out = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
        st = torch.cuda.current_stream().cuda_stream

        def call(lib):
            rc = lib.sglq_fp8_blockwise_scaled_mm(x.data_ptr(), k, wq.data_ptr(), k, sa.data_ptr(), sa.stride(0), sa.stride(1), wsc.data_ptr(),
                                                  wsc.stride(1), wsc.stride(0), out.data_ptr(), n, 0, m, n, k, ws.data_ptr(), ws.numel(), st)
            assert rc == 0, rc

        outs = {}
        for rnd in range(4):
            for name, lib in libs:
                for _ in range(60):
                    call(lib)
                c0 = bk.clock_sample()
                s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                s.record()
                for _ in range(60):
                    call(lib)
                e.record()
                c1 = bk.clock_sample()
                torch.cuda.synchronize()
                us = s.elapsed_time(e) / 60 * 1e3
                mhz = bk.clock_mhz(c0, c1)
                tf = 2.0 * m * n * k / us / 1e6
                outs[name] = out.clone()
                print(json.dumps({"library": name, "M": m, "N": n, "K": k, "round": rnd, "kernel": lib.sglq_debug_last_gemm_kernel().decode(),
                                  "us": round(us, 1), "TFLOPs": round(tf, 1), "clock_mhz": round(mhz),
                                  "mfma_pipe_utilisation": round(tf * 1e12 / (bk.cus * 8192.0 * max(mhz, 1.0) * 1e6), 3)}), flush=True)
        print(json.dumps({"M": m, "N": n, "K": k, "outputs_equal": bool(torch.equal(outs["other"], outs["tree"]))}), flush=True)
        del wq, x, out


def run_fill(args):
    """bench.py --fill: what the compute units take in through their LDS with the GEMM kernels' global -> LDS copies and
    nothing else (lds_fill_kernel of libsglq_bench.so: 8 waves per block, one block per CU, every wave keeps stages - 1
    stages of its own copies in flight, no barrier, no arithmetic), per source of the bytes: windows that stay in the
    XCDs' L2s, windows shared by four blocks of one XCD, and windows of 2.75 MB per block that come from HBM (the K
    walk of a 7168-byte row pitch).  One JSON line: per case the median rate per block and the sum over the blocks."""
    import torch

    dev = torch.device("cuda:0")
    bk = BenchKernels(dev)
    cus = bk.cus
    cases = []
    for stages in (2, 3):
        # (label, rows per stage, row pitch, 128-byte steps per row, blocks sharing a window, blocks)
        cases += [("hbm: a window of 384 rows x 7168 B per block", stages, 384, 7168, 56, 1, cus),
                  ("hbm, a quarter of the CUs", stages, 384, 7168, 56, 1, cus // 4),
                  ("four blocks of an XCD share a window of 384 rows x 7168 B (704 MB / 4 in all)", stages, 384, 7168, 56, 4, cus),
                  ("L2: four blocks share a window of 384 rows x 1024 B (3 MB per XCD)", stages, 384, 1024, 8, 4, cus),
                  ("L2: a window of 256 rows x 512 B per block (4 MB per XCD)", stages, 256, 512, 4, 1, cus),
                  ("L2: a window of 128 rows x 512 B per block (2 MB per XCD), 16 KiB stages", stages, 128, 512, 4, 1, cus)]
    cases += [("L2: a window of 128 rows x 512 B per block (2 MB per XCD), 16 KiB stages", 4, 128, 512, 4, 1, cus),
              ("hbm: a window of 256 rows x 7168 B per block", 4, 256, 7168, 56, 1, cus)]
    out = {"what": "global -> LDS copy loop (buffer_load_dwordx4 ... lds, 1 KiB per wave instruction), 8 waves per block, one block per CU, no arithmetic",
           "cus": cus, "cases": []}
    for label, stages, rows, pitch, steps, share, blocks in cases:
        window = ((rows - 1) * pitch + steps * 128 + 4095) // 4096 * 4096
        windows = -(-blocks // (8 * share)) * 8
        src = torch.empty(windows * window, dtype=torch.uint8, device=dev)
        src.random_(0, 255)
        clocks = torch.zeros(blocks * 2, dtype=torch.int64, device=dev)
        sink = torch.zeros(blocks, dtype=torch.int32, device=dev)
        stage_bytes = rows * 128
        iters = max(steps * 4, 2_000_000_000 // (blocks * stage_bytes) // steps * steps)
        run = lambda: bk.lib.sglqb_lds_fill(stages, src.data_ptr(), rows, pitch, steps, window, share, iters, clocks.data_ptr(), sink.data_ptr(),
                                            blocks, bk._stream())
        rc = run()
        assert rc == 0, (rc, label)
        torch.cuda.synchronize()
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        rc = run()
        e.record()
        torch.cuda.synchronize()
        assert rc == 0, (rc, label)
        ticks = clocks.view(blocks, 2)[:, 1].double().cpu()  # 100 MHz ticks of each block's loop
        per_block = (iters * stage_bytes) / (ticks * 1e-8) / 1e9
        out["cases"].append({"source": label, "stages": stages, "stage_KiB": stage_bytes // 1024, "in_flight_KiB_per_CU": (stages - 1) * stage_bytes // 1024,
                             "blocks": blocks, "bytes_per_block_MB": round(iters * stage_bytes / 1e6, 1), "footprint_MB": round(windows * window / 1e6, 1),
                             "GBs_per_block_median": round(float(per_block.median()), 1), "GBs_per_block_min": round(float(per_block.min()), 1),
                             "TBs_all_blocks": round(blocks * iters * stage_bytes / (s.elapsed_time(e) * 1e-3) / 1e12, 2)})
        del src
    print(json.dumps(out), flush=True)


def run_ceiling(args):
    """bench.py --ceiling: the MFMA pipe's sustained rate under a register-only loop (no memory traffic), for the
    instruction mixes of the two GEMM families and two kinds of operand bytes.  One JSON line."""
    import torch

    dev = torch.device("cuda:0")
    bk = BenchKernels(dev)
    out = {"what": "register-only MFMA loop, 8 waves per CU, 20000 K steps of a 128 x 64 wave tile per wave",
           "published_peak_TFLOPs": PEAK_FP8_TFLOPS, "cus": bk.cus, "runs": []}
    for kind in ("random", "small_integers"):
        ops = bk.operands(kind)
        for v in range(5):
            r = bk.mfma_ceiling(v, ops)
            r["operands"] = kind
            r["frac_of_published_peak"] = round(r["TFLOPs"] / PEAK_FP8_TFLOPS, 3)
            out["runs"].append(r)
    print(json.dumps(out), flush=True)


class Timer:
    """Sums event-timed durations of individual launches on the current stream."""

    def __init__(self):
        self.pairs = []

    def time(self, fn):
        import torch

        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        s.record()
        out = fn()
        e.record()
        self.pairs.append((s, e))
        return out

    def total_ms(self):
        return sum(s.elapsed_time(e) for s, e in self.pairs)

    def count(self):
        return len(self.pairs)

    def each_ms(self):
        return sorted(s.elapsed_time(e) for s, e in self.pairs)


def cpu_baseline(m_sample):
    """The torch restatement of the same step on the host cores, on the first
    m_sample activation rows of every shape (weights in full)."""
    import torch

    from oracle import w8a8_oracle as O

    cores = torch.get_num_threads()
    flops = 0.0
    secs = 0.0
    PASSES = 2  # about 16 s of host time on the 16 cores of a one-GPU box
    for i, (n, k) in enumerate(DSV3_NK):
        x = O.gen_activation(m_sample, k, seed=2000 + i)
        w = torch.randn((n, k), generator=torch.Generator().manual_seed(i)) * 0.02
        wq, ws = O.block_quant_weight(w)
        del w
        for _ in range(PASSES):
            t0 = time.perf_counter()
            xq, xs = O.per_token_group_quant_fp8(x, 128)
            O.fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16)
            secs += time.perf_counter() - t0
            flops += 2.0 * m_sample * n * k
    # configuration 0 (the reference's own CPU-runnable case) in full: quantize A[256, 7168] with outliers, then the
    # block-scaled GEMM against W[2048, 7168]; the fastest of three passes
    x0 = O.gen_activation(256, 7168, seed=0, outliers=True)
    wq0, ws0 = O.block_quant_weight(O.gen_weight(2048, 7168, seed=0))
    cfg0_q = cfg0_g = float("inf")
    for _ in range(3):
        t0 = time.perf_counter()
        xq0, xs0 = O.per_token_group_quant_fp8(x0, 128)
        t1 = time.perf_counter()
        O.fp8_blockwise_scaled_mm(xq0, wq0.t(), xs0, ws0.t(), torch.bfloat16)
        t2 = time.perf_counter()
        cfg0_q, cfg0_g = min(cfg0_q, t1 - t0), min(cfg0_g, t2 - t1)
    return {
        "value": round(flops / secs / 1e12, 4),
        "unit": "TFLOP/s",
        "cores": cores,
        "kind": "port",
        "sample": f"{m_sample} of 4096 activation rows of each of the 5 shapes, full weights, {PASSES} passes, {secs:.1f} s of CPU time",
        "cfg0_quant_ms": round(cfg0_q * 1e3, 3),
        "cfg0_quant_GBs": round(group_quant_bytes(256, 7168) / cfg0_q / 1e9, 3),
        "cfg0_gemm_ms": round(cfg0_g * 1e3, 3),
        "cfg0_gemm_TFLOPs": round(2.0 * 256 * 2048 * 7168 / cfg0_g / 1e12, 4),
        "cfg0_sample": "configuration 0 in full (A[256,7168] with outliers -> group quant -> block-FP8 GEMM with W[2048,7168]), fastest of 3 passes",
    }


def ue8m0_summary(args, layers, m, bk, ops_rand):
    """The headline step once more with power-of-two (UE8M0) scales: per_token_group_quant_fp8_pow2 and
    fp8_blockwise_scaled_mm_ue8m0, whose matrix instructions apply the scales and accumulate in place (the reference's
    deepgemm_w8a8_block_fp8_linear_with_fallback under DEEPGEMM_SCALE_UE8M0).  Reported next to the headline, which
    stays the fp32-scale operator; same shapes, same timing method (wall clock over the timed steps, then a pass with
    events per launch)."""
    import torch

    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import per_token_group_quant_fp8_pow2
    from sglang_amd.sgl_kernel.gemm import fp8_blockwise_scaled_mm_ue8m0

    lib = _lib.load()
    ws2 = [torch.exp2(torch.ceil(torch.log2(ws))) for (_, _, _, _, ws) in layers]
    hw = {}

    def step(tq=None, tg=None):
        for li, (n, k, x, wq, _) in enumerate(layers):
            if tq is None:
                xq, xs = per_token_group_quant_fp8_pow2(x, 128, column_major_scales=True)
                fp8_blockwise_scaled_mm_ue8m0(xq, wq.t(), xs, ws2[li].t(), torch.bfloat16)
            else:
                xq, xs = tq[li].time(lambda: per_token_group_quant_fp8_pow2(x, 128, column_major_scales=True))
                tg[li].time(lambda: fp8_blockwise_scaled_mm_ue8m0(xq, wq.t(), xs, ws2[li].t(), torch.bfloat16))
                hw[li] = (lib.sglq_debug_last_gemm_kernel().decode(), bool(lib.sglq_debug_last_gemm_hw_scaled()))

    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.05:  # (the clocks are settled by the headline's steps; a few more to switch kernels)
        step()
        torch.cuda.synchronize()
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    tq, tg = [Timer() for _ in layers], [Timer() for _ in layers]
    for _ in range(args.steps):
        step(tq, tg)
    torch.cuda.synchronize()
    flops_step = sum(2.0 * m * n * k for n, k, *_ in layers)
    ms_per_step = wall * 1e3 / args.steps
    per_shape = []
    for li, ((n, k, *_), a, b) in enumerate(zip(layers, tq, tg)):
        qm, gm = a.total_ms() / args.steps, b.total_ms() / args.steps
        per_shape.append({"N": n, "K": k, "gemm_kernel": hw[li][0], "scales_applied_by_the_mfma": hw[li][1],
                          "quant_us": round(qm * 1e3, 1), "quant_GBs": round(group_quant_bytes(m, k) / qm / 1e6, 1),
                          "gemm_us": round(gm * 1e3, 1), "gemm_TFLOPs": round(2.0 * m * n * k / gm / 1e9, 1),
                          "gemm_frac": round(2.0 * m * n * k / gm / 1e9 / PEAK_FP8_TFLOPS, 4)})
    dom = max(range(len(layers)), key=lambda i: tg[i].total_ms())
    dom_tflops = per_shape[dom]["gemm_TFLOPs"]
    gemm_ms = sum(t.total_ms() for t in tg) / args.steps
    ceil = bk.mfma_ceiling(4, ops_rand, iters=10000)
    return {
        "what": "the same step with power-of-two (UE8M0) scales: per_token_group_quant_fp8_pow2 + fp8_blockwise_scaled_mm_ue8m0, "
                "the MFMAs apply the scales (v_mfma_scale_f32_16x16x128_f8f6f4) and accumulate in place; weights' block scales "
                "rounded up to powers of two, values synthetic",
        "value": round(flops_step / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "ms_per_step": round(ms_per_step, 4),
        "roofline": {"kernel": f"fp8_blockwise_scaled_mm_ue8m0: sglq::{per_shape[dom]['gemm_kernel']} on {m} x {layers[dom][0]} x {layers[dom][1]}",
                     "bound": "mfma", "achieved": dom_tflops, "peak": PEAK_FP8_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(dom_tflops / PEAK_FP8_TFLOPS, 4),
                     "avg_launch_ms": round(tg[dom].total_ms() / tg[dom].count(), 4),
                     "practical_peak": {"value": ceil["TFLOPs"], "clock_mhz": ceil["clock_mhz"],
                                        "mfma_pipe_utilisation": ceil["mfma_pipe_utilisation"],
                                        "what": "register-only loop of the scaled MFMA accumulating in place, N(0,1) e4m3 operands",
                                        "frac_of_it": round(dom_tflops / ceil["TFLOPs"], 4)},
                     "all_gemm_launches_of_the_step": {"achieved": round(flops_step / (gemm_ms * 1e-3) / 1e12, 2),
                                                       "frac": round(flops_step / (gemm_ms * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4)}},
        "per_shape": per_shape,
    }


def run_headline(args):
    import torch

    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm

    _lib.load()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    m = 4096
    layers = []
    for i, (n, k) in enumerate(DSV3_NK):
        wq, ws = make_block_weight(n, k, 2000 + i, dev)
        layers.append((n, k, make_activation(m, k, 2000 + i, dev), wq, ws))
    torch.cuda.synchronize()

    kernel_of = {}

    def step(tq=None, tg=None):
        for li, (n, k, x, wq, ws) in enumerate(layers):
            if tq is None:
                xq, xs = sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True)
                fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16)
            else:
                xq, xs = tq[li].time(lambda: sglang_per_token_group_quant_fp8(x, 128, column_major_scales=True))
                tg[li].time(lambda: fp8_blockwise_scaled_mm(xq, wq.t(), xs, ws.t(), torch.bfloat16))
                kernel_of[li] = _lib.load().sglq_debug_last_gemm_kernel().decode()

    if args.calibrate_copy:
        calibrate_copy(dev)

    # The chip needs about 60 steps (60 ms) of this load before its step time settles (962 us per step over
    # steps 10-20, 933 over 20-30, 890-900 from step 60 on; measured): run untimed steps for 150 ms first, so
    # that W and K of any size see the settled clocks.  Then W untimed steps and exactly K timed ones.
    prewarm_steps = 0
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < args.prewarm_ms * 1e-3:
        step()
        torch.cuda.synchronize()
        prewarm_steps += 1
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    wall_graph = None
    bk = BenchKernels(dev)
    # The K timed steps, three times over (one box's step time moves by a few per cent between blocks of steps):
    # `value` comes from the fastest block, all three are listed.
    walls, block_clocks = [], []
    for _ in range(TIMED_BLOCKS):
        clk0 = bk.clock_sample()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            step()
        torch.cuda.synchronize()
        walls.append(time.perf_counter() - t0)
        clk1 = bk.clock_sample()
        torch.cuda.synchronize()
        block_clocks.append(bk.clock_mhz(clk0, clk1))
    wall = min(walls)
    step_clock_mhz = block_clocks[walls.index(wall)]
    if args.graph:
        # the same K steps replayed as one HIP graph, for comparison (measured: no faster than the launches above)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(args.steps):
                step()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        wall_graph = time.perf_counter() - t0

    # per-kernel durations on the launch stream (separate pass so the events do not perturb the wall clock above)
    tq, tg = [Timer() for _ in layers], [Timer() for _ in layers]
    for _ in range(args.steps):
        step(tq, tg)
    torch.cuda.synchronize()

    flops_step = sum(2.0 * m * n * k for n, k, *_ in layers)
    qbytes_step = sum(group_quant_bytes(m, k) for _, k, *_ in layers)
    ms_per_step = wall * 1e3 / args.steps
    gemm_ms = sum(t.total_ms() for t in tg) / args.steps
    quant_ms = sum(t.total_ms() for t in tq) / args.steps
    per_shape = []
    for (n, k, *_), a, b in zip(layers, tq, tg):
        qm, gm = a.total_ms() / args.steps, b.total_ms() / args.steps
        per_shape.append({"N": n, "K": k, "gemm_kernel": kernel_of.get(len(per_shape), ""), "quant_us": round(qm * 1e3, 1),
                          "quant_GBs": round(group_quant_bytes(m, k) / qm / 1e6, 1),
                          "gemm_us": round(gm * 1e3, 1), "gemm_TFLOPs": round(2.0 * m * n * k / gm / 1e9, 1)})
    big = max(range(len(layers)), key=lambda i: layers[i][1])  # the launch with the most activation bytes
    quant_in_step_gbs = per_shape[big]["quant_GBs"]
    # the same launch back to back on two alternating inputs: the kernel on its own, without the
    # write-back of the preceding GEMM's output competing for HBM
    xs_iso = [layers[big][2], layers[big][2].clone()]
    iso = Timer()
    for i in range(2 + 10):
        if i < 2:
            sglang_per_token_group_quant_fp8(xs_iso[i % 2], 128, column_major_scales=True)
        else:
            iso.time(lambda: sglang_per_token_group_quant_fp8(xs_iso[i % 2], 128, column_major_scales=True))
    torch.cuda.synchronize()
    quant_big_gbs = round(group_quant_bytes(m, layers[big][1]) / (iso.total_ms() / iso.count()) / 1e6, 1)
    del xs_iso
    # the clock while the dominant GEMM launch alone repeats (settled), and the MFMA pipe's ceiling right after
    dom = max(range(len(layers)), key=lambda i: tg[i].total_ms())
    n_d, k_d, x_d, wq_d, ws_d = layers[dom]
    xq_d, xs_d = sglang_per_token_group_quant_fp8(x_d, 128, column_major_scales=True)
    for _ in range(20):
        fp8_blockwise_scaled_mm(xq_d, wq_d.t(), xs_d, ws_d.t(), torch.bfloat16)
    c0 = bk.clock_sample()
    for _ in range(20):
        fp8_blockwise_scaled_mm(xq_d, wq_d.t(), xs_d, ws_d.t(), torch.bfloat16)
    c1 = bk.clock_sample()
    torch.cuda.synchronize()
    dom_clock_mhz = bk.clock_mhz(c0, c1)
    ops_rand = bk.operands("random")
    ceil_fold = bk.mfma_ceiling(1, ops_rand, iters=10000)
    ceil_acc = bk.mfma_ceiling(0, ops_rand, iters=10000)
    # the dominant kernel: the GEMM launch that takes the largest share of the step
    props = torch.cuda.get_device_properties(dev)
    dom_n, dom_k = layers[dom][0], layers[dom][1]
    dom_ms = tg[dom].total_ms() / tg[dom].count()
    dom_each = tg[dom].each_ms()
    dom_flops = 2.0 * m * dom_n * dom_k
    dom_tflops = dom_flops / (dom_ms * 1e-3) / 1e12
    traffic = traffic_all = None
    tfile = ROOT / "profiles" / "headline_traffic.json"
    if tfile.exists():
        tj = json.loads(tfile.read_text())
        traffic = tj.get("hbm_bytes_per_launch", {}).get(f"{dom_n}x{dom_k}")
        traffic_all = tj.get("gemm_hbm_bytes_per_launch_avg")
    gemm_tflops = flops_step / (gemm_ms * 1e-3) / 1e12
    quant_gbs = qbytes_step / (quant_ms * 1e-3) / 1e9

    out = {
        "metric": "block-FP8 GEMM TFLOPS (% of FP8 MFMA peak); quant kernel GB/s (% of HBM)",
        "value": round(flops_step / (ms_per_step * 1e-3) / 1e12, 2),
        "unit": "TFLOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_blocks": [round(w * 1e3 / args.steps, 4) for w in walls],
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "fp8_e4m3fn (fp32 accumulate, bf16 out)",
        "data": "synthetic",
        "config": {
            "workload": "cfg2 DeepSeek-V3 block-FP8 linears, M=4096, (N,K) in "
                        "{(24576,1536),(32768,512),(7168,16384),(4096,7168),(2112,7168)}: "
                        "per-token-group-128 FP8 quant + 128x128 block-scaled FP8 GEMM, bf16 in/out",
            "value_is": "sum of 2MNK over the 5 GEMMs / wall time of the whole step (quant kernels included); the K timed steps are run "
                        f"{TIMED_BLOCKS} times and the fastest block is `ms_per_step` (all in ms_per_step_blocks)",
            "prewarm": f"{prewarm_steps} untimed steps over {args.prewarm_ms} ms before the {args.warmup} warm-up steps (clock settling)",
        },
        "roofline": {
            "kernel": f"fp8_blockwise_scaled_mm: sglq::{kernel_of.get(dom, '')} (block-scaled FP8, bf16 out) on "
                      f"{m} x {dom_n} x {dom_k}, the launch with the largest share of the step",
            "bound": "mfma",
            "achieved": round(dom_tflops, 2),
            "peak": PEAK_FP8_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(dom_tflops / PEAK_FP8_TFLOPS, 4),
            "practical_peak": {
                "value": ceil_fold["TFLOPs"],
                "unit": "TFLOP/s",
                "what": "register-only loop of this kernel's MFMA mix (v_mfma_f32_16x16x128_f8f6f4 from a zero accumulator + 4 fold "
                        "FMAs, 8 waves per CU) on N(0,1) e4m3 operands, no memory traffic, measured in this run: what the matrix "
                        "pipe sustains at the clock the chip settles to under that load",
                "clock_mhz": ceil_fold["clock_mhz"],
                "mfma_pipe_utilisation": ceil_fold["mfma_pipe_utilisation"],
                "frac_of_it": round(dom_tflops / ceil_fold["TFLOPs"], 4),
                "accumulate_in_place_TFLOPs": ceil_acc["TFLOPs"],
                "accumulate_in_place_clock_mhz": ceil_acc["clock_mhz"],
            },
            "clock_mhz": round(dom_clock_mhz, 0),
            "mfma_pipe_utilisation": round(dom_tflops * 1e12 / (props.multi_processor_count * 8192.0 * max(dom_clock_mhz, 1.0) * 1e6), 3),
            "traffic": traffic,
            "traffic_source": "profiles/headline_traffic.json (rocprofv3 FETCH_SIZE / WRITE_SIZE of this launch, scaled by a plain copy "
                              "kernel's readings; a committed constant, not measured in this run)",
            "avg_launch_ms": round(dom_ms, 4),
            "min_launch_ms": round(dom_each[0], 4),
            "median_launch_ms": round(dom_each[len(dom_each) // 2], 4),
            "frac_at_median": round(dom_flops / (dom_each[len(dom_each) // 2] * 1e-3) / 1e12 / PEAK_FP8_TFLOPS, 4),
            "flops_per_launch": dom_flops,
            # scalars that restate what the nested objects below and beside hold
            "practical_peak_tflops": ceil_fold["TFLOPs"],
            "practical_peak_clock_mhz": ceil_fold["clock_mhz"],
            "frac_of_practical_peak": round(dom_tflops / ceil_fold["TFLOPs"], 4),
            "step_gemm_tflops": round(gemm_tflops, 2),
            "step_gemm_frac": round(gemm_tflops / PEAK_FP8_TFLOPS, 4),
            "quant_GBs_in_step": quant_in_step_gbs,
            "quant_frac_hbm_in_step": round(quant_in_step_gbs / PEAK_HBM_GBS, 4),
            "quant_GBs_isolated": quant_big_gbs,
            "quant_frac_hbm_isolated": round(quant_big_gbs / PEAK_HBM_GBS, 4),
            "quant_all_launches_frac_hbm_in_step": round(quant_gbs / PEAK_HBM_GBS, 4),
            "all_gemm_launches_of_the_step": {
                "achieved": round(gemm_tflops, 2),
                "frac": round(gemm_tflops / PEAK_FP8_TFLOPS, 4),
                "avg_launch_ms": round(gemm_ms / len(layers), 4),
                "flops_per_launch_avg": flops_step / len(layers),
                "traffic_per_launch_avg": traffic_all,
            },
        },
        "quant": {
            "kernel": "sgl_per_token_group_quant_fp8 (group_quant_kernel)",
            "bound": "hbm",
            "launch": f"A[4096,{layers[big][1]}] bf16 -> e4m3fn + fp32 scales (largest of the step)",
            "achieved": quant_in_step_gbs,
            "peak": PEAK_HBM_GBS,
            "unit": "GB/s",
            "frac": round(quant_in_step_gbs / PEAK_HBM_GBS, 4),
            "bytes_per_launch": group_quant_bytes(m, layers[big][1]),
            "measured": "inside the timed step (right after the preceding GEMM, whose output write-back shares HBM with it), "
                        "events on the launch stream",
            "same_launch_isolated_GBs": quant_big_gbs,
            "same_launch_isolated_frac": round(quant_big_gbs / PEAK_HBM_GBS, 4),
            "isolated_measured": "10 back-to-back launches on 2 alternating inputs",
            "all_launches_inside_the_step_GBs": round(quant_gbs, 1),
            "all_launches_inside_the_step_frac": round(quant_gbs / PEAK_HBM_GBS, 4),
        },
        "graph_ms_per_step": None if wall_graph is None else round(wall_graph * 1e3 / args.steps, 4),
        "per_shape": per_shape,
        "device": {"name": props.name, "cus": props.multi_processor_count,
                   "clock_mhz": round(step_clock_mhz, 0),
                   "clock_is": "average shader clock over the timed steps: shader-cycle counter against the 100 MHz reference "
                               "counter, sampled per compute unit on the launch stream before and after them (median over the CUs)",
                   "nominal_clock_mhz": getattr(props, "clock_rate", 0) // 1000},
    }
    out["ue8m0_scales"] = ue8m0_summary(args, layers, m, bk, ops_rand)
    # (a different operator: it needs weights re-quantized to power-of-two block scales, and its parity rests on the
    # block-scaled oracle evaluated with such scales; reported beside the headline, never as `value`)
    out["roofline"]["ue8m0_frac"] = out["ue8m0_scales"]["roofline"]["frac"]
    out["roofline"]["ue8m0_step_tflops"] = out["ue8m0_scales"]["value"]
    if not args.no_configs:
        out["configs"] = config_summary(args)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(args.cpu_rows)
    print(json.dumps(out), flush=True)


# ---------------------------------------------------------------------------
# --sweep: every configuration, one JSON line per (config, shape)
# ---------------------------------------------------------------------------
def time_kernel(fn, iters, rotate=1):
    """Device-side time per call: `iters` calls captured into one HIP graph (no host
    launch gaps inside), inputs rotated so that consecutive calls do not reuse cached data."""
    import torch

    for i in range(max(2, rotate)):
        fn(i % rotate)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    iters = max(iters, rotate)  # every copy takes its turn inside the graph
    with torch.cuda.graph(g):
        for i in range(iters):
            fn(i % rotate)
    # replay untimed for 20 ms (a kernel measured right after a pause or after a different one runs several per
    # cent slower than in a steady sequence of itself), then the fastest of three timed replays
    t0 = time.perf_counter()
    while True:
        g.replay()
        torch.cuda.synchronize()
        if time.perf_counter() - t0 >= 0.02:
            break
    s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    best = float("inf")
    for _ in range(3):
        s.record()
        g.replay()
        e.record()
        torch.cuda.synchronize()
        best = min(best, s.elapsed_time(e) / iters)
    return best


def config_summary(args):
    """Every configuration of the baseline, graph-timed as --sweep does, condensed for the one JSON line:
    per (config, shape) the quantization and GEMM device times and the fraction of the roofline that bounds
    the GEMM there: of the two lower bounds on its time, algorithmic bytes / 8 TB/s and operations / 5 P(FL)OP/s,
    the larger one."""
    rows = []
    run_sweep(args, collect=rows, cfg2_ms=(1, 64, 512, 8192), only={"0", "1", "2", "3", "4"})
    out = {}
    for r in rows:
        cfg = f"cfg{r['cfg']}"
        if r.get("op") == "total":
            out.setdefault(cfg, {}).setdefault("totals", []).append({"M": r["M"], "total_us": r["total_us"], "TFLOPs": r["TFLOPs"],
                                                                      "frac_mfma": round(r["TFLOPs"] / PEAK_FP8_TFLOPS, 4)})
            continue
        m = r["M"]
        hbm_bound = r["gemm_frac_hbm"] >= r["gemm_frac_mfma"]
        e = {"M": m, "N": r["N"], "K": r["K"], "quant_us": r["quant_us"], "gemm_us": r["gemm_us"],
             "bound": "hbm" if hbm_bound else "mfma",
             "frac": r["gemm_frac_hbm"] if hbm_bound else r["gemm_frac_mfma"]}
        e["rate"] = f"{r['gemm_GBs']} GB/s" if hbm_bound else f"{r.get('gemm_TFLOPs', r.get('gemm_TOPs'))} T(FL)OP/s"
        if "quant_GBs" in r:
            e["quant_frac_hbm"] = round(r["quant_GBs"] / PEAK_HBM_GBS, 4)
        if "linear_us" in r:  # quantization and GEMM through the one-call operator (fused kernel where it is chosen)
            e["linear_us"], e["linear_kernel"] = r["linear_us"], r["linear_kernel"]
        out.setdefault(cfg, {}).setdefault("shapes", []).append(e)
    for cfg, d in out.items():
        sh = d.get("shapes", [])
        if sh:
            d["linear_us_sum"] = round(sum(x.get("linear_us", x["quant_us"] + x["gemm_us"]) for x in sh), 1)
    out["timing"] = ("device time per call from a HIP graph of 20 calls or more, the weights rotated over copies of 320 MB and more in total "
                     "(past the 256 MiB last-level cache), every copy inside the graph")
    return out


def run_sweep(args, collect=None, cfg2_ms=None, only=None):
    import torch

    from sglang_amd import _lib
    from sglang_amd.quantization.fp8_kernel import sglang_per_token_group_quant_fp8, sglang_per_token_quant_fp8
    from sglang_amd.quantization.int8_kernel import per_token_quant_int8
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_scaled_mm
    from sglang_amd.sgl_kernel.gemm import block_fp8_linear, fp8_linear, int8_linear

    _lib.load()
    dev = torch.device("cuda:0")
    # untimed load for 150 ms first (the clocks take that long to settle, see run_headline)
    spin = torch.randn((4096, 4096), device=dev)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.15:
        torch.mm(spin, spin)
        torch.cuda.synchronize()
    del spin
    f = None
    if collect is None:
        out_path = Path(args.sweep)
        out_path.parent.mkdir(parents=True, exist_ok=True)
        f = open(out_path, "w")

    def emit(**kw):
        if collect is not None:
            collect.append(kw)
            return
        f.write(json.dumps(kw) + "\n")
        f.flush()
        print(json.dumps(kw), flush=True)

    def rot_count(nbytes):  # activations: up to eight copies (they come from the layer before and are cache-warm in use)
        return max(1, min(8, int(600e6 // max(nbytes, 1))))

    def weight_copies(nbytes):  # weights: enough copies to exceed the 256 MiB last-level cache (320 MB and more in rotation)
        return max(2, min(48, -(-320_000_000 // max(nbytes, 1))))

    def block_case(cfg, name, m, n, k, seed):
        wq, ws = make_block_weight(n, k, seed, dev)
        r = rot_count(3 * m * k)
        xs_in = [make_activation(m, k, seed + j, dev) for j in range(r)]
        tq = time_kernel(lambda j: sglang_per_token_group_quant_fp8(xs_in[j], 128, column_major_scales=True), args.iters, r)
        xq, xs = sglang_per_token_group_quant_fp8(xs_in[0], 128, column_major_scales=True)
        rw = weight_copies(n * k)
        wqs = [wq] + [wq.clone() for _ in range(rw - 1)]
        tg = time_kernel(lambda j: fp8_blockwise_scaled_mm(xq, wqs[j].t(), xs, ws.t(), torch.bfloat16), args.iters, rw)
        fl = 2.0 * m * n * k
        extra = {}
        if m <= 4:  # decode rows: the whole linear through the one operator that the glue calls for them
            tl = time_kernel(lambda j: block_fp8_linear(xs_in[0], wqs[j].t(), ws.t()), args.iters, rw)
            extra = dict(linear_us=round(tl * 1e3, 2), linear_kernel=_lib.load().sglq_debug_last_gemm_kernel().decode())
        emit(cfg=cfg, op="group_quant_fp8+fp8_blockwise_scaled_mm", name=name, M=m, N=n, K=k, **extra,
             quant_us=round(tq * 1e3, 2), quant_GBs=round(group_quant_bytes(m, k) / tq / 1e6, 1),
             quant_frac_hbm=round(group_quant_bytes(m, k) / tq / 1e6 / PEAK_HBM_GBS, 4),
             gemm_us=round(tg * 1e3, 2), gemm_TFLOPs=round(fl / tg / 1e9, 2),
             gemm_frac_mfma=round(fl / tg / 1e9 / PEAK_FP8_TFLOPS, 4),
             gemm_GBs=round(block_gemm_bytes(m, n, k) / tg / 1e6, 1),
             gemm_frac_hbm=round(block_gemm_bytes(m, n, k) / tg / 1e6 / PEAK_HBM_GBS, 4))
        return tq, tg

    if only is None:
        only = None if not args.sweep_only else set(args.sweep_only.split(","))

    def want(cfg):
        return only is None or str(cfg) in only

    # cfg 0
    if want(0):
        block_case(0, "cfg0", 256, 2048, 7168, 0)
    # cfg 1
    g = torch.Generator(device=dev).manual_seed(1000)
    n, k = 14336, 4096
    w8 = torch.randint(-127, 128, (n, k), generator=g, device=dev, dtype=torch.int8)
    s_b = torch.rand((n,), generator=g, device=dev) * 9e-3 + 1e-3
    bias = (torch.randn((n,), generator=g, device=dev) * 0.1).to(torch.bfloat16)
    w8s = [w8] + [w8.clone() for _ in range(7)]
    for m in (1, 16, 128, 1024) if want(1) else ():
        x = make_activation(m, k, 1000 + m, dev)
        tq = time_kernel(lambda j: per_token_quant_int8(x), args.iters)
        xq, xs = per_token_quant_int8(x)
        tg = time_kernel(lambda j: int8_scaled_mm(xq, w8s[j].t(), xs, s_b, torch.bfloat16, bias), args.iters, 8)
        fl = 2.0 * m * n * k
        extra = {}
        if m <= 2:
            tl = time_kernel(lambda j: int8_linear(x, w8s[j].t(), s_b, bias), args.iters, 8)
            extra = dict(linear_us=round(tl * 1e3, 2), linear_kernel=_lib.load().sglq_debug_last_gemm_kernel().decode())
        emit(cfg=1, op="per_token_quant_int8+int8_scaled_mm", M=m, N=n, K=k, quant_us=round(tq * 1e3, 2), **extra,
             quant_GBs=round(token_quant_bytes(m, k) / tq / 1e6, 1), gemm_us=round(tg * 1e3, 2),
             gemm_TOPs=round(fl / tg / 1e9, 2), gemm_frac_mfma=round(fl / tg / 1e9 / PEAK_INT8_TOPS, 4),
             gemm_GBs=round(rowcol_gemm_bytes(m, n, k, True) / tg / 1e6, 1),
             gemm_frac_hbm=round(rowcol_gemm_bytes(m, n, k, True) / tg / 1e6 / PEAK_HBM_GBS, 4))
    del w8s
    # cfg 2
    for i, (n, k) in enumerate(DSV3_NK if want(2) else ()):
        for m in cfg2_ms or (1, 8, 64, 512, 4096, 8192):
            block_case(2, "dsv3", m, n, k, 2000 + i)
    # cfg 3
    for i, (n, k) in enumerate(LLAMA8B_NK if want(3) else ()):
        g = torch.Generator(device=dev).manual_seed(3000 + i)
        w = torch.randn((n, k), generator=g, device=dev) * 0.02
        sc = w.abs().amax() / 448.0
        wq = (w / sc).clamp(-448, 448).to(torch.float8_e4m3fn)
        ws = sc.reshape(1, 1).expand(n, 1).contiguous()
        rw = weight_copies(n * k)
        wqs = [wq] + [wq.clone() for _ in range(rw - 1)]
        for m in (1, 32, 256, 2048):
            x = make_activation(m, k, 3000 + m, dev)
            tq = time_kernel(lambda j: sglang_per_token_quant_fp8(x), args.iters)
            xq, xs = sglang_per_token_quant_fp8(x)
            tg = time_kernel(lambda j: fp8_scaled_mm(xq, wqs[j].t(), xs, ws, torch.bfloat16, None), args.iters, rw)
            fl = 2.0 * m * n * k
            extra = {}
            if m <= 2:
                tl = time_kernel(lambda j: fp8_linear(x, wqs[j].t(), ws), args.iters, rw)
                extra = dict(linear_us=round(tl * 1e3, 2), linear_kernel=_lib.load().sglq_debug_last_gemm_kernel().decode())
            emit(cfg=3, op="per_token_quant_fp8+fp8_scaled_mm", M=m, N=n, K=k, quant_us=round(tq * 1e3, 2), **extra,
                 quant_GBs=round(token_quant_bytes(m, k) / tq / 1e6, 1), gemm_us=round(tg * 1e3, 2),
                 gemm_TFLOPs=round(fl / tg / 1e9, 2), gemm_frac_mfma=round(fl / tg / 1e9 / PEAK_FP8_TFLOPS, 4),
                 gemm_GBs=round(rowcol_gemm_bytes(m, n, k) / tg / 1e6, 1),
                 gemm_frac_hbm=round(rowcol_gemm_bytes(m, n, k) / tg / 1e6 / PEAK_HBM_GBS, 4))
        del wqs
    # cfg 4
    for m in (4096, 64) if want(4) else ():
        tot = 0.0
        fl_tot = 0.0
        for i, (name, n, k) in enumerate(LLAMA70B_NK):
            tq, tg = block_case(4, name, m, n, k, 4000 + i)
            tot += tq + tg
            fl_tot += 2.0 * m * n * k
            torch.cuda.empty_cache()
        emit(cfg=4, op="total", M=m, total_us=round(tot * 1e3, 1), TFLOPs=round(fl_tot / tot / 1e9, 2))
    # grouped (MoE) block-FP8 GEMM, DeepSeek-V3 expert shapes: 256 experts (one GPU holding all of them) and
    # 32 (an 8-way expert-parallel share), equal groups of `rows` routed rows; every expert's weight is read once
    from sglang_amd.sgl_kernel import fp8_blockwise_scaled_grouped_mm

    for e in (32, 256) if want("moe") else ():
        for (n, k) in ((4096, 7168), (7168, 2048)):
            g = torch.Generator(device=dev).manual_seed(5000 + e)
            b = (torch.randn((e, n, k), generator=g, device=dev) * 0.5).to(torch.float8_e4m3fn)
            sb = torch.rand((e, k // 128, n // 128), generator=g, device=dev) * 1e-3 + 1e-4
            for rows in (2, 32, 128, 256):
                total = e * rows
                a = torch.randn((total, k), generator=g, device=dev).to(torch.float8_e4m3fn)
                sa = torch.rand((total, k // 128), generator=g, device=dev) * 1e-2 + 1e-3
                ps = torch.tensor([[rows, n, k]] * e, dtype=torch.int32, device=dev)
                eo = torch.arange(e, dtype=torch.int32, device=dev) * rows
                out = torch.empty((total, n), dtype=torch.bfloat16, device=dev)
                i64 = torch.empty((e,), dtype=torch.int64, device=dev)
                lay = torch.zeros((e, 5), dtype=torch.int32, device=dev)
                ws = torch.empty((1 << 20,), dtype=torch.uint8, device=dev)
                tg = time_kernel(lambda j: fp8_blockwise_scaled_grouped_mm(out, i64, i64, i64, i64, i64, a, b.transpose(1, 2), sa, sb,
                                                                           i64, i64, i64, lay, lay, ps, eo, ws), max(2, args.iters // 4))
                fl = 2.0 * total * n * k
                nbytes = e * n * k + total * k + 2 * total * n + 4 * total * (k // 128) + 4 * e * (k // 128) * (n // 128)
                emit(cfg="moe", op="fp8_blockwise_scaled_grouped_mm", experts=e, rows_per_expert=rows, N=n, K=k,
                     kernel=_lib.load().sglq_debug_last_gemm_kernel().decode(), gemm_us=round(tg * 1e3, 1),
                     gemm_TFLOPs=round(fl / tg / 1e9, 2), gemm_frac_mfma=round(fl / tg / 1e9 / PEAK_FP8_TFLOPS, 4),
                     gemm_GBs=round(nbytes / tg / 1e6, 1), gemm_frac_hbm=round(nbytes / tg / 1e6 / PEAK_HBM_GBS, 4))
            del b
            torch.cuda.empty_cache()
    # the whole expert layer (routing tables, gathers, two grouped GEMMs, SiLU-and-multiply, quantization, combine) on
    # DeepSeek-V3's expert shape, 32 local experts, top-8 routing among them: per-step device times and the layer's
    # (the layer runs the first quantization and the two gathers as one kernel, "quant_to_expert_rows_fused", and
    # SiLU-and-multiply and the second quantization as another, "silu_quant_fused"; the separate operators are timed
    # beside them and left out of the steps' sum)
    SEPARATE = ("quant1", "gather_codes", "gather_scales", "silu_and_mul", "quant2")
    if want("moe_layer"):
        from sglang_amd.moe.cutlass_moe import cutlass_fused_experts_fp8
        from sglang_amd.sgl_kernel import apply_shuffle_mul_sum, prepare_moe_input, shuffle_rows, silu_and_mul
        from sglang_amd.sgl_kernel.moe import per_token_group_quant_fp8_to_expert_rows, silu_and_mul_per_token_group_quant_fp8

        e, k, n, topk = 32, 7168, 2048, 8
        g = torch.Generator(device=dev).manual_seed(6000)
        w1 = (torch.randn((e, 2 * n, k), generator=g, device=dev) * 0.5).to(torch.float8_e4m3fn).transpose(1, 2)
        w2 = (torch.randn((e, k, n), generator=g, device=dev) * 0.5).to(torch.float8_e4m3fn).transpose(1, 2)
        s1 = torch.rand((e, k // 128, 2 * n // 128), generator=g, device=dev) * 1e-3 + 1e-4
        s2 = torch.rand((e, n // 128, k // 128), generator=g, device=dev) * 1e-3 + 1e-4
        i64 = torch.empty((e,), dtype=torch.int64, device=dev)
        lay = torch.zeros((e, 5), dtype=torch.int32, device=dev)
        ws = torch.empty((1 << 20,), dtype=torch.uint8, device=dev)
        offs = torch.empty((e + 1,), dtype=torch.int32, device=dev)
        ps1, ps2 = torch.empty((e, 3), dtype=torch.int32, device=dev), torch.empty((e, 3), dtype=torch.int32, device=dev)
        for m in (16, 512, 4096):
            x = make_activation(m, k, 6000 + m, dev)
            ids = torch.rand((m, e), generator=g, device=dev).argsort(dim=1)[:, :topk].to(torch.int32).contiguous()
            tw = torch.softmax(torch.rand((m, topk), generator=g, device=dev), dim=-1)
            rows = m * topk
            a_map = torch.empty((rows,), dtype=torch.int32, device=dev)
            c_map = torch.empty((rows,), dtype=torch.int32, device=dev)
            iters = max(2, args.iters // 4)
            t = {}
            t["prepare"] = time_kernel(lambda j: prepare_moe_input(ids, offs, ps1, ps2, a_map, c_map, e, n, k), iters)
            t["quant1"] = time_kernel(lambda j: sglang_per_token_group_quant_fp8(x, 128), iters)
            a_q, a_s = sglang_per_token_group_quant_fp8(x, 128)
            t["gather_codes"] = time_kernel(lambda j: shuffle_rows(a_q, a_map, (rows, k)), iters)
            t["gather_scales"] = time_kernel(lambda j: shuffle_rows(a_s, a_map, (rows, k // 128)), iters)
            t["quant_to_expert_rows_fused"] = time_kernel(lambda j: per_token_group_quant_fp8_to_expert_rows(x, c_map, topk, 128), iters)
            rq, rs = shuffle_rows(a_q, a_map, (rows, k)), shuffle_rows(a_s, a_map, (rows, k // 128))
            c1 = torch.empty((rows, 2 * n), dtype=torch.bfloat16, device=dev)
            c2 = torch.empty((rows, k), dtype=torch.bfloat16, device=dev)
            gmm = lambda out, a, b, sa, sb, ps: fp8_blockwise_scaled_grouped_mm(out, i64, i64, i64, i64, i64, a, b, sa, sb, i64, i64, i64,
                                                                                lay, lay, ps, offs[:-1], ws)
            t["gemm1"] = time_kernel(lambda j: gmm(c1, rq, w1, rs, s1, ps1), iters)
            t["silu_and_mul"] = time_kernel(lambda j: silu_and_mul(c1), iters)
            inter = silu_and_mul(c1)
            t["quant2"] = time_kernel(lambda j: sglang_per_token_group_quant_fp8(inter, 128), iters)
            t["silu_quant_fused"] = time_kernel(lambda j: silu_and_mul_per_token_group_quant_fp8(c1, 128), iters)
            iq, isc = sglang_per_token_group_quant_fp8(inter, 128)
            t["gemm2"] = time_kernel(lambda j: gmm(c2, iq, w2, isc, s2, ps2), iters)
            res = torch.empty((m, k), dtype=torch.bfloat16, device=dev)
            twb = tw.to(torch.bfloat16)
            t["combine"] = time_kernel(lambda j: apply_shuffle_mul_sum(c2, res, c_map, twb), iters)
            layer = time_kernel(lambda j: cutlass_fused_experts_fp8(x, w1, w2, s1, s2, tw, ids, i64, i64, i64, i64, ws, i64, i64, i64, i64,
                                                                    i64, offs, ps1, ps2), iters)
            fl = 2.0 * rows * (2 * n * k + n * k)
            moved = {"gather_codes": 2 * rows * k, "gather_scales": 8 * rows * (k // 128), "silu_and_mul": 6 * rows * n,
                     "quant1": group_quant_bytes(m, k), "quant2": group_quant_bytes(rows, n),
                     "silu_quant_fused": 5 * rows * n + 4 * rows * (n // 128),
                     "quant_to_expert_rows_fused": 2 * m * k + rows * k + 4 * rows * (k // 128), "combine": 2 * rows * k + 2 * m * k}
            emit(cfg="moe_layer", op="cutlass_fused_experts_fp8", experts=e, topk=topk, M=m, hidden=k, intermediate=n,
                 layer_us=round(layer * 1e3, 1), layer_TFLOPs=round(fl / layer / 1e9, 2),
                 steps_us={s: round(v * 1e3, 1) for s, v in t.items()}, steps_sum_us=round(sum(v for s, v in t.items() if s not in SEPARATE) * 1e3, 1),
                 steps_GBs={s: round(b / t[s] / 1e6, 1) for s, b in moved.items()})
    if f is not None:
        f.close()


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--cpu-rows", type=int, default=4096, help="activation rows in the CPU-baseline sample")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 256 MiB copy kernel first (reference point for the rocprofv3 byte counters)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-configs", action="store_true", help="skip the `configs` block (every baseline configuration, graph-timed)")
    ap.add_argument("--launches", type=str, default=None,
                    help='"M,N,K;M,N,K;...": run these block-FP8 linears as plain launches in this order and exit (for profiler counter runs)')
    ap.add_argument("--launch-reps", type=int, default=5)
    ap.add_argument("--force-tile", type=int, default=0, help="with --launches: the kernel code of sglq_debug_force_tile for every GEMM (0 = the selection rules)")
    ap.add_argument("--ab", type=str, default=None, metavar="OTHER.so",
                    help="with --launches: alternate the block-FP8 GEMM of another build of libsglq.so with the tree's in one process")
    ap.add_argument("--rotate-weights", action="store_true",
                    help="with --launches: rotate the weight over copies of 320 MB and more in total (weights come from HBM every time)")
    ap.add_argument("--kind", type=str, default="block_fp8", choices=("block_fp8", "fp8", "int8"),
                    help="with --launches: the block-scaled FP8 linear (default), or the per-token FP8 / INT8 one")
    ap.add_argument("--ue8m0", action="store_true",
                    help="with --launches: power-of-two scales (per_token_group_quant_fp8_pow2 + fp8_blockwise_scaled_mm_ue8m0)")
    ap.add_argument("--fill", action="store_true", help="only measure what the compute units take in through their LDS (copy loop without arithmetic) and exit")
    ap.add_argument("--ceiling", action="store_true", help="only measure the MFMA pipe's sustained rate (register-only loop) and exit")
    ap.add_argument("--graph", action="store_true", help="also time the K steps replayed as one HIP graph (graph_ms_per_step)")
    ap.add_argument("--prewarm-ms", type=float, default=150.0, help="untimed steps for this long before the warm-up steps")
    ap.add_argument("--sweep", type=str, default=None, help="write per-shape lines for every configuration to this file")
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--sweep-only", type=str, default=None,
                    help="with --sweep: comma-separated configurations to run (0, 1, 2, 3, 4, moe, moe_layer); default all")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path is measured on one GPU only (it needs no exchange between GPUs; "
              "a tensor-parallel deployment shards N or K per rank and all-reduces outside it). Run with --gpus 1.",
              file=sys.stderr)
        sys.exit(2)
    if args.launches and args.ab:
        run_ab(args)
    elif args.launches:
        run_launches(args)
    elif args.fill:
        run_fill(args)
    elif args.ceiling:
        run_ceiling(args)
    elif args.sweep:
        run_sweep(args)
    else:
        run_headline(args)


if __name__ == "__main__":
    main()
