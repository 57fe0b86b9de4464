"""Tunes the kernel selection of the block-scaled FP8 GEMM for given (N, K) over a grid of batch
sizes and writes the table that tuned_configs.load_tuned_configs reads: the counterpart of the
reference's benchmark/kernels/quantization/tuning_block_wise_kernel.py for its Triton kernel.

    python -m sglang_amd.quantization.tune_block_fp8 --N 4096 --K 7168 [--M 1 8 64 ...] [--out DIR] [--dtype int8_w8a8]

(--dtype int8_w8a8 tunes the block-scaled INT8 GEMM, w8a8_block_int8_matmul, instead; fp8_w8a8_channel / int8_w8a8_channel
tune fp8_scaled_mm / int8_scaled_mm, whose kernel the reference picks per M bucket in C++, sgl-kernel/csrc/gemm/fp8_gemm_kernel.cu:751-791,
int8_gemm_kernel.cu:585-661.)

Every candidate (kernel code, split-K factor) is timed from HIP-graph replays with the weights
rotated through more than the last-level cache; an entry is written only where a candidate beats
the built-in selection by more than --margin (default 4 %; its slowest of three runs against the built-in
selection's fastest of three), otherwise {"tile": 0, "splits": 0}.

    python -m sglang_amd.quantization.tune_block_fp8 --verify [--fix] [--verify-margin 0.03] [--dir DIR]
    python -m sglang_amd.quantization.tune_block_fp8 --apply VERIFY_OUTPUT

re-times every entry of every shipped table against the built-in selection of the library at hand (alternated,
as above) and lists the entries that no longer win by more than the margin; --fix resets those to the built-in
selection in their files (--apply does the same from the saved output of a --verify run, on a machine without a GPU).
Run it after a kernel or a selection rule has changed."""

from __future__ import annotations

import argparse
import json
import time

import torch

DEFAULT_M = [1, 2, 4, 8, 16, 24, 32, 48, 64, 96, 128, 256, 512, 1024, 1536, 2048, 3072, 4096, 8192]


def candidates(m: int, n: int, k: int):
    """(tile code, splits) pairs worth timing for this shape."""
    out = [(0, 0)]
    nkb = k // 128
    if k % 128:
        return out
    if m <= 64 and k >= 512:
        out += [(16, 0), (32, 0)]
    if m <= 512:
        out += [(64, s) for s in (0, 2, 4, 8) if s == 0 or s <= nkb // 2]
        if m > 32:
            out += [(66, s) for s in (0, 1, 2, 4) if s <= 1 or s <= nkb // 4]
            if k >= 512:
                out += [(68, 0), (69, 0)]
    out += [(128, s) for s in (0, 2, 4) if s == 0 or s <= nkb // 4]
    if k >= 384 and m > 64:
        out += [(130, s) for s in (0, 1, 2, 4, 8) if s <= 1 or (nkb % s == 0 and nkb // s >= 3)]
        out += [(258, s) for s in (0, 1, 2, 4) if s <= 1 or (nkb % s == 0 and nkb // s >= 3)]
        if m > 256:
            out += [(192, 0), (224, 0), (257, 0), (193, 0)]  # (193: 192 x 192 tiles, block FP8 only; elsewhere the rules' choice)
    return out


class Harness:
    """Times the block-scaled GEMM of one (N, K) under a forced (kernel code, split-K factor) for any M: HIP-graph
    replays, the weights rotated over copies of 320 MB and more in total (past the 256 MiB last-level cache)."""

    def __init__(self, n: int, k: int, iters: int, dev, dtype: str = "fp8_w8a8"):
        from sglang_amd import _lib

        self.n, self.k, self.dev, self.int8 = n, k, dev, dtype.startswith("int8_w8a8")
        self.channel = dtype.endswith("_channel")  # per-token / per-channel scales: int8_scaled_mm, fp8_scaled_mm
        self.lib = _lib.load()
        self.g = torch.Generator(device=dev).manual_seed(n + k)
        if self.int8:
            w = torch.randint(-127, 128, (n, k), generator=self.g, device=dev, dtype=torch.int32).to(torch.int8)
        else:
            w = (torch.randn((n, k), generator=self.g, device=dev) * 0.5).to(torch.float8_e4m3fn)
        self.ws = torch.rand(((n + 127) // 128, (k + 127) // 128), generator=self.g, device=dev) * 1e-2 + 1e-3
        if self.channel:
            self.ws = torch.rand((n, 1), generator=self.g, device=dev) * 9e-3 + 1e-3
        # weights in rotation past the 256 MiB last-level cache (320 MB and more), as a model's layers come by in use
        self.copies = max(2, min(48, -(-320_000_000 // (n * k))))
        self.iters = max(iters, self.copies)
        self.wq = [w] + [w.clone() for _ in range(self.copies - 1)]
        self.m = None

    def set_m(self, m: int):
        n, k, g, dev = self.n, self.k, self.g, self.dev
        if self.channel:
            if self.int8:
                self.a = torch.randint(-127, 128, (m, k), generator=g, device=dev, dtype=torch.int32).to(torch.int8)
            else:
                self.a = (torch.randn((m, k), generator=g, device=dev) * 2).to(torch.float8_e4m3fn)
            self.sa = torch.rand((m, 1), generator=g, device=dev) * 1e-2 + 1e-3
        elif self.int8:
            self.a = torch.randint(-127, 128, (m, k), generator=g, device=dev, dtype=torch.int32).to(torch.int8)
            self.sa = torch.rand((m, k // 128), generator=g, device=dev) * 1e-2 + 1e-3  # row-major, as the INT8 quantizer writes it
        else:
            self.a = (torch.randn((m, k), generator=g, device=dev) * 2).to(torch.float8_e4m3fn)
            self.sa = (torch.rand((k // 128, m), generator=g, device=dev) * 1e-2 + 1e-3).t()  # column-major [m, k / 128]
        self.m = m

    def run(self, j):
        from sglang_amd.quantization.int8_kernel import w8a8_block_int8_matmul
        from sglang_amd.sgl_kernel import fp8_blockwise_scaled_mm, fp8_scaled_mm, int8_scaled_mm

        if self.channel:
            return (int8_scaled_mm if self.int8 else fp8_scaled_mm)(self.a, self.wq[j].t(), self.sa, self.ws, torch.bfloat16, None)
        if self.int8:
            return w8a8_block_int8_matmul(self.a, self.wq[j], self.sa, self.ws, [128, 128], torch.bfloat16)
        return fp8_blockwise_scaled_mm(self.a, self.wq[j].t(), self.sa, self.ws.t(), torch.bfloat16)

    def time_it(self):
        copies, iters = self.copies, self.iters
        for j in range(max(2, copies)):
            self.run(j % copies)
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for i in range(iters):
                self.run(i % copies)
        t0 = time.perf_counter()
        while True:  # untimed replays for 10 ms: a kernel timed right after a different one runs slower
            graph.replay()
            torch.cuda.synchronize()
            if time.perf_counter() - t0 >= 0.01:
                break
        s, e = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        best = float("inf")
        for _ in range(3):
            s.record()
            graph.replay()
            e.record()
            torch.cuda.synchronize()
            best = min(best, s.elapsed_time(e) / iters)
        return best

    def timed(self, tile: int, splits: int):
        """(ms per call, kernel name) under the forced selection; (0, 0) = the library's own choice."""
        self.lib.sglq_debug_force_tile(tile)
        self.lib.sglq_debug_force_splits(splits)
        try:
            return self.time_it(), self.lib.sglq_debug_last_gemm_kernel().decode()
        finally:
            self.lib.sglq_debug_force_tile(0)
            self.lib.sglq_debug_force_splits(0)

    def confirm(self, tile: int, splits: int, base: float, t: float, rounds: int = 2):
        """The entry against the built-in selection in alternation: the built-in's fastest and the entry's slowest."""
        for _ in range(rounds):
            base = min(base, self.timed(0, 0)[0])
            t = max(t, self.timed(tile, splits)[0])
        return base, t


def settle(dev):
    # untimed load for 150 ms first: the chip's clocks take that long to settle
    spin = torch.randn((4096, 4096), device=dev)
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < 0.15:
        torch.mm(spin, spin)
        torch.cuda.synchronize()


def tune(n: int, k: int, ms, iters: int, margin: float, dev, dtype: str = "fp8_w8a8"):
    h = Harness(n, k, iters, dev, dtype)
    h.lib.sglq_tuned_clear()
    settle(dev)
    table = {}
    for m in ms:
        h.set_m(m)
        results = {}
        for tile, splits in candidates(m, n, k):
            results[(tile, splits)] = h.timed(tile, splits)
        (tile, splits), (t, name) = min(results.items(), key=lambda kv: kv[1][0])
        base = results[(0, 0)][0]
        if (tile, splits) != (0, 0) and t < base * (1.0 - margin):
            # the same pair measured twice can differ by a few per cent: confirm the winner against the
            # built-in selection in alternation before it is written down
            base, t = h.confirm(tile, splits, base, t)
        if t < base * (1.0 - margin):
            table[m] = {"tile": tile, "splits": splits}
        else:
            table[m] = {"tile": 0, "splits": 0}
        print(json.dumps({"M": m, "N": n, "K": k, "default_us": round(base * 1e3, 2), "default_kernel": results[(0, 0)][1],
                          "best_us": round(t * 1e3, 2), "best": [tile, splits], "best_kernel": name, "chosen": table[m]}), flush=True)
    return table


def verify(config_dir, iters: int, margin: float, dev, fix: bool):
    """Every entry of every shipped table against the built-in selection of this library.  Returns
    (entries checked, entries that no longer win by more than `margin`)."""
    from pathlib import Path

    from sglang_amd.quantization import tuned_configs as T

    directory = Path(config_dir or T.CONFIG_DIR)
    settle(dev)
    checked, stale = 0, []
    for path in sorted(directory.iterdir()):
        parsed = T.parse_file_name(path.name)
        if parsed is None or parsed[2] != T.DEVICE_NAME or parsed[3] not in T.KIND_OF_DTYPE:
            continue
        n, k, _, dtype = parsed
        with open(path) as f:
            table = {int(key): val for key, val in json.load(f).items()}
        entries = [(m, int(v.get("tile", 0)), int(v.get("splits", 0))) for m, v in sorted(table.items())]
        entries = [e for e in entries if e[1] or e[2]]
        if not entries:
            continue
        h = Harness(n, k, iters, dev, dtype)
        h.lib.sglq_tuned_clear()  # (0, 0) must mean the built-in selection, not this table's entry
        changed = False
        for m, tile, splits in entries:
            h.set_m(m)
            base, base_kernel = h.timed(0, 0)
            t, kernel = h.timed(tile, splits)
            base, t = h.confirm(tile, splits, base, t, rounds=1)
            checked += 1
            wins = t < base * (1.0 - margin)
            row = {"dtype": dtype, "N": n, "K": k, "M": m, "entry": [tile, splits], "entry_kernel": kernel, "entry_us": round(t * 1e3, 2),
                   "builtin_kernel": base_kernel, "builtin_us": round(base * 1e3, 2), "gain": round(1.0 - t / base, 4), "still_wins": wins}
            print(json.dumps(row), flush=True)
            if not wins:
                stale.append(row)
                if fix:
                    table[m] = {"tile": 0, "splits": 0}
                    changed = True
        if changed:
            T.save_config(n, k, table, directory, dtype=dtype)
        del h
        torch.cuda.empty_cache()
    print(json.dumps({"checked": checked, "no_longer_winning": len(stale), "margin": margin, "fixed": bool(fix)}), flush=True)
    T.load_tuned_configs()
    return checked, stale


def apply_verify_log(log_path, config_dir=None):
    """Resets, in the tables' files, the entries that a --verify run (its output saved to `log_path`) lists with
    "still_wins": false.  Needs no GPU: the verification can run on one machine and the tables be edited on another."""
    from pathlib import Path

    from sglang_amd.quantization import tuned_configs as T

    directory = Path(config_dir or T.CONFIG_DIR)
    dropped = 0
    for line in open(log_path):
        if not line.startswith('{"dtype"'):
            continue
        row = json.loads(line)
        if row["still_wins"]:
            continue
        table = T.get_w8a8_block_fp8_configs(row["N"], row["K"], config_dir=directory, dtype=row["dtype"])
        if table is None or row["M"] not in table:
            continue
        entry = table[row["M"]]
        if [int(entry.get("tile", 0)), int(entry.get("splits", 0))] != row["entry"]:
            continue
        table[row["M"]] = {"tile": 0, "splits": 0}
        T.save_config(row["N"], row["K"], table, directory, dtype=row["dtype"])
        dropped += 1
    print(f"reset {dropped} entries")
    return dropped


def main():
    from sglang_amd.quantization.tuned_configs import save_config

    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--N", type=int, default=None)
    ap.add_argument("--K", type=int, default=None)
    ap.add_argument("--verify", action="store_true", help="re-time every shipped table entry against the built-in selection and list those that no longer win")
    ap.add_argument("--fix", action="store_true", help="with --verify: reset the entries that no longer win to the built-in selection in their files")
    ap.add_argument("--verify-margin", type=float, default=0.03)
    ap.add_argument("--apply", type=str, default=None, metavar="LOG",
                    help="reset the entries that the saved output of a --verify run lists as no longer winning (no GPU needed)")
    ap.add_argument("--dir", type=str, default=None, help="with --verify: directory of the tables (default: the package's configs/)")
    ap.add_argument("--M", type=int, nargs="*", default=DEFAULT_M)
    ap.add_argument("--iters", type=int, default=8)
    ap.add_argument("--margin", type=float, default=0.04)
    ap.add_argument("--out", type=str, default=None, help="directory for the table (default: the package's configs/)")
    ap.add_argument("--dtype", choices=["fp8_w8a8", "int8_w8a8", "fp8_w8a8_channel", "int8_w8a8_channel"], default="fp8_w8a8",
                    help="block-scaled FP8 or block-scaled INT8 GEMM; with _channel: fp8_scaled_mm / int8_scaled_mm (per-token and per-channel scales)")
    args = ap.parse_args()
    if args.apply:
        apply_verify_log(args.apply, args.dir)
        return
    dev = torch.device("cuda:0")
    if args.verify:
        verify(args.dir, args.iters, args.verify_margin, dev, args.fix)
        return
    if args.N is None or args.K is None:
        ap.error("--N and --K are required (or --verify)")
    table = tune(args.N, args.K, args.M, args.iters, args.margin, dev, args.dtype)
    path = save_config(args.N, args.K, table, args.out, dtype=args.dtype)
    print("wrote", path)


if __name__ == "__main__":
    main()
