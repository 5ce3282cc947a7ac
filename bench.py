"""Benchmark of the blockwise int8 hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload (the configuration the headline metric is quoted on): int8 block GEMM with fused dequantize at
M = N = K = 8192, block 128, bf16 out, operands = block-quantized bf16 N(0,1) activations and 0.02*N(0,1)
weights (seed 0), already resident in HBM; next to it the block quantize -> dequantize round trip of a bf16
[8192,8192] tensor with 0.1% x50 outliers at blocks 32/64/128, and ("extras") the block-64 GEMM, the decode GEMM
and the transposed quantizer.  A "step" is one GEMM launch through the drop-in operator.  Prints ONE JSON line.

Kernel durations are measured with HIP events recorded on the stream the kernels are launched on (torch's
current stream), around runs of back-to-back launches.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5000.0        # MI355X, dense int8 MFMA, as published (256 CUs x 8192 ops/clk/CU x 2.4 GHz = 5033)
HBM_PEAK_GBS = 8000.0          # HBM3E, 8 TB/s
# Bytes that cross the L2 <-> fabric boundary in one 8192^3 block-128 launch of the headline kernel: FETCH_SIZE and
# WRITE_SIZE of rocprofv3 --pmc runs of this file, scaled by what the same counters read for a 256 MiB copy
# (x2.0 and x1.0); the runs and figures are in profiles/gemm_wide_8192x8192x8192_block128.md.  Counters cannot be read
# from inside the process, so this is a constant from those runs, labelled as such in the output ("traffic_source").
GEMM_8192_TRAFFIC_BYTES = 966965985
GEMM_8192_TRAFFIC_SOURCE = ("profiles/gemm_wide_8192x8192x8192_block128.md: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this "
                            "command, scaled by a 256 MiB copy; a constant, not measured in this run")
PREROLL_MAX = 400              # launches
PREROLL_BATCH = 10


def event_ms(fn, iters: int) -> float:
    """average duration of one `fn()` launch: `iters` back-to-back launches between two events"""
    import torch
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(iters):
        fn()
    stop.record()
    stop.synchronize()
    return start.elapsed_time(stop) / iters


def median_ms(fn, iters: int, reps: int = 3) -> float:
    """median of `reps` averages over `iters` back-to-back launches"""
    ts = sorted(event_ms(fn, iters) for _ in range(reps))
    return ts[len(ts) // 2]


def preroll(fn, torch):
    """Untimed launches until the chip's clocks have settled: after idle the first launches run at ramping clocks (up
    to 30 % slower, for about a hundred launches).  Batches of PREROLL_BATCH launches are timed with events until three
    batches in a row agree within 0.7 %, at most PREROLL_MAX launches.  Returns (launches made, ms per launch of the last batch)."""
    done, hist = 0, []
    while done < PREROLL_MAX:
        hist.append(event_ms(fn, PREROLL_BATCH))
        done += PREROLL_BATCH
        if len(hist) >= 3 and max(hist[-3:]) <= 1.007 * min(hist[-3:]):
            break
    return done, hist[-1]


def bench_quantize(pkg, torch, iters: int):
    """block quantize / dequantize of bf16 [8192,8192] with outliers, through the C ABI with preallocated outputs.
    Three independent sets of buffers are used in rotation (576 MiB in total), so that successive launches do
    not find their operands in the 256 MiB memory-side cache left there by the launch before."""
    from blockwise_int8_linear_amd import _lib
    lib = _lib.load()
    M = K = 8192
    E = M * K
    NSETS = 3
    xs = []
    for i in range(NSETS):
        gen = torch.Generator(device="cuda").manual_seed(i)
        x = torch.randn(M, K, device="cuda", generator=gen, dtype=torch.float32)
        gen1 = torch.Generator(device="cuda").manual_seed(100 + i)
        pos = torch.randperm(E, device="cuda", generator=gen1)[:E // 1000]      # distinct positions: exactly 0.1 %
        x.view(-1)[pos] *= 50.0
        del pos
        xs.append(x.to(torch.bfloat16))
        del x
    st = torch.cuda.current_stream().cuda_stream
    out = {}
    for B in (32, 64, 128):
        qs = [torch.empty(M, K, device="cuda", dtype=torch.int8) for _ in range(NSETS)]
        ss = [torch.empty(K // B, M, device="cuda", dtype=torch.float32) for _ in range(NSETS)]
        ds = [torch.empty(M, K, device="cuda", dtype=torch.bfloat16) for _ in range(NSETS)]
        turn = [0]

        def fq():
            i = turn[0] = (turn[0] + 1) % NSETS
            rc = lib.bi8_quantize_rowwise(xs[i].data_ptr(), 1, qs[i].data_ptr(), ss[i].data_ptr(), M, K, K, K, B, st)
            assert rc == 0

        def fd():
            i = turn[0] = (turn[0] + 1) % NSETS
            rc = lib.bi8_dequantize_rowwise(qs[i].data_ptr(), ss[i].data_ptr(), ds[i].data_ptr(), 1, M, K, K, K, B, st)
            assert rc == 0

        for f in (fq, fd):
            for _ in range(2 * NSETS):
                f()
        torch.cuda.synchronize()
        # five averages over `iters` launches each: the median is the figure reported, the best one next to it
        tqs = sorted(event_ms(fq, iters) for _ in range(5))
        tds = sorted(event_ms(fd, iters) for _ in range(5))
        tq, td = tqs[2], tds[2]
        nbytes = E * 3 + 4 * E // B                 # read 2 B + write 1 B per element (or the reverse) + scales
        mse = ((ds[0].float() - xs[0].float()) ** 2).mean().item()
        out[f"block{B}"] = {
            "bytes": nbytes,
            "quantize_us": round(tq * 1e3, 2), "quantize_GBps": round(nbytes / tq / 1e6, 1),
            "quantize_frac_hbm": round(nbytes / tq / 1e6 / HBM_PEAK_GBS, 4),
            "dequantize_us": round(td * 1e3, 2), "dequantize_GBps": round(nbytes / td / 1e6, 1),
            "dequantize_frac_hbm": round(nbytes / td / 1e6 / HBM_PEAK_GBS, 4),
            "quantize_best_us": round(tqs[0] * 1e3, 2), "dequantize_best_us": round(tds[0] * 1e3, 2),
            "timing": f"median of 5 averages over {iters} launches (best next to it)",
            "roundtrip_mse": mse,
        }
        del qs, ss, ds
    return out


def bench_extras(pkg, torch):
    """secondary figures of the same path (each the median of three averages over a run of back-to-back launches), all
    through the C ABI with preallocated outputs: the block-64 GEMM at
    8192^3, the few-row (decode) GEMM at Llama-7B shapes with the weights rotated through ~600 MB so that they come
    from HBM (and the one-token eval-path linear, quantize included, as two launches and as one kernel), the
    transposed quantizer of the backward pass and the quantizer that writes both directions from one read"""
    from blockwise_int8_linear_amd import _lib
    lib = _lib.load()
    st = torch.cuda.current_stream().cuda_stream
    out = {}
    S, B = 8192, 64
    a = torch.randint(-127, 128, (S, S), device="cuda", dtype=torch.int8)
    w = torch.randint(-127, 128, (S, S), device="cuda", dtype=torch.int8)
    sa = torch.rand(S // B, S, device="cuda") + 0.5
    sw = torch.rand(S // B, S, device="cuda") * 0.02
    c = torch.empty(S, S, device="cuda", dtype=torch.bfloat16)

    def g64():
        assert lib.bi8_gemm_nt_dequant(a.data_ptr(), w.data_ptr(), sa.data_ptr(), sw.data_ptr(), None, 0, c.data_ptr(), 1,
                                       S, S, S, S, S, S, B, st) == 0
    g64()
    t = median_ms(g64, 10)
    out["gemm_block64_8192"] = {"ms": round(t, 4), "TOPS": round(2.0 * S ** 3 / t / 1e9, 1)}
    del sa, sw
    sa = torch.rand(S // 32, S, device="cuda") + 0.5
    sw = torch.rand(S // 32, S, device="cuda") * 0.02

    def g32():
        assert lib.bi8_gemm_nt_dequant(a.data_ptr(), w.data_ptr(), sa.data_ptr(), sw.data_ptr(), None, 0, c.data_ptr(), 1,
                                       S, S, S, S, S, S, 32, st) == 0
    g32()
    t = median_ms(g32, 10)
    out["gemm_block32_8192"] = {"ms": round(t, 4), "TOPS": round(2.0 * S ** 3 / t / 1e9, 1)}
    del sa, sw, c

    # Context, not part of the path: the vendor library's PLAIN int8 GEMM (int32 out, no scales, no fold) on random
    # codes of the same shape, and the block-128 kernel on all-zero codes.  Both show how far the chip's power
    # management moves the ceiling with the data: the published peak is quoted at 2.4 GHz, which the chip holds only
    # when the operands do not toggle.
    try:
        wt = w.t()
        for _ in range(30):
            torch._int_mm(a, wt)
        t = median_ms(lambda: torch._int_mm(a, wt), 30)
        out["context_vendor_plain_int8_gemm_8192_random_codes"] = {"ms": round(t, 4), "TOPS": round(2.0 * S ** 3 / t / 1e9, 1),
                                                                   "what": "torch._int_mm (hipBLASLt), int32 out, no dequantize"}
    except Exception as e:                          # not every torch build has it: the figure is context only
        out["context_vendor_plain_int8_gemm_8192_random_codes"] = {"error": repr(e)[:120]}
    del a, w
    z = torch.zeros(S, S, device="cuda", dtype=torch.int8)
    sa = torch.rand(S // 128, S, device="cuda") + 0.5
    sw = torch.rand(S // 128, S, device="cuda") * 0.02
    c = torch.empty(S, S, device="cuda", dtype=torch.bfloat16)

    def gz():
        assert lib.bi8_gemm_nt_dequant(z.data_ptr(), z.data_ptr(), sa.data_ptr(), sw.data_ptr(), None, 0, c.data_ptr(), 1,
                                       S, S, S, S, S, S, 128, st) == 0
    for _ in range(30):
        gz()
    t = median_ms(gz, 20)
    out["context_gemm_block128_8192_zero_codes"] = {"ms": round(t, 4), "TOPS": round(2.0 * S ** 3 / t / 1e9, 1)}
    del z, sa, sw, c

    B = 128
    for (K, N) in ((4096, 11008), (11008, 4096)):
        nset = max(2, int(600e6 // (N * K)))
        ws = [torch.randint(-127, 128, (N, K), device="cuda", dtype=torch.int8) for _ in range(nset)]
        sw = torch.rand(K // B, N, device="cuda") * 0.02
        for M in (1, 16, 32):
            x = torch.randint(-127, 128, (M, K), device="cuda", dtype=torch.int8)
            sx = torch.rand(K // B, M, device="cuda") + 0.5
            c = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            turn = [0]
            need = lib.bi8_gemm_workspace_bytes(M, N, K, B)          # scratch memory, as the Python operator passes it
            scratch = torch.empty(max(need, 16), device="cuda", dtype=torch.uint8)

            def gv():
                i = turn[0] = (turn[0] + 1) % nset
                assert lib.bi8_gemm_nt_dequant_ws(x.data_ptr(), ws[i].data_ptr(), sx.data_ptr(), sw.data_ptr(), None, 0, c.data_ptr(), 1,
                                                  M, N, K, K, K, N, B, scratch.data_ptr(), need, st) == 0
            for _ in range(5):
                gv()
            t = median_ms(gv, 50)
            nbytes = N * K + 4 * (K // B) * (N + M) + M * K + 2 * M * N
            out[f"decode_gemm_M{M}_K{K}_N{N}"] = {"us": round(t * 1e3, 2), "GBps": round(nbytes / t / 1e6, 1),
                                                  "frac_hbm": round(nbytes / t / 1e6 / HBM_PEAK_GBS, 4),
                                                  "kernel": lib.bi8_gemm_kernel_name(M, N, K, K, K, B, need).decode()}
            if M == 1:
                # the whole eval-path linear for one token: row quantizer + GEMM as two launches, and as the one kernel
                xf = torch.randn(M, K, device="cuda").to(torch.bfloat16)
                xq = torch.empty(M, K, device="cuda", dtype=torch.int8)

                def two():
                    i = turn[0] = (turn[0] + 1) % nset
                    assert lib.bi8_quantize_rowwise(xf.data_ptr(), 1, xq.data_ptr(), sx.data_ptr(), M, K, K, K, B, st) == 0
                    assert lib.bi8_gemm_nt_dequant(xq.data_ptr(), ws[i].data_ptr(), sx.data_ptr(), sw.data_ptr(), None, 0,
                                                   c.data_ptr(), 1, M, N, K, K, K, N, B, st) == 0

                def one():
                    i = turn[0] = (turn[0] + 1) % nset
                    assert lib.bi8_linear_few_rows(xf.data_ptr(), 1, ws[i].data_ptr(), sw.data_ptr(), None, 0, c.data_ptr(),
                                                   M, N, K, K, K, N, B, st) == 0
                for _ in range(5):
                    two(), one()
                t2 = median_ms(two, 50)
                t1 = median_ms(one, 50)
                out[f"decode_linear_M1_K{K}_N{N}"] = {"one_kernel_us": round(t1 * 1e3, 2), "two_launches_us": round(t2 * 1e3, 2)}
        del ws

    # The Llama-7B GEMM shapes at 2048 (and, against 4096 columns, 1024) and at 128 rows of activations (prefill; a decode
    # batch), and 512 tokens against GPT-2-small's layers: through the entry point that takes scratch memory, as the Python operator calls it (problems
    # of few tiles run on narrow tiles, one per CU, or split K over the workgroups)
    shapes = [(M, K, N) for M in (2048, 128) for (K, N) in ((4096, 4096), (4096, 11008), (11008, 4096), (4096, 12288))]
    shapes += [(512, 768, 2304), (512, 768, 3072), (512, 3072, 768)]
    shapes += [(1024, 4096, 4096), (1024, 11008, 4096)]          # 1024 tokens against N = 4096: 256 tiles of 128 x 128
    for (M, K, N) in shapes:
        if True:
            x = torch.randint(-127, 128, (M, K), device="cuda", dtype=torch.int8)
            # up to 512 rows the time is the pass over W: W comes from HBM (rotated through 600 MB, as for the decode shapes)
            nset = max(1, int(600e6 // (N * K))) if M <= 512 else 1
            wsets = [torch.randint(-127, 128, (N, K), device="cuda", dtype=torch.int8) for _ in range(nset)]
            sx = torch.rand(K // B, M, device="cuda") + 0.5
            sw = torch.rand(K // B, N, device="cuda") * 0.02
            c = torch.empty(M, N, device="cuda", dtype=torch.bfloat16)
            need = lib.bi8_gemm_workspace_bytes(M, N, K, B)
            ws = torch.empty(max(need, 16), device="cuda", dtype=torch.uint8)
            turn = [0]

            def gp():
                i = turn[0] = (turn[0] + 1) % nset
                assert lib.bi8_gemm_nt_dequant_ws(x.data_ptr(), wsets[i].data_ptr(), sx.data_ptr(), sw.data_ptr(), None, 0, c.data_ptr(), 1,
                                                  M, N, K, K, K, N, B, ws.data_ptr(), need, st) == 0
            for _ in range(100 if M < 1024 else 20):          # (short kernels: the clock needs a few hundred microseconds of work to settle)
                gp()
            t = median_ms(gp, 30)
            out[f"{'prefill' if M >= 1024 else 'batch128' if M == 128 else 'tokens512'}_gemm_M{M}_K{K}_N{N}"] = {
                "us": round(t * 1e3, 1), "TOPS": round(2.0 * M * N * K / t / 1e9, 1),
                "frac_int8_peak": round(2.0 * M * N * K / t / 1e9 / INT8_PEAK_TOPS, 4),
                "kernel": lib.bi8_gemm_kernel_name(M, N, K, K, K, B, need).decode()}
            del x, wsets, c, ws

    M = K = 8192
    xs = [torch.randn(M, K, device="cuda", dtype=torch.float32).to(torch.bfloat16) for _ in range(3)]
    qs = [torch.empty(K, M, device="cuda", dtype=torch.int8) for _ in range(3)]
    ss = [torch.empty(M // 128, K, device="cuda", dtype=torch.float32) for _ in range(3)]
    turn = [0]

    def qt():
        i = turn[0] = (turn[0] + 1) % 3
        assert lib.bi8_quantize_transposed(xs[i].data_ptr(), 1, qs[i].data_ptr(), ss[i].data_ptr(), M, K, K, M, 128, st) == 0
    for _ in range(6):
        qt()
    t = median_ms(qt, 30)
    nbytes = M * K * 3 + 4 * M * K // 128
    out["quantize_transposed_bf16_8192"] = {"us": round(t * 1e3, 2), "GBps": round(nbytes / t / 1e6, 1),
                                            "frac_hbm": round(nbytes / t / 1e6 / HBM_PEAK_GBS, 4)}

    # both directions from one read (three buffer sets again)
    qr = [torch.empty(M, K, device="cuda", dtype=torch.int8) for _ in range(3)]
    sr = [torch.empty(K // 128, M, device="cuda", dtype=torch.float32) for _ in range(3)]

    def qd():
        i = turn[0] = (turn[0] + 1) % 3
        assert lib.bi8_quantize_dual(xs[i].data_ptr(), 1, qr[i].data_ptr(), sr[i].data_ptr(), qs[i].data_ptr(), ss[i].data_ptr(),
                                     M, K, K, K, M, 128, st) == 0
    for _ in range(6):
        qd()
    t = median_ms(qd, 30)
    nbytes = M * K * 4 + 8 * M * K // 128
    out["quantize_dual_bf16_8192"] = {"us": round(t * 1e3, 2), "GBps": round(nbytes / t / 1e6, 1),
                                      "frac_hbm": round(nbytes / t / 1e6 / HBM_PEAK_GBS, 4)}

    # Context, not part of the path: what torch's device-to-device copy of the same 128 MiB (the dual quantizer's input;
    # it writes as many bytes again) reaches on this chip, three buffer pairs in rotation.  For scale only: a hand-written
    # copy kernel with non-temporal 16-byte accesses measured 6.2 TB/s, the row quantizer's rate.
    ds = [torch.empty_like(x) for x in xs]

    def cp():
        i = turn[0] = (turn[0] + 1) % 3
        ds[i].copy_(xs[i])
    for _ in range(6):
        cp()
    t = median_ms(cp, 30)
    nbytes = 2 * xs[0].numel() * xs[0].element_size()
    out["context_device_copy_128MiB"] = {"us": round(t * 1e3, 2), "GBps": round(nbytes / t / 1e6, 1),
                                         "frac_hbm": round(nbytes / t / 1e6 / HBM_PEAK_GBS, 4), "what": "torch dst.copy_(src), read + write"}
    return out


def cpu_baseline(torch, xq, wq, sx, sw, B, chunk: int = 2048):
    """the PyTorch CPU restatement of the reference math (oracle/oracle_torch.py) on this host's cores: the same
    8192^3 problem, in row chunks so that the int32 partials of one chunk fit comfortably in memory"""
    from oracle import oracle_torch
    M, K = xq.shape
    N = wq.shape[0]
    t0 = time.perf_counter()
    for r0 in range(0, M, chunk):
        oracle_torch.int8_matmul_block_dequantize(xq[r0:r0 + chunk], wq, sx[:, r0:r0 + chunk].contiguous(), sw, B, None, torch.bfloat16)
    dt = time.perf_counter() - t0
    return {
        "value": round(2.0 * M * N * K / dt / 1e12, 4), "unit": "TOPS", "cores": torch.get_num_threads(), "kind": "port",
        "sample": f"oracle/oracle_torch.py (PyTorch eager: fp32 bmm per K-block, exact for int8 codes, + fp32 rescale) on the whole "
                  f"{M}x{N}x{K} problem, block {B}, bf16 out, in {M // chunk} row chunks: {dt:.1f} s on {torch.get_num_threads()} "
                  f"threads ({os.cpu_count()} logical CPUs)",
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=50)
    ap.add_argument("--size", type=int, default=8192, help="M = N = K of the GEMM (the metric is quoted at 8192)")
    ap.add_argument("--shape", type=int, nargs=3, metavar=("M", "N", "K"), default=None,
                    help="another GEMM shape in place of the headline one (for profiles of the kernels that run other shapes)")
    ap.add_argument("--block", type=int, default=None, help="block size of the GEMM with --shape (default 128)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-quantize", action="store_true")
    ap.add_argument("--no-extras", action="store_true", help="skip the secondary figures (their small launches share kernel names with the round trip)")
    ap.add_argument("--no-preroll", action="store_true", help="skip the untimed launches that let the clocks settle before the warm-up")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch a plain 256 MiB device-to-device copy 5 times (a kernel of known traffic, for scaling "
                         "the FETCH_SIZE / WRITE_SIZE counters of a rocprofv3 --pmc run)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build is a one-GPU path (no collectives, no sharding); run it with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch

    import blockwise_int8_linear_amd as pkg
    from blockwise_int8_linear_amd import _lib
    _lib.load()                                     # fails loudly if libbi8.so is not built
    assert torch.cuda.is_available(), "bench.py needs the GPU"
    torch.cuda.set_device(0)
    cfg = pkg.block_linear_config
    B = cfg.GROUP_SIZE
    assert B == 128 and cfg.INPUT_OUTPUT_TORCH_TYPE == torch.bfloat16
    S = args.size
    M, N, K = args.shape if args.shape else (S, S, S)
    if args.shape and args.block:
        B = cfg.GROUP_SIZE = args.block

    if args.calibrate_copy:
        src = torch.empty(256 * 1024 * 1024, device="cuda", dtype=torch.uint8).random_(0, 255)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    torch.manual_seed(0)
    x = torch.randn(M, K, device="cuda", dtype=torch.float32).to(torch.bfloat16)
    w = (torch.randn(N, K, device="cuda", dtype=torch.float32) * 0.02).to(torch.bfloat16)
    xq, sx = pkg.quantize_block_rowwise(x)
    wq, sw = pkg.quantize_block_rowwise(w)
    wqt = wq.t()
    del x, w

    def step():
        return pkg.int8_matmul_block64_rowwise_dequantize(xq, wqt, sx, sw)

    step()
    torch.cuda.synchronize()
    # For the record, the figure WITHOUT the pre-roll below: `warmup` launches, then `steps` timed ones, straight from an
    # idle chip, whose shader clock is still ramping (reported as roofline.cold_start_avg_launch_ms; not the headline)
    for _ in range(args.warmup):
        step()
    cold_ms = event_ms(step, args.steps)
    preroll_launches, preroll_ms = (0, None) if args.no_preroll else preroll(step, torch)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    # the timed region: exactly `steps` launches, wall clock between two synchronizations, and HIP events on the
    # stream the kernel runs on (torch's current stream) before the first and after every launch: the kernel's
    # average duration is (last - first) / steps, the per-launch durations give the median
    evs = [torch.cuda.Event(enable_timing=True) for _ in range(args.steps + 1)]
    t0 = time.perf_counter()
    evs[0].record()
    for i in range(args.steps):
        step()
        evs[i + 1].record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps

    # context: the vendor library's plain int8 GEMM (int32 out, no scales, nothing folded) on the SAME operands, right
    # after the timed region, with the clocks where the timed launches left them
    vendor_ms = None
    try:
        for _ in range(10):
            torch._int_mm(xq, wqt)
        vendor_ms = median_ms(lambda: torch._int_mm(xq, wqt), args.steps)
    except Exception:                               # not every torch build has it: the figure is context only
        pass

    ops_per_launch = 2.0 * M * N * K
    kern_ms = evs[0].elapsed_time(evs[-1]) / args.steps
    per_launch = sorted(evs[i].elapsed_time(evs[i + 1]) for i in range(args.steps))
    launch_median = per_launch[len(per_launch) // 2] if len(per_launch) % 2 else 0.5 * (per_launch[len(per_launch) // 2 - 1] + per_launch[len(per_launch) // 2])
    achieved = ops_per_launch / kern_ms / 1e9       # TOPS
    lib = _lib.load()
    kernel = lib.bi8_gemm_kernel_name(M, N, K, K, K, B, lib.bi8_gemm_workspace_bytes(M, N, K, B)).decode()
    headline = (M, N, K, B) == (8192, 8192, 8192, 128)

    res = {
        "metric": "int8 block GEMM TOPS (% int8 MFMA peak) at 8192^3; quantize GB/s (% HBM)",
        "value": round(ops_per_launch / wall_ms / 1e9, 2), "unit": "TOPS",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(wall_ms, 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8", "data": "synthetic",
        "config": {"workload": f"int8 block GEMM + fused dequantize, M={M} N={N} K={K}, block {B}, bf16 out; A = quantize(bf16 N(0,1)), "
                               f"W = quantize(bf16 0.02*N(0,1)), seed 0; one launch per step via "
                               f"int8_matmul_block64_rowwise_dequantize",
                   "block": B, "out_dtype": "bf16"},
        "roofline": {"bound": "mfma", "achieved": round(achieved, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                     "frac": round(achieved / INT8_PEAK_TOPS, 4),
                     "traffic": GEMM_8192_TRAFFIC_BYTES if headline else None,
                     "traffic_source": GEMM_8192_TRAFFIC_SOURCE if headline else None,
                     "kernel": f"{kernel}<{B},bf16> (the library's choice for this shape: bi8_gemm_kernel_name)",
                     "ops_per_launch": ops_per_launch, "avg_launch_ms": round(kern_ms, 4), "median_launch_ms": round(launch_median, 4),
                     "frac_of_5033_TOPs_at_2p4GHz": round(achieved / 5033.2, 4),
                     "preroll_launches": preroll_launches, "preroll_last_batch_ms": None if preroll_ms is None else round(preroll_ms, 4),
                     "cold_start_avg_launch_ms": round(cold_ms, 4),
                     "context_vendor_plain_int8_gemm_same_operands_ms": None if vendor_ms is None else round(vendor_ms, 4),
                     "time_relative_to_vendor_plain_int8_gemm": None if vendor_ms is None else round(kern_ms / vendor_ms, 3)},
    }
    if not args.no_quantize:
        res["quantize_roundtrip"] = bench_quantize(pkg, torch, 50)
    if not args.no_quantize and not args.no_extras:
        res["extras"] = bench_extras(pkg, torch)
    if not args.no_cpu_baseline:
        res["cpu_baseline"] = cpu_baseline(torch, xq.cpu(), wq.cpu(), sx.cpu(), sw.cpu(), B)
    print(json.dumps(res))


if __name__ == "__main__":
    main()
