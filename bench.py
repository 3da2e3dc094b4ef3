#!/usr/bin/env python3
"""Benchmark of the fused 2-bit quantize step on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one error-feedback quantize pass (a = g + r; codes; r' written back;
16 codes packed per word) over the GPT-2-medium-sized gradient of 354,823,168
fp32 elements, inputs resident in HBM.  Prints one JSON line:

  value        GB/s = 12.25 bytes/element * N / wall time per step
               (read g 4 + read r 4 + write r' 4 + write codes 0.25)
  roofline     the same bytes over the average kernel time between two HIP
               events on the launch stream, against the 8 TB/s HBM peak
  cpu_baseline the C restatement of the reference kernel (oracle/), OpenMP over
               the host cores, timed on a slab of the same gradient
  extras       decode (elements/s), 8-payload fixed-order sum, plain copy

The CPU checker is used for the cpu_baseline leg only, never for the GPU path.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

N_ELEMS = 354_823_168          # GPT-2-medium parameter count
THRD = 2e-3
HBM_PEAK_GBPS = 8000.0         # MI355X HBM3E, published
BYTES_QUANT = 12.25            # per element, fused step
BYTES_DEQUANT = 4.25           # per element, decode (overwrite)
K_PAYLOADS = 8                 # receive side: local + 7 peers


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--elems", type=int, default=N_ELEMS, help="gradient length (default: the headline size)")
    ap.add_argument("--chunk", type=int, default=0,
                    help="elements per launch (multiple of 16); 0 = the whole gradient in one launch. "
                         "The HBM-sizing workload is --elems 2800000000 --chunk 268435456")
    ap.add_argument("--cpu-seconds", type=float, default=20.0, help="CPU-baseline time budget; 0 skips it")
    ap.add_argument("--legs", default="deq,acc,copy,cpu",
                    help="extra legs after the timed quantize steps: deq, acc, copy, cpu, and (off by "
                         "default) matrix, multi (comma list, '' = none)")
    return ap.parse_args()


def student_t3(n, gen, torch):
    """1e-3 * Student-t(3) on the GPU: z / sqrt(chi2_3 / 3), built slab-wise to bound scratch memory."""
    out = torch.empty(n, dtype=torch.float32, device="cuda")
    slab = 1 << 26
    for lo in range(0, n, slab):
        m = min(slab, n - lo)
        z = torch.randn(m, device="cuda", generator=gen)
        chi = torch.zeros(m, device="cuda")
        for _ in range(3):
            chi += torch.randn(m, device="cuda", generator=gen) ** 2
        out[lo:lo + m] = z * torch.rsqrt(chi / 3.0) * 1e-3
    return out


def time_region(torch, fn, steps):
    """Wall time and HIP-event time (ms) of `steps` back-to-back calls on the current stream."""
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    e0.record()
    for _ in range(steps):
        fn()
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    return wall_ms, e0.elapsed_time(e1)


def _time_passes(fn, budget_s, max_reps=10000):
    fn()  # warm: page in, spin up threads
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or reps >= max_reps:
            return reps, el


def cpu_baseline(g_slab, r_slab, budget_s):
    """Time the CPU restatement of the reference kernel on a slab of the workload: the C version on
    all host threads (the headline baseline), on one thread, and the numpy version."""
    import numpy as np
    import oracle
    threads = oracle.c.threads()
    n = g_slab.shape[0]
    c = np.empty((n + 15) // 16, dtype=np.uint32)
    r = r_slab.copy()
    reps, el = _time_passes(lambda: oracle.c.fused_quantize_inplace(g_slab, r, c, THRD), budget_s * 0.6)
    oracle.c.set_threads(1)
    reps1, el1 = _time_passes(lambda: oracle.c.fused_quantize_inplace(g_slab, r, c, THRD), budget_s * 0.2)
    oracle.c.set_threads(threads)
    m = min(n, 1 << 22)
    repsn, eln = _time_passes(lambda: oracle.vec.quantize(g_slab[:m], THRD, R_in=r_slab[:m]), budget_s * 0.2)
    return {
        "value": round(BYTES_QUANT * n * reps / el / 1e9, 3),
        "unit": "GB/s",
        "cores": threads,
        "kind": "port",
        "elements_per_s": round(n * reps / el),
        "sample": f"{reps} passes over the first {n} elements of the same gradient "
                  f"({el:.1f} s, C restatement of necklace/cuda/quantize.py, OpenMP {threads} threads)",
        "one_thread_GBps": round(BYTES_QUANT * n * reps1 / el1 / 1e9, 3),
        "numpy_one_thread_GBps": round(BYTES_QUANT * m * repsn / eln / 1e9, 3),
    }


def main():
    args = parse()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this path runs on ONE GPU (no collectives are part of it); "
              "use --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.chunk < 0 or args.chunk % 16:
        print("bench.py: --chunk must be a non-negative multiple of 16", file=sys.stderr)
        sys.exit(2)

    import torch
    from necklace_amd.csrc import build as hip_build
    hip_build.ensure_built()  # compiles only when no library is there; a failed build raises
    from necklace_amd import _lib
    from necklace_amd.cuda import quantize as q  # noqa: F401  (fails loudly if the library is missing)

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(2)
    torch.cuda.set_device(0)
    L = _lib.lib()
    n = args.elems
    gen = torch.Generator(device="cuda")
    gen.manual_seed(4)
    g = student_t3(n, gen, torch)
    r0 = torch.randn(n, device="cuda", generator=gen) * 1e-4
    r = r0.clone()
    c = torch.empty(_lib.packed_words(n), dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    chunk = args.chunk or n
    pieces = [(lo, min(n, lo + chunk)) for lo in range(0, n, chunk)]
    gp, rp, cp = g.data_ptr(), r.data_ptr(), c.data_ptr()

    def step():
        for lo, hi in pieces:
            _lib.check(L.nklq_quantize_f32(gp + 4 * lo, rp + 4 * lo, rp + 4 * lo, cp + 4 * (lo // 16),
                                           hi - lo, 1, THRD, 1, stream))

    for _ in range(args.warmup):
        step()
    wall_ms, ev_ms = time_region(torch, step, args.steps)
    ms_per_step = wall_ms / args.steps
    kernel_ms = ev_ms / args.steps / len(pieces)
    bytes_per_launch = BYTES_QUANT * n / len(pieces)
    value = BYTES_QUANT * n / (ms_per_step * 1e-3) / 1e9
    achieved = bytes_per_launch / (kernel_ms * 1e-3) / 1e9

    # spread of single steps (outside the timed region): one event pair per step
    pairs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(30)]
    for e0, e1 in pairs:
        e0.record()
        step()
        e1.record()
    torch.cuda.synchronize()
    singles = sorted(e0.elapsed_time(e1) for e0, e1 in pairs)

    # HBM bytes per launch from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs of this same command
    # (a separate, committed measurement: counters cannot be read from inside the process)
    traffic = None
    tpath = os.path.join(ROOT, "profiles", "quant_flat_355M_pmc.txt")
    if os.path.exists(tpath) and n == N_ELEMS and len(pieces) == 1:
        import re
        m = re.search(r"^\s*total\s+([0-9,]+) B\s+vs algorithmic", open(tpath).read(), re.M)
        if m:
            traffic = int(m.group(1).replace(",", ""))

    res = {
        "metric": "fused 2-bit quantize GB/s (355M fp32 grad)" if n == N_ELEMS
                  else f"fused 2-bit quantize GB/s ({n}-element fp32 grad)",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {
            "workload": ("GPT-2-medium-sized" if n == N_ELEMS else f"{n}-element")
                        + " flat fp32 gradient, fused quantize + residual update + pack",
            "elements": n,
            "gradient": "1e-3 * Student-t(df=3), generated on the GPU",
            "residual": "N(0, sigma=1e-4) at step 0, carried in place across steps",
            "thrd": THRD,
            "layout": "flat (N,1): word w packs elements 16w..16w+15",
            "launches_per_step": len(pieces),
            "launch_geometry": {"chunks_per_wave": _lib.tune(_lib.TUNE_CHUNKS_PER_WAVE),
                                "workgroup": _lib.tune(_lib.TUNE_WORKGROUP_SIZE),
                                "nontemporal": _lib.tune(_lib.TUNE_NONTEMPORAL),
                                "xcd_interleave_log2": _lib.tune(_lib.TUNE_XCD_INTERLEAVE_LOG2)},
        },
        "pct_hbm_peak": round(100.0 * value / HBM_PEAK_GBPS, 2),
        "roofline": {
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "traffic": traffic,
            "kernel": "quant_flat_kernel",
            "bytes_per_launch": bytes_per_launch,
            "avg_launch_ms": round(kernel_ms, 4),
        },
        "single_step_ms": {"median": round(singles[len(singles) // 2], 4), "min": round(singles[0], 4),
                           "max": round(singles[-1], 4), "samples": len(singles)},
    }

    legs = {x for x in args.legs.split(",") if x}
    if legs & {"deq", "copy"}:
        out = torch.empty(n, dtype=torch.float32, device="cuda")
    if "deq" in legs:

        def deq():
            _lib.check(L.nklq_dequantize_f32(out.data_ptr(), c.data_ptr(), n, 1, THRD, stream))

        for _ in range(5):
            deq()
        _, ev = time_region(torch, deq, max(20, args.steps // 4))
        deq_ms = ev / max(20, args.steps // 4)
        res["dequant"] = {
            "elements_per_s": round(n / (deq_ms * 1e-3)),
            "ms": round(deq_ms, 4),
            "GBps": round(BYTES_DEQUANT * n / (deq_ms * 1e-3) / 1e9, 1),
            "frac_hbm_peak": round(BYTES_DEQUANT * n / (deq_ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        }

    if "acc" in legs:
        # receive side at bucket size: 8 payloads (local + 7 synthetic peers, P(0) = 0.9) into one buffer
        nb = 8_000_000 - 3
        wb = _lib.packed_words(nb)
        import ctypes as ct
        u = torch.rand(K_PAYLOADS, wb * 16, device="cuda", generator=gen)
        codes = (u < 0.05).to(torch.int64) + 2 * ((u >= 0.05) & (u < 0.10)).to(torch.int64)
        shifts = (2 * torch.arange(16, device="cuda", dtype=torch.int64)).view(1, 1, 16)
        words = (codes.view(K_PAYLOADS, wb, 16) << shifts).sum(-1)
        payloads = (words & 0xFFFFFFFF).to(torch.int64)
        payloads = torch.where(payloads >= 2 ** 31, payloads - 2 ** 32, payloads).to(torch.int32).contiguous()
        del u, codes, words
        acc = torch.empty(nb, dtype=torch.float32, device="cuda")
        ptrs = (ct.c_void_p * K_PAYLOADS)(*[payloads[p].data_ptr() for p in range(K_PAYLOADS)])

        def accum():
            _lib.check(L.nklq_dequant_accumulate_f32(acc.data_ptr(), ptrs, K_PAYLOADS, nb, THRD, 0, stream))

        for _ in range(5):
            accum()
        _, ev = time_region(torch, accum, 50)
        acc_ms = ev / 50
        acc_bytes = (0.25 * K_PAYLOADS + 4) * nb
        res["dequant_accumulate"] = {
            "payloads": K_PAYLOADS, "elements": nb,
            "elements_per_s": round(nb / (acc_ms * 1e-3)),
            "ms": round(acc_ms, 4),
            "GBps": round(acc_bytes / (acc_ms * 1e-3) / 1e9, 1),
        }
        del payloads, acc
        # the same sum at gradient size: 8 random payloads (the kernel's time does not depend on the codes)
        if n >= 1 << 24:
            wl = _lib.packed_words(n)
            big = torch.randint(-2 ** 31, 2 ** 31 - 1, (K_PAYLOADS, wl), dtype=torch.int32, device="cuda",
                                generator=gen)
            accl = torch.empty(n, dtype=torch.float32, device="cuda")
            ptrl = (ct.c_void_p * K_PAYLOADS)(*[big[p].data_ptr() for p in range(K_PAYLOADS)])

            def accum_large():
                _lib.check(L.nklq_dequant_accumulate_f32(accl.data_ptr(), ptrl, K_PAYLOADS, n, THRD, 0, stream))

            for _ in range(3):
                accum_large()
            _, ev = time_region(torch, accum_large, 20)
            res["dequant_accumulate_large"] = {
                "payloads": K_PAYLOADS, "elements": n,
                "elements_per_s": round(n / (ev / 20 * 1e-3)),
                "ms": round(ev / 20, 4),
                "GBps": round((0.25 * K_PAYLOADS + 4) * n / (ev / 20 * 1e-3) / 1e9, 1),
            }
            del big, accl

    if "matrix" in legs:
        # the reference's own layout: (n, k) matrix, codes packed down the columns
        side = 8192
        A = g[:side * side].view(side, side)
        R = torch.zeros(side, side, device="cuda")
        C = torch.empty(side // 16, side, dtype=torch.int32, device="cuda")

        def mq():
            _lib.check(L.nklq_quantize_f32(A.data_ptr(), R.data_ptr(), R.data_ptr(), C.data_ptr(),
                                           side, side, THRD, 1, stream))

        def md():
            _lib.check(L.nklq_dequantize_f32(R.data_ptr(), C.data_ptr(), side, side, THRD, stream))

        for _ in range(5):
            mq()
        _, ev = time_region(torch, mq, 50)
        res["matrix_8192x8192"] = {"fused_GBps": round(BYTES_QUANT * side * side / (ev / 50 * 1e-3) / 1e9, 1)}
        for _ in range(5):
            md()
        _, ev = time_region(torch, md, 50)
        res["matrix_8192x8192"]["decode_GBps"] = round(BYTES_DEQUANT * side * side / (ev / 50 * 1e-3) / 1e9, 1)
        del A, R, C

    if "multi" in legs:
        # a ResNet-50-shaped list of gradient tensors through the trainer-side buffers
        from necklace_amd.frmwrk.pytorch import ptcomp
        sizes = [64 * 3 * 7 * 7, 64, 64]
        inpl = 64
        for planes, blocks in ((64, 3), (128, 4), (256, 6), (512, 3)):
            for b in range(blocks):
                sizes += [planes * inpl, planes, planes, planes * planes * 9, planes, planes,
                          4 * planes * planes, 4 * planes, 4 * planes]
                if b == 0:
                    sizes += [4 * planes * inpl, 4 * planes, 4 * planes]
                inpl = 4 * planes
        sizes += [1000 * 2048, 1000]
        gcomp = ptcomp.GradCompressor(sizes, K_PAYLOADS, thrd=THRD)
        gl, pos = [], 0
        for sz in sizes:
            gl.append(g[pos:pos + sz])
            pos += sz
        gcomp.recv.random_(-2 ** 31, 2 ** 31 - 1)
        outs = [torch.empty(sz, device="cuda") for sz in sizes]
        nel = sum(sz for sz in sizes if sz >= 1001)
        for _ in range(5):
            gcomp.compress(gl)
            gcomp.decompress_sum(outs)
        _, ev = time_region(torch, lambda: gcomp.compress(gl), 50)
        _, ev2 = time_region(torch, lambda: gcomp.decompress_sum(outs), 50)
        res["resnet50_tensor_list"] = {
            "tensors": len(sizes), "compressed_elements": nel,
            "compress_us": round(ev / 50 * 1e3, 1), "decompress_sum_us": round(ev2 / 50 * 1e3, 1),
        }

    if "copy" in legs:
        def cp():
            _lib.check(L.nklq_copy_f32(out.data_ptr(), g.data_ptr(), n, stream))

        for _ in range(5):
            cp()
        _, ev = time_region(torch, cp, 20)
        res["copy_GBps"] = round(8.0 * n / (ev / 20 * 1e-3) / 1e9, 1)

    if "cpu" in legs and args.cpu_seconds > 0:
        slab = min(n, 1 << 25)
        res["cpu_baseline"] = cpu_baseline(g[:slab].cpu().numpy(), r0[:slab].cpu().numpy(),
                                           args.cpu_seconds)
    print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
