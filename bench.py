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
  extras       decode (elements/s), 8-payload fixed-order sum, plain copy, the other four
               synthetic workloads (config1, config2, config3, config5: kernel time, GB/s of
               algorithmic bytes, fraction of the HBM peak), wall time per call of the
               reference-named wrapper at small sizes, the matrix form on eight shapes (wide,
               rows off cache lines, a few columns), a ResNet-50-shaped list of 161 gradient
               tensors through the trainer-side buffers

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
    ap.add_argument("--legs", default="deq,coldcodes,acc,configs,wrapper,matrix,multi,copy,cpu",
                    help="extra legs after the timed quantize steps: deq, coldcodes, acc, configs, wrapper, matrix, "
                         "multi, copy, cpu, and (off by default) accsweep, geometry (comma list, '' = none)")
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


def warm_for(torch, fn, seconds):
    """Keeps the GPU under the load of `fn` for about `seconds` before a timed region.  After a leg of
    many tiny launches the first few milliseconds of streaming work have measured up to 30 % slower
    (the clocks of an idle-looking GPU come back with a delay), whichever kernel runs."""
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        for _ in range(10):
            fn()
        torch.cuda.synchronize()


def _time_passes(fn, budget_s, max_reps=10000):
    fn()  # warm: page in, spin up threads
    reps, t0 = 0, time.perf_counter()
    while True:
        fn()
        reps += 1
        el = time.perf_counter() - t0
        if el >= budget_s or reps >= max_reps:
            return reps, el


def cpu_baseline(g_slab, r_slab, budget_s, thrd=THRD):
    """Time the CPU restatement of the reference kernel on a slab of the workload: the C version on
    all host threads (the headline baseline), on one thread, and the numpy version."""
    import numpy as np
    import oracle
    threads = oracle.c.threads()
    n = g_slab.shape[0]
    c = np.empty((n + 15) // 16, dtype=np.uint32)
    r = r_slab.copy()
    reps, el = _time_passes(lambda: oracle.c.fused_quantize_inplace(g_slab, r, c, thrd), budget_s * 0.6)
    oracle.c.set_threads(1)
    reps1, el1 = _time_passes(lambda: oracle.c.fused_quantize_inplace(g_slab, r, c, thrd), budget_s * 0.2)
    oracle.c.set_threads(threads)
    m = min(n, 1 << 22)
    repsn, eln = _time_passes(lambda: oracle.vec.quantize(g_slab[:m], thrd, R_in=r_slab[:m]), budget_s * 0.2)
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
        # the reference's own CPU route would be numba's CUDA simulator; it is used only if it is there
        "numba_installed": __import__("importlib.util").util.find_spec("numba") is not None,
    }


def cpu_baseline_small(g, r0, thrd, budget_s, what):
    """The same C restatement, all host threads, on another workload's own data."""
    import numpy as np
    import oracle
    n = g.shape[0]
    c = np.empty((n + 15) // 16, dtype=np.uint32)
    r = r0.copy()
    reps, el = _time_passes(lambda: oracle.c.fused_quantize_inplace(g, r, c, thrd), budget_s)
    return {"value": round(BYTES_QUANT * n * reps / el / 1e9, 3), "unit": "GB/s", "cores": oracle.c.threads(),
            "kind": "port", "elements_per_s": round(n * reps / el),
            "sample": f"{reps} fused passes over {what} ({el:.1f} s)"}


def source_stamp():
    """First 16 hex digits of the SHA-256 of the kernel source: ties a counter summary under
    profiles/ to the code it measured."""
    import hashlib
    with open(os.path.join(ROOT, "necklace_amd", "csrc", "nklq.hip"), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def hbm_traffic_from_profile(name):
    """(bytes per launch, stale) from the committed rocprofv3 FETCH_SIZE / WRITE_SIZE summary: the
    figure is only quoted when the summary was taken from the kernel source as it is now."""
    import re
    tpath = os.path.join(ROOT, "profiles", name)
    if not os.path.exists(tpath):
        return None, False
    text = open(tpath).read()
    m = re.search(r"^\s*total\s+([0-9,]+) B\s+vs algorithmic", text, re.M)
    st = re.search(r"kernel source sha256\[:16\]:\s*([0-9a-f]{16})", text)
    if not m:
        return None, False
    if not st or st.group(1) != source_stamp():
        return None, True
    return int(m.group(1).replace(",", "")), False


def sparse_payloads(torch, k, words, gen, p_zero=0.9):
    """[k, words] packed payloads (int32 bits) of i.i.d. codes: P(0) = p_zero, P(01) = P(10), never 11."""
    half = (1.0 - p_zero) / 2
    out = torch.empty(k, words, dtype=torch.int32, device="cuda")
    shifts = (2 * torch.arange(16, device="cuda", dtype=torch.int64)).view(1, 16)
    for p in range(k):
        u = torch.rand(words, 16, device="cuda", generator=gen)
        codes = (u < half).to(torch.int64) + 2 * ((u >= half) & (u < 2 * half)).to(torch.int64)
        w = (codes << shifts).sum(-1)
        out[p] = torch.where(w >= 2 ** 31, w - 2 ** 32, w).to(torch.int32)
    return out


def frac(gbps):
    return round(gbps / HBM_PEAK_GBPS, 4)


def bench_configs(torch, L, _lib, stream, gen, res, cpu_seconds):
    """The four synthetic workloads that are not the headline one (BASELINE.json configs 1, 2, 3, 5)."""
    import ctypes as ct
    import numpy as np
    check = _lib.check

    # ---- config 1: 1,048,576 elements, N(0, 0.01), zero residual, thrd 0.005; flat and as 1024 x 1024
    n1, t1 = 1 << 20, 0.005
    g1 = torch.randn(n1, device="cuda", generator=gen) * 0.01
    r1 = torch.zeros(n1, device="cuda")
    c1 = torch.empty(n1 // 16, dtype=torch.int32, device="cuda")
    f_flat = lambda: check(L.nklq_quantize_f32(g1.data_ptr(), r1.data_ptr(), r1.data_ptr(), c1.data_ptr(), n1, 1, t1, 1, stream))
    f_sq = lambda: check(L.nklq_quantize_f32(g1.data_ptr(), r1.data_ptr(), r1.data_ptr(), c1.data_ptr(), 1024, 1024, t1, 1, stream))
    out = {}
    for name, f in (("flat", f_flat), ("square_1024x1024", f_sq)):
        for _ in range(20):
            f()
        _, ev = time_region(torch, f, 500)
        us = ev / 500 * 1e3
        out[name] = {"us": round(us, 2), "GBps": round(BYTES_QUANT * n1 / us / 1e3, 1),
                     "frac_hbm_peak": frac(BYTES_QUANT * n1 / us / 1e3), "elements_per_s": round(n1 / us * 1e6)}
    out["note"] = "12.8 MB per launch: launch latency, not HBM, bounds it"
    if cpu_seconds > 0:
        out["cpu_baseline"] = cpu_baseline_small(g1.cpu().numpy(), np.zeros(n1, np.float32), t1, cpu_seconds * 0.1,
                                                 "config 1's 1,048,576 elements")
    res["config1"] = out

    # ---- config 2: 25,557,032 elements = 161 segments, per-segment sigma log-uniform [1e-4, 1e-2], thrd 1e-3,
    # 10 error-feedback steps with a fresh gradient each, packed as ONE flat vector (last word: 8 codes)
    sizes = resnet50_sizes()
    n2, t2, steps2 = sum(sizes), 1e-3, 10
    sig = 10.0 ** (torch.rand(len(sizes), device="cuda", generator=gen) * 2 - 4)
    scale = torch.repeat_interleave(sig, torch.tensor(sizes, device="cuda"))
    grads = [torch.randn(n2, device="cuda", generator=gen) * scale for _ in range(steps2)]
    r2 = torch.zeros(n2, device="cuda")
    c2 = torch.empty(_lib.packed_words(n2), dtype=torch.int32, device="cuda")
    state = {"i": 0}

    def step2():
        g = grads[state["i"] % steps2]
        state["i"] += 1
        check(L.nklq_quantize_f32(g.data_ptr(), r2.data_ptr(), r2.data_ptr(), c2.data_ptr(), n2, 1, t2, 1, stream))

    for _ in range(steps2):
        step2()
    r2.zero_()
    state["i"] = 0
    _, ev = time_region(torch, step2, steps2)
    us = ev / steps2 * 1e3
    res["config2"] = {"elements": n2, "segments": len(sizes), "steps": steps2, "us_per_step": round(us, 2),
                      "GBps": round(BYTES_QUANT * n2 / us / 1e3, 1), "frac_hbm_peak": frac(BYTES_QUANT * n2 / us / 1e3),
                      "elements_per_s": round(n2 / us * 1e6),
                      "note": "one launch per step over the flat vector; 10 different gradients (1 GB) so "
                              "that no step finds its input in the 256 MB memory-side cache"}
    if cpu_seconds > 0:
        res["config2"]["cpu_baseline"] = cpu_baseline_small(grads[0].cpu().numpy(), np.zeros(n2, np.float32), t2,
                                                            cpu_seconds * 0.2, "config 2's 25,557,032 elements")
    del grads, scale, r2, c2

    # ---- config 3: 64 buckets of 1M..8M elements (not multiples of 16), 8 payloads each (local + 7 peers,
    # P(0) = 0.9), fixed-order sum into a fresh fp32 buffer
    rng = np.random.default_rng(3)
    lens = []
    while len(lens) < 64:
        v = int(rng.integers(1_000_000, 8_000_001))
        if v % 16:
            lens.append(v)
    words = [_lib.packed_words(v) for v in lens]
    woff = np.concatenate([[0], np.cumsum([-(-w // 16) * 16 for w in words])]).astype(np.int64)  # 64 B aligned
    total_words, total = int(woff[-1]), sum(lens)
    msgs = sparse_payloads(torch, K_PAYLOADS, total_words, gen)      # one contiguous message per worker
    accs = [torch.empty(v, device="cuda") for v in lens]
    ptr_tabs = [(ct.c_void_p * K_PAYLOADS)(*[msgs[p].data_ptr() + 4 * int(woff[b]) for p in range(K_PAYLOADS)])
                for b in range(64)]

    def per_bucket():
        for b in range(64):
            check(L.nklq_dequant_accumulate_f32(accs[b].data_ptr(), ptr_tabs[b], K_PAYLOADS, lens[b], 1e-3, 0, stream))

    acc_arr = (ct.c_void_p * 64)(*[a.data_ptr() for a in accs])
    n_arr = (ct.c_uint64 * 64)(*lens)
    wo_arr = (ct.c_uint64 * 64)(*[int(w) for w in woff[:64]])
    base_arr = (ct.c_void_p * K_PAYLOADS)(*[msgs[p].data_ptr() for p in range(K_PAYLOADS)])

    def one_launch():
        check(L.nklq_dequant_accumulate_multi_f32(64, acc_arr, n_arr, wo_arr, base_arr, K_PAYLOADS, 1e-3, 0, 1.0, stream))

    c3 = {"buckets": 64, "payloads": K_PAYLOADS, "elements": total}
    byt = (0.25 * K_PAYLOADS + 4) * total
    for name, f in (("one_launch_per_bucket", per_bucket), ("all_buckets_one_launch", one_launch)):
        for _ in range(3):
            f()
        _, ev = time_region(torch, f, 10)
        ms = ev / 10
        c3[name] = {"ms": round(ms, 4), "elements_per_s": round(total / ms * 1e3), "GBps": round(byt / ms / 1e6, 1),
                    "frac_hbm_peak": frac(byt / ms / 1e6)}
    res["config3"] = c3
    del msgs, accs

    # ---- config 5: 2.8e9 elements (11.2 GB + 11.2 GB + 0.7 GB resident), N(0, 5e-3), thrd 1e-2, 5 steps in
    # chunks of 268,435,456 elements
    n5, t5, chunk5, steps5 = 2_800_000_000, 1e-2, 268_435_456, 5
    free, _ = torch.cuda.mem_get_info()
    if free > 2 * 4 * n5 + n5 // 4 + (4 << 30):
        g5 = torch.empty(n5, device="cuda")
        for lo in range(0, n5, 1 << 28):
            hi = min(n5, lo + (1 << 28))
            torch.randn(hi - lo, device="cuda", generator=gen, out=g5[lo:hi])
            g5[lo:hi] *= 5e-3
        r5 = torch.zeros(n5, device="cuda")
        c5 = torch.empty(_lib.packed_words(n5), dtype=torch.int32, device="cuda")
        pieces = [(lo, min(n5, lo + chunk5)) for lo in range(0, n5, chunk5)]
        gp, rp, cp = g5.data_ptr(), r5.data_ptr(), c5.data_ptr()

        def step5():
            for lo, hi in pieces:
                check(L.nklq_quantize_f32(gp + 4 * lo, rp + 4 * lo, rp + 4 * lo, cp + 4 * (lo // 16), hi - lo, 1, t5, 1, stream))

        step5()
        r5.zero_()
        _, ev = time_region(torch, step5, steps5)
        ms = ev / steps5
        slab5 = g5[:1 << 26].cpu().numpy() if cpu_seconds > 0 else None
        res["config5"] = {"elements": n5, "chunk": chunk5, "launches_per_step": len(pieces), "steps": steps5,
                          "ms_per_step": round(ms, 4), "GBps": round(BYTES_QUANT * n5 / ms / 1e6, 1),
                          "frac_hbm_peak": frac(BYTES_QUANT * n5 / ms / 1e6), "elements_per_s": round(n5 / ms * 1e3),
                          "resident_GB": round((2 * 4 * n5 + 4 * _lib.packed_words(n5)) / 1e9, 2)}
        del g5, r5, c5
        if slab5 is not None:
            res["config5"]["cpu_baseline"] = cpu_baseline_small(slab5, np.zeros(1 << 26, np.float32), t5, cpu_seconds * 0.2,
                                                                "a 67,108,864-element slice of config 5")
    else:
        res["config5"] = {"skipped": f"only {free / 1e9:.0f} GB of HBM free"}


def bench_wrapper(torch, L, _lib, stream, res):
    """Wall time per call of the reference-named wrapper (necklace/cuda/quantize.py:96-115 creates a
    stream and blocks on it every call) at sizes where the kernel takes a few microseconds."""
    from necklace_amd.cuda import quantize as q
    out = {}
    for name, shape in (("1048576", (1 << 20,)), ("224x224", (224, 224))):
        A = torch.randn(*shape, device="cuda") * 0.01
        R = torch.zeros_like(A)
        m = (shape[0] + 15) // 16
        C = torch.empty((m,) + tuple(shape[1:]), dtype=torch.int32, device="cuda")
        n, k = (shape[0], 1) if len(shape) == 1 else shape
        raw = lambda: _lib.check(L.nklq_quantize_f32(A.data_ptr(), R.data_ptr(), R.data_ptr(), C.data_ptr(), n, k, 0.005, 1, stream))
        for _ in range(50):
            raw()
        _, ev = time_region(torch, raw, 1000)
        row = {"kernel_us": round(ev, 2)}          # ev is ms for 1000 launches = us per launch
        for label, kw in (("sync_true", {}), ("sync_false", {"sync": False})):
            f = lambda: q.cu_fn_matrix_quantize_e(A, C, R, 0.005, add_residual=True, **kw)
            for _ in range(50):
                f()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(1000):
                f()
            torch.cuda.synchronize()
            row[f"wall_us_per_call_{label}"] = round((time.perf_counter() - t0) * 1e3, 2)
        t0 = time.perf_counter()
        for _ in range(1000):
            raw()
        torch.cuda.synchronize()
        row["wall_us_per_call_c_abi_async"] = round((time.perf_counter() - t0) * 1e3, 2)
        out[name] = row
    res["wrapper_call_overhead"] = out


def resnet50_sizes():
    """Element counts of ResNet-50's 161 parameter tensors, in module order (25,557,032 in all)."""
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
    return sizes


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

    def tuning():
        """The measurement build of the same source (copy kernel, every launch geometry, interleaved sum)."""
        hip_build.ensure_built(tuning=True)
        return _lib.tuning_lib()

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
    # (a separate, committed measurement: counters cannot be read from inside the process).  The
    # summary carries the hash of the kernel source it was taken from; after any change to the
    # source the figure is withheld until the counters have been collected again.
    traffic, traffic_stale = None, False
    if n == N_ELEMS and len(pieces) == 1:
        traffic, traffic_stale = hbm_traffic_from_profile("quant_flat_355M_pmc.txt")

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
            "traffic_stale": traffic_stale,
            "kernel": "quant_flat_kernel",
            "kernel_source_sha256_16": source_stamp(),
            "bytes_per_launch": bytes_per_launch,
            "avg_launch_ms": round(kernel_ms, 4),
        },
        "single_step_ms": {"median": round(singles[len(singles) // 2], 4), "min": round(singles[0], 4),
                           "max": round(singles[-1], 4), "samples": len(singles)},
    }

    legs = {x for x in args.legs.split(",") if x}
    if legs & {"deq", "coldcodes", "copy", "geometry"}:
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

    if "coldcodes" in legs:
        # The decode loop above finds its 89 MB of code words in the 256 MB memory-side cache (they were read by
        # the launch before; after an exchange they would have just been written).  Here 0.25 GB of other memory
        # is read between the launches, so the words come from HBM: each launch timed on its own, median of 12,
        # without and with the decode's prefetch workgroups (nklq_tune knob NKLQ_TUNE_DECODE_PREFETCH; left to
        # itself the library switches them on from 2^30 elements, where the words cannot all be in that cache)
        other = torch.ones(62_500_000, device="cuda")

        def one_cold_decode():
            other.sum()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            _lib.check(L.nklq_dequantize_f32(out.data_ptr(), c.data_ptr(), n, 1, THRD, stream))
            e1.record()
            torch.cuda.synchronize()
            return e0.elapsed_time(e1)

        res["dequant_code_words_from_hbm"] = {}
        before = _lib.tune(_lib.TUNE_DECODE_PREFETCH)
        for label, knob in (("without_prefetch", 2), ("with_prefetch", 1)):
            _lib.tune(_lib.TUNE_DECODE_PREFETCH, knob)
            ts = sorted([one_cold_decode() for _ in range(15)][3:])   # the first three are warm-up
            ms = ts[len(ts) // 2]
            res["dequant_code_words_from_hbm"][label] = {
                "ms": round(ms, 4), "frac_hbm_peak": frac(BYTES_DEQUANT * n / (ms * 1e-3) / 1e9)}
        _lib.tune(_lib.TUNE_DECODE_PREFETCH, before)
        del other

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
            "frac_hbm_peak": frac(acc_bytes / (acc_ms * 1e-3) / 1e9),
            "note": "50 MB working set: served by the 256 MB memory-side cache when repeated",
        }
        del payloads, acc
        # the size necklace reduces at a time: one 256 MB bucket (nccl_reduce_bucket_size,
        # necklace/frmwrk/pytorch/ptprms.py:253) = 67,108,864 elements, 8 payloads of 16 MB that another
        # kernel has just written (as an all-gather would have) before every sum; only the sums are timed
        nk = 1 << 26
        wk = _lib.packed_words(nk)
        arrived = torch.randint(-2 ** 31, 2 ** 31 - 1, (K_PAYLOADS, wk), dtype=torch.int32, device="cuda", generator=gen)
        inbox = torch.empty_like(arrived)
        acck = torch.empty(nk, dtype=torch.float32, device="cuda")
        ptrk = (ct.c_void_p * K_PAYLOADS)(*[inbox[p].data_ptr() for p in range(K_PAYLOADS)])
        pairs_k = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(30)]
        for i in range(40):
            inbox.copy_(arrived)
            if i >= 10:
                pairs_k[i - 10][0].record()
            _lib.check(L.nklq_dequant_accumulate_f32(acck.data_ptr(), ptrk, K_PAYLOADS, nk, THRD, 0, stream))
            if i >= 10:
                pairs_k[i - 10][1].record()
        torch.cuda.synchronize()
        tk_ms = sorted(a.elapsed_time(b) for a, b in pairs_k)[len(pairs_k) // 2]
        gbk = (0.25 * K_PAYLOADS + 4) * nk / (tk_ms * 1e-3) / 1e9
        res["dequant_accumulate_256MB_bucket"] = {
            "payloads": K_PAYLOADS, "elements": nk, "elements_per_s": round(nk / (tk_ms * 1e-3)),
            "ms": round(tk_ms, 4), "GBps": round(gbk, 1), "frac_hbm_peak": frac(gbk),
            "note": "median of 30 sums, each right after its 128 MB of payloads were written",
        }
        del arrived, inbox, acck
        # the same sum at gradient size: 8 random payloads (the kernel's time does not depend on the codes)
        if n >= 1 << 24:
            wl = _lib.packed_words(n)
            big = torch.randint(-2 ** 31, 2 ** 31 - 1, (K_PAYLOADS, wl), dtype=torch.int32, device="cuda",
                                generator=gen)
            accl = torch.empty(n, dtype=torch.float32, device="cuda")
            ptrl = (ct.c_void_p * K_PAYLOADS)(*[big[p].data_ptr() for p in range(K_PAYLOADS)])

            def accum_large():
                _lib.check(L.nklq_dequant_accumulate_f32(accl.data_ptr(), ptrl, K_PAYLOADS, n, THRD, 0, stream))

            for _ in range(25):  # the first few dozen launches on fresh buffers run 2-5 % slower
                accum_large()
            _, ev = time_region(torch, accum_large, 20)
            res["dequant_accumulate_large"] = {
                "payloads": K_PAYLOADS, "elements": n,
                "elements_per_s": round(n / (ev / 20 * 1e-3)),
                "ms": round(ev / 20, 4),
                "GBps": round((0.25 * K_PAYLOADS + 4) * n / (ev / 20 * 1e-3) / 1e9, 1),
                "frac_hbm_peak": frac((0.25 * K_PAYLOADS + 4) * n / (ev / 20 * 1e-3) / 1e9),
            }
            del big, accl

    if "configs" in legs and n == N_ELEMS:
        bench_configs(torch, L, _lib, stream, gen, res, args.cpu_seconds if "cpu" in legs else 0.0)

    if "wrapper" in legs:
        bench_wrapper(torch, L, _lib, stream, res)

    if "accsweep" in legs:
        # the fixed-order sum against the number of payloads, at gradient size: where the payloads stop
        # fitting the 256 MB memory-side cache (K >= 4 here) the time per payload jumps
        import ctypes as ct
        wl = _lib.packed_words(n)
        big = torch.randint(-2 ** 31, 2 ** 31 - 1, (16, wl), dtype=torch.int32, device="cuda", generator=gen)
        accl = torch.empty(n, dtype=torch.float32, device="cuda")
        ptrl = (ct.c_void_p * 16)(*[big[p].data_ptr() for p in range(16)])
        res["dequant_accumulate_by_payloads"] = {}
        for kp in (1, 2, 3, 4, 6, 8, 12, 16):
            f = lambda: _lib.check(L.nklq_dequant_accumulate_f32(accl.data_ptr(), ptrl, kp, n, THRD, 0, stream))
            for _ in range(10):
                f()
            _, ev = time_region(torch, f, 20)
            gb = (0.25 * kp + 4) * n / (ev / 20 * 1e-3) / 1e9
            res["dequant_accumulate_by_payloads"][str(kp)] = {
                "us": round(ev / 20 * 1e3, 1), "GBps": round(gb, 1), "frac_hbm_peak": frac(gb),
                "payload_MB": round(4 * wl * kp / 1e6)}
        del big
        # The same 8 payloads' worth of words, the same bytes read and written, but the payloads
        # alternate inside ONE array in runs of 2^s words: from 256 B runs (the 8 reads of a tile are one
        # contiguous 2 KiB) to runs longer than a payload (8 streams far apart, the layout above).  If
        # the number of distinct read streams were what slows the sum, short runs would be faster.
        T = tuning()
        nt = n - n % 1024
        res["dequant_accumulate_by_interleave"] = {"payloads": K_PAYLOADS, "elements": nt}
        top = max(6, (nt // 16 - 1).bit_length())
        for s_log2 in (6, 8, 10, 12, 16, 20, top):
            run = 1 << s_log2
            runs = (nt // 16 + run - 1) // run
            words = torch.randint(-2 ** 31, 2 ** 31 - 1, (runs * K_PAYLOADS * run,), dtype=torch.int32,
                                  device="cuda", generator=gen)
            f = lambda: _lib.check(T.nklq_tuning_sum_interleaved_f32(accl.data_ptr(), words.data_ptr(), K_PAYLOADS,
                                                                     nt, s_log2, THRD, stream))
            for _ in range(10):
                f()
            _, ev = time_region(torch, f, 20)
            gb = (0.25 * K_PAYLOADS + 4) * nt / (ev / 20 * 1e-3) / 1e9
            res["dequant_accumulate_by_interleave"][f"run_{4 * run}_bytes"] = {
                "us": round(ev / 20 * 1e3, 1), "GBps": round(gb, 1), "frac_hbm_peak": frac(gb)}
            del words
        del accl

    if "geometry" in legs:
        # the launch knobs of nklq_tune on the three flat kernels at gradient size: the shipped defaults
        # against their neighbours (results never depend on them, only the time does)
        import ctypes as ct
        Lg = tuning()     # the geometries other than the default exist in the measurement build only
        tune = lambda i, v=-1: Lg.nklq_tune(i, v)
        default = [tune(i) for i in range(_lib.N_TUNE)]
        wl = _lib.packed_words(n)
        pay = torch.randint(-2 ** 31, 2 ** 31 - 1, (K_PAYLOADS, wl), dtype=torch.int32, device="cuda", generator=gen)
        ptrg = (ct.c_void_p * K_PAYLOADS)(*[pay[p].data_ptr() for p in range(K_PAYLOADS)])
        kernels = {
            "quantize": (lambda: _lib.check(Lg.nklq_quantize_f32(gp, rp, rp, cp, n, 1, THRD, 1, stream)), BYTES_QUANT),
            "decode": (lambda: _lib.check(Lg.nklq_dequantize_f32(out.data_ptr(), cp, n, 1, THRD, stream)), BYTES_DEQUANT),
            "sum8": (lambda: _lib.check(Lg.nklq_dequant_accumulate_f32(out.data_ptr(), ptrg, K_PAYLOADS, n, THRD, 0, stream)),
                     0.25 * K_PAYLOADS + 4),
        }
        sweeps = {   # kernel -> [(label, {knob: value})]
            "quantize": [(f"interleave 2^{x}", {_lib.TUNE_XCD_INTERLEAVE_LOG2: x}) for x in range(7)]
                        + [(f"{u} chunks per wave", {_lib.TUNE_CHUNKS_PER_WAVE: u}) for u in (2, 4)]
                        + [(f"workgroup {b}", {_lib.TUNE_WORKGROUP_SIZE: b}) for b in (64, 128, 512, 1024)]
                        + [("cached loads and stores", {_lib.TUNE_NONTEMPORAL: 0})],
            "decode": [(f"interleave 2^{x}", {_lib.TUNE_XCD_INTERLEAVE_LOG2_DECODE: x}) for x in range(7)]
                      + [("cached stores", {_lib.TUNE_NONTEMPORAL: 0})],
            "sum8": [(f"interleave 2^{x}", {_lib.TUNE_XCD_INTERLEAVE_LOG2_ACCUMULATE: x}) for x in range(7)],
        }
        res["launch_geometry"] = {"defaults": default}
        for name, (fn, bpe) in kernels.items():
            rows_ = {}
            for label, knobs in [("defaults", {})] + sweeps[name]:
                for i, v in enumerate(default):
                    assert tune(i, v) >= 0
                for kk, v in knobs.items():
                    assert tune(kk, v) >= 0
                for _ in range(5):
                    fn()
                _, ev = time_region(torch, fn, 10)
                gb = bpe * n / (ev / 10 * 1e-3) / 1e9
                rows_[label] = {"us": round(ev / 10 * 1e3, 1), "frac_hbm_peak": frac(gb)}
            res["launch_geometry"][name] = rows_
        for i, v in enumerate(default):
            tune(i, v)
        del pay

    if "matrix" in legs:
        # the reference's own layout: (n, k) matrix, codes packed down the columns; wide and narrow,
        # rows on and off 128-byte lines
        res["matrix"] = {}
        # this leg follows legs of many tiny launches: without 50 ms of streaming load first, the decode of
        # the first shape has measured 0.67-0.75 of the HBM peak here and 0.92-0.96 in any other place, with
        # either of the two kernels that can run it
        warm_for(torch, lambda: _lib.check(L.nklq_quantize_f32(gp, rp, rp, cp, n, 1, THRD, 1, stream)), 0.05)
        # (the last three: fewer than 8 bands of 16 rows, rows off 128-byte lines)
        for rows, cols in ((8192, 8192), (8191, 8191), (16384, 16383), (100000, 1000), (150_000, 401),
                           (20_000_000, 3), (4_000_000, 17), (1_000_000, 65),
                           (16, 4_000_001), (100, 1_000_003), (144, 500_001)):
            tot = rows * cols
            A = g[:tot] if tot <= n else torch.randn(tot, device="cuda", generator=gen) * 1e-3
            R = torch.zeros(tot, device="cuda")
            C = torch.empty(_lib.packed_words(rows, cols), dtype=torch.int32, device="cuda")

            def mq():
                _lib.check(L.nklq_quantize_f32(A.data_ptr(), R.data_ptr(), R.data_ptr(), C.data_ptr(),
                                               rows, cols, THRD, 1, stream))

            def md():
                _lib.check(L.nklq_dequantize_f32(R.data_ptr(), C.data_ptr(), rows, cols, THRD, stream))

            for _ in range(5):
                mq()
            _, ev = time_region(torch, mq, 30)
            fq = BYTES_QUANT * tot / (ev / 30 * 1e-3) / 1e9
            for _ in range(5):
                md()
            _, ev2 = time_region(torch, md, 30)
            fd = BYTES_DEQUANT * tot / (ev2 / 30 * 1e-3) / 1e9
            res["matrix"][f"{rows}x{cols}"] = {"fused_us": round(ev / 30 * 1e3, 1), "fused_GBps": round(fq, 1),
                                               "fused_frac_hbm_peak": frac(fq), "decode_us": round(ev2 / 30 * 1e3, 1),
                                               "decode_GBps": round(fd, 1), "decode_frac_hbm_peak": frac(fd)}
            if cols > 384 and cols % 32:
                # rows off 128-byte lines: with the new residual in a buffer of its own (no in-place partner)
                # the tiles move each row's window onto lines; in place they cannot (a neighbour would
                # read elements another workgroup has already replaced)
                R2 = torch.empty(tot, device="cuda")

                def mq2():
                    _lib.check(L.nklq_quantize_f32(A.data_ptr(), R.data_ptr(), R2.data_ptr(), C.data_ptr(),
                                                   rows, cols, THRD, 1, stream))

                for _ in range(5):
                    mq2()
                _, ev3 = time_region(torch, mq2, 30)
                fo = BYTES_QUANT * tot / (ev3 / 30 * 1e-3) / 1e9
                res["matrix"][f"{rows}x{cols}"].update({"fused_out_of_place_us": round(ev3 / 30 * 1e3, 1),
                                                        "fused_out_of_place_frac_hbm_peak": frac(fo)})
                del R2
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
        gcomp = ptcomp.GradCompressor(sizes, K_PAYLOADS, thrd=THRD, rank=0)
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
        # host side of a steady-state call (gradients keep their storage): wall time until the call
        # returns, launches left in flight (200 calls stay far below the depth of the launch queue)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(200):
            gcomp.compress(gl)
        host_us = (time.perf_counter() - t0) / 200 * 1e6
        torch.cuda.synchronize()
        res["resnet50_tensor_list"] = {
            "tensors": len(sizes), "compressed_elements": nel,
            "compress_us": round(ev / 50 * 1e3, 1), "decompress_sum_us": round(ev2 / 50 * 1e3, 1),
            "host_us_per_call": round(host_us, 1),
        }

    if "copy" in legs:
        T = tuning()   # the copy kernel is a measurement aid: it is not in the product library

        def cp():
            _lib.check(T.nklq_copy_f32(out.data_ptr(), g.data_ptr(), n, stream))

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
