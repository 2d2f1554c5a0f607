#!/usr/bin/env python3
"""Benchmark of the quantized Gram build (the hot path of hyacinTsvdFit) on one MI355X.

A step = hyacinXquantizeScaleBatch + hyacinXherkBatch on a synthetic matrix that is already resident in
HBM: per-column exponents, int8 CRT-residue / limb quantization, the int8 MFMA contraction and the
reconstruction of the exact integer Gram.  Prints ONE JSON line:
  value      effective Gram TFLOP/s = M N (N+1) (x4 complex) / step time  (the FP SYRK/HERK flops replaced)
  roofline   the contraction kernel alone, timed with HIP events on its stream: algorithmic int8 ops / time
             against the dense INT8 MFMA peak
  cpu_baseline  the same limb / CRT algorithm compiled for the host (the oracle), timed on a row sample, with
             OpenBLAS DSYRK / ZHERK on the same sample and LAPACK syevd / heevd on its N x N Gram beside it
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

INT8_PEAK_TOPS = 5000.0   # MI355X dense INT8 MFMA peak, 5.0 POP/s
HBM_PEAK_GBS = 8000.0     # MI355X HBM3E peak, 8 TB/s

# HBM bytes per launch of the contraction kernel, from rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script
# (profiles/gram_ring_kernel_target_hbm_traffic.md), each scaled by what the counter reads for copy_kernel's known 1 GiB.
MEASURED_TRAFFIC = {("target", 0): 5.65e9 + 0.12e9}

WORKLOADS = {
    # name: (type, opA, M, N, K, eps, algorithm, description)
    "target": (0, "N", 131072, 2048, 1024, 1e-12, b"A", "real FP64 M=131072 N=2048 eps=1e-12 (CRT real, 14 moduli)"),
    "cfg1": (0, "N", 4096, 256, 256, 1e-10, b"L", "real FP64 M=4096 N=256 eps=1e-10 (limbs, 6 digits)"),
    "cfg2": (2, "T", 65536, 1024, 512, 1e-5, b"A", "real FP32 opA=T M=65536 N=1024 eps=1e-5 (CRT real, 8 moduli)"),
    "cfg3": (1, "N", 131072, 2048, 1024, 1e-12, b"A", "complex FP64 M=131072 N=2048 eps=1e-12 (CRT complex, 15 moduli)"),
    "cfg4": (5, "C", 262144, 4096, 256, 1e-3, b"L", "complex FP16 opA=C M=262144 N=4096 eps=1e-3 (limbs, 3 digits x 3 groups)"),
    "cfg5": (0, "N", 1048576, 4096, 2048, 1e-8, b"A", "real FP64 M=1048576 N=4096 eps=1e-8 (CRT real, 11 moduli)"),
}


def synth_low_rank(torch, M, N, rank, noise, seed):
    """Configuration 4's own recipe: a rank-`rank` product L R with entries complex N(0, 1 / 256) plus complex Gaussian
    noise of size `noise`, cast to half; column-major M x N (the tensor is [N][M][re, im])."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    s = (1.0 / 512.0) ** 0.5                                   # real and imaginary part: variance 1 / 512 each
    Lt = torch.view_as_complex(torch.randn((rank, M, 2), generator=g, device="cuda", dtype=torch.float32) * s)   # L^T
    Rt = torch.view_as_complex(torch.randn((N, rank, 2), generator=g, device="cuda", dtype=torch.float32) * s)   # R^T
    out = torch.empty((N, M, 2), device="cuda", dtype=torch.float16)
    step = 512                                                  # columns per slab: keeps the FP32 product at 1 GB
    for j in range(0, N, step):
        P = torch.view_as_real(Rt[j:j + step] @ Lt)             # (L R)^T, rows j .. j + step
        P.add_(torch.randn(P.shape, generator=g, device="cuda", dtype=torch.float32), alpha=noise * 0.5 ** 0.5)
        out[j:j + step] = P.half()
    return out


def synth(torch, at, M, N, seed):
    """Column-scaled Gaussian test matrix generated on the device, column-major M x N."""
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    real = torch.float64 if at in (0, 1) else torch.float32
    comps = 2 if at & 1 else 1
    decades = 2.0 if at in (4, 5) else 8.0          # FP16 storage holds five decades in all
    scale = torch.pow(10.0, -torch.arange(N, device="cuda", dtype=torch.float64) * (decades / N)).to(real)
    A = torch.randn((N, M, comps), generator=g, device="cuda", dtype=real)
    A.mul_(scale[:, None, None])
    return A.half().contiguous() if at in (4, 5) else A.contiguous()


def algorithmic_ops(alg, order, cplx, M, N):
    if alg == "C":
        if not cplx:
            return order * M * N * (N + 1)
        return min(order, 20) * 2 * M * N * N + max(order - 20, 0) * (M * N * (N + 1) + 2 * M * N * N)
    ops = order * M * N * (N + 1) + order * (order - 1) * M * N * N
    return ops + (order * order * 2 * M * N * N if cplx else 0)


def cpu_baseline(at, M, N, eps, alg, order, u, sample_rows):
    """The oracle's quantize + int8 Gram + reconstruction on the first sample_rows rows, all host cores."""
    import numpy as np
    from oracle import ho
    rng = np.random.default_rng(3)
    cplx = at & 1
    A = rng.standard_normal((sample_rows, N)) * 10.0 ** (-np.arange(N) / (N / 8.0))
    if cplx:
        A = A + 1j * rng.standard_normal((sample_rows, N)) * 10.0 ** (-np.arange(N) / (N / 8.0))
    A = A.astype({0: np.float64, 1: np.complex128, 2: np.float32, 3: np.complex64}[at])
    ho.build()
    t0 = time.perf_counter()
    vexp = ho.quantize_scale_batch(A, 1, sample_rows, sample_rows, u)
    kind = "crt" if alg == "C" else "limbs"
    K = (sample_rows + 127) // 128 * 128
    panels = ho.quantize(kind, A, order, vexp, ldb=K)
    ho.i8herk(kind, cplx, N, order, panels, 0, 2)
    dt = time.perf_counter() - t0
    feff = sample_rows * N * (N + 1) * (4 if cplx else 1)
    threads = int(os.environ.get("OMP_NUM_THREADS") or len(os.sched_getaffinity(0)))   # what the OpenMP loops of the oracle run on
    out = {"value": feff / dt / 1e12, "unit": "TFLOP/s (FP-equivalent Gram flops)", "cores": threads, "kind": "port",
           "sample": "first %d of %d rows (int8 work is linear in rows), %s order %d, %.2f s" % (sample_rows, M, kind, order, dt)}
    try:   # FP reference: SYRK / HERK from the BLAS scipy ships, on the same sample
        from scipy.linalg import blas
        t0 = time.perf_counter()
        G = (blas.zherk if cplx else blas.dsyrk)(1.0, np.asfortranarray(A.astype(np.complex128 if cplx else np.float64)), trans=2 if cplx else 1)
        out["fp_blas_tflops"] = feff / (time.perf_counter() - t0) / 1e12
        # eigenvalues of the N x N Gram with LAPACK's divide and conquer: the FP counterpart of the fit's tail
        from scipy.linalg import lapack
        t0 = time.perf_counter()
        (lapack.zheevd if cplx else lapack.dsyevd)(G, compute_v=1, lower=0)
        out["fp_lapack_syevd_ms"] = (time.perf_counter() - t0) * 1e3
    except Exception as e:  # pragma: no cover
        out["fp_blas_tflops"] = None
        out["fp_blas_note"] = "BLAS unavailable: %s" % e
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=5)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--workload", default="target", choices=sorted(WORKLOADS))
    ap.add_argument("--no-fit", action="store_true", help="skip the end-to-end hyacinTsvdFit timing")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline")
    ap.add_argument("--no-stages", action="store_true", help="skip the separate timing of the HBM-bound stages (exponents, quantize, dequantize)")
    ap.add_argument("--no-ceiling", action="store_true", help="skip the register-only MFMA ceiling measurement")
    ap.add_argument("--cpu-rows", type=int, default=65536, help="rows of the workload the CPU baseline is timed on (about 15 s of host work)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="before the timed region, run three plain 1 GiB -> 1 GiB device copies (copy_kernel): the known-size reference for HBM traffic counters")
    ap.add_argument("--slab", type=int, default=-1, help="contraction kernel variant: 0 direct-to-LDS ring, 128-byte rows (default); 2 direct-to-LDS, 64-byte rows; 64 / 128 register-staged")
    a = ap.parse_args()
    if a.gpus != 1:
        print("bench.py measures one GPU: the Gram path of this build has no multi-GPU leg (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch
    import hyacinth_amd as ha
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    L = ha.lib()
    at, opA, M, N, K, eps, alg, desc = WORKLOADS[a.workload]
    if a.slab >= 0:
        assert L.hykGramSetSlab(a.slab) == 0
    stream = torch.cuda.current_stream().cuda_stream
    h = ha.create_handle(stream=stream, GramMatrixAlgorithm=alg)
    cplx = at & 1
    A = synth_low_rank(torch, M, N, 256, 1e-4, 0x4859) if a.workload == "cfg4" else synth(torch, at, M, N, 0x4859)          # stored column-major M x N; opA='T' workloads are benchmarked on the transposed copy the fit makes
    lda = M
    u, cP, lP, stride = ha.herk_batch_init(h, eps, M, N, at)
    seg = min(h.GramSegmentK, M) if h.GramSegmentK > 0 else M
    batches, lastM = (M + seg - 1) // seg, M - (M - 1) // seg * seg
    vexp = torch.zeros((batches + 1) * N, dtype=torch.int32, device="cuda")
    Cq = torch.zeros(cP * lP * stride, dtype=torch.int64, device="cuda")
    pA, pV, pC = C.c_void_p(A.data_ptr()), C.c_void_p(vexp.data_ptr()), C.c_void_p(Cq.data_ptr())

    def step():
        L.hyacinXquantizeScaleBatch(C.byref(h), batches, seg, lastM, N, at, pA, lda, u, pV)
        L.hyacinXherkBatch(C.byref(h), batches, seg, lastM, N, at, pA, lda, u, pV, 0, lP, pC)

    if a.copy_calibration:
        src = torch.ones(2 ** 27, dtype=torch.float64, device="cuda")
        dst = torch.empty_like(src)
        for _ in range(3):   # 2^20 x 128 FP64: reads 1 GiB, writes 1 GiB
            assert L.hykMatcopy(stream, b"A", 2 ** 20, 128, 0, C.c_void_p(src.data_ptr()), 2 ** 20, 0, C.c_void_p(dst.data_ptr()), 2 ** 20) == 0
        torch.cuda.synchronize()
        del src, dst

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    L.hykGramProfile(1)
    t0 = time.perf_counter()
    for _ in range(a.steps):
        step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / a.steps
    kms, kn = C.c_double(), C.c_int32()
    L.hykGramProfileRead(C.byref(kms), C.byref(kn))
    L.hykGramProfile(0)

    # the plan the library followed (same planner, host side)
    from oracle import ho
    plan_alg, order, plan_rows = ho.gram_algorithm(alg.decode(), M if batches <= 1 else M, u + cplx, cplx, h.TCGemmTargetK, h.StrideBatchPerfPenalty)
    ops = algorithmic_ops(plan_alg, order, cplx, M, N)
    feff = M * N * (N + 1) * (4 if cplx else 1)
    launches_per_step = max(1, kn.value // a.steps)
    t_kernel = kms.value / 1e3 / a.steps            # contraction kernel time per step
    achieved = ops / t_kernel / 1e12 if t_kernel > 0 else 0.0

    ceiling = None
    if not a.no_ceiling:   # what a register-only MFMA loop sustains on this device with random operands (power-limited clock)
        tops, ghz = C.c_double(), C.c_double()
        if L.hykMfmaCeiling(stream, h.DeviceSMs, 20000, 1, C.byref(tops), C.byref(ghz)) == 0:
            ceiling = {"value": tops.value, "unit": "TFLOP/s", "clock_ghz": ghz.value,
                       "what": "register-only v_mfma_i32_32x32x32_i8 loop, random int8 operands, one workgroup of 4 waves per CU"}

    # HBM-bound stages on their own (HIP events on the launch stream, outside the timed region): algorithmic bytes / time
    def timed_ms(fn, reps=3):
        best = None
        for _ in range(reps):
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record(); fn(); e1.record(); torch.cuda.synchronize()
            t = e0.elapsed_time(e1)
            best = t if best is None or t < best else best
        return best
    eb = {0: 8, 1: 16, 2: 4, 3: 8, 4: 2, 5: 4}[at]
    stages = {}
    if not a.no_stages:
        t = timed_ms(lambda: L.hyacinXquantizeScaleBatch(C.byref(h), batches, seg, lastM, N, at, pA, lda, u, pV))
        stages["column_exponents"] = {"ms": t, "bytes": M * N * eb, "GB/s": M * N * eb / t / 1e6, "frac_of_hbm_peak": M * N * eb / t / 1e6 / HBM_PEAK_GBS}
        rows = min(M, plan_rows) if plan_alg == "C" and plan_rows > 0 else M   # the rows the library quantizes per call (one residue chunk, or all)
        if plan_alg == "C":
            npan = 2 * min(order, 20) + 3 * max(order - 20, 0) if cplx else order
        else:
            npan = 3 * order if cplx else order
        ldb = (rows + 127) // 128 * 128
        ldb += 256 if ldb % 4096 == 0 else 0   # the row padding the library applies to its panels
        panels = torch.empty(npan * N * ldb, dtype=torch.int8, device="cuda")
        pB = C.c_void_p(panels.data_ptr())
        if plan_alg == "C":
            quant = lambda: L.hykQuantizeCrt(stream, rows, N, order, at, pA, lda, pV, pB, ldb, u + cplx)
        else:
            quant = lambda: L.hykQuantizeLimbs(stream, rows, N, order, at, pA, lda, pV, pB, ldb)
        assert quant() == 0
        t = timed_ms(quant)
        qbytes = rows * N * eb + npan * rows * N
        stages["quantize"] = {"ms": t, "rows": rows, "panels": npan, "bytes": qbytes, "GB/s": qbytes / t / 1e6, "frac_of_hbm_peak": qbytes / t / 1e6 / HBM_PEAK_GBS}
        del panels
        gt, gb = C.c_int(), C.c_int32()
        L.hyacinXdequantizeInit(C.byref(h), N, lP, pC, pV, at, C.byref(gt), C.byref(gb))
        G = torch.empty(N * N * gb.value, dtype=torch.uint8, device="cuda")
        t = timed_ms(lambda: L.hyacinXdequantize(C.byref(h), N, lP, pC, pV, gt.value, C.c_void_p(G.data_ptr()), N))
        dbytes = cP * lP * stride * 8 + N * N * gb.value
        stages["dequantize"] = {"ms": t, "bytes": dbytes, "GB/s": dbytes / t / 1e6, "frac_of_hbm_peak": dbytes / t / 1e6 / HBM_PEAK_GBS}
        del G

    fit_ms = None
    if not a.no_fit:
        S = torch.zeros(K, dtype=torch.float64, device="cuda")
        V = torch.zeros(N * K * (2 if cplx else 1), dtype=torch.float64 if at in (0, 1) else torch.float32, device="cuda")
        times = []
        for i in range(3):
            torch.cuda.synchronize()
            t1 = time.perf_counter()
            rank = L.hyacinTsvdFit(C.byref(h), eps, b"N", M, N, K, pA, lda, C.c_void_p(S.data_ptr()), C.c_void_p(V.data_ptr()), N, 0, at)
            torch.cuda.synchronize()
            times.append((time.perf_counter() - t1) * 1e3)
        fit_ms = sorted(times[1:])[len(times[1:]) // 2]

    out = {
        "metric": "Gram-build effective TFLOPS (+ % INT8 MFMA peak; hyacinTsvdFit wall ms)",
        "value": feff / dt / 1e12, "unit": "TFLOP/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": dt * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 (i32 accumulate)", "data": "synthetic",
        "config": {"workload": "%s: %s" % (a.workload, desc), "M": M, "N": N, "eps": eps, "algorithm": plan_alg, "order": order,
                   "quant_bits": u, "gram_limbs": lP, "row_slices": batches},
        "pct_int8_mfma_peak": 100.0 * achieved / INT8_PEAK_TOPS,
        "tsvd_fit_ms": fit_ms,
        "hbm_stages": stages,
        "roofline": {"bound": "mfma", "achieved": achieved, "peak": INT8_PEAK_TOPS, "unit": "TFLOP/s", "frac": achieved / INT8_PEAK_TOPS,
                     "traffic": MEASURED_TRAFFIC.get((a.workload, max(a.slab, 0))),
                     "kernel": "gram_ring_kernel" if a.slab <= 0 else ("gram_dma_kernel" if a.slab == 2 else "gram_kernel<%d>" % a.slab), "ops": "int8 multiply-adds x2, upper triangle only", "launches_per_step": launches_per_step,
                     "avg_launch_ms": kms.value / max(1, kn.value), "algorithmic_ops_per_step": ops,
                     "sustained_mfma_ceiling": ceiling},
    }
    if not a.no_cpu:
        rows = min(a.cpu_rows, M)
        out["cpu_baseline"] = cpu_baseline(at, M, N, eps, plan_alg, order, u, rows)
    ha.destroy_handle(h)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
