"""Where the pivoted Cholesky and a Jacobi round spend their time, from the measurement build of the library.

    python -m hyacinth_amd.build --timing
    HYACIN_LIBRARY=hyacinth_amd/libhyacin_timing.so python -m hyacinth_amd.phase_timing

The measurement build compiles potrfp.hip with -DHYK_POTRFP_TIMING (the first agent adds up 10 ns wall-clock ticks per phase
of its steps into the control words of the workspace) and tail.hip with -DHYK_JACOBI_TIMING (the first thread of workgroup 1
adds shader-clock differences between the phases of a round to the words behind the sweep's rotation counter).  The stamps cost
time themselves: the totals are a few per cent above those of the product build.
"""
import ctypes as C
import os
import sys

import numpy as np


def potrfp_phases(L, torch, N, gtype):
    cplx, dd = gtype & 1, gtype >= 6
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    A = torch.randn((N + 64, N), generator=g, device="cuda", dtype=torch.float64)
    if cplx:
        A = torch.complex(A, torch.randn((N + 64, N), generator=g, device="cuda", dtype=torch.float64))
    A = A * torch.pow(10.0, -torch.arange(N, device="cuda", dtype=torch.float64) * (6.0 / N))[None, :]
    Gt = (A.conj().T @ A).T.contiguous()
    W = 2 if dd else 1
    raw = torch.zeros((N, N, W * (2 if cplx else 1)), device="cuda", dtype=torch.float64)
    raw[..., 0] = Gt.real if cplx else Gt
    if cplx:
        raw[..., W] = Gt.imag
    ws = torch.zeros(L.hykPotrfpWorkspaceBytes(N, gtype), dtype=torch.uint8, device="cuda")
    rk = torch.zeros(1, dtype=torch.int32).pin_memory()
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    best = None
    for _ in range(3):
        Gc = raw.clone()
        Rt = torch.zeros(N * N * raw.shape[2], device="cuda", dtype=torch.float64)
        jp = torch.zeros(N, dtype=torch.int32, device="cuda")
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        rc = L.hykPotrfp(st, 256, 1e-13, N, N, gtype, C.c_void_p(Gc.data_ptr()), N, C.c_void_p(Rt.data_ptr()), N, C.c_void_p(jp.data_ptr()), C.c_void_p(ws.data_ptr()), C.c_void_p(rk.data_ptr()))
        e1.record()
        torch.cuda.synchronize()
        assert rc == 0 and int(rk[0]) > 0
        ms = e0.elapsed_time(e1)
        if best is None or ms < best[0]:
            off = (N * 4 + 255) // 256 * 256 + 2 * 128 * 16 * 8            # position table, exchange records, then the control words
            t = ws[off + 40 * 8: off + 50 * 8].cpu().numpy().view(np.int64)
            best = (ms, int(rk[0]), t.copy())
    ms, rank, t = best
    steps = max(1, int(t[9]))
    us = t[:8] / 100.0
    print("potrfp N %d type %d: %.2f ms, rank %d, %d steps, %d started on the fetched-ahead column" % (N, gtype, ms, rank, steps, int(t[8])))
    print("   first agent, us in all: waiting for the update %.0f | loads + dot %.0f | reduce %.0f | publish + fetch ahead %.0f | collect %.0f | panel summary %.0f | update %.0f | rest %.0f"
          % (us[0], us[1], us[2], us[3], us[4], us[5], us[6], us[7]))
    print("   per step, us: loads + dot %.2f | reduce %.2f | publish + fetch ahead %.2f | collect %.2f" % (us[1] / steps, us[2] / steps, us[3] / steps, us[4] / steps))


def jacobi_phases(L, torch, cplx, N, r, sweeps=3):
    g = torch.Generator(device="cuda")
    g.manual_seed(3)
    def rnd(n):
        a = torch.randn((n, n), generator=g, device="cuda", dtype=torch.float64)
        return torch.complex(a, torch.randn((n, n), generator=g, device="cuda", dtype=torch.float64)) if cplx else a
    Q, _ = torch.linalg.qr(rnd(N))
    Q2, _ = torch.linalg.qr(rnd(N))
    s = torch.pow(10.0, -torch.arange(N, device="cuda", dtype=torch.float64) / 128.0)
    Bm = ((Q * s[None, :]) @ Q2)[:, :r].T.contiguous()                      # column-major N x r: dense, singular values s
    B = torch.view_as_real(Bm).contiguous() if cplx else Bm
    cnt = torch.zeros(16, dtype=torch.int32, device="cuda")
    carry = torch.zeros(L.hykJacobiCarryBytes(r), dtype=torch.uint8, device="cuda")
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    rounds = r // (4 if cplx else 8) - 1
    for sw in range(sweeps):
        cnt.zero_()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        rc = L.hykJacobiSweepCarry(st, cplx, N, r, C.c_void_p(B.data_ptr()), 6.25e-14, C.c_void_p(cnt.data_ptr()), C.c_void_p(carry.data_ptr()))
        b.record()
        torch.cuda.synchronize()
        assert rc == 0
        h = cnt.cpu().numpy()
        t = h[4:16].view(np.int64) / float(rounds)
        print("jacobi %s N %d r %d sweep %d: %.2f ms, %d rotations; shader cycles per round: load %.0f | sums %.0f | waiting for the slowest wavefront %.0f | steps %.0f | replay of the first wavefront's rows %.0f | store %.0f | sum %.0f"
              % ("complex" if cplx else "real", N, r, sw, a.elapsed_time(b), int(h[0]), t[0], t[1], t[2], t[3], t[4], t[5], t.sum()))


def main():
    if "timing" not in os.path.basename(os.environ.get("HYACIN_LIBRARY", "")):
        sys.exit("set HYACIN_LIBRARY to the measurement build (python -m hyacinth_amd.build --timing): the product build has no stamps")
    import torch
    import hyacinth_amd as ha
    L = ha.lib()
    for N, gtype in ((2048, 6), (2048, 7), (2048, 0), (4096, 6)):
        potrfp_phases(L, torch, N, gtype)
    jacobi_phases(L, torch, 0, 2048, 2048)
    jacobi_phases(L, torch, 0, 1024, 1024)
    jacobi_phases(L, torch, 1, 2048, 2048)


if __name__ == "__main__":
    main()
