"""GPU-side helpers for the tests: device buffers through torch, calls through the C ABI of libhyacin.so."""
import ctypes as C

import numpy as np
import torch

import hyacinth_amd as ha

DEV = "cuda:0"


def dev(a):
    """numpy -> device tensor of raw bytes (keeps layout)."""
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a.view(np.uint8).reshape(-1).copy()).to(DEV)


def host(t, dtype, shape=None):
    a = t.cpu().numpy().view(dtype)
    return a.reshape(shape) if shape is not None else a


def zeros(nbytes):
    return torch.zeros(int(nbytes), dtype=torch.uint8, device=DEV)


def ptr(t):
    return C.c_void_p(t.data_ptr())


def stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def sync():
    torch.cuda.synchronize()


def colmajor_bytes(A):
    """Column-major device copy of a test matrix; returns (tensor, lda, precision enum)."""
    from oracle import ho
    Af, lda = ho.colmajor(A)
    if Af.ndim == 2:
        flat = np.ascontiguousarray(Af.T)      # [col][row] contiguous == column-major
    else:
        flat = Af                              # complex half is already [col][row][2]
    return dev(flat), lda, ho.atype_of(A)


def stored_transpose(A, op, pad=0):
    """The stored N x M matrix S with op(S) = A (op 'T' or 'C'), column-major with leading dimension N + pad: returns
    (device tensor, lda, precision enum).  S[j + k lda] = A[k, j], conjugated for 'C'; the padding holds NaN."""
    from oracle import ho
    at = ho.atype_of(A)
    M, N = A.shape[0], A.shape[1]
    if A.ndim == 3:                                   # complex half as [M, N, 2]
        body = A.copy()
        if op == "C":
            body[..., 1] = -body[..., 1]
        buf = np.full((M, N + pad, 2), np.nan, np.float16)
        buf[:, :N] = body
    else:
        body = np.conj(A) if (op == "C" and np.iscomplexobj(A)) else A
        buf = np.full((M, N + pad), np.nan, A.dtype)
        buf[:, :N] = body
    return dev(buf), N + pad, at


def check(rc):
    assert rc == 0, "kernel layer returned %d" % rc


class Lib:
    def __init__(self):
        self.L = ha.lib()

    def column_exponents(self, A, batches, segM, lastM, u):
        d, lda, at = colmajor_bytes(A)
        N = A.shape[1]
        vexp = zeros(4 * (max(batches, 0) + 1) * N)
        check(self.L.hykColumnExponents(stream(), batches, segM, lastM, N, at, ptr(d), lda, u, ptr(vexp)))
        sync()
        return host(vexp, np.int32)

    def column_exponents_op(self, A, op, batches, segM, lastM, u, pad=0):
        d, lda, at = stored_transpose(A, op, pad)
        N = A.shape[1]
        vexp = zeros(4 * (max(batches, 0) + 1) * N)
        check(self.L.hykColumnExponentsOp(stream(), op.encode(), batches, segM, lastM, N, at, ptr(d), lda, u, ptr(vexp)))
        sync()
        return host(vexp, np.int32)

    def quantize_op(self, kind, A, op, order, vexp, ldb=None, max_bits=0, pad=0):
        from oracle import ho
        d, lda, at = stored_transpose(A, op, pad)
        M, N = A.shape[0], A.shape[1]
        ldb = ldb or M
        panels = ho.n_panels(kind, order, at & 1)
        B = zeros(panels * N * ldb)
        dv = dev(np.ascontiguousarray(vexp[:N]))
        if kind == "limbs":
            check(self.L.hykQuantizeLimbsOp(stream(), op.encode(), M, N, order, at, ptr(d), lda, ptr(dv), ptr(B), ldb))
        else:
            check(self.L.hykQuantizeCrtOp(stream(), op.encode(), M, N, order, at, ptr(d), lda, ptr(dv), ptr(B), ldb, max_bits))
        sync()
        return host(B, np.int8, (panels, N, ldb))

    def quantize(self, kind, A, order, vexp, ldb=None, row_offset=0, max_bits=0):
        from oracle import ho
        d, lda, at = colmajor_bytes(A)
        M, N = A.shape[0], A.shape[1]
        ldb = ldb or (M + row_offset)
        panels = ho.n_panels(kind, order, at & 1)
        B = zeros(panels * N * ldb)
        dv = dev(np.ascontiguousarray(vexp[:N]))
        out = C.c_void_p(B.data_ptr() + row_offset)
        if kind == "limbs":
            check(self.L.hykQuantizeLimbs(stream(), M, N, order, at, ptr(d), lda, ptr(dv), out, ldb))
        else:
            check(self.L.hykQuantizeCrt(stream(), M, N, order, at, ptr(d), lda, ptr(dv), out, ldb, max_bits))
        sync()
        return host(B, np.int8, (panels, N, ldb))

    def gram(self, kind, cplx, N, order, panels, orderC, beta=0, Cin=None, K=None):
        """panels: int8 [p][N][ldb] host array."""
        ldb = panels.shape[2]
        K = K or ldb
        T = N * (N + 1) // 2
        dP = dev(panels)
        Cd = zeros(8 * (1 + cplx) * orderC * T) if Cin is None else dev(Cin)
        code = ha.GRAM_LIMBS if kind == "limbs" else ha.GRAM_CRT
        wsb = self.L.hykGramWorkspaceBytes(code, cplx, N, order)
        ws = torch.empty(int(wsb), dtype=torch.uint8, device=DEV).fill_(0x5A)
        check(self.L.hykGramWorkspaceClear(stream(), ptr(ws), wsb))
        fn = self.L.hykGramLimbs if kind == "limbs" else self.L.hykGramCrt
        check(fn(stream(), cplx, N, order, ptr(dP), ldb, K, beta, orderC, ptr(Cd), ptr(ws)))
        sync()
        assert not bool(ws.any()), "workspace must be zero again after the call"
        return host(Cd, np.uint64)
