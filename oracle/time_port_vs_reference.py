"""TEST INFRASTRUCTURE ONLY.  Times the AVX2 restatement of the reference CPU GEMM (cpu_gemm_port.c, what
bench.py's cpu_baseline leg runs on the GPU box) against the compiled reference itself (oracle/_ref, build
container only) on the same matrices and thread count, best of N calls each, so that the restatement can stand in
for the reference as a clock.

    python -m oracle.time_port_vs_reference [threads] [repeats]
"""
import ctypes
import json
import os
import subprocess
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
SHAPES = [(1024, 1024, 1024), (1000, 1500, 777)]


def time_port(A, B, threads, repeats):
    from oracle import binding as b
    M, K = A.shape; N = B.shape[1]
    L = b.lib()
    a, lda = b.aligned_f32(M, K); a[:, :K] = A
    bb, ldb = b.aligned_f32(K, N); bb[:, :N] = B
    d, ldd = b.aligned_f32(M, N)
    scratch, _ = b.aligned_f32(1, int(L.cpu_port_scratch_floats(K, N)))
    fp = ctypes.POINTER(ctypes.c_float)
    args = [x.ctypes.data_as(fp) for x in (a, bb)] + [None, d.ctypes.data_as(fp), M, N, K, lda, ldb, 0, ldd,
                                                      scratch.ctypes.data_as(fp), threads]
    best = 1e30
    for _ in range(repeats):
        t0 = time.perf_counter()
        assert L.cpu_port_gemm_f32(*args) == 0
        best = min(best, (time.perf_counter() - t0) * 1e3)
    return best, d[:, :N].copy()


def time_reference_child(M, N, K, threads, repeats):
    """One child process per shape (the reference's planner does not survive a change of shape reliably)."""
    code = ("import sys, ctypes, numpy as np; sys.path.insert(0, %r)\n"
            "from oracle import binding as b; from decx_amd import synth\n"
            "ld = ctypes.CDLL(b._HERE + '/_ref/libref_loader.so'); ld.ref_loader_sym.restype = ctypes.c_void_p\n"
            "ld.ref_loader_sym.argtypes = [ctypes.c_char_p, ctypes.c_char_p]\n"
            "addr = ld.ref_loader_sym((b._HERE + '/_ref/libdecx_ref_cpu.so').encode(), b'ref_cpu_gemm_f32_timed')\n"
            "fp = ctypes.POINTER(ctypes.c_float); u = ctypes.c_uint32\n"
            "fn = ctypes.CFUNCTYPE(ctypes.c_int, fp, fp, fp, u, u, u, u, u, ctypes.POINTER(ctypes.c_double))(addr)\n"
            "A = synth.uniform_f32(%d, %d, 11); B = synth.uniform_f32(%d, %d, 12); D = np.empty((%d, %d), np.float32)\n"
            "ms = ctypes.c_double()\n"
            "e = fn(A.ctypes.data_as(fp), B.ctypes.data_as(fp), D.ctypes.data_as(fp), %d, %d, %d, %d, %d, ctypes.byref(ms))\n"
            "np.save(sys.argv[1], D); print('REFMS', e, ms.value)\n" % (ROOT, M, K, K, N, M, N, M, N, K, threads, repeats))
    import tempfile
    with tempfile.TemporaryDirectory() as tmp:
        out = os.path.join(tmp, "D.npy")
        for _ in range(4):                                   # the reference crashes intermittently
            done = subprocess.run([sys.executable, "-c", code, out], capture_output=True, text=True, timeout=600)
            for l in done.stdout.splitlines():
                if l.startswith("REFMS") and done.returncode == 0:
                    return float(l.split()[2]), np.load(out)
    return None, None


def measure(threads=8, repeats=7):
    from oracle import binding as b
    from decx_amd import synth
    rows = []
    for M, N, K in SHAPES:
        A = synth.uniform_f32(M, K, 11); B = synth.uniform_f32(K, N, 12)
        port_ms, Dp = time_port(A, B, threads, repeats)
        ref_ms, Dr = (None, None)
        if b.reference_available():
            ref_ms, Dr = time_reference_child(M, N, K, threads, repeats)
        rows.append({"shape": [M, N, K], "threads": threads, "port_ms": round(port_ms, 2),
                     "reference_ms": None if ref_ms is None else round(ref_ms, 2),
                     "port_over_reference": None if ref_ms is None else round(port_ms / ref_ms, 3),
                     "bit_equal": None if Dr is None else bool(np.array_equal(Dp.view(np.uint32), Dr.view(np.uint32)))})
    return rows


if __name__ == "__main__":
    t = int(sys.argv[1]) if len(sys.argv) > 1 else 8
    r = int(sys.argv[2]) if len(sys.argv) > 2 else 7
    for row in measure(t, r):
        print(json.dumps(row))
