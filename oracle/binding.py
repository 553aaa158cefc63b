"""ctypes bindings of the CPU oracle (liboracle.so) and, when it has been built in the
build container, of the compiled reference CPU GEMM (oracle/_ref).  TEST INFRASTRUCTURE ONLY."""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_f32p = ctypes.POINTER(ctypes.c_float)
_f64p = ctypes.POINTER(ctypes.c_double)
_u16p = ctypes.POINTER(ctypes.c_uint16)
_u32p = ctypes.POINTER(ctypes.c_uint32)
_u32 = ctypes.c_uint32
_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        path = os.path.join(_HERE, "liboracle.so")
        if not os.path.exists(path):
            build()
        L = ctypes.CDLL(path)
        L.oracle_half_to_float.restype = ctypes.c_float
        L.oracle_half_to_float.argtypes = [ctypes.c_uint16]
        L.oracle_float_to_half.restype = ctypes.c_uint16
        L.oracle_float_to_half.argtypes = [ctypes.c_float]
        L.oracle_fill_uniform_f32.argtypes = [_f32p, _u32, _u32, _u32, ctypes.c_uint64]
        L.oracle_gemm_f32_chain.argtypes = [_f32p, _f32p, _f32p, _f32p] + [_u32] * 7 + [_u32p, _u32]
        L.oracle_gemm_f32_chain_scalar.argtypes = [_f32p, _f32p, _f32p, _f32p] + [_u32] * 7
        L.oracle_gemm_f32_axpby.argtypes = ([_f32p, _f32p, _f32p, _f32p] + [_u32] * 7 +
                                            [ctypes.c_float, ctypes.c_float, _u32p, _u32])
        L.oracle_gemm_f16.argtypes = ([_u16p, _u16p, _u16p, _u16p] + [_u32] * 7 +
                                      [ctypes.c_float, ctypes.c_float, _u32p, _u32])
        L.oracle_gemm_f64_brute.argtypes = ([_f32p, _f32p, _f32p, _f64p] + [_u32] * 7 +
                                            [ctypes.c_double, ctypes.c_double])
        L.cpu_port_scratch_floats.restype = ctypes.c_size_t
        L.cpu_port_scratch_floats.argtypes = [_u32, _u32]
        L.cpu_port_max_threads.restype = _u32
        L.cpu_port_gemm_f32.restype = ctypes.c_int
        L.cpu_port_gemm_f32.argtypes = [_f32p, _f32p, _f32p, _f32p] + [_u32] * 7 + [_f32p, _u32]
        L.oracle_gemm_f64_chain.argtypes = [_f64p, _f64p, _f64p, _f64p] + [_u32] * 7 + [_u32p, _u32]
        L.oracle_gemm_f64_axpby.argtypes = ([_f64p, _f64p, _f64p, _f64p] + [_u32] * 7 +
                                            [ctypes.c_double, ctypes.c_double, _u32p, _u32])
        L.oracle_conv2d_out_dims.argtypes = [_u32] * 6 + [ctypes.c_int, _u32p, _u32p]
        L.oracle_conv2d_f32.argtypes = [_f32p] + [_u32] * 3 + [_f32p] + [_u32] * 5 + [ctypes.c_int, _f32p]
        _lib = L
    return _lib


def _p(a, ty):
    return a.ctypes.data_as(ty) if a is not None else None


def _rows(rows):
    if rows is None:
        return None, None, 0
    r = np.ascontiguousarray(rows, dtype=np.uint32)
    return r, _p(r, _u32p), len(r)


def _ld(a):
    assert a.strides[1] == a.itemsize, "row-major with unit column stride required"
    return a.strides[0] // a.itemsize


def gemm_f32(A, B, C=None, alpha=None, beta=None, rows=None):
    """Scalar-chain oracle.  A (M,K), B (K,N), optional C (M,N): 2-D float32 views with
    unit column stride (row pitch may exceed the width).  alpha/beta None -> chain seeded
    with C (the CPU semantics); otherwise fma(C, beta, alpha*chain0) (the GPU entry point).
    rows: optional subset of output rows; the result then has len(rows) rows."""
    M, K = A.shape
    K2, N = B.shape
    assert K == K2
    keep, rp, nr = _rows(rows)
    out = np.empty((nr if rows is not None else M, N), np.float32)
    if alpha is None:
        lib().oracle_gemm_f32_chain(_p(A, _f32p), _p(B, _f32p), _p(C, _f32p), _p(out, _f32p), M, N, K,
                                    _ld(A), _ld(B), _ld(C) if C is not None else 0, N, rp, nr)
    else:
        assert C is not None
        lib().oracle_gemm_f32_axpby(_p(A, _f32p), _p(B, _f32p), _p(C, _f32p), _p(out, _f32p), M, N, K,
                                    _ld(A), _ld(B), _ld(C), N, alpha, beta, rp, nr)
    return out


def gemm_f64(A, B, C=None, alpha=None, beta=None, rows=None):
    """Double-precision chain oracle; same conventions as gemm_f32."""
    M, K = A.shape
    K2, N = B.shape
    assert K == K2 and A.dtype == np.float64 and B.dtype == np.float64
    keep, rp, nr = _rows(rows)
    out = np.empty((nr if rows is not None else M, N), np.float64)
    if alpha is None:
        lib().oracle_gemm_f64_chain(_p(A, _f64p), _p(B, _f64p), _p(C, _f64p), _p(out, _f64p), M, N, K,
                                    _ld(A), _ld(B), _ld(C) if C is not None else 0, N, rp, nr)
    else:
        assert C is not None
        lib().oracle_gemm_f64_axpby(_p(A, _f64p), _p(B, _f64p), _p(C, _f64p), _p(out, _f64p), M, N, K,
                                    _ld(A), _ld(B), _ld(C), N, alpha, beta, rp, nr)
    return out


def complex_embed(B):
    """The real 2K x 2N matrix whose product with an interleaved complex row gives the interleaved complex result."""
    K, N = B.shape
    rt = np.float32 if B.dtype == np.complex64 else np.float64
    X = np.empty((2 * K, 2 * N), rt)
    X[0::2, 0::2] = B.real; X[0::2, 1::2] = B.imag
    X[1::2, 0::2] = -B.imag; X[1::2, 1::2] = B.real
    return X


def gemm_complex(A, B, C=None):
    """Complex A.B (+ C): per element re = chain of fma(ar, br, .), fma(ai, -bi, .) and im = chain of fma(ar, bi, .),
    fma(ai, br, .), k ascending, seeded with 0 or C -- i.e. the real chain oracle on the real expansion of B."""
    assert A.dtype == B.dtype and A.dtype in (np.complex64, np.complex128)
    rt = np.float32 if A.dtype == np.complex64 else np.float64
    Ar = np.ascontiguousarray(A).view(rt)
    Cr = np.ascontiguousarray(C).view(rt) if C is not None else None
    fn = gemm_f32 if rt == np.float32 else gemm_f64
    return np.ascontiguousarray(fn(Ar, complex_embed(B), Cr)).view(A.dtype)


def gemm_f32_scalar(A, B, C=None):
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N), np.float32)
    lib().oracle_gemm_f32_chain_scalar(_p(A, _f32p), _p(B, _f32p), _p(C, _f32p), _p(out, _f32p), M, N, K,
                                       _ld(A), _ld(B), _ld(C) if C is not None else 0, N)
    return out


def gemm_f16(A, B, C=None, alpha=1.0, beta=1.0, rows=None):
    """A, B, C: float16 arrays (2-D, unit column stride).  Returns float16."""
    M, K = A.shape
    N = B.shape[1]
    keep, rp, nr = _rows(rows)
    out = np.empty((nr if rows is not None else M, N), np.float16)
    lib().oracle_gemm_f16(_p(A, _u16p), _p(B, _u16p), _p(C, _u16p), _p(out, _u16p), M, N, K,
                          _ld(A), _ld(B), _ld(C) if C is not None else 0, N, alpha, beta, rp, nr)
    return out


def gemm_f64_brute(A, B, C=None, alpha=1.0, beta=1.0):
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N), np.float64)
    lib().oracle_gemm_f64_brute(_p(A, _f32p), _p(B, _f32p), _p(C, _f32p), _p(out, _f64p), M, N, K,
                                _ld(A), _ld(B), _ld(C) if C is not None else 0, N, alpha, beta)
    return out


def fill_uniform_f32(rows, cols, seed):
    out = np.empty((rows, cols), np.float32)
    lib().oracle_fill_uniform_f32(_p(out, _f32p), rows, cols, cols, seed)
    return out


def aligned_f32(rows, cols, fill=0.0):
    """Host matrix in the reference's host layout: pitch = width rounded up to 8 floats,
    base 32-byte aligned.  Returns (view rows x cols, pitch)."""
    pitch = (cols + 7) // 8 * 8
    raw = np.empty(rows * pitch + 8, np.float32)
    off = (-raw.ctypes.data // 4) % 8
    buf = raw[off:off + rows * pitch].reshape(rows, pitch)
    buf[...] = fill
    return buf, pitch


def cpu_port_gemm_f32(A, B, C=None, threads=8):
    """The multithreaded AVX2 restatement of the reference CPU GEMM.  Inputs are copied into
    host-layout buffers; returns an (M, N) array."""
    M, K = A.shape
    N = B.shape[1]
    a, lda = aligned_f32(M, K); a[:, :K] = A
    b, ldb = aligned_f32(K, N); b[:, :N] = B
    d, ldd = aligned_f32(M, N)
    c = None; ldc = 0
    if C is not None:
        c, ldc = aligned_f32(M, N); c[:, :N] = C
    scratch, _ = aligned_f32(1, int(lib().cpu_port_scratch_floats(K, N)))
    rc = lib().cpu_port_gemm_f32(_p(a, _f32p), _p(b, _f32p), _p(c, _f32p), _p(d, _f32p), M, N, K,
                                 lda, ldb, ldc, ldd, _p(scratch, _f32p), threads)
    assert rc == 0, rc
    return d[:, :N].copy()


# --------------------------------------------------------------------------- compiled reference

_ref_fn = None


def reference_available():
    return (os.path.exists(os.path.join(_HERE, "_ref", "libdecx_ref_cpu.so")) and
            os.path.exists(os.path.join(_HERE, "_ref", "libref_loader.so")) and
            (os.cpu_count() or 99) <= 16)   # the reference's thread pool overruns its 16 slots beyond that


def _reference_call(A, B, C, threads):
    """Element type by A.dtype: float32 or float64."""
    global _ref_fn
    if _ref_fn is None:
        ld = ctypes.CDLL(os.path.join(_HERE, "_ref", "libref_loader.so"))
        ld.ref_loader_sym.restype = ctypes.c_void_p
        ld.ref_loader_sym.argtypes = [ctypes.c_char_p, ctypes.c_char_p]
        path = os.path.join(_HERE, "_ref", "libdecx_ref_cpu.so").encode()
        a32, a64 = ld.ref_loader_sym(path, b"ref_cpu_gemm_f32"), ld.ref_loader_sym(path, b"ref_cpu_gemm_f64")
        ac32 = ld.ref_loader_sym(path, b"ref_cpu_gemm_c32")
        assert a32 and a64 and ac32, "could not load the compiled reference"
        f32sig = ctypes.CFUNCTYPE(ctypes.c_int, _f32p, _f32p, _f32p, _f32p, _u32, _u32, _u32, _u32)
        _ref_fn = {np.dtype(np.float32): (f32sig(a32), _f32p),
                   np.dtype(np.float64): (ctypes.CFUNCTYPE(ctypes.c_int, _f64p, _f64p, _f64p, _f64p, _u32, _u32, _u32, _u32)(a64), _f64p),
                   np.dtype(np.complex64): (f32sig(ac32), _f32p)}
    fn, pt = _ref_fn[A.dtype]
    M, K = A.shape
    N = B.shape[1]
    out = np.empty((M, N), A.dtype)
    err = fn(_p(A, pt), _p(B, pt), _p(C, pt), _p(out, pt), M, N, K, threads)
    return out, err


def reference_cpu_gemm_c32(A, B, C=None, threads=8):
    """The same for the reference's single-precision complex CPU GEMM (complex64 arrays)."""
    return reference_cpu_gemm_f32(A, B, C, threads, dtype=np.complex64)


def reference_cpu_gemm_f64(A, B, C=None, threads=8):
    """The same for the reference's double-precision CPU GEMM."""
    return reference_cpu_gemm_f32(A, B, C, threads, dtype=np.float64)


def reference_cpu_gemm_f32(A, B, C=None, threads=8, dtype=np.float32):
    """de::blas::cpu::GEMM of the compiled reference (build container only).  Every call runs
    in a process of its own: the reference's cached planner does not survive a change of
    shape or thread count reliably, and a crash must not take the test run with it.  Some
    shapes crash inside the reference's planner as the first call of a process and work
    after any earlier call, others the other way round; so the child is tried first cold,
    then with one 64x64x64 single-thread call in front, up to three times each (the crashes
    are intermittent).  Returns (D, error_type); raises RuntimeError if every child died."""
    import tempfile
    A = np.ascontiguousarray(A, dtype); B = np.ascontiguousarray(B, dtype)
    with tempfile.TemporaryDirectory() as tmp:
        np.save(os.path.join(tmp, "A.npy"), A)
        np.save(os.path.join(tmp, "B.npy"), B)
        if C is not None:
            np.save(os.path.join(tmp, "C.npy"), np.ascontiguousarray(C, dtype))
        for warm in ("", "w = np.zeros((64, 64), np.float32); b._reference_call(w, w, None, 1);") * 3:
            code = ("import sys, os, numpy as np; sys.path.insert(0, %r); from oracle import binding as b; t = %r;"
                    "A = np.load(t + '/A.npy'); B = np.load(t + '/B.npy');"
                    "C = np.load(t + '/C.npy') if os.path.exists(t + '/C.npy') else None;"
                    "%s"
                    "D, e = b._reference_call(A, B, C, %d); np.save(t + '/D.npy', D); open(t + '/err', 'w').write(str(e))"
                    % (os.path.dirname(_HERE), tmp, warm, threads))
            done = subprocess.run([os.sys.executable, "-c", code], timeout=600)
            if done.returncode == 0:
                return np.load(os.path.join(tmp, "D.npy")), int(open(os.path.join(tmp, "err")).read())
        raise RuntimeError("the compiled reference crashed on %s x %s, %d threads" % (A.shape, B.shape, threads))


def conv2d_out_dims(W, H, KW, KH, sx=1, sy=1, extend=False):
    ow, oh = _u32(), _u32()
    lib().oracle_conv2d_out_dims(W, H, KW, KH, sx, sy, int(extend), ctypes.byref(ow), ctypes.byref(oh))
    return ow.value, oh.value


def conv2d_f32(image, kernels, sx=1, sy=1, extend=False):
    """image [H][W][C], kernels [OC][KH][KW][C] -> [OH][OW][OC]; fmaf chain over (kh, kw, ic)."""
    image = np.ascontiguousarray(image, np.float32); kernels = np.ascontiguousarray(kernels, np.float32)
    H, W, C = image.shape
    OC, KH, KW, C2 = kernels.shape
    assert C == C2
    ow, oh = conv2d_out_dims(W, H, KW, KH, sx, sy, extend)
    out = np.empty((oh, ow, OC), np.float32)
    lib().oracle_conv2d_f32(_p(image, _f32p), W, H, C, _p(kernels, _f32p), OC, KW, KH, sx, sy, int(extend), _p(out, _f32p))
    return out
