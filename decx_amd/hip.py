"""ctypes view of the C ABI (include/decx_hip.h) plus small numpy conveniences used by the
tests, the smoke check and the benchmark.  There is no fallback: if the native library is
missing or no GPU answers, this raises."""
import ctypes
import os

import numpy as np

_PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_PKG, "lib", "libdecx_hip.so")

TILE_AUTO, TILE_LARGE, TILE_MEDIUM, TILE_SMALL, PATH_GEMV, PATH_GEVM = -1, 0, 1, 2, 16, 17

_vp = ctypes.c_void_p
_u32 = ctypes.c_uint32
_f = ctypes.c_float
_sz = ctypes.c_size_t
_int = ctypes.c_int


class DeviceProps(ctypes.Structure):
    _fields_ = [("name", ctypes.c_char * 64), ("arch", ctypes.c_char * 32), ("compute_units", ctypes.c_int32),
                ("clock_khz", ctypes.c_int32), ("memory_clock_khz", ctypes.c_int32),
                ("memory_bus_bits", ctypes.c_int32), ("lds_bytes_per_block", ctypes.c_int32),
                ("wavefront_size", ctypes.c_int32), ("global_mem_bytes", ctypes.c_uint64)]


class Plan(ctypes.Structure):
    _fields_ = [("path", ctypes.c_int32), ("edge", ctypes.c_int32), ("tile_m", _u32), ("tile_n", _u32),
                ("grid", _u32), ("k_splits", _u32), ("whole_tiles", _u32)]


# name -> (restype, argtypes): every symbol include/decx_hip.h declares
SYMBOLS = {
    "decx_hip_init": (_int, [_int]),
    "decx_hip_get_device_props": (_int, [ctypes.POINTER(DeviceProps)]),
    "decx_hip_error_string": (ctypes.c_char_p, [_int]),
    "decx_hip_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "decx_hip_free": (_int, [_vp]),
    "decx_hip_host_malloc": (_int, [ctypes.POINTER(_vp), _sz]),
    "decx_hip_host_free": (_int, [_vp]),
    "decx_hip_memset_async": (_int, [_vp, _int, _sz, _vp]),
    "decx_hip_mem_info": (_int, [ctypes.POINTER(_sz), ctypes.POINTER(_sz)]),
    "decx_hip_reset_split_counters": (_int, []),
    "decx_hip_split_counter_stats": (_int, [ctypes.POINTER(ctypes.c_uint64)]),
    "decx_hip_memcpy2d_async": (_int, [_vp, _sz, _vp, _sz, _sz, _sz, _int, _vp]),
    "decx_hip_stream_create": (_int, [ctypes.POINTER(_vp)]),
    "decx_hip_stream_destroy": (_int, [_vp]),
    "decx_hip_stream_sync": (_int, [_vp]),
    "decx_hip_event_create": (_int, [ctypes.POINTER(_vp)]),
    "decx_hip_event_destroy": (_int, [_vp]),
    "decx_hip_event_record": (_int, [_vp, _vp]),
    "decx_hip_stream_wait_event": (_int, [_vp, _vp]),
    "decx_hip_event_sync": (_int, [_vp]),
    "decx_hip_event_elapsed_ms": (_int, [_vp, _vp, ctypes.POINTER(_f)]),
    "decx_hip_gemm_f32": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp]),
    "decx_hip_gemm_f16": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp]),
    "decx_hip_gemm_f32_workspace": (ctypes.c_size_t, [_u32] * 3),
    "decx_hip_gemm_f32_ws": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp, ctypes.c_size_t, _vp]),
    "decx_hip_gemm_f32_static": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp]),
    "decx_hip_gemm_workspace": (ctypes.c_size_t, [_int] + [_u32] * 3),
    "decx_hip_gemm_f16_ws": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp, ctypes.c_size_t, _vp]),
    "decx_hip_gemm_f64_ws": (_int, [_vp] * 4 + [_u32] * 7 + [ctypes.c_double, ctypes.c_double, _vp, ctypes.c_size_t, _vp]),
    "decx_hip_gemv_f32": (_int, [_vp] * 4 + [_u32] * 6 + [_f, _f, _vp]),
    "decx_hip_gemv_f16": (_int, [_vp] * 4 + [_u32] * 6 + [_f, _f, _int, _vp]),
    "decx_hip_gevm_f32": (_int, [_vp] * 4 + [_u32] * 6 + [_f, _f, _vp]),
    "decx_hip_gevm_f16": (_int, [_vp] * 4 + [_u32] * 6 + [_f, _f, _int, _vp]),
    "decx_hip_gevm_f32_ws": (_int, [_vp] * 4 + [_u32] * 6 + [_f, _f, _vp, _sz, _vp]),
    "decx_hip_gevm_f16_ws": (_int, [_vp] * 4 + [_u32] * 6 + [_f, _f, _int, _vp, _sz, _vp]),
    "decx_hip_conv2d_pack_kernels_f32": (_int, [_vp, _vp] + [_u32] * 5 + [ctypes.c_uint64] + [_u32] * 3 + [_vp]),
    "decx_hip_conv2d_f32": (_int, [_vp] * 3 + [_u32] * 12 + [_vp]),
    "decx_hip_conv2d_f32_depth": (_int, [_vp] * 3 + [_u32] * 13 + [_vp]),
    "decx_hip_gemm_f64": (_int, [_vp] * 4 + [_u32] * 7 + [ctypes.c_double, ctypes.c_double, _vp]),
    "decx_hip_gemm_f64_tile": (_int, [_vp] * 4 + [_u32] * 7 + [ctypes.c_double, ctypes.c_double, _vp, _int, _int]),
    "decx_hip_gemm_complex_workspace": (ctypes.c_size_t, [_int, _u32, _u32]),
    "decx_hip_gemm_c32": (_int, [_vp] * 4 + [_u32] * 7 + [_f] * 4 + [_vp, ctypes.c_size_t, _vp]),
    "decx_hip_gemm_c64": (_int, [_vp] * 4 + [_u32] * 7 + [ctypes.c_double] * 4 + [_vp, ctypes.c_size_t, _vp]),
    "decx_hip_gemm_f32_tile": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp, _int, _int]),
    "decx_hip_gemm_f16_tile": (_int, [_vp] * 4 + [_u32] * 7 + [_f, _f, _vp, _int, _int]),
    "decx_hip_gemm_plan": (_int, [_int, _u32, _u32, _u32, _int, ctypes.POINTER(Plan)]),
    "decx_hip_calibration_copy": (_int, [_vp, _vp, _sz, _vp]),
    "decx_hip_calibration_read": (_int, [_vp, _sz, _vp, _sz, _vp]),
    "decx_hip_gemm_forced_plan": (_int, [_int] + [_vp] * 4 + [_u32] * 7 + [ctypes.c_double, ctypes.c_double, _int, _u32, _u32, _vp, _sz, _vp]),
    "decx_hip_calibration_mfma": (_int, [_int, _vp, _sz, _vp, _sz, _u32, ctypes.POINTER(ctypes.c_double), _vp]),
    "decx_hip_float_to_half": (ctypes.c_uint16, [_f]),
    "decx_hip_half_to_float": (_f, [ctypes.c_uint16]),
}

_lib = None


class HipError(RuntimeError):
    pass


def lib():
    """Loads libdecx_hip.so (built in-tree by decx_amd.build) and types its symbols."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise HipError("native library missing: %s (run `python -m decx_amd.build`)" % LIB_PATH)
        L = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(L, name)       # AttributeError if the library does not export it
            fn.restype, fn.argtypes = res, args
        _lib = L
    return _lib


def check(rc, what=""):
    if rc != 0:
        raise HipError("%s failed: %d (%s)" % (what or "decx_hip call", rc, lib().decx_hip_error_string(rc).decode()))


_inited = False


def init(device=0):
    global _inited
    if not _inited:
        check(lib().decx_hip_init(device), "decx_hip_init")
        _inited = True


def device_props():
    init()
    p = DeviceProps()
    check(lib().decx_hip_get_device_props(ctypes.byref(p)))
    return p


def plan(elem_bytes, M, N, K, aligned=True):
    p = Plan()
    check(lib().decx_hip_gemm_plan(elem_bytes, M, N, K, 1 if aligned else 0, ctypes.byref(p)))
    return p


class DeviceMatrix:
    """A pitched row-major matrix in HBM.  `pitch` in elements; padding columns are filled
    with `pad_value` (NaN by default in tests) so that any kernel that touches them shows."""

    def __init__(self, rows, cols, dtype, pitch=None, data=None, pad_value=None, offset_elems=0):
        init()
        self.rows, self.cols = rows, cols
        self.dtype = np.dtype(dtype)
        self.pitch = pitch if pitch is not None else cols
        assert self.pitch >= cols
        self.offset = offset_elems                  # deliberately misaligned bases for tests
        self.nbytes = (max(rows, 1) * self.pitch + offset_elems) * self.dtype.itemsize
        raw = _vp()
        check(lib().decx_hip_malloc(ctypes.byref(raw), self.nbytes), "decx_hip_malloc")
        self.raw = raw
        self.ptr = _vp(raw.value + offset_elems * self.dtype.itemsize)
        if data is not None or pad_value is not None:
            host = np.empty((rows, self.pitch), self.dtype)
            if pad_value is not None:
                host[...] = pad_value
            if data is not None:
                host[:, :cols] = data
            elif pad_value is None:
                host[:, :cols] = 0
            self.upload_raw(host)

    def upload_raw(self, host):
        host = np.ascontiguousarray(host, self.dtype)
        assert host.shape == (self.rows, self.pitch)
        if host.size:
            check(lib().decx_hip_memcpy2d_async(self.ptr, host.nbytes, host.ctypes.data, host.nbytes,
                                                host.nbytes, 1, 0, None), "upload")
            check(lib().decx_hip_stream_sync(None))

    def download_raw(self):
        host = np.empty((self.rows, self.pitch), self.dtype)
        if host.size:
            check(lib().decx_hip_memcpy2d_async(host.ctypes.data, host.nbytes, self.ptr, host.nbytes,
                                                host.nbytes, 1, 1, None), "download")
            check(lib().decx_hip_stream_sync(None))
        return host

    def download(self):
        return self.download_raw()[:, :self.cols].copy()

    def free(self):
        if self.raw is not None:
            lib().decx_hip_free(self.raw)
            self.raw = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def gemm(A, B, D, C=None, alpha=1.0, beta=1.0, stream=None, tile=TILE_AUTO, force_edge=False, workspace=None):
    """D = A.B or fma(C, beta, alpha*A.B) on DeviceMatrix operands through the C ABI.  workspace: a DeviceMatrix the
    fp32 product may split K through (decx_hip_gemm_f32_ws)."""
    assert A.dtype == B.dtype == D.dtype
    M, K, N = A.rows, A.cols, B.cols
    assert B.rows == K and D.rows == M and D.cols == N
    L = lib()
    f16 = A.dtype == np.float16
    args = [A.ptr, B.ptr, C.ptr if C is not None else None, D.ptr, M, N, K, A.pitch, B.pitch,
            C.pitch if C is not None else 0, D.pitch, alpha, beta, stream]
    if A.dtype in (np.complex64, np.complex128):
        real_bytes = 4 if A.dtype == np.complex64 else 8
        need = L.decx_hip_gemm_complex_workspace(real_bytes, N, K)
        ws = DeviceMatrix(1, max(need // 16, 1), np.complex128)
        a, b = complex(alpha), complex(beta)
        fn = L.decx_hip_gemm_c32 if real_bytes == 4 else L.decx_hip_gemm_c64
        rc = fn(A.ptr, B.ptr, C.ptr if C is not None else None, D.ptr, M, N, K, A.pitch, B.pitch,
                C.pitch if C is not None else 0, D.pitch, a.real, a.imag, b.real, b.imag, ws.ptr, need, stream)
        check(lib().decx_hip_stream_sync(stream))          # the workspace dies with this call
        ws.free()
        check(rc, "gemm")
        return
    if A.dtype == np.float64:
        if workspace is not None and tile == TILE_AUTO and not force_edge:
            check(L.decx_hip_gemm_f64_ws(*args[:-1], workspace.ptr, workspace.rows * workspace.pitch * workspace.dtype.itemsize, stream), "gemm")
        elif tile == TILE_AUTO and not force_edge:
            check(L.decx_hip_gemm_f64(*args), "gemm")
        else:
            check(L.decx_hip_gemm_f64_tile(*args, tile, 1 if force_edge else 0), "gemm")
        return
    if workspace is not None and tile == TILE_AUTO and not force_edge:
        fn = L.decx_hip_gemm_f16_ws if f16 else L.decx_hip_gemm_f32_ws
        rc = fn(*args[:-1], workspace.ptr, workspace.rows * workspace.pitch * workspace.dtype.itemsize, stream)
    elif tile == TILE_AUTO and not force_edge:
        rc = (L.decx_hip_gemm_f16 if f16 else L.decx_hip_gemm_f32)(*args)
    else:
        rc = (L.decx_hip_gemm_f16_tile if f16 else L.decx_hip_gemm_f32_tile)(*args, tile, 1 if force_edge else 0)
    check(rc, "gemm")


def _as_vector(V, n):
    """(pointer, element stride) of a DeviceMatrix used as a vector of n elements: 1 x n is contiguous,
    n x 1 strides by the pitch."""
    if V.rows == 1 and V.cols == n:
        return V.ptr, 1
    assert V.cols == 1 and V.rows == n, "vector operand must be 1 x n or n x 1"
    return V.ptr, V.pitch


def gemv(A, x, y, c=None, alpha=1.0, beta=1.0, stream=None):
    """y (M) = alpha * A (M x K) . x (K) + beta * c through decx_hip_gemv_f32 / _f16; y may be fp32 for fp16 inputs."""
    M, K = A.rows, A.cols
    (xp, incx), (yp, incy) = _as_vector(x, K), _as_vector(y, M)
    cp, incc = _as_vector(c, M) if c is not None else (None, 0)
    L = lib()
    if A.dtype == np.float16:
        assert x.dtype == np.float16 and y.dtype in (np.float16, np.float32)
        rc = L.decx_hip_gemv_f16(A.ptr, xp, cp, yp, M, K, A.pitch, incx, incc, incy, alpha, beta,
                                 1 if y.dtype == np.float32 else 0, stream)
    else:
        assert x.dtype == y.dtype == np.float32
        rc = L.decx_hip_gemv_f32(A.ptr, xp, cp, yp, M, K, A.pitch, incx, incc, incy, alpha, beta, stream)
    check(rc, "gemv")


def gevm(x, B, y, c=None, alpha=1.0, beta=1.0, stream=None, workspace=None):
    """y (N) = alpha * x (K) . B (K x N) + beta * c through decx_hip_gevm_f32 / _f16, or their _ws forms when a
    workspace (a DeviceMatrix) is given."""
    K, N = B.rows, B.cols
    (xp, incx), (yp, incy) = _as_vector(x, K), _as_vector(y, N)
    cp, incc = _as_vector(c, N) if c is not None else (None, 0)
    L = lib()
    ws = () if workspace is None else (workspace.ptr, workspace.rows * workspace.pitch * workspace.dtype.itemsize)
    if B.dtype == np.float16:
        assert x.dtype == np.float16 and y.dtype in (np.float16, np.float32)
        fn = L.decx_hip_gevm_f16 if workspace is None else L.decx_hip_gevm_f16_ws
        rc = fn(xp, B.ptr, cp, yp, K, N, B.pitch, incx, incc, incy, alpha, beta, 1 if y.dtype == np.float32 else 0, *ws, stream)
    else:
        assert x.dtype == y.dtype == np.float32
        fn = L.decx_hip_gevm_f32 if workspace is None else L.decx_hip_gevm_f32_ws
        rc = fn(xp, B.ptr, cp, yp, K, N, B.pitch, incx, incc, incy, alpha, beta, *ws, stream)
    check(rc, "gevm")


def _align(v, a):
    return (v + a - 1) // a * a


def conv2d(image, kernels, stride_x=1, stride_y=1, extend=False, stream=None, pad_value=np.nan, channel_pad_value=0.0):
    """dst[oy][ox][oc] = sum image[oy*sy+kh][ox*sx+kw][ic] * kernels[oc][kh][kw][ic] through decx_hip_conv2d_f32_depth.
    image [H][W][C], kernels [OC][KH][KW][C] (numpy fp32).  Device layouts follow the original's device tensors:
    channel pitch = C rounded up to 4, row pitch = W rounded up to 8 columns; unused columns hold `pad_value`,
    unused channels zero.  extend: zero-extended borders, output W/sx x H/sy."""
    image = np.ascontiguousarray(image, np.float32); kernels = np.ascontiguousarray(kernels, np.float32)
    H, W, C = image.shape
    OC, KH, KW, _ = kernels.shape
    L = lib()
    dp = _align(C, 4)
    if extend:
        ow, oh = W // stride_x, H // stride_y
        left, top = KW // 2, KH // 2
        PW = max((ow - 1) * stride_x + KW, W + left) if ow else W + left
        PH = max((oh - 1) * stride_y + KH, H + top) if oh else H + top
        host_img = np.zeros((PH, PW, C), np.float32)
        host_img[top:top + H, left:left + W] = image
    else:
        ow, oh = (W - KW + 1) // stride_x, (H - KH + 1) // stride_y
        PH, PW, host_img = H, W, image
    wp = _align(PW, 8)
    raw = np.full((PH, wp, dp), pad_value, np.float32)
    raw[:, :PW, :] = channel_pad_value
    raw[:, :PW, :C] = host_img
    d_img = DeviceMatrix(PH, wp * dp, np.float32, data=raw.reshape(PH, wp * dp))
    kdp, kwp = _align(C, 4), _align(KW, 8)
    kraw = np.zeros((OC, KH, kwp, kdp), np.float32)
    kraw[:, :, :KW, :C] = kernels
    d_ker = DeviceMatrix(OC, KH * kwp * kdp, np.float32, data=kraw.reshape(OC, -1))
    kp = _align(OC, 4)
    d_kmat = DeviceMatrix(KH * KW * dp, kp, np.float32)
    check(L.decx_hip_conv2d_pack_kernels_f32(d_ker.ptr, d_kmat.ptr, KW, KH, C, kdp, kwp, KH * kwp * kdp, OC, kp, dp, stream),
          "conv2d pack")
    odp, owp = _align(OC, 4), _align(max(ow, 1), 8)
    d_out = DeviceMatrix(max(oh, 1), owp * odp, np.float32)
    d_out.upload_raw(np.full((max(oh, 1), owp * odp), -555.0, np.float32))
    check(L.decx_hip_conv2d_f32_depth(d_img.ptr, d_kmat.ptr, d_out.ptr, ow, oh, OC, KW, KH, C, dp, wp, stride_x, stride_y, kp, odp,
                                      owp, stream), "conv2d")
    check(L.decx_hip_stream_sync(stream))
    out_raw = d_out.download_raw().reshape(max(oh, 1), owp, odp)
    for d in (d_img, d_ker, d_kmat, d_out):
        d.free()
    return out_raw[:oh, :ow, :OC].copy(), out_raw


def mem_free_bytes():
    """Free device memory as the runtime reports it."""
    free, total = _sz(), _sz()
    check(lib().decx_hip_mem_info(ctypes.byref(free), ctypes.byref(total)), "mem info")
    return free.value


def split_counter_stats():
    """{"taken", "wraps", "refused", "events", "reserved", "ring"}: what the split-K counter windows have seen so far."""
    out = (ctypes.c_uint64 * 6)()
    check(lib().decx_hip_split_counter_stats(out), "split counter stats")
    return dict(zip(("taken", "wraps", "refused", "events", "reserved", "ring"), (int(v) for v in out)))


class Stream:
    def __init__(self):
        init()
        self.handle = _vp()
        check(lib().decx_hip_stream_create(ctypes.byref(self.handle)), "stream create")

    def sync(self):
        check(lib().decx_hip_stream_sync(self.handle), "stream sync")

    def destroy(self):
        if self.handle is not None:
            check(lib().decx_hip_stream_destroy(self.handle), "stream destroy")
            self.handle = None


def sync(stream=None):
    check(lib().decx_hip_stream_sync(stream), "stream sync")


class Timer:
    """HIP events on the stream the kernels are launched on."""

    def __init__(self):
        init()
        self.a, self.b = _vp(), _vp()
        check(lib().decx_hip_event_create(ctypes.byref(self.a)))
        check(lib().decx_hip_event_create(ctypes.byref(self.b)))

    def start(self, stream=None):
        check(lib().decx_hip_event_record(self.a, stream))

    def stop(self, stream=None):
        check(lib().decx_hip_event_record(self.b, stream))
        check(lib().decx_hip_event_sync(self.b))
        ms = _f()
        check(lib().decx_hip_event_elapsed_ms(self.a, self.b, ctypes.byref(ms)))
        return ms.value
