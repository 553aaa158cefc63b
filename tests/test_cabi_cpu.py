"""CPU-only checks of the C ABI: the library loads, exports every symbol the header declares,
and the parts that need no GPU (planner, half conversion, argument checks) behave."""
import ctypes
import os
import re

import numpy as np
import pytest

from decx_amd import hip

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    names = set()
    for fn in os.listdir(os.path.join(ROOT, "include")):
        if fn.endswith(".h"):
            text = open(os.path.join(ROOT, "include", fn)).read()
            names.update(re.findall(r"DECX_HIP_API\s+[\w\s\*]+?\b(decx_hip_\w+)\s*\(", text))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 25
    raw = ctypes.CDLL(hip.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "libdecx_hip.so does not export " + n
    assert set(names) == set(hip.SYMBOLS), "ctypes table and header disagree"
    hip.lib()


def test_half_conversion_matches_ieee_rne():
    L = hip.lib()
    h = np.arange(65536, dtype=np.uint16)
    want = h.view(np.float16).astype(np.float32)
    got = np.array([L.decx_hip_half_to_float(int(v)) for v in h], np.float32)
    ok = ~np.isnan(want)
    assert np.array_equal(np.isnan(got), ~ok)
    assert np.array_equal(got[ok].view(np.uint32), want[ok].view(np.uint32))
    rng = np.random.default_rng(3)
    vals = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 5,
                           (rng.standard_normal(4000) * 1e-6).astype(np.float32),
                           (rng.standard_normal(2000) * 4e4).astype(np.float32),
                           np.array([0.0, -0.0, 65504, 65519.99, 65520, 65536, 1e30, -1e30, 2.0 ** -24, 2.0 ** -25,
                                     np.nextafter(np.float32(2.0 ** -25), np.float32(1)), 2.0 ** -14,
                                     np.inf, -np.inf], np.float32)])
    hh = np.arange(0x0001, 0x7bff, 37, dtype=np.uint16).view(np.float16).astype(np.float32)
    vals = np.concatenate([vals, (hh[:-1] + hh[1:]) / np.float32(2)])           # ties and near-ties
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([L.decx_hip_float_to_half(float(v)) for v in vals], np.uint16)
    assert np.array_equal(got, want)


def test_planner_choices():
    # headline shapes take the big tile, the unpredicated variant
    for eb, (M, N, K) in [(4, (8192, 8192, 8192)), (2, (4096, 4096, 4096)), (4, (65536, 256, 1024))]:
        p = hip.plan(eb, M, N, K)
        # the largest tile: 256 x 128 in fp32 (two workgroups per CU), 256 x 256 in fp16
        assert (p.path, p.edge, p.tile_m, p.tile_n) == (hip.TILE_LARGE, 0, 256, 128 if eb == 4 else 256)
        assert p.grid == (M // p.tile_m) * (N // p.tile_n)
    assert hip.plan(4, 8192, 8192, 8192, aligned=False).tile_n == 256     # the register-staged family keeps 256 x 256
    # small and ragged problems take smaller tiles so the chip fills; they stay on the direct-to-LDS
    # kernels as long as the operands are 16-byte aligned
    p = hip.plan(4, 1000, 1500, 777)
    # 384 tiles of 64 x 64 are 1.5 per CU: with a workspace every CU gets one tile whole and one half of another
    # (256 whole + 128 on two ranges of K: 23.5 us; all 384 on two ranges 25.6, the whole product 28.2)
    assert p.edge == 0 and p.tile_m == 64 and (p.k_splits, p.whole_tiles, p.grid) == (2, 256, 256 + 2 * 128)
    assert hip.plan(4, 1024, 1024, 1024).k_splits == 1 and hip.plan(4, 2048, 2048, 2048).k_splits == 1
    assert hip.plan(4, 1000, 1500, 777, aligned=False).edge == 1
    assert hip.plan(2, 1000, 1500, 777).edge == 0 and hip.plan(2, 1000, 1500, 777).tile_m == 64
    assert hip.plan(2, 2048, 2048, 2048).tile_m == 128 and hip.plan(2, 1000, 1500, 777, aligned=False).edge == 1
    assert hip.plan(4, 1024, 1024, 1024).tile_m == 64
    assert hip.plan(4, 2048, 2048, 2048).tile_m == 128     # 256 tiles of 128 x 128, one per CU: 121.5 us (1024 small ones, four per CU: 122.9)
    assert hip.plan(4, 6144, 6144, 6144).tile_m == 128
    assert hip.plan(4, 3000, 3000, 3000).tile_m == 64
    assert hip.plan(4, 1024, 1024, 1024, aligned=False).edge == 1
    # N == 1 goes to the row-dot kernel and M == 1 to the column-sum kernel, in both element types
    for eb in (4, 2):
        p = hip.plan(eb, 8192, 1, 8192)
        assert (p.path, p.grid) == (hip.PATH_GEMV, 8192 // 32)
        p = hip.plan(eb, 1, 8192, 8192)
        assert (p.path, p.grid) == (hip.PATH_GEVM, 256)    # 128-byte column groups in fp32, 64-byte ones in fp16: 256 either way
    assert hip.plan(2, 1, 32768, 64).tile_n == 64 and hip.plan(4, 1, 4096, 64).tile_n == 16
    assert hip.plan(4, 0, 5, 5).grid == 0
    # few tiles and a long K: the plan reports the split a workspace makes possible
    p = hip.plan(4, 300, 300, 8192)
    assert p.k_splits > 1 and p.grid == 25 * p.k_splits and hip.plan(4, 8192, 8192, 8192).k_splits == 1
    assert hip.plan(4, 300, 300, 400).k_splits == 1 and hip.plan(2, 256, 256, 65536).k_splits > 1
    # a few hundred tiles that do not divide among 256 CUs and a long K: even rounds of workgroups on the small tile
    p = hip.plan(4, 1280, 1024, 8192)                      # 320 tiles of 64 x 64: a whole one per CU and 64 on 4 ranges, one of those per CU
    assert (p.tile_m, p.k_splits, p.whole_tiles, p.grid) == (64, 4, 256, 256 + 64 * 4)     # 150 us; all on 8 ranges 163, whole 239
    p = hip.plan(4, 1536, 1024, 8192)                      # 384 tiles on 2 ranges: three per CU
    assert (p.tile_m, p.k_splits) == (64, 2)
    assert hip.plan(4, 2048, 2048, 8192).k_splits == 1
    p = hip.plan(4, 1280, 1024, 2048)                      # 1.25 tiles per CU: whole 65.6 us, all on 3 ranges 47.1, 256 whole + 64 on 4 ranges 44.4
    assert (p.k_splits, p.whole_tiles) == (4, 256)
    p = hip.plan(4, 1536, 1536, 1536)                      # 2.25 per CU: two whole and a quarter (62.0 -> 55.1 us)
    assert (p.k_splits, p.whole_tiles, p.grid) == (4, 512, 512 + 64 * 4)
    assert hip.plan(4, 1536, 1280, 1024).k_splits == 1     # 480 tiles: the 224 beyond one per CU do not fit beside them on two ranges
    p = hip.plan(2, 1536, 1024, 8192)                      # fp16: 96 tiles of 128 x 128 on 2 ranges
    assert (p.tile_m, p.k_splits) == (128, 2)
    p = hip.plan(2, 1024, 1024, 6144)                      # 64 tiles of 128 x 128 on 4 ranges, one per CU: 29.6 -> 23.5 us
    assert (p.tile_m, p.k_splits) == (128, 4)
    assert hip.plan(2, 768, 768, 16384).k_splits == 6 and hip.plan(2, 2048, 2048, 8192).k_splits == 1
    assert hip.plan(2, 4096, 512, 2048).k_splits == 1 and hip.plan(2, 896, 896, 4096).k_splits == 1    # on ranges: 20.7 and 18.3 us, whole 14.1 and 14.7
    p = hip.plan(2, 2560, 2048, 4096)                      # 320 tiles of 128 x 128: 256 whole + 64 on 4 ranges (52.5 us; all on 3 ranges 57.4)
    assert (p.tile_m, p.k_splits, p.whole_tiles) == (128, 4, 256)
    assert hip.plan(2, 3072, 2048, 8192).k_splits == 1     # 1.5 per CU, power-bound either way: whole 100.9 us, 4 ranges 115.3
    assert hip.plan(2, 2560, 2048, 2048).k_splits == 1 and hip.plan(2, 2560, 2048, 8192).whole_tiles == 0
    p = hip.plan(2, 300, 300, 8192)                        # few tiles: 8 ranges on 64 x 64 (12.9 us; the 20 that two
    assert (p.tile_m, p.k_splits) == (64, 8)               # workgroups per CU would ask for: 17.8, the whole product 38.8)
    # more tiles than the chip holds at once: the full rounds stay whole, only the ragged last round is split
    p = hip.plan(4, 2112, 2112, 2112)                      # 1089 tiles: 1024 whole, 65 on 7 ranges each (161.5 -> 143.7 us)
    assert (p.tile_m, p.k_splits, p.whole_tiles, p.grid) == (64, 7, 1024, 1024 + 65 * 7)
    p = hip.plan(8, 1536, 1536, 1536)                      # fp64, two workgroups per CU: 512 whole + 64 x 4 (146 -> 112 us)
    assert (p.tile_m, p.k_splits, p.whole_tiles, p.grid) == (64, 4, 512, 512 + 64 * 4)
    assert hip.plan(4, 2048, 2048, 2048).whole_tiles == 0 and hip.plan(4, 640, 640, 8192).whole_tiles == 0
    p = hip.plan(8, 1280, 1024, 2048)                      # fp64: 320 tiles of 64 x 64, 256 whole + 64 on 4 ranges (whole 128.5 us, all on 4 ranges 87.1, this 77.3)
    assert (p.tile_m, p.k_splits, p.whole_tiles) == (64, 4, 256)
    p = hip.plan(8, 1000, 1500, 777)                       # 48.2 -> 39.4 us
    assert (p.tile_m, p.k_splits, p.whole_tiles) == (64, 2, 256)
    p = hip.plan(8, 1280, 1024, 8192)
    assert p.tile_m == 64 and p.k_splits > 1 and hip.plan(8, 4096, 4096, 4096).k_splits == 1
    # the vector corners: rows per workgroup of the row-dot kernel, ranges of K for few columns, fp64 on the same kernels
    assert [hip.plan(4, M, 1, 4096).tile_m for M in (9000, 5000, 3000, 1500, 600, 100)] == [32, 16, 8, 4, 2, 1]
    p = hip.plan(4, 1, 512, 32768)
    assert (p.path, p.tile_n) == (hip.PATH_GEVM, 32) and p.k_splits > 1 and p.grid == 16 * p.k_splits
    assert hip.plan(4, 1, 512, 8192).k_splits == 1 and hip.plan(4, 1, 8192, 8192).k_splits == 1
    assert hip.plan(2, 1, 8192, 8192).k_splits == 2        # 128 groups of whole cache lines, two ranges: a workgroup per CU
    assert hip.plan(8, 8192, 1, 8192).path == hip.PATH_GEMV and hip.plan(8, 1, 8192, 8192).path == hip.PATH_GEVM
    assert hip.plan(8, 1, 8192, 8192).tile_n == 16
    bad = hip.Plan()
    assert hip.lib().decx_hip_gemm_plan(3, 4, 4, 4, 1, ctypes.byref(bad)) == -1


def test_compute_entry_points_refuse_to_run_uninitialised():
    """Fresh process, no decx_hip_init: every GPU entry point reports NOT_INIT (-2) instead of
    touching the device or falling back to anything."""
    import subprocess
    import sys
    code = (
        "import sys, ctypes; sys.path.insert(0, %r); from decx_amd import hip; L = hip.lib();"
        "p = ctypes.c_void_p(16); q = ctypes.c_void_p();"
        "assert L.decx_hip_gemm_f32(p, p, None, p, 4, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None) == -2;"
        "assert L.decx_hip_gemm_f16(p, p, None, p, 4, 4, 4, 4, 4, 0, 4, 1.0, 1.0, None) == -2;"
        "assert L.decx_hip_gemv_f32(p, p, None, p, 4, 4, 4, 1, 1, 1, 1.0, 1.0, None) == -2;"
        "assert L.decx_hip_gevm_f32(p, p, None, p, 4, 4, 4, 1, 1, 1, 1.0, 1.0, None) == -2;"
        "assert L.decx_hip_gemv_f16(p, p, None, p, 4, 4, 4, 1, 1, 1, 1.0, 1.0, 1, None) == -2;"
        "assert L.decx_hip_gevm_f16(p, p, None, p, 4, 4, 4, 1, 1, 1, 1.0, 1.0, 0, None) == -2;"
        "assert L.decx_hip_malloc(ctypes.byref(q), 64) == -2;"
        "assert L.decx_hip_stream_create(ctypes.byref(q)) == -2;"
        "assert b'init' in L.decx_hip_error_string(-2)" % ROOT)
    subprocess.run([sys.executable, "-c", code], check=True, timeout=120)


def test_missing_library_is_an_error_not_a_fallback():
    """Without the built HIP library the Python layer raises; there is no CPU path behind it."""
    import subprocess
    import sys
    code = ("from decx_amd import hip\n"
            "hip.LIB_PATH = '/nonexistent/libdecx_hip.so'\n"
            "try:\n"
            "    hip.lib()\n"
            "except hip.HipError as e:\n"
            "    assert 'native library missing' in str(e); print('raised')\n")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=root, timeout=120)
    assert out.returncode == 0 and out.stdout.strip() == "raised", out.stderr


def test_error_strings():
    L = hip.lib()
    assert L.decx_hip_error_string(0) == b"success"
    assert b"invalid argument" in L.decx_hip_error_string(-1)
    assert L.decx_hip_error_string(-99) == b"unknown error"


def test_device_pass_applies_the_no_packed_fp32_switch(tmp_path):
    """The build's feature switch keeps packed-fp32 VALU forms out of gfx950 code: the same float2 multiply-add
    compiles to v_pk_fma_f32 without it and to scalar fmas with it (the host pass, which warns that it does not know
    the feature, is not what is compiled here)."""
    import subprocess
    from decx_amd import build
    src = tmp_path / "pk.hip"
    src.write_text("#include <hip/hip_runtime.h>\n"
                   "__global__ void k(float2* a, const float2* b, const float2* c) { const int i = threadIdx.x;\n"
                   "  const float2 x = b[i], y = c[i], z = a[i]; a[i] = make_float2(x.x * y.x + z.x, x.y * y.y + z.y); }\n")
    def asm(flags):
        out = tmp_path / "pk.s"
        subprocess.run([build.HIPCC, "--offload-arch=gfx950", "-O3", "--cuda-device-only", "-S", str(src), "-o", str(out)] + flags,
                       check=True, capture_output=True)
        return out.read_text()
    switch = [f for f in build.HIP_FLAGS if f in ("-Xclang", "-target-feature", "-packed-fp32-ops")]
    assert switch == ["-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]
    assert "v_pk_fma_f32" in asm([])
    with_switch = asm(switch)
    assert "v_pk_" not in with_switch and "v_fma_f32" in with_switch
