"""Register budgets the schedules rely on (CPU only: hipcc's own resource report for gfx950, nothing runs).

How many workgroups share a CU is part of every kernel's design here -- two independent 256 x 128 fp32 workgroups take
turns on the matrix pipe, four 64 x 64 ones hide each other's latencies, two 1024-thread vector workgroups fit a CU --
and a change in an epilogue can take it away without any test of results noticing.  A SIMD has 512 registers per lane
(vector and accumulation registers together); the figure checked is the compiler's own."""
import os
import re
import subprocess

import pytest

from decx_amd import build

CSRC = os.path.join(os.path.dirname(os.path.abspath(build.__file__)), "csrc")


def resource_report(source, tmp_path):
    """{mangled kernel name: (wavefronts per SIMD its registers allow, scratch bytes per lane)}, as the compiler reports them"""
    done = subprocess.run([build.HIPCC] + build.HIP_FLAGS + ["--cuda-device-only", "-c", os.path.join(CSRC, source), "-o",
                           str(tmp_path / "k.o"), "-Rpass-analysis=kernel-resource-usage"], capture_output=True, text=True)
    assert done.returncode == 0, done.stderr[-2000:]
    out = {}
    name = None
    for line in done.stderr.splitlines():
        m = re.search(r"Function Name: (\S+)", line)
        if m:
            name = m.group(1)
            out[name] = [0, 0]
            continue
        for i, key in enumerate(("Occupancy [waves/SIMD]: ", "ScratchSize [bytes/lane]: ")):
            if name and key in line:
                out[name][i] = int(line.split(key)[1].split()[0])
    return {k: tuple(v) for k, v in out.items()}


def find(report, *parts):
    hits = [k for k in report if all(p in k for p in parts)]
    assert len(hits) == 1, (parts, hits)
    return report[hits[0]]


@pytest.mark.timeout(600)
def test_fp32_kernels_keep_their_workgroups_per_cu(tmp_path):
    r = resource_report("gemm_f32_dma.hip", tmp_path)
    for k, (waves, scratch) in r.items():
        assert scratch == 0, (k, "spills")
    # 256 x 128, 4 wavefronts: two workgroups per CU = 2 wavefronts per SIMD
    waves, _ = find(r, "gemm_f32_dma_kernelILi256ELi128ELi2ELi2ELi16ELi2ELb0ELi0ELb0ELb0E")
    assert waves >= 2
    # 128 x 128: three per CU (compiled for that; four fit)
    waves, _ = find(r, "gemm_f32_dma_kernelILi128ELi128ELi2ELi2ELi16ELi2ELb1ELi0ELb0ELb0E")
    assert waves >= 3
    # 64 x 64 whole and on ranges of K (with and without C loaded early): four per CU
    for tail in ("Lb0ELb0E", "Lb1ELb0E", "Lb1ELb1E"):
        waves, _ = find(r, "gemm_f32_dma_kernelILi64ELi64ELi2ELi2ELi32ELi2ELb1ELi0E" + tail)
        assert waves >= 4, tail


@pytest.mark.timeout(600)
def test_fp16_and_fp64_kernels_keep_their_workgroups_per_cu(tmp_path):
    r = resource_report("gemm_f16_dma.hip", tmp_path)
    for k, (waves, scratch) in r.items():
        assert scratch == 0, (k, "spills")
    for split in (0, 1):                                                                # 8 wavefronts, one workgroup per CU; whole and
        waves, _ = find(r, "gemm_f16_dma_kernelILi256ELi256ELi2ELi4ELi64ELi2ELb%dE" % split)   # on ranges of K (the last round's tiles)
        assert waves >= 2, split
    for shape in ("Li192ELi192ELi4ELi2E", "Li192ELi256ELi2ELi4E", "Li256ELi192ELi4ELi2E"):    # the tiles of 192 rows or columns: the same
        waves, _ = find(r, "gemm_f16_dma_kernelI" + shape + "Li64ELi2ELb0E")
        assert waves >= 2, shape
    # (the compiler's figure counts LDS in: the rings of 4 stages are those of workgroups that have a CU to themselves)
    for stages, want in ((2, 4), (4, 2)):                                               # 128 x 128, 8 wavefronts: two per CU / one
        for split in (0, 1):
            waves, _ = find(r, "gemm_f16_dma_kernelILi128ELi128ELi2ELi4ELi64ELi%dELb%dE" % (stages, split))
            assert waves >= want, (stages, split)
    for stages, want in ((2, 4), (4, 2)):                                               # 64 x 64, 4 wavefronts: four per CU / two
        for split in (0, 1):
            waves, _ = find(r, "gemm_f16_dma_kernelILi64ELi64ELi2ELi2ELi64ELi%dELb%dE" % (stages, split))
            assert waves >= want, (stages, split)
    r = resource_report("gemm_f64.hip", tmp_path)
    for k, (waves, scratch) in r.items():
        assert scratch == 0, (k, "spills")
    waves, _ = find(r, "gemm_f64_dma_kernelILi256ELi128ELi4ELi2ELi16ELi3ELb0E")          # 8 wavefronts, one workgroup per CU
    assert waves >= 2
    for split in (0, 1):                                                                # 64 x 64, 8 wavefronts: two per CU
        waves, _ = find(r, "gemm_f64_dma_kernelILi64ELi64ELi4ELi2ELi16ELi4ELb%dE" % split)
        assert waves >= 4, split


@pytest.mark.timeout(600)
def test_vector_kernels_fit_two_workgroups_of_1024_threads_per_cu(tmp_path):
    r = resource_report("gemv.hip", tmp_path)
    checked = 0
    for k, (waves, scratch) in r.items():
        if "gemv_kernel" in k or "gevm_kernel" in k:
            assert scratch == 0 and waves >= 8, (k, waves, scratch)       # 2 x 16 wavefronts on 4 SIMDs
            checked += 1
    assert checked >= 30
