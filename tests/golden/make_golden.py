"""Writes the golden fixtures in this directory.  Run in the build container:

    python tests/golden/make_golden.py

`ref_f32_*.npz` / `ref_f64_*.npz` hold outputs of the *reference's own* CPU GEMM (de::blas::cpu::GEMM,
compiled from the mounted reference tree by oracle/build_ref.sh) at shapes and thread
counts inside the envelope where it is correct; the inputs are regenerated from the seeds
stored beside them (fp16 fixtures store their inputs, which pass through libm).  `orc_*.npz` hold outputs the reference cannot produce (fp16, the
alpha/beta form, ragged shapes it gets wrong); those come from the CPU oracle and are
regression anchors, not reference outputs.
"""
import os
import sys
import zlib

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from decx_amd import synth          # noqa: E402
from oracle import binding as orc   # noqa: E402

REF_CASES = [  # (M, N, K, threads)
    (64, 64, 64, 1),
    (96, 80, 72, 4),      # wrong at 1 and 2 threads
    (128, 64, 96, 2),
    (200, 112, 136, 4),   # (200, 120, 136) is outside the envelope: the reference gets it wrong at every thread count
]
REF64_CASES = [  # (M, N, K, threads, with_C): the reference's double-precision CPU GEMM, correct also with C
    (64, 64, 64, 1, False),
    (96, 80, 72, 4, True),
    (100, 150, 77, 4, False),
    (200, 112, 136, 4, True),
]
REFC32_CASES = [  # (M, N, K, threads): the reference's single-precision complex CPU GEMM (compared with a tolerance:
    (64, 64, 64, 1),   #  its blocked complex arithmetic rounds in another order than the oracle's chain)
    (96, 80, 72, 4),
]
ORC_F32 = [  # (M, N, K, with_C, alpha, beta)   alpha None => chain seeded with C
    (37, 53, 29, False, None, None),
    (37, 53, 29, True, None, None),
    (100, 150, 77, False, None, None),
    (100, 150, 77, True, 1.0, 1.0),
    (65, 130, 67, True, -0.75, 2.5),
]
ORC_F16 = [
    (64, 64, 64, False, 1.0, 1.0),
    (45, 70, 83, False, 1.0, 1.0),
    (45, 70, 83, True, 1.5, -0.5),
]


def crc(a):
    return zlib.crc32(np.ascontiguousarray(a).tobytes()) & 0xFFFFFFFF


def main():
    if not orc.reference_available():
        sys.exit("compiled reference missing: run oracle/build_ref.sh first")
    for idx, (M, N, K, T) in enumerate(REF_CASES):
        sa, sb = 0x6000 + idx, 0x7000 + idx
        A = synth.uniform_f32(M, K, sa)
        B = synth.uniform_f32(K, N, sb)
        D, err = orc.reference_cpu_gemm_f32(A, B, None, threads=T)
        assert err == 0
        np.savez(os.path.join(HERE, f"ref_f32_{M}x{N}x{K}.npz"), M=M, N=N, K=K, threads=T,
                 seed_a=sa, seed_b=sb, D=D, crc=crc(D))
    for idx, (M, N, K, T, with_c) in enumerate(REF64_CASES):
        sa, sb, sc = 0x6400 + idx, 0x7400 + idx, 0x8400 + idx
        A = synth.uniform_f64(M, K, sa)
        B = synth.uniform_f64(K, N, sb)
        C = synth.uniform_f64(M, N, sc) if with_c else None
        D, err = orc.reference_cpu_gemm_f64(A, B, C, threads=T)
        assert err == 0
        np.savez(os.path.join(HERE, f"ref_f64_{'abc' if with_c else 'ab'}_{M}x{N}x{K}.npz"), M=M, N=N, K=K, threads=T,
                 with_c=with_c, seed_a=sa, seed_b=sb, seed_c=sc, D=D, crc=crc(D))
    for idx, (M, N, K, T) in enumerate(REFC32_CASES):
        sa, sb = 0x6500 + idx, 0x7500 + idx
        A = synth.uniform_f32(M, 2 * K, sa).view(np.complex64)
        B = synth.uniform_f32(K, 2 * N, sb).view(np.complex64)
        D, err = orc.reference_cpu_gemm_c32(A, B, None, threads=T)
        assert err == 0
        np.savez(os.path.join(HERE, f"ref_c32_{M}x{N}x{K}.npz"), M=M, N=N, K=K, threads=T, seed_a=sa, seed_b=sb, D=D, crc=crc(D))
    for idx, (M, N, K, with_c, alpha, beta) in enumerate(ORC_F32):
        sa, sb, sc = 0x6100 + idx, 0x7100 + idx, 0x8100 + idx
        A = synth.uniform_f32(M, K, sa)
        B = synth.uniform_f32(K, N, sb)
        C = synth.uniform_f32(M, N, sc) if with_c else None
        D = orc.gemm_f32(A, B, C, alpha, beta)
        tag = "ab" if not with_c else ("abc" if alpha is None else "axpby")
        np.savez(os.path.join(HERE, f"orc_f32_{tag}_{M}x{N}x{K}.npz"), M=M, N=N, K=K, with_c=with_c,
                 alpha=np.float32(np.nan if alpha is None else alpha),
                 beta=np.float32(np.nan if beta is None else beta),
                 seed_a=sa, seed_b=sb, seed_c=sc, D=D, crc=crc(D))
    for idx, (M, N, K, with_c, alpha, beta) in enumerate(ORC_F16):
        sa, sb, sc = 0x6200 + idx, 0x7200 + idx, 0x8200 + idx
        A = synth.normal_half(M, K, sa)
        B = synth.normal_half(K, N, sb)
        C = synth.normal_half(M, N, sc) if with_c else None
        D = orc.gemm_f16(A, B, C, alpha, beta)
        tag = "axpby" if with_c else "ab"
        np.savez(os.path.join(HERE, f"orc_f16_{tag}_{M}x{N}x{K}.npz"), M=M, N=N, K=K, with_c=with_c,
                 alpha=np.float32(alpha), beta=np.float32(beta),
                 A=A.view(np.uint16), B=B.view(np.uint16),
                 C=(C.view(np.uint16) if with_c else np.zeros((0, 0), np.uint16)),
                 D=D.view(np.uint16), crc=crc(D))
    print("golden fixtures written to", HERE)


if __name__ == "__main__":
    main()
