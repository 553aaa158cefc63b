// fp16 GEMM, the full-tile fast path for gfx950: 256 x 256 block tile, K slabs of 64,
// global -> LDS by direct (LDS-DMA) 128-bit loads, B fragments by the transposing LDS read.
//
// Why this shape.  v_mfma_f32_32x32x16_f16 takes 8 consecutive k per lane for BOTH
// operands.  A (row-major M x K) has them contiguous.  B (row-major K x N) does not, and
// the reference solves that with a separate transpose pass over A for its "_T" kernels
// (srcs/common/Basic_process/transpose/CUDA/transpose_kernels.cuh:204-236).  On gfx950
// neither a pass nor a register shuffle is needed:
//   * both operand slabs are copied global -> LDS untouched by `global_load_lds_dwordx4`
//     (each lane fetches 16 bytes, the wave's 1 KB lands contiguously at a wave-uniform
//     LDS base), so the copy costs no VGPRs, no ds_write and no VALU;
//   * B fragments are read with `ds_read_b64_tr_b16`: a group of 16 lanes hands in the
//     addresses of a 4(k) x 16(n) block (lane s: row s/4, 8-byte segment s%4) and lane i
//     receives column i of it, i.e. 4 consecutive k of one n.  Two such reads give the 8 k
//     a lane needs.
// Bank conflicts are removed by permuting 16-byte chunks inside each row -- done on the
// global side of the copy, since the LDS side of a direct load is fixed:
//   A slab  [256 rows][8 chunks]   chunk c of row r sits in slot c ^ ((r >> 1) & 7)
//   B slab  [64 k-rows][32 chunks] chunk c of row k sits in slot c ^ (4 * (k & 3))
// With these, 16 lanes reading one k-chunk of 16 consecutive A rows, and 32 lanes reading
// four k-rows of B through the transposing read, each touch every bank exactly once.
//
// Pipeline: two LDS stages of 64 KB.  While slab s is multiplied, the direct loads of
// slab s+1 are in flight into the other stage; one `s_waitcnt vmcnt(0)` + barrier per
// slab.  Inside a slab the fragments of k-step i+1 are fetched while the 16 MFMAs of
// k-step i run (two register sets).  4 wavefronts, each a 128 x 128 tile = 256 accumulator
// registers; one workgroup per CU.
#include "gemm_common.hpp"
#include <cstdlib>

namespace decx_hip {

namespace {

constexpr int BM = 256, BN = 256;
constexpr int NT = 256;                              // 4 wavefronts, 2 x 2

typedef __attribute__((address_space(3))) void lds_void;
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

__device__ __forceinline__ halfx8 join(shortx4 lo, shortx4 hi)
{
    union { struct { shortx4 a, b; } s; halfx8 v; } u;
    u.s.a = lo; u.s.b = hi;
    return u.v;
}

// Waits until at most N of this wave's direct loads are still in flight, and until its LDS
// reads have returned, then joins the workgroup barrier.  Deliberately not __syncthreads():
// that carries a fence which drains every outstanding load and would undo the prefetch.
template <int N> __device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(N) : "memory");
}

}  // namespace

// BK: slab depth (32 or 64).  STAGES: LDS stages; slab s+STAGES-1 is fetched while slab s is
// multiplied, so a direct load has (STAGES-1) slabs of MFMA time to land.
template <int BK, int STAGES>
__global__ void __launch_bounds__(NT)
gemm_f16_pipelined_kernel(const GemmArgs g)
{
    constexpr int RB = BK * 2;                       // bytes of one A row in a slab
    constexpr int CPR = RB / 16;                     // 16-byte chunks per A row (8 or 4)
    constexpr int RPB = 16 / CPR;                    // A rows per 256 bytes (one sweep over the banks)
    constexpr int A_STAGE_BYTES = BM * RB;
    constexpr int B_STAGE_BYTES = BK * BN * 2;
    constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
    constexpr int A_LOADS = A_STAGE_BYTES / 1024 / 4;   // direct-load instructions per wave per slab
    constexpr int B_LOADS = B_STAGE_BYTES / 1024 / 4;
    constexpr int LOADS = A_LOADS + B_LOADS;
    constexpr int KS = BK / 16;                      // MFMA k-steps per slab
    static_assert(STAGES >= 2 && STAGES * STAGE_BYTES <= 160 * 1024, "LDS budget");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");

    __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE_BYTES];

    uint32_t tile_m, tile_n;
    block_to_tile(g, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave >> 1) * 128, wn0 = (wave & 1) * 128;
    const int l32 = lane & 31, h = lane >> 5;

    const unsigned char* __restrict__ A = (const unsigned char*)g.A;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B;
    const size_t lda_b = (size_t)g.lda * 2, ldb_b = (size_t)g.ldb * 2;

    // ---- global -> LDS copy plan.
    // A instruction I covers rows (64/CPR)*I ..: lane -> row (64/CPR)*I + lane/CPR, slot lane%CPR.
    // B instruction I covers k-rows 2I, 2I+1:    lane -> k 2I + lane/32, slot lane%32.
    // Chunk permutation (see the file header): A slot = chunk ^ ((row / RPB) % CPR),
    // B slot = chunk ^ (4 * (k & 3)).
    const unsigned char* a_src[A_LOADS];
    const unsigned char* b_src[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int I = wave * A_LOADS + i;
        const int row = (64 / CPR) * I + lane / CPR;
        const int chunk = (lane % CPR) ^ ((row / RPB) % CPR);
        a_src[i] = A + (size_t)(m0 + row) * lda_b + chunk * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int I = wave * B_LOADS + i;
        const int k = 2 * I + (lane >> 5);
        const int bchunk = (lane & 31) ^ (4 * (k & 3));
        b_src[i] = B + (size_t)k * ldb_b + (size_t)n0 * 2 + bchunk * 16;
    }

    // The direct loads are issued from inline assembly on purpose: the compiler's wait-count
    // pass cannot tell that a load into one LDS stage does not alias a read of another
    // and would put `s_waitcnt vmcnt(0)` in front of every fragment read, serialising the
    // copy with the arithmetic.  M0 carries the wave-uniform LDS destination.
    auto issue_loads = [&](uint32_t slab) {
        const uint32_t stage = slab % STAGES;
        const uint32_t sa = stage * STAGE_BYTES;
        const uint32_t sb = sa + A_STAGE_BYTES;
        const uint32_t k0 = slab * BK;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(sa + (uint32_t)(wave * A_LOADS + i) * 1024u);
            const unsigned char* src = a_src[i] + (size_t)k0 * 2;
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(dst), "v"(src) : "memory", "m0");
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(sb + (uint32_t)(wave * B_LOADS + i) * 1024u);
            const unsigned char* src = b_src[i] + (size_t)k0 * ldb_b;
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(dst), "v"(src) : "memory", "m0");
        }
    };

    // ---- fragment addressing (byte offsets inside a stage)
    // A fragment (tile i, k-step ks): row = wm0 + 32 i + l32, chunk = 2 ks + h; the row's
    // permutation key does not depend on i (32 i is a multiple of RPB * CPR = 16).
    const int a_row = wm0 + l32;
    const int a_sw = (a_row / RPB) % CPR;
    const int a_off = a_row * RB;
    // B fragment (tile j, k-step ks, half r): a 16-lane group handles the n half (lane>>4)&1;
    // lane s = lane & 15 supplies k = 16 ks + 8 h + 4 r + s/4 and the 8-byte segment s%4 of
    // the 16 columns starting at wn0 + 32 j + 16 * nhalf.
    const int s16 = lane & 15;
    const int b_krow = 8 * h + (s16 >> 2);                    // + 16 ks + 4 r
    const int b_col = wn0 + 16 * ((lane >> 4) & 1) + 4 * (s16 & 3);   // + 32 j ; in halves
    const int b_sw = 4 * (b_krow & 3);                        // k & 3 is unchanged by + 16 ks + 4 r

    auto load_frags = [&](uint32_t stage, int ks, halfx8 (&af)[4], halfx8 (&bf)[4]) {
        const unsigned char* sa = lds + stage * STAGE_BYTES;
        const unsigned char* sb = sa + A_STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < 4; ++i)
            af[i] = *(const halfx8*)(sa + a_off + i * 32 * RB + (((2 * ks + h) ^ a_sw) * 16));
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            const int col = b_col + 32 * j;                    // halves
            const int chunk = (col >> 3) ^ b_sw;
            const int within = (col & 7) * 2;                  // bytes inside the 16-byte chunk (0 or 8)
            const unsigned char* p0 = sb + (16 * ks + b_krow) * 512 + chunk * 16 + within;
            const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)p0);
            const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(p0 + 4 * 512));
            bf[j] = join(lo, hi);
        }
    };

    floatx16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    auto multiply = [&](const halfx8 (&af)[4], const halfx8 (&bf)[4]) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
    };

    // Software pipeline.  Every phase = "fetch the next fragments, then issue 16 MFMAs on
    // the current ones"; sched_barrier pins that order so the LDS latency of a fetch hides
    // behind the 512 cycles of MFMA issue of the phase before it.  The last phase of a slab
    // is multiplied after the barrier, under the first fetch of the next slab.
    const uint32_t slabs = g.K / BK;
#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if ((uint32_t)p < slabs) issue_loads(p);
    if (slabs >= (uint32_t)(STAGES - 1)) wait_loads_and_barrier<LOADS * (STAGES - 2)>();
    else wait_loads_and_barrier<0>();

    halfx8 afx[4], bfx[4], afy[4], bfy[4];
    for (uint32_t s = 0; s < slabs; ++s) {
        const uint32_t stage = s % STAGES;
        const bool more = s + STAGES - 1 < slabs;
        // the stage that held slab s-1 is free: every wave passed the barrier after reading it
        if (more) issue_loads(s + STAGES - 1);
#pragma unroll
        for (int ks = 0; ks < KS; ks += 2) {
            load_frags(stage, ks, afx, bfx);
            __builtin_amdgcn_sched_barrier(0);
            if (s > 0 || ks > 0) multiply(afy, bfy);           // the k-step before this one
            __builtin_amdgcn_sched_barrier(0);
            load_frags(stage, ks + 1, afy, bfy);
            __builtin_amdgcn_sched_barrier(0);
            multiply(afx, bfx);
            __builtin_amdgcn_sched_barrier(0);
        }
        // slab s+1 must have landed (ours: vmcnt; everyone's: barrier).  Loads of the
        // STAGES-2 slabs after it may stay in flight.
        if (more) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
    }
    multiply(afy, bfy);

    // Epilogue: register r of lane (l32, h) is row 8*(r/4) + 4*h + r%4, column l32 of a tile.
    const _Float16* __restrict__ C = (const _Float16*)g.C;
    _Float16* __restrict__ D = (_Float16*)g.D;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const uint32_t col = n0 + wn0 + 32 * j + l32;
                float o = acc[i][j][r];
                if (C) o = __builtin_fmaf((float)C[(size_t)row * g.ldc + col], g.beta, g.alpha * o);
                D[(size_t)row * g.ldd + col] = (_Float16)o;
            }
        }
    }
}

static int g_variant = -1;
void set_f16_pipelined_variant(int v) { g_variant = v; }

// Full tiles only: M, N multiples of 256, K a positive multiple of 64, 16-byte aligned
// bases and pitches.  The caller checks.
int launch_gemm_f16_pipelined(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = g.M / BM;
    g.tiles_n = g.N / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    g.xcd_remap = (nb % kXcds == 0) ? 1u : 0u;
    if (g_variant < 0) {
        const char* e = getenv("DECX_HIP_F16_VARIANT");
        g_variant = e ? atoi(e) : 0;
    }
    switch (g_variant) {
    case 1:  hipLaunchKernelGGL((gemm_f16_pipelined_kernel<32, 4>), dim3(nb), dim3(NT), 0, stream, g); break;
    case 2:  hipLaunchKernelGGL((gemm_f16_pipelined_kernel<32, 5>), dim3(nb), dim3(NT), 0, stream, g); break;
    default: hipLaunchKernelGGL((gemm_f16_pipelined_kernel<64, 2>), dim3(nb), dim3(NT), 0, stream, g); break;
    }
    return (int)hipGetLastError();
}

}  // namespace decx_hip
