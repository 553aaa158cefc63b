// fp16 GEMM, the full-tile fast path for gfx950: 256 x 256 block tile, global -> LDS by
// direct (LDS-DMA) 128-bit loads, B fragments by the transposing LDS read, and a hand-ordered
// instruction stream in which every MFMA is followed by the LDS reads / direct loads that
// should issue in its shadow.
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
//   A slab  [256 rows][CPR chunks]  chunk c of row r sits in slot c ^ ((r / RPB) % CPR)
//   B slab  [BK k-rows][32 chunks]  chunk c of row k sits in slot c ^ (4 * (k & 3))
// With these, 16 lanes reading one k-chunk of 16 consecutive A rows, and 32 lanes reading
// four k-rows of B through the transposing read, each touch every bank exactly once.
//
// The MFMA is issued with its operands swapped (B fragment first): it then produces the
// transposed 32x32 tile, in which a lane owns 4 *adjacent columns* of one output row per
// register group, so the epilogue stores 8 bytes per lane instead of 2.
//
// Pipeline.  STAGES LDS stages of one K slab each.  The k-steps of all slabs form one
// sequence of phases; phase p issues the 16 MFMAs of k-step p and, interleaved behind
// them, the 12 fragment reads of k-step p+1 (two register sets) and 4 direct loads.  A
// stage is free as soon as the fragments of its last k-step are in registers, so slab
// s + STAGES is fetched from the last phase of slab s on; one wait + barrier per slab,
// placed before that last phase.  Three things are taken out of the compiler's hands:
// the direct loads are inline assembly (otherwise it puts `s_waitcnt vmcnt(0)` in front of
// every LDS read that follows one, because it cannot prove the stages do not alias); the
// barrier is a bare `s_barrier` with an explicit vmcnt wait (__syncthreads() drains all
// loads); and `sched_group_barrier` pins the MFMA / LDS-read interleave (left alone it
// issues all reads of a k-step in a clump in front of the MFMAs).
#include "gemm_common.hpp"
#include <type_traits>

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

#define DECX_DMA16(lds_dst, gptr) \
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(lds_dst), "v"(gptr) : "memory", "m0")

// Waits until at most N of this wave's direct loads are in flight and all its LDS reads have
// returned, then joins the workgroup barrier.  Not __syncthreads(): that carries a fence
// which drains every outstanding load and would undo the prefetch.
template <int N> __device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(N) : "memory");
}

// scheduling-group masks of __builtin_amdgcn_sched_group_barrier
constexpr int SG_MFMA = 0x008, SG_DS_READ = 0x100;

}  // namespace

// BK: slab depth (32 or 64).  STAGES: LDS stages.
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
    constexpr int KS = BK / 16;                      // MFMA k-steps (= phases) per slab
    constexpr int DMA_PER_PHASE = LOADS / KS;        // 4
    static_assert(STAGES >= 2 && STAGES * STAGE_BYTES <= 160 * 1024, "LDS budget");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
    static_assert(KS % 2 == 0 && DMA_PER_PHASE == 4 && A_LOADS % DMA_PER_PHASE == 0, "phase plan");

    __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE_BYTES];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)lds;

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

    // One direct load: index q in [0, LOADS) of slab `slab` (A instructions first).
    auto dma = [&](uint32_t slab, auto qc) {
        constexpr int q = decltype(qc)::value;
        const uint32_t stage_off = lds_base + (slab % STAGES) * STAGE_BYTES;
        if constexpr (q < A_LOADS) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(stage_off + (uint32_t)(wave * A_LOADS + q) * 1024u);
            const unsigned char* src = a_src[q] + (size_t)slab * (BK * 2);
            DECX_DMA16(dst, src);
        } else {
            constexpr int qb = q - A_LOADS;
            const uint32_t dst = __builtin_amdgcn_readfirstlane(stage_off + A_STAGE_BYTES +
                                                                (uint32_t)(wave * B_LOADS + qb) * 1024u);
            const unsigned char* src = b_src[qb] + (size_t)slab * BK * ldb_b;
            DECX_DMA16(dst, src);
        }
    };
    auto dma_batch = [&](uint32_t slab, auto bc) {       // batch b of KS: loads 4b .. 4b+3
        constexpr int b = decltype(bc)::value;
        dma(slab, std::integral_constant<int, 4 * b + 0>{});
        dma(slab, std::integral_constant<int, 4 * b + 1>{});
        dma(slab, std::integral_constant<int, 4 * b + 2>{});
        dma(slab, std::integral_constant<int, 4 * b + 3>{});
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
    int b_off[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        const int col = b_col + 32 * j;
        b_off[j] = A_STAGE_BYTES + b_krow * 512 + (((col >> 3) ^ b_sw) * 16) + (col & 7) * 2;
    }

    struct Frags { halfx8 a[4], b[4]; };

    auto read_a = [&](Frags& f, const unsigned char* st, int ks, int i) {
        f.a[i] = *(const halfx8*)(st + a_off + i * 32 * RB + (((2 * ks + h) ^ a_sw) * 16));
    };
    auto read_b = [&](Frags& f, const unsigned char* st, int ks, int j) {
        const unsigned char* p0 = st + b_off[j] + ks * 16 * 512;
        const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)p0);
        const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(p0 + 4 * 512));
        f.b[j] = join(lo, hi);
    };

    // accT[j][i]: n-tile j, m-tile i, held transposed (see the file header)
    floatx16 accT[4][4];
#pragma unroll
    for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int r = 0; r < 16; ++r) accT[j][i][r] = 0.f;

    auto mfma4 = [&](const Frags& cur, int j) {           // the 4 MFMAs of n-tile j
#pragma unroll
        for (int i = 0; i < 4; ++i)
            accT[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(cur.b[j], cur.a[i], accT[j][i], 0, 0, 0);
    };

    // One phase: the 16 MFMAs of the current k-step, the 12 fragment reads of the next
    // k-step (8 LDS instructions for B, 4 for A) spread behind them, and -- if `dma_ok` --
    // one direct load in front of each quarter.  Source order = intended issue order; the
    // group barriers make the scheduler keep the "one MFMA, one LDS read" alternation.
    // Only the direct loads are conditional (tiny uniform branches): the arithmetic is
    // never duplicated, so the 256 accumulators stay put.
    auto quarter = [&](bool dma_ok, uint32_t dma_slab, auto qc) {
        if (dma_ok) dma(dma_slab, qc);
    };
    auto phase = [&](const Frags& cur, Frags& nxt, const unsigned char* nst, int nks,
                     bool dma_ok, uint32_t dma_slab, auto dbc) {
        constexpr int db = decltype(dbc)::value;
        quarter(dma_ok, dma_slab, std::integral_constant<int, 4 * db + 0>{});
        read_b(nxt, nst, nks, 0); read_a(nxt, nst, nks, 0);
        mfma4(cur, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        quarter(dma_ok, dma_slab, std::integral_constant<int, 4 * db + 1>{});
        read_a(nxt, nst, nks, 1); read_a(nxt, nst, nks, 2); read_a(nxt, nst, nks, 3);
        mfma4(cur, 1);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        quarter(dma_ok, dma_slab, std::integral_constant<int, 4 * db + 2>{});
        read_b(nxt, nst, nks, 1); read_b(nxt, nst, nks, 2);
        mfma4(cur, 2);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        quarter(dma_ok, dma_slab, std::integral_constant<int, 4 * db + 3>{});
        read_b(nxt, nst, nks, 3);
        mfma4(cur, 3);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 2, 0);
    };
    auto I0 = std::integral_constant<int, 0>{};

    const uint32_t slabs = g.K / BK;

    // ---- prologue: slabs 0 .. STAGES-2 entirely, plus the first batch of slab STAGES-1
    // (its other batches are issued by phases 0 .. KS-2 of slab 0).
#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p) {
        if ((uint32_t)p < slabs) {
            dma_batch(p, std::integral_constant<int, 0>{});
            dma_batch(p, std::integral_constant<int, 1>{});
            if constexpr (KS == 4) {
                dma_batch(p, std::integral_constant<int, 2>{});
                dma_batch(p, std::integral_constant<int, 3>{});
            }
        }
    }
    if ((uint32_t)(STAGES - 1) < slabs) dma_batch(STAGES - 1, std::integral_constant<int, 0>{});
    wait_loads_and_barrier<0>();

    Frags f0, f1;
#pragma unroll
    for (int q = 0; q < 4; ++q) { read_a(f0, lds, 0, q); read_b(f0, lds, 0, q); }

    for (uint32_t s = 0; s < slabs; ++s) {
        const unsigned char* st = lds + (s % STAGES) * STAGE_BYTES;
        const unsigned char* st_next = lds + ((s + 1) % STAGES) * STAGE_BYTES;
        const bool dma_mid = s + STAGES - 1 < slabs;          // slab s+STAGES-1 exists (its batches 1..KS-1)
        const bool dma_last = s + STAGES < slabs;             // slab s+STAGES exists (its batch 0)

        // phases 0 .. KS-2: fetch k-step ks+1 of this slab
        phase(f0, f1, st, 1, dma_mid, s + STAGES - 1, std::integral_constant<int, 1>{});
        if constexpr (KS == 4) {
            phase(f1, f0, st, 2, dma_mid, s + STAGES - 1, std::integral_constant<int, 2>{});
            phase(f0, f1, st, 3, dma_mid, s + STAGES - 1, std::integral_constant<int, 3>{});
        }

        // Last phase of the slab.  Its fragments are in registers (lgkmcnt(0) in the wait), so
        // every wave is done with this stage; slab s+1 must have landed: ours by vmcnt,
        // everyone's by the barrier.  Loads of the STAGES-2 slabs behind it may stay in flight.
        // It fetches k-step 0 of the next slab; after the final slab that read returns stale
        // LDS contents which nothing uses.
        if (dma_mid) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
        phase(f1, f0, st_next, 0, dma_last, s + STAGES, I0);
    }

    // Epilogue.  Transposed tile layout: lane (l32, h) holds output row l32 of the m-tile;
    // register 4 q + e is column 8 q + 4 h + e of the n-tile, so the two half-waves hold the
    // two 4-column halves of every 8-column group of a row.  `v_permlane32_swap` trades the
    // halves of an even and an odd group between lane l and lane l + 32; after it the lower
    // lane owns all 8 columns of the even group and the upper lane those of the odd group,
    // and each lane stores 16 bytes.
    const _Float16* __restrict__ C = (const _Float16*)g.C;
    _Float16* __restrict__ D = (_Float16*)g.D;
    auto pack2 = [](float lo, float hi) -> uint32_t {
        union { _Float16 f[2]; uint32_t u; } w;
        w.f[0] = (_Float16)lo; w.f[1] = (_Float16)hi;
        return w.u;
    };
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const uint32_t row = m0 + wm0 + 32 * i + l32;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int qp = 0; qp < 2; ++qp) {
                uint32_t w[2][2];                      // [even / odd group][dword]
#pragma unroll
                for (int o = 0; o < 2; ++o) {
                    const int q = 2 * qp + o;
                    float v[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = accT[j][i][4 * q + e];
                    if (C) {
                        const uint32_t col = n0 + wn0 + 32 * j + 8 * q + 4 * h;
                        const halfx4 cv = *(const halfx4*)(C + (size_t)row * g.ldc + col);
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)cv[e], g.beta, g.alpha * v[e]);
                    }
                    w[o][0] = pack2(v[0], v[1]);
                    w[o][1] = pack2(v[2], v[3]);
                }
                const auto s0 = __builtin_amdgcn_permlane32_swap(w[0][0], w[1][0], false, false);
                const auto s1 = __builtin_amdgcn_permlane32_swap(w[0][1], w[1][1], false, false);
                const uintx4 out = {s0[0], s1[0], s0[1], s1[1]};
                const uint32_t col = n0 + wn0 + 32 * j + 8 * (2 * qp + h);
                *(uintx4*)(D + (size_t)row * g.ldd + col) = out;
            }
        }
    }
}

// Full tiles only: M, N multiples of 256, K a positive multiple of 32, 16-byte aligned
// bases and pitches.  The caller checks.  32-deep slabs in a ring of 4 stages measured best
// (equal to 64 x 2 at 4096^3, 4 % faster at 8192^3; 32 x 5 is slower).
int launch_gemm_f16_pipelined(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = g.M / BM;
    g.tiles_n = g.N / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    g.xcd_remap = (nb % kXcds == 0) ? 1u : 0u;
    hipLaunchKernelGGL((gemm_f16_pipelined_kernel<32, 4>), dim3(nb), dim3(NT), 0, stream, g);
    return (int)hipGetLastError();
}

}  // namespace decx_hip
