// fp16 GEMM (fp32 accumulate, fp16 out) for gfx950, any M, N, K on 16-byte aligned operands:
// BM x BN block tiles whose K slabs are copied global -> LDS by direct (LDS-DMA) 128-bit
// loads into a ring of STAGES stages, ragged edges included.
//
// Replaces the reference's cu_GEMM_fp16_[F_]kernel_* family and the transpose pass in front of
// its "_T" kernels (srcs/modules/BLAS/GEMM/CUDA/large_squares/fp16/, srcs/common/Basic_process/
// transpose/CUDA/transpose_kernels.cuh:204-236).
//
// The matrix instruction is v_mfma_f32_16x16x32_f16, not the 32x32x16 form: fp16 products of this size run
// under the board's power cap, and per flop the 16x16x32 form moves a fifth less through the register file
// (half the accumulator traffic per flop).  A register-only loop on random operands sustains 1 900 TFLOP/s
// with it against 1 680 with 32x32x16; this kernel gained 12 % from the change.
//
// The instruction takes 8 consecutive k per lane for BOTH operands: lane (kg = lane / 16, l16 = lane % 16)
// supplies row / column l16 and k = 8 kg .. 8 kg + 7 of a 32-deep step.  A (row-major M x K) has them
// contiguous: A fragments are 128-bit LDS reads.  B (row-major K x N) does not; its fragments come from the
// transposing read `ds_read_b64_tr_b16` straight out of the row-major B slab: a group of 16 lanes hands in
// the addresses of a 4 (k) x 16 (n) block (lane s: row s / 4, 8-byte segment s % 4) and lane i receives
// column i of it, 4 consecutive k of one n; two such reads give the 8 k a lane needs.  So neither a
// transpose pass nor a register shuffle is needed.
// The MFMA is issued with its operands swapped (B fragment first): it then produces the transposed
// 16 x 16 tile, in which a lane owns 4 adjacent columns of one output row.  A wave turns 16 rows of its
// tile around through LDS so that it stores whole rows (WN * 2 contiguous bytes per row instead of 8).
//
// Slabs reach LDS by `global_load_lds_dwordx4` (no VGPRs, no ds_write).  These are inline assembly
// and the slab barrier is a bare `s_barrier` behind an explicit vmcnt wait, because the compiler
// would otherwise drain every outstanding load in front of each LDS read and at each
// __syncthreads(); `sched_group_barrier` pins the MFMA / LDS-read alternation.
//   * tile shapes from 256 x 256 down to 64 x 64, so small problems still cover the chip;
//   * ragged M and N without predicated loads: a copy lane whose row or column chunk lies outside
//     the matrix fetches the last valid row / chunk (mapped memory); what it brings only reaches
//     accumulators of rows / columns that are never stored;
//   * ragged K: the partial last slab goes through registers, zero-filled beyond K.
//
// LDS layout of a stage.  A: [BM rows][CPR chunks of 16 bytes], chunk c of row r in slot
// c ^ ((r / RPB) % CPR): the 16 lanes of a read phase (16 consecutive rows, one chunk) cover all banks.
// B: [BK k rows][BN / 8 chunks], chunk c of row k in slot c ^ key(k), key(k) = 4 (k & 3) ^ 2 ((k >> 3) & 1)
// for rows of 256 bytes or more and 4 ((k >> 1) & 1) ^ 2 ((k >> 3) & 1) for 128-byte rows: a half-wave
// of the transposing read takes 4 k rows x 32 bytes from each of two k groups 8 rows apart, and the 16
// pieces land in 16 different bank groups.  Both permutations are applied on the global side of the copy.
#include "gemm_common.hpp"
#include "split_k_exchange.hpp"
#include <type_traits>

namespace decx_hip {

namespace {

typedef __attribute__((address_space(3))) void lds_void;
typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) shortx4 lds_shortx4;

__device__ __forceinline__ halfx8 join(shortx4 lo, shortx4 hi)
{
    union { struct { shortx4 a, b; } s; halfx8 v; } u;
    u.s.a = lo; u.s.b = hi;
    return u.v;
}

template <int N> __device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(N) : "memory");
}

constexpr int SG_MFMA = 0x008, SG_DS_READ = 0x100;

// `mfmas` MFMAs and `reads` LDS reads, alternating one to one while both last
template <int MFMAS, int READS> __device__ __forceinline__ void interleave()
{
    constexpr int PAIRS = MFMAS < READS ? MFMAS : READS;
    static_for<0, PAIRS>([&](auto) {
        __builtin_amdgcn_sched_group_barrier(SG_MFMA, 1, 0);
        __builtin_amdgcn_sched_group_barrier(SG_DS_READ, 1, 0);
    });
    if constexpr (READS > PAIRS) __builtin_amdgcn_sched_group_barrier(SG_DS_READ, READS - PAIRS, 0);
    if constexpr (MFMAS > PAIRS) __builtin_amdgcn_sched_group_barrier(SG_MFMA, MFMAS - PAIRS, 0);
}

}  // namespace

// SPLIT: grid.y workgroups share each tile, each with its own range of K; the one that finishes last adds their fp32
// partial products and rounds once (split_k_exchange).
template <int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES, bool SPLIT = false>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
__attribute__((amdgpu_waves_per_eu((BM * BN >= 192 * 192 || STAGES > 2) ? 2 : 4)))     // as scheduled: one workgroup of 192 x 192 and up per CU, two of 128 x 128, four of 64 x 64 (rings of 2 stages)
gemm_f16_dma_kernel(const GemmArgs g_in)
{
    struct Nothing {};
    std::conditional_t<SPLIT, GemmArgs, Nothing> g_split;
    uint32_t tile_m, tile_n;
    SplitBlock sb = {0u, 0u, 1u};
    if constexpr (SPLIT) {                                 // this workgroup's tile, its share of K and its partial product
        sb = split_block(g_in, tile_m, tile_n);
        g_split = g_in;
        if (sb.splits > 1) {
            const uint32_t k0 = sb.z * g_in.split_len;
            g_split.A = (const unsigned char*)g_in.A + (size_t)k0 * 2;
            g_split.B = (const unsigned char*)g_in.B + (size_t)k0 * g_in.ldb * 2;
            g_split.K = sb.z + 1 == sb.splits ? g_in.K - k0 : g_in.split_len;     // the last range: what is left (more or less than split_len)
            if (g_in.split_urgent) __builtin_amdgcn_s_setprio(3);
        }
    } else {
        block_to_tile(g_in, tile_m, tile_n);
    }
    const GemmArgs& g = [&]() -> const GemmArgs& { if constexpr (SPLIT) return g_split; else return g_in; }();
    constexpr int WAVES = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 16, TN = WN / 16;
    constexpr int HALVES = TM >= 8 ? 2 : 1, TMH = TM / HALVES;        // the A fragments of a k step come in this many parts
    constexpr int RB = BK * 2, CPR = RB / 16, RPB = 16 / CPR;         // A row bytes, chunks per row, rows per 256 bytes
    constexpr int BRB = BN * 2, CBR = BRB / 16;                       // B row bytes, chunks per row
    constexpr int A_STAGE_BYTES = BM * RB, B_STAGE_BYTES = BK * BRB, STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
    constexpr int A_LOADS = A_STAGE_BYTES / 1024 / WAVES, B_LOADS = B_STAGE_BYTES / 1024 / WAVES, LOADS = A_LOADS + B_LOADS;
    constexpr int KS = BK / 32;                                       // MFMA k steps per slab
    constexpr int UNITS = KS * HALVES;
    static_assert(TM >= 1 && TN >= 1 && BK == 64 && UNITS % 2 == 0, "shape");
    static_assert(BN == 64 || BN == 128 || BN == 192 || BN == 256, "B row must be 128, 256, 384 or 512 bytes");
    static_assert(A_LOADS >= 1 && B_LOADS >= 1 && A_LOADS * WAVES * 1024 == A_STAGE_BYTES &&
                  B_LOADS * WAVES * 1024 == B_STAGE_BYTES, "copy plan must divide evenly");
    constexpr int LDS_BYTES = STAGES * STAGE_BYTES;
    static_assert(STAGES >= 2 && LDS_BYTES <= 160 * 1024, "LDS budget");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[LDS_BYTES];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)lds;

    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l16 = lane & 15, kg = lane >> 4;                 // row / column inside a 16 x 16 tile, group of 8 k

    const unsigned char* __restrict__ A = (const unsigned char*)g.A;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B;
    const size_t lda_b = (size_t)g.lda * 2, ldb_b = (size_t)g.ldb * 2;

    // chunk permutation of B row k: the transposing read of a half-wave takes 4 k rows from each of two groups of
    // 8 k (rows 8 apart), 32 bytes each: all 16 pieces must fall into different 16-byte bank groups.  (384-byte rows:
    // consecutive rows already lie half the banks apart, so the key tells apart the rows two apart and eight apart.)
    auto b_key = [](int k) {
        if constexpr (BN == 192) return (4 * ((k >> 3) & 1)) ^ (2 * ((k >> 1) & 1));
        else return (BN >= 128 ? 4 * (k & 3) : 4 * ((k >> 1) & 1)) ^ (2 * ((k >> 3) & 1));
    };

    const unsigned char* a_src[A_LOADS];
    const unsigned char* b_src[B_LOADS];
    // chunk of its row that copy lane i of A fetches / k row of copy lane i of B (functions, not arrays: the partial last
    // slab is the only other place that wants them, and registers that live across the K loop are scarce)
    auto a_chunk_of = [&](int i) { const int row = (64 / CPR) * (wave * A_LOADS + i) + lane / CPR; return (lane % CPR) ^ ((row / RPB) % CPR); };
    // (a direct load fills 1024 contiguous bytes of the stage: 16-byte piece 64 I + lane of the B slab, whatever the row length)
    auto b_krow_of = [&](int i) { return (64 * (wave * B_LOADS + i) + lane) / CBR; };
    const uint32_t last_row = g.M - 1, last_col_chunk = (g.N - 1) / 8;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int I = wave * A_LOADS + i;
        const int row = (64 / CPR) * I + lane / CPR;
        const uint32_t grow = (m0 + row) < last_row ? (m0 + row) : last_row;
        a_src[i] = A + (size_t)grow * lda_b + a_chunk_of(i) * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int krow = b_krow_of(i);
        const int chunk = ((64 * (wave * B_LOADS + i) + lane) % CBR) ^ b_key(krow);
        const uint32_t gchunk = (n0 / 8 + chunk) < last_col_chunk ? (n0 / 8 + chunk) : last_col_chunk;
        b_src[i] = B + (size_t)krow * ldb_b + (size_t)gchunk * 16;
    }

    const uint32_t full_slabs = g.K / BK, k_tail = g.K % BK;
    const uint32_t slabs = full_slabs + (k_tail ? 1u : 0u);

    const size_t b_step = (size_t)BK * ldb_b;
    uint32_t a_voff[A_LOADS], b_voff[B_LOADS];
    const unsigned char* a_base = A + (size_t)m0 * lda_b;
    const unsigned char* b_base = B;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) a_voff[i] = (uint32_t)(a_src[i] - a_base);
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) b_voff[i] = (uint32_t)(b_src[i] - b_base);
    // Slabs are issued in ascending order.  A direct load takes its address as a scalar base (the tile's
    // first row of A / B's row k, running along K) plus a 32-bit lane offset that never changes, so that
    // advancing to the next slab is scalar arithmetic.
    auto issue_direct = [&](uint32_t stage) {               // a whole slab, straight into LDS
        const uint32_t stage_off = lds_base + stage * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const uint32_t dst = stage_off + (uint32_t)(wave * A_LOADS + i) * 1024u;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(dst), "v"(a_voff[i]), "s"(a_base) : "memory", "m0");
        }
        a_base += RB;
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const uint32_t dst = stage_off + A_STAGE_BYTES + (uint32_t)(wave * B_LOADS + i) * 1024u;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(dst), "v"(b_voff[i]), "s"(b_base) : "memory", "m0");
        }
        b_base += b_step;
    };
    auto issue_loads = [&](uint32_t slab) {
        const uint32_t stage = slab % STAGES;
        if (slab < full_slabs) {
            issue_direct(stage);
        } else {
            // the partial last slab: through registers, zero beyond K
            unsigned char* st = lds + stage * STAGE_BYTES;
            const uint32_t k0 = full_slabs * BK;
#pragma unroll
            for (int i = 0; i < A_LOADS; ++i) {
                const uint32_t k = k0 + a_chunk_of(i) * 8;
                halfx8 v = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
                if (k < g.K) {
                    v = *(const halfx8*)(a_base + a_voff[i]);             // inside the pitch: lda is a multiple of 8
#pragma unroll
                    for (int e = 1; e < 8; ++e) if (k + e >= g.K) v[e] = (_Float16)0;
                }
                *(halfx8*)(st + (wave * A_LOADS + i) * 1024 + lane * 16) = v;
            }
#pragma unroll
            for (int i = 0; i < B_LOADS; ++i) {
                halfx8 v = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
                if (k0 + b_krow_of(i) < g.K) v = *(const halfx8*)(b_base + b_voff[i]);
                *(halfx8*)(st + A_STAGE_BYTES + (wave * B_LOADS + i) * 1024 + lane * 16) = v;
            }
        }
    };

    // ---- fragment addressing (byte offsets inside a stage)
    // A fragment (tile i, k step ks): lane (kg, l16) takes row wm0 + 16 i + l16, k = 32 ks + 8 kg .. + 7: chunk 4 ks + kg.
    const int a_row = wm0 + l16;
    const int a_sw = (a_row / RPB) % CPR;                  // wm0 + 16 i leaves it unchanged (multiples of 16 rows)
    int a_off = a_row * RB;
    // B fragment (tile j, k step ks, half r): the 16 lanes of group kg hand in the 4 k rows 32 ks + 8 kg + 4 r + (0..3),
    // lane s = l16 the row s / 4 and the 8-byte segment s % 4 of the 16 columns from wn0 + 16 j; lane l16 receives
    // column l16, 4 consecutive k.
    const int bk_row = 8 * kg + (l16 >> 2);
    const int bk_col = wn0 + 4 * (l16 & 3);
    const int bk_sw = b_key(bk_row);                       // unchanged by + 32 ks + 4 r
    int b_off[TN];
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        const int col = bk_col + 16 * j;
        b_off[j] = A_STAGE_BYTES + bk_row * BRB + (((col >> 3) ^ bk_sw) * 16) + (col & 7) * 2;
    }

    struct FragA { halfx8 a[TMH]; };
    struct FragB { halfx8 b[TN]; };
    FragA fa[2];
    FragB fb[2];
    // unit u = (k step ks = u / HALVES, part u % HALVES of the A rows)
    auto read_unit = [&](const unsigned char* st, auto uc) {
        constexpr int u = decltype(uc)::value, ks = u / HALVES, part = u % HALVES;
#pragma unroll
        for (int i = 0; i < TMH; ++i)
            fa[u & 1].a[i] = *(const halfx8*)(st + a_off + (part * TMH + i) * 16 * RB + (((4 * ks + kg) ^ a_sw) * 16));
        if constexpr (part == 0) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                const unsigned char* p0 = st + b_off[j] + ks * 32 * BRB;
                const shortx4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)p0);
                const shortx4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4*)(p0 + 4 * BRB));
                fb[ks & 1].b[j] = join(lo, hi);
            }
        }
    };

    floatx4 accT[TN][TM];                                  // n tile j, m tile i, transposed
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int r = 0; r < 4; ++r) accT[j][i][r] = 0.f;

    auto multiply_unit = [&](auto uc) {
        constexpr int u = decltype(uc)::value, ks = u / HALVES, part = u % HALVES;
#pragma unroll
        for (int i = 0; i < TMH; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                accT[j][part * TMH + i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(fb[ks & 1].b[j], fa[u & 1].a[i], accT[j][part * TMH + i], 0, 0, 0);
    };
    constexpr int MFMAS = TMH * TN;
    constexpr int READS_FIRST = TMH + 2 * TN, READS_NEXT = TMH;      // a unit that opens a k step also reads the B fragments

#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if ((uint32_t)p < slabs) issue_loads(p);
    if (slabs >= (uint32_t)(STAGES - 1)) wait_loads_and_barrier<LOADS * (STAGES - 2)>();
    else wait_loads_and_barrier<0>();

    // The last unit of a slab is multiplied after the slab barrier, behind the fragment reads of the next slab's
    // first unit (before the first slab it multiplies zeros).
#pragma unroll
    for (int i = 0; i < TMH; ++i) fa[(UNITS - 1) & 1].a[i] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
    for (int j = 0; j < TN; ++j) fb[(KS - 1) & 1].b[j] = halfx8{0, 0, 0, 0, 0, 0, 0, 0};

    // One slab.  STAGE >= 0: its stage is known at compile time and the slab that is asked for meanwhile is a whole one;
    // a loop over STAGES such slabs is one block of code with neither a branch nor address arithmetic between its MFMAs
    // (every LDS address a register that never changes plus an immediate).  STAGE < 0: the general form, for the last slabs.
    auto slab_body = [&](uint32_t s, auto stage_c) {
        constexpr int STAGE = decltype(stage_c)::value;
        constexpr bool STEADY = STAGE >= 0;
        const unsigned char* st;
        if constexpr (STEADY) st = lds + STAGE * STAGE_BYTES; else st = lds + (s % STAGES) * STAGE_BYTES;
        const bool more = STEADY || s + STAGES - 1 < slabs;

        read_unit(st, std::integral_constant<int, 0>{});
        multiply_unit(std::integral_constant<int, UNITS - 1>{});
        interleave<MFMAS, READS_FIRST>();
        __builtin_amdgcn_sched_barrier(0);
        // the stage that held slab s-1 is free: every wave passed the barrier after reading it
        if constexpr (STEADY) {
            issue_direct((uint32_t)((STAGE + STAGES - 1) % STAGES));
            __builtin_amdgcn_sched_barrier(0);
        } else if (more) issue_loads(s + STAGES - 1);

        static_for<0, UNITS - 1>([&](auto uc) {
            constexpr int u = decltype(uc)::value;
            read_unit(st, std::integral_constant<int, u + 1>{});
            multiply_unit(uc);
            interleave<MFMAS, ((u + 1) % HALVES == 0) ? READS_FIRST : READS_NEXT>();
            __builtin_amdgcn_sched_barrier(0);
        });

        if (more) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
    };
    const uint32_t steady = __builtin_amdgcn_readfirstlane(full_slabs > (uint32_t)(STAGES - 1) ? (full_slabs - (uint32_t)(STAGES - 1)) / STAGES * STAGES : 0u);
    uint32_t s = 0;
    for (; s < steady; s += STAGES) static_for<0, STAGES>([&](auto jc) { slab_body(s + decltype(jc)::value, jc); });
    // (the general form derives its LDS addresses from these afresh: computed in front of the loop above they would
    // have to live across it, and it has no register to spare)
    asm volatile("" : "+v"(a_off));
#pragma unroll
    for (int j = 0; j < TN; ++j) asm volatile("" : "+v"(b_off[j]));
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) asm volatile("" : "+v"(a_voff[i]));
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) asm volatile("" : "+v"(b_voff[i]));
    for (; s < slabs; ++s) slab_body(s, std::integral_constant<int, -1>{});
    multiply_unit(std::integral_constant<int, UNITS - 1>{});

    // Epilogue.  Lane (kg, l16) holds, of the 16 x 16 tile (i, j), row l16 and the 4 adjacent columns 4 kg .. 4 kg + 3.
    if constexpr (SPLIT) {
        // piece c of a lane: the four fp32 accumulators of its 16 x 16 tile (c % TM, c / TM).  The ring is free: every
        // LDS read precedes the last slab barrier.
        const bool last = sb.splits == 1 || split_k_exchange<WAVES * 64, TM * TN, floatx4, (BM <= 64)>(g_in, sb, (uint32_t*)lds,
            [&](auto cc) { constexpr int c = decltype(cc)::value; return accT[c / TM][c % TM]; },
            [&](auto cc, const floatx4& v, bool first) {
                constexpr int c = decltype(cc)::value;
                floatx4& a = accT[c / TM][c % TM];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float old = a[e], w = v[e];
                    a[e] = first ? w : old + w;
                }
            },
            [] {});
        if (!last) return;
    }
    const _Float16* __restrict__ C = (const _Float16*)g.C;
    _Float16* __restrict__ D = (_Float16*)g.D;
    auto pack2 = [](float lo, float hi) -> uint32_t {
        union { _Float16 f[2]; uint32_t u; } w;
        w.f[0] = (_Float16)lo; w.f[1] = (_Float16)hi;
        return w.u;
    };
    const bool interior = (m0 + BM <= g.M) && (n0 + BN <= g.N);
    // The tile goes through LDS once more (the ring is free: every wave has passed the last slab barrier): a lane
    // holds 8 bytes of a row, 4 lanes 32 contiguous bytes.  Each wave turns 16 rows x WN columns around in a private
    // buffer (two of them, taking turns) and stores whole rows: WN * 2 contiguous bytes per row.  Tiles on a ragged
    // edge take the same way and leave out rows beyond M and 16-byte pieces beyond N; only a piece that straddles N is
    // stored element by element (stored that way as a whole, a 256 x 256 edge tile took a third longer than an interior one).
    // (Rows of 192 bytes -- a wave tile 96 columns wide -- are not permuted but laid 16 bytes further apart.)
    constexpr int ROW_BYTES = WN * 2, PPR = WN / 8, STORES = PPR / 4;
    constexpr bool POW2 = (PPR & (PPR - 1)) == 0;
    constexpr int ROW_PITCH = POW2 ? ROW_BYTES : ROW_BYTES + 16, RPG = POW2 ? 256 / ROW_BYTES : 1;
    static_assert(PPR == 4 || PPR == 8 || PPR == 12 || PPR == 16, "staging rows of 64, 128, 192 or 256 bytes");
    static_assert(WAVES * 2 * 16 * ROW_PITCH <= LDS_BYTES, "staging rows must fit in the ring");
    auto piece_slot = [](int piece, int row) { if constexpr (POW2) return piece ^ ((row / RPG) % PPR); else return piece; };
    auto wave_sync = [] {
        __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        __builtin_amdgcn_wave_barrier();
        __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    };
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const uint32_t row = m0 + wm0 + 16 * i + l16;
        unsigned char* stage_rows = lds + (wave * 2 + (i & 1)) * (16 * ROW_PITCH);
        // interior tiles ask for the C values of all TN blocks of the row before the first is used (one load, its wait and
        // the fmas block by block made the C term cost 6 to 12 %)
        halfx4 c_row[TN];
        const bool c_ahead = C != nullptr && interior;
        if (c_ahead) {
#pragma unroll
            for (int j = 0; j < TN; ++j) c_row[j] = *(const halfx4*)(C + (size_t)row * g.ldc + (n0 + wn0 + 16 * j + 4 * kg));
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            float v[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = accT[j][i][e];
            if (c_ahead) {
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)c_row[j][e], g.beta, g.alpha * v[e]);
            } else if (C) {
                const uint32_t col = n0 + wn0 + 16 * j + 4 * kg;
                if (interior || (row < g.M && col + 4 <= g.N)) {
                    const halfx4 cv = *(const halfx4*)(C + (size_t)row * g.ldc + col);
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = __builtin_fmaf((float)cv[e], g.beta, g.alpha * v[e]);
                } else if (row < g.M) {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (col + e < g.N) v[e] = __builtin_fmaf((float)C[(size_t)row * g.ldc + col + e], g.beta, g.alpha * v[e]);
                }
            }
            const uintx2 out = {pack2(v[0], v[1]), pack2(v[2], v[3])};
            // piece p (16 bytes) of row l16, half kg & 1 of it; pieces XOR-permuted so that the 32 lanes of a write
            // and the 16 lanes of a read-back each cover all banks once
            const int p = 2 * j + (kg >> 1);
            *(uintx2*)(stage_rows + l16 * ROW_PITCH + piece_slot(p, l16) * 16 + (kg & 1) * 8) = out;
        }
        wave_sync();
#pragma unroll
        for (int t2 = 0; t2 < STORES; ++t2) {
            const int r = (64 * t2 + lane) / PPR, pc = (64 * t2 + lane) % PPR;
            const uintx4 v = *(const uintx4*)(stage_rows + r * ROW_PITCH + piece_slot(pc, r) * 16);
            const uint32_t grow = m0 + wm0 + 16 * i + r, gcol = n0 + wn0 + 8 * pc;
            _Float16* out = D + (size_t)grow * g.ldd + gcol;
            if (interior || (grow < g.M && gcol + 8 <= g.N)) {
                // the streaming hint: 2048^3 904 -> 943 TFLOP/s, 16384 x 2048 x 512 876 -> 958, 4096^3 1399 -> 1415
                // (8192 x 8192 x 1024: 1196 -> 1166)
                __builtin_nontemporal_store(v, (uintx4*)out);
            } else if (grow < g.M && gcol < g.N) {
                union { uintx4 u; _Float16 h[8]; } w;
                w.u = v;
#pragma unroll
                for (int e = 0; e < 8; ++e)
                    if (gcol + e < g.N) out[e] = w.h[e];
            }
        }
        wave_sync();
    }
}

namespace {

template <int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES>
int launch_dma(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    if (g.split_len) {                                     // (the tiles of 192 rows or columns have no split form)
        if constexpr ((BM <= 128 && BN <= 128) || (BM == 256 && BN == 256)) {
            const uint32_t splits = g.split_count;
            hipLaunchKernelGGL((gemm_f16_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES, true>), dim3(g.split_first + (nb - g.split_first) * splits),
                               dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
            return (int)hipGetLastError();
        } else {
            return (int)hipErrorInvalidValue;
        }
    }
    hipLaunchKernelGGL((gemm_f16_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES>), dim3(nb), dim3(WAVES_M * WAVES_N * 64),
                       0, stream, g);
    return (int)hipGetLastError();
}

}  // namespace

// M, N, K >= 1; 16-byte aligned bases and pitches (the caller checks).  Shapes measured on MI355X:
//   256 x 256: 8 wavefronts of 128 x 64 on 64-deep slabs in 2 stages (1177 TFLOP/s at 4096^3, 1222 at
//     8192^3); 4 wavefronts of 128 x 128 reach 1075-1124, 16 wavefronts 1144, 32-deep slabs 1100-1124.
//     Two wavefronts per SIMD take turns on the matrix pipe while the other waits for LDS or the barrier.
//     Spreading the direct loads over the k steps, or raising the wave priority around the MFMAs, is 3-4 % slower.
//   128 x 128: 8 wavefronts of 64 x 32 (1536^3: 526 TFLOP/s against 453 with 4 of 64 x 64; the same from 2560^3 up),
//     64-deep slabs; a ring of 4 stages when there is at most one workgroup per CU (784 TFLOP/s at 2048^3), else of
//     2 stages so that two workgroups share a CU (4096^3: 994 against 940 with 32-deep slabs in 4 stages, 6144^3:
//     1035 against 960).
//   64 x 64: 4 wavefronts of 32 x 32, 64-deep slabs in 4 stages (327 TFLOP/s at 1024^3), in 2 stages once more
//     than two workgroups per CU are there to hide the copies (1536^3: 447 against 388).
int launch_gemm_f16_dma(int shape, const GemmArgs& args, hipStream_t stream)
{
    // workgroups of a launch on b x b tiles: whole tiles, and splits of the others
    const auto workgroups = [&](uint32_t b) {
        const uint64_t tiles = (uint64_t)((args.M + b - 1) / b) * ((args.N + b - 1) / b);
        return args.split_len ? args.split_first + (tiles - args.split_first) * args.split_count : tiles;
    };
    switch (shape) {
    case TILE_LARGE: return launch_dma<256, 256, 2, 4, 64, 2>(args, stream);
    case TILE_MEDIUM: {
        const uint64_t blocks = workgroups(128);
        return blocks <= 256 ? launch_dma<128, 128, 2, 4, 64, 4>(args, stream)
                             : launch_dma<128, 128, 2, 4, 64, 2>(args, stream);
    }
    case TILE_SMALL: {
        const uint64_t blocks = workgroups(64);
        return blocks <= 512 ? launch_dma<64, 64, 2, 2, 64, 4>(args, stream)
                             : launch_dma<64, 64, 2, 2, 64, 2>(args, stream);
    }
    // tiles between 128 x 128 and 256 x 256, one workgroup of 8 wavefronts per CU, for outputs that the largest tile
    // cuts into an awkward number of pieces (3000^3: 144 tiles of 256 x 256 on 256 CUs, but 256 of 192 x 192)
    case TILE_F16_192x192: return launch_dma<192, 192, 4, 2, 64, 2>(args, stream);     // wavefronts of 48 x 96
    case TILE_F16_192x256: return launch_dma<192, 256, 2, 4, 64, 2>(args, stream);     // 96 x 64
    case TILE_F16_256x192: return launch_dma<256, 192, 4, 2, 64, 2>(args, stream);     // 64 x 96
    default:           return (int)hipErrorInvalidValue;
    }
}

}  // namespace decx_hip
