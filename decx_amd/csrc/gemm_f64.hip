// fp64 GEMM for gfx950 on the fp64 matrix cores (v_mfma_f64_16x16x4_f64).
//
// Replaces the reference's cu_GEMM_fp64_*_16_64_64 kernels and their runner
// (srcs/modules/BLAS/GEMM/CUDA/large_squares/GEMM_kernels.cuh:182-189, GEMM_LS.cu:164-211).
// Same data movement as the fp32 / fp16 kernels: K slabs go global -> LDS by direct 128-bit
// loads into a ring of STAGES stages (inline assembly, bare s_barrier behind an explicit vmcnt
// wait), ragged M / N by fetching the last valid row / column chunk, ragged K through registers
// with zero fill.
//
// Fragment scheme.  One MFMA multiplies a 16 x 4 by a 4 x 16 block: lane l supplies A(l % 16, q)
// and B(q, l % 16) with q = l / 16, and holds D(4 i + q, l % 16) in result element i.  A lane
// fetches two consecutive k of its A row with one 128-bit LDS read and uses them in two
// successive k steps: step 2 t + e takes k = 8 t + 2 q + e (any assignment of k's to steps is valid
// as long as A and B agree).  Columns are dealt to lanes in pairs (lane c owns columns
// 32 jj + 2 c, 32 jj + 2 c + 1 of the wave tile), so B fragments are 128-bit reads of adjacent
// lanes and the epilogue stores 16 bytes per lane.
//
// LDS layout of a stage: A as [BM rows][BK / 2 chunks of 16 bytes], chunk c of row r in slot
// c ^ ((r / RP) % CPR); B as [BK][BN] doubles, straight.
//
// A plain one-thread-per-element kernel serves operands that are not 16-byte aligned, and K == 0.
#include "gemm_common.hpp"
#include "split_k_exchange.hpp"
#include <type_traits>

namespace decx_hip {

namespace {

typedef double doublex2 __attribute__((ext_vector_type(2)));
typedef double doublex4 __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) void lds_void;

template <int N> __device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(N) : "memory");
}

}  // namespace

// SPLIT: grid.y workgroups share each tile, each with its own range of K; the one that finishes last adds their
// partial products (split_k_exchange).
template <int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES, bool SPLIT = false>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
__attribute__((amdgpu_waves_per_eu(BM * BN >= 128 * 128 ? 2 : 4)))     // as scheduled: one workgroup of 8 wavefronts per CU on the two larger tiles, two of 64 x 64
gemm_f64_dma_kernel(const GemmArgs g_in)
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
            g_split.A = (const unsigned char*)g_in.A + (size_t)k0 * 8;
            g_split.B = (const unsigned char*)g_in.B + (size_t)k0 * g_in.ldb * 8;
            g_split.K = sb.z + 1 == sb.splits ? g_in.K - k0 : g_in.split_len;     // the last range: what is left (more or less than split_len)
            if (g_in.split_urgent) __builtin_amdgcn_s_setprio(3);
        }
    } else {
        block_to_tile(g_in, tile_m, tile_n);
    }
    const GemmArgs& g = [&]() -> const GemmArgs& { if constexpr (SPLIT) return g_split; else return g_in; }();
    constexpr int WAVES = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 16, TN = WN / 16, TP = TN / 2;
    constexpr int RBYTES = BK * 8, CPR = RBYTES / 16, RP = 16 / CPR;       // A row bytes, chunks per row, rows per 256 bytes
    constexpr int CB = BN / 2, RB = 64 / CB;                               // B chunks per k row, k rows per direct load
    constexpr int A_STAGE_BYTES = BM * RBYTES, B_STAGE_BYTES = BK * BN * 8, STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
    constexpr int A_LOADS = A_STAGE_BYTES / 1024 / WAVES, B_LOADS = B_STAGE_BYTES / 1024 / WAVES, LOADS = A_LOADS + B_LOADS;
    constexpr int STEPS = BK / 4, GROUPS = BK / 8;                          // MFMA k steps, 8-deep k groups per slab
    // GROUPS must be even: the A pairs of a slab's last k group (af[1]) have to survive the reads of the next
    // slab's first group (af[0]) until the deferred last step is issued
    static_assert(TM >= 1 && TN >= 2 && TN % 2 == 0 && BK == 16, "shape");
    static_assert(CB <= 64 && 64 % CB == 0, "B copy plan");
    static_assert(A_LOADS >= 1 && B_LOADS >= 1 && A_LOADS * WAVES * 1024 == A_STAGE_BYTES &&
                  B_LOADS * WAVES * 1024 == B_STAGE_BYTES, "copy plan must divide evenly");
    static_assert(STAGES >= 2 && STAGES * STAGE_BYTES <= 160 * 1024, "LDS budget");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE_BYTES];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)lds;

    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);      // uniform: LDS destinations stay in scalar registers
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l16 = lane & 15, q = lane >> 4;

    const unsigned char* __restrict__ A = (const unsigned char*)g.A;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B;
    const size_t lda_b = (size_t)g.lda * 8, ldb_b = (size_t)g.ldb * 8;

    // ---- copy plan (rows beyond M and column chunks beyond N are replaced by the last valid ones)
    const unsigned char* a_src[A_LOADS];
    const unsigned char* b_src[B_LOADS];
    int a_chunk[A_LOADS], b_krow[B_LOADS];
    const uint32_t last_row = g.M - 1, last_col_chunk = (g.N - 1) / 2;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int I = wave * A_LOADS + i;
        const int row = I * (64 / CPR) + lane / CPR;
        a_chunk[i] = (lane % CPR) ^ ((row / RP) % CPR);
        const uint32_t grow = (m0 + row) < last_row ? (m0 + row) : last_row;
        a_src[i] = A + (size_t)grow * lda_b + a_chunk[i] * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int I = wave * B_LOADS + i;
        b_krow[i] = I * RB + lane / CB;
        const uint32_t chunk = lane % CB;
        const uint32_t gchunk = (n0 / 2 + chunk) < last_col_chunk ? (n0 / 2 + chunk) : last_col_chunk;
        b_src[i] = B + (size_t)b_krow[i] * ldb_b + (size_t)gchunk * 16;
    }

    const uint32_t full_slabs = g.K / BK, k_tail = g.K % BK;
    const uint32_t slabs = full_slabs + (k_tail ? 1u : 0u);

    // Slabs are issued in ascending order.  A direct load takes its address as a scalar base (the tile's
    // first row of A / B's row k, running along K) plus a 32-bit lane offset that never changes, so that
    // advancing to the next slab is scalar arithmetic.
    const size_t b_step = (size_t)BK * ldb_b;
    uint32_t a_voff[A_LOADS], b_voff[B_LOADS];
    const unsigned char* a_base = A + (size_t)m0 * lda_b;
    const unsigned char* b_base = B;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) a_voff[i] = (uint32_t)(a_src[i] - a_base);           // < BM * lda_b: the launcher checks
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) b_voff[i] = (uint32_t)(b_src[i] - b_base);           // < BK * ldb_b
    auto issue_one = [&](uint32_t stage, auto ic) {        // direct load ic of a full slab: A first, then B
        constexpr int idx = decltype(ic)::value;
        const uint32_t stage_off = lds_base + stage * STAGE_BYTES;
        if constexpr (idx < A_LOADS) {
            constexpr int i = idx;
            const uint32_t dst = stage_off + (uint32_t)(wave * A_LOADS + i) * 1024u;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(dst), "v"(a_voff[i]), "s"(a_base) : "memory", "m0");
            if constexpr (i == A_LOADS - 1) a_base += RBYTES;
        } else {
            constexpr int i = idx - A_LOADS;
            const uint32_t dst = stage_off + A_STAGE_BYTES + (uint32_t)(wave * B_LOADS + i) * 1024u;
            asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(dst), "v"(b_voff[i]), "s"(b_base) : "memory", "m0");
            if constexpr (i == B_LOADS - 1) b_base += b_step;
        }
    };
    auto issue_tail = [&](uint32_t stage) {                // the partial last slab: through registers, zero beyond K
        unsigned char* st = lds + stage * STAGE_BYTES;
        const uint32_t k0 = full_slabs * BK;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const uint32_t k = k0 + a_chunk[i] * 2;
            doublex2 v = doublex2{0.0, 0.0};
            if (k < g.K) {
                v = *(const doublex2*)(a_base + a_voff[i]);    // inside the pitch: lda is even
                if (k + 1 >= g.K) v[1] = 0.0;
            }
            *(doublex2*)(st + (wave * A_LOADS + i) * 1024 + lane * 16) = v;
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            doublex2 v = doublex2{0.0, 0.0};
            if (k0 + b_krow[i] < g.K) v = *(const doublex2*)(b_base + b_voff[i]);
            *(doublex2*)(st + A_STAGE_BYTES + (wave * B_LOADS + i) * 1024 + lane * 16) = v;
        }
    };
    auto issue_loads = [&](uint32_t slab) {                // a whole slab in one burst
        if (slab < full_slabs) static_for<0, LOADS>([&](auto ic) { issue_one(slab % STAGES, ic); });
        else issue_tail(slab % STAGES);
    };

    // ---- fragment addressing inside a stage
    const int a_row = wm0 + l16;                       // + 16 i leaves (row / RP) % CPR unchanged
    const int a_sw = (a_row / RP) % CPR;
    int a_off[GROUPS];                                 // byte offset of chunk 4 t + q of this lane's row
#pragma unroll
    for (int tt = 0; tt < GROUPS; ++tt) a_off[tt] = a_row * RBYTES + (((4 * tt + q) ^ a_sw) * 16);
    const int b_col = wn0 + 2 * l16;                   // + 32 jj
    const int b_off = A_STAGE_BYTES + (2 * q) * BN * 8 + b_col * 8;       // + (8 t + e) rows

    doublex4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j) acc[i][j] = doublex4{0.0, 0.0, 0.0, 0.0};

#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if ((uint32_t)p < slabs) issue_loads(p);
    if (slabs >= (uint32_t)(STAGES - 1)) wait_loads_and_barrier<LOADS * (STAGES - 2)>();
    else wait_loads_and_barrier<0>();

    // af[t & 1] holds the A pairs of k group t, bf[step & 1] the B pairs of a k step.  Fragments are fetched one
    // step ahead; the MFMAs of the last step of a slab are issued after the slab barrier, behind the first
    // fragment reads of the next slab (before the first slab they multiply zeros).
    doublex2 af[2][TM];
    constexpr int BF_AHEAD = 2, BFM = 3;                   // B fragments are read 2 k steps ahead into a ring of 4
    doublex2 bf[BFM + 1][TP];
#pragma unroll
    for (int i = 0; i < TM; ++i) af[(GROUPS - 1) & 1][i] = doublex2{0.0, 0.0};
#pragma unroll
    for (int jj = 0; jj < TP; ++jj) bf[(STEPS - 1) & BFM][jj] = doublex2{0.0, 0.0};

    // MFMAs FIRST .. LAST-1 (in i-major order) of a k step
    auto multiply_part = [&](auto stc, auto firstc, auto lastc) {
        constexpr int step = decltype(stc)::value;
        constexpr int tt = step / 2, e = step % 2;
        static_for<decltype(firstc)::value, decltype(lastc)::value>([&](auto nc) {
            constexpr int i = decltype(nc)::value / TN, j = decltype(nc)::value % TN;
            acc[i][j] = __builtin_amdgcn_mfma_f64_16x16x4f64(af[tt & 1][i][e], bf[step & BFM][j / 2][j % 2], acc[i][j], 0, 0, 0);
        });
    };
    auto multiply = [&](auto stc) {
        multiply_part(stc, std::integral_constant<int, 0>{}, std::integral_constant<int, TM * TN>{});
    };
    auto read_b = [&](const unsigned char* st, auto stc) {
        constexpr int step = decltype(stc)::value;
#pragma unroll
        for (int jj = 0; jj < TP; ++jj)
            bf[step & BFM][jj] = *(const doublex2*)(st + b_off + (8 * (step / 2) + step % 2) * BN * 8 + jj * 32 * 8);
    };
    auto read_a = [&](const unsigned char* st, auto tc) {
        constexpr int tt = decltype(tc)::value;
#pragma unroll
        for (int i = 0; i < TM; ++i) af[tt & 1][i] = *(const doublex2*)(st + a_off[tt] + i * 16 * RBYTES);
    };
    // the direct loads of a slab go out PER_STEP per k step, each group behind the first MFMA of its step
    constexpr int PER_STEP = (LOADS + STEPS - 2) / (STEPS - 1);

    // One slab.  STAGE >= 0: its stage is known at compile time and the slab that is asked for meanwhile is a whole one;
    // a loop over STAGES such slabs is one block of code with neither a branch nor address arithmetic between its MFMAs.
    // STAGE < 0: the general form, for the last slabs.
    auto slab_body = [&](uint32_t s, auto stage_c) {
        constexpr int STAGE = decltype(stage_c)::value;
        constexpr bool STEADY = STAGE >= 0;
        const unsigned char* st;
        if constexpr (STEADY) st = lds + STAGE * STAGE_BYTES; else st = lds + (s % STAGES) * STAGE_BYTES;
        const bool more = STEADY || s + STAGES - 1 < slabs;

        read_a(st, std::integral_constant<int, 0>{});
        static_for<0, BF_AHEAD>([&](auto stc) { read_b(st, stc); });
        multiply(std::integral_constant<int, STEPS - 1>{});
        __builtin_amdgcn_sched_group_barrier(0x100, TM + BF_AHEAD * TP, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
        __builtin_amdgcn_sched_barrier(0);
        // the stage that held slab s-1 is free: every wave passed the barrier after reading it
        const uint32_t nstage = STEADY ? (uint32_t)((STAGE + STAGES - 1) % STAGES) : (s + STAGES - 1) % STAGES;
        const bool direct = STEADY || s + STAGES - 1 < full_slabs;
        if constexpr (!STEADY) { if (more && !direct) issue_tail(nstage); }

        static_for<0, STEPS - 1>([&](auto stc) {
            constexpr int step = decltype(stc)::value;
            constexpr int tt = step / 2, e = step % 2;                 // group tt + 1 of A is read during group tt, half per step
            constexpr bool next_b = step + BF_AHEAD < STEPS;
            constexpr int a_lo = (tt + 1 < GROUPS) ? (e * TM + 1) / 2 : 0, a_hi = (tt + 1 < GROUPS) ? ((e + 1) * TM + 1) / 2 : 0;
            constexpr int reads = (next_b ? TP : 0) + (a_hi - a_lo);
            if constexpr (next_b) read_b(st, std::integral_constant<int, step + BF_AHEAD>{});
            static_for<a_lo, a_hi>([&](auto ic) {
                constexpr int i = decltype(ic)::value;
                af[(tt + 1) & 1][i] = *(const doublex2*)(st + a_off[(tt + 1) % GROUPS] + i * 16 * RBYTES);
            });
            multiply_part(stc, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            if constexpr (reads > 0) __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (step * PER_STEP < LOADS) {
                if (direct)
                    static_for<step * PER_STEP, (step + 1) * PER_STEP < LOADS ? (step + 1) * PER_STEP : LOADS>(
                        [&](auto ic) { issue_one(nstage, ic); });
                __builtin_amdgcn_sched_barrier(0);
            }
            multiply_part(stc, std::integral_constant<int, 1>{}, std::integral_constant<int, TM * TN>{});
            __builtin_amdgcn_sched_barrier(0);
        });

        if (more) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
    };
    const uint32_t steady = __builtin_amdgcn_readfirstlane(full_slabs > (uint32_t)(STAGES - 1) ? (full_slabs - (uint32_t)(STAGES - 1)) / STAGES * STAGES : 0u);
    uint32_t s = 0;
    for (; s < steady; s += STAGES) static_for<0, STAGES>([&](auto jc) { slab_body(s + decltype(jc)::value, jc); });
    for (; s < slabs; ++s) slab_body(s, std::integral_constant<int, -1>{});
    multiply(std::integral_constant<int, STEPS - 1>{});

    if constexpr (SPLIT) {
        // piece c of a lane: elements 2 (c % 2), + 1 of its 16 x 16 tile c / 2.  The ring is free: every LDS read
        // precedes the last slab barrier.
        const bool last = sb.splits == 1 || split_k_exchange<WAVES * 64, TM * TN * 2, doublex2>(g_in, sb, (uint32_t*)lds,
            [&](auto cc) {
                constexpr int c = decltype(cc)::value, tile = c / 2, e0 = 2 * (c % 2);
                const doublex4& a = acc[tile / TN][tile % TN];
                return doublex2{a[e0], a[e0 + 1]};
            },
            [&](auto cc, const doublex2& v, bool first) {
                constexpr int c = decltype(cc)::value, tile = c / 2, e0 = 2 * (c % 2);
                doublex4& a = acc[tile / TN][tile % TN];
#pragma unroll
                for (int e = 0; e < 2; ++e) {
                    const double old = a[e0 + e], w = v[e];
                    a[e0 + e] = first ? w : old + w;
                }
            },
            [] {});
        if (!last) return;
    }

    // Epilogue: element i of tile (ti, tj) is row 16 ti + 4 i + q; tiles 2 jj, 2 jj + 1 are the adjacent columns
    // 32 jj + 2 l16, + 1.
    const double* __restrict__ C = (const double*)g.C;
    double* __restrict__ D = (double*)g.D;
    const bool interior = (m0 + BM <= g.M) && (n0 + BN <= g.N);
#pragma unroll
    for (int ti = 0; ti < TM; ++ti) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const uint32_t row = m0 + wm0 + 16 * ti + 4 * i + q;
            // interior tiles ask for a row's C values before the first is used
            doublex2 c_row[TP];
            const bool c_ahead = C != nullptr && interior;
            if (c_ahead) {
#pragma unroll
                for (int jj = 0; jj < TP; ++jj) c_row[jj] = *(const doublex2*)(C + (size_t)row * g.ldc + (n0 + b_col + 32 * jj));
            }
#pragma unroll
            for (int jj = 0; jj < TP; ++jj) {
                const uint32_t col = n0 + b_col + 32 * jj;
                double v0 = acc[ti][2 * jj][i], v1 = acc[ti][2 * jj + 1][i];
                if (interior || (row < g.M && col + 2 <= g.N)) {
                    if (c_ahead) {
                        v0 = __builtin_fma(c_row[jj][0], g.beta64, g.alpha64 * v0);
                        v1 = __builtin_fma(c_row[jj][1], g.beta64, g.alpha64 * v1);
                    } else if (C) {
                        const doublex2 cv = *(const doublex2*)(C + (size_t)row * g.ldc + col);
                        v0 = __builtin_fma(cv[0], g.beta64, g.alpha64 * v0);
                        v1 = __builtin_fma(cv[1], g.beta64, g.alpha64 * v1);
                    }
                    __builtin_nontemporal_store(doublex2{v0, v1}, (doublex2*)(D + (size_t)row * g.ldd + col));     // the streaming hint: 2048^3 73.9 -> 74.4 TFLOP/s
                } else if (row < g.M) {
                    if (col < g.N) {
                        if (C) v0 = __builtin_fma(C[(size_t)row * g.ldc + col], g.beta64, g.alpha64 * v0);
                        D[(size_t)row * g.ldd + col] = v0;
                    }
                    if (col + 1 < g.N) {
                        if (C) v1 = __builtin_fma(C[(size_t)row * g.ldc + col + 1], g.beta64, g.alpha64 * v1);
                        D[(size_t)row * g.ldd + col + 1] = v1;
                    }
                }
            }
        }
    }
}

// One thread per output element, k ascending: any alignment, any K (also 0).
__global__ void __launch_bounds__(256) gemm_f64_plain_kernel(const GemmArgs g)
{
    // tiles of 16 x 16 outputs on a 1-D grid (neither dimension is bound by the 65 535 blocks of grid.y)
    const uint32_t tiles_n = (g.N + 15) / 16;
    const uint32_t col = (blockIdx.x % tiles_n) * 16 + (threadIdx.x & 15), row = (blockIdx.x / tiles_n) * 16 + (threadIdx.x >> 4);
    if (row >= g.M || col >= g.N) return;
    const double* a = (const double*)g.A + (size_t)row * g.lda;
    const double* b = (const double*)g.B + col;
    double acc = 0.0;
    for (uint32_t k = 0; k < g.K; ++k) acc = __builtin_fma(a[k], b[(size_t)k * g.ldb], acc);
    if (g.C) acc = __builtin_fma(((const double*)g.C)[(size_t)row * g.ldc + col], g.beta64, g.alpha64 * acc);
    ((double*)g.D)[(size_t)row * g.ldd + col] = acc;
}

namespace {

template <int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES>
int launch_dma(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    if (g.split_len) {                                     // the planner splits K on the smallest tile only
        if constexpr (BM == 64) {
            const uint32_t splits = g.split_count;
            hipLaunchKernelGGL((gemm_f64_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES, true>), dim3(g.split_first + (nb - g.split_first) * splits),
                               dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
            return (int)hipGetLastError();
        } else {
            return (int)hipErrorInvalidValue;
        }
    }
    hipLaunchKernelGGL((gemm_f64_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES>), dim3(nb), dim3(WAVES_M * WAVES_N * 64),
                       0, stream, g);
    return (int)hipGetLastError();
}

}  // namespace

// shape: TILE_LARGE stands for the largest fp64 tile, 256 x 128 (eight wavefronts of 64 x 64).  The smaller tiles
// run eight wavefronts too (128 x 128: 64 x 32 each, 64 x 64: 16 x 32 each): measured 70 against 61 TFLOP/s at
// 2048^3 and 56 against 50 at 1024^3 with four.
int launch_gemm_f64(int shape, bool plain, const GemmArgs& args, hipStream_t stream)
{
    if (plain || !args.vec_ok || args.K == 0 || !dma_offsets_fit(args, 8)) {
        const uint64_t tiles = (uint64_t)((args.N + 15) / 16) * ((args.M + 15) / 16);
        if (tiles > 0x7fffffffull) return (int)hipErrorInvalidValue;
        hipLaunchKernelGGL(gemm_f64_plain_kernel, dim3((unsigned)tiles), dim3(256), 0, stream, args);
        return (int)hipGetLastError();
    }
    switch (shape) {
    case TILE_LARGE: return launch_dma<256, 128, 4, 2, 16, 3>(args, stream);
    case TILE_MEDIUM: return launch_dma<128, 128, 2, 4, 16, 2>(args, stream);
    case TILE_SMALL:   return launch_dma< 64,  64, 4, 2, 16, 4>(args, stream);
    default:           return (int)hipErrorInvalidValue;
    }
}

}  // namespace decx_hip
