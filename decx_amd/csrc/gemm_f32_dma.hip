// fp32 GEMM for gfx950, any M, N, K on 16-byte aligned operands: BM x BN block tiles whose K
// slabs are copied global -> LDS by direct (LDS-DMA) 128-bit loads into a ring of STAGES
// stages, ragged edges included.
//
// Replaces the reference's SIMT kernels cu_GEMM_fp32_[F_]kernel_* and their transposed-A
// variants (srcs/modules/BLAS/GEMM/CUDA/large_squares/fp32/GEMM_fp32_B128_kernels.cu,
// GEMM_fp32_B64_kernels.cu) and the separate A-transpose pass: one kernel family, no scratch,
// no reliance on zero-filled pitch padding.
//
// Arithmetic: v_mfma_f32_32x32x2_f32; the lower / upper half-wave supply k and k + 4 of each
// 8-deep chunk (any pairing of k's is valid as long as A and B agree), which lets a lane fetch
// A four k's at a time with one 128-bit LDS read; a wave's TN column tiles are interleaved (lane
// j owns columns TN j .. TN j + TN - 1), so one 32/64/128-bit read feeds all TN MFMAs of a k
// step and the epilogue stores TN contiguous floats per lane.  Epilogue D = fma(C, beta,
// alpha * acc) as the reference's F kernels do (GEMM_fp32_B128_kernels.cu:725-744).
//
// Data movement: `global_load_lds_dwordx4` writes LDS directly (no staging registers, no
// ds_write), so late loads are absorbed by the ring and by the other workgroups of the CU.  The direct
// loads are inline assembly and the slab barrier is a bare `s_barrier` behind an explicit vmcnt
// wait, because the compiler would otherwise wait for every outstanding load in front of each
// LDS read and at each __syncthreads().  (The compiler does not look into inline assembly for
// hazards: the `s_nop 0` between the write of M0, which carries the LDS destination, and the
// load that reads it is the wait state this part asks for.)  Fragment reads are pinned behind MFMAs with
// `sched_group_barrier`; the MFMAs of the last k step of a slab are issued after the slab
// barrier, behind the first fragment reads of the next slab.
//   * tile shapes from 256 x 128 (four wavefronts of 128 x 64, two workgroups per CU; the
//     convolution keeps 256 x 256 with eight) down to 64 x 64 (four wavefronts of 32 x 32), so
//     that small problems still put a workgroup on every CU; wave tiles that small issue one
//     MFMA per k step, less than an LDS read takes, so their fragments are fetched a whole
//     8-deep chunk ahead;
//   * ragged M and N without predicated loads: a copy lane whose row or column chunk
//     lies outside the matrix fetches the last valid row / chunk instead (always mapped
//     memory); what it brings lands in accumulators of rows / columns that are never stored;
//   * ragged K: the last, partial slab goes through registers (zero-filled beyond K) into
//     its LDS stage, so no product ever sees bytes from outside the operands.
//
// LDS layout of a stage: A as [BM rows][BK / 4 chunks of 16 bytes], chunk c of row r in
// slot c ^ ((r / RP) % CPR) (CPR chunks per row, RP = 16 / CPR rows per 256 bytes): the
// 128-bit fragment reads of 16 consecutive rows then cover 16 distinct 16-byte bank
// groups.  B as [BK][BN] floats; for 32-column wave tiles the chunks of k rows 4..7 (mod 8)
// are shifted by 128 bytes so the two half-waves read different banks.  Both permutations
// are applied on the global side of the copy: a direct load always writes 1 KB contiguous.
#include "gemm_common.hpp"
#include "split_k_exchange.hpp"
#include <type_traits>

namespace decx_hip {

namespace {

typedef __attribute__((address_space(3))) void lds_void;

template <int N> __device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(N) : "memory");
}

template <int TN> struct BFrag;
template <> struct BFrag<1> { typedef float type; };
template <> struct BFrag<2> { typedef floatx2 type; };
template <> struct BFrag<4> { typedef floatx4 type; };

template <int TN> __device__ __forceinline__ float lane_of(const typename BFrag<TN>::type& v, int j)
{
    if constexpr (TN == 1) return v; else return v[j];
}

}  // namespace

// CONV: 0 plain GEMM; 1 convolution, every copy lane walks the image on its own; 2 convolution whose runs of
// contiguous bytes are whole slabs, so that all lanes hop to the next image row in the same slab.
// SPLIT: grid.y workgroups share each tile, each with its own range of K (a separate instantiation, so that the
// plain kernel keeps reading its arguments straight from the kernel-argument segment).  They meet in the workspace:
// every workgroup stores its accumulators to its slot and counts itself in at the tile's counter; the last one to
// arrive adds the slots in range order and runs the epilogue.  No workgroup waits for another.
template <int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES, bool CHUNK_AHEAD, int CONV = 0, bool SPLIT = false, bool SPLIT_WITH_C = false>
// The wavefronts per SIMD every tile is scheduled for (two workgroups of the largest tile per CU, three of 128 x 128, four of
// the smaller ones) are told to the compiler: it then keeps the accumulators in the unified register file's VGPR half and
// fits the epilogue below into the budget, where its own choice was 142 VGPRs beside 128 accumulation registers (one
// workgroup of the 256 x 128 tile per CU) for any epilogue that keeps loads in flight across rows.
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
__attribute__((amdgpu_waves_per_eu(BM * BN >= 256 * 128 ? 2 : BM * BN >= 128 * 128 ? 3 : 4)))
gemm_f32_dma_kernel(const GemmArgs g_in)
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
            g_split.A = (const unsigned char*)g_in.A + (size_t)k0 * 4;
            g_split.B = (const unsigned char*)g_in.B + (size_t)k0 * g_in.ldb * 4;
            g_split.K = sb.z + 1 == sb.splits ? g_in.K - k0 : g_in.split_len;     // the last range: what is left (more or less than split_len)
            if (g_in.split_urgent) __builtin_amdgcn_s_setprio(3);
        }
    } else {
        block_to_tile(g_in, tile_m, tile_n);
    }
    const GemmArgs& g = [&]() -> const GemmArgs& { if constexpr (SPLIT) return g_split; else return g_in; }();
    constexpr int WAVES = WAVES_M * WAVES_N;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / 32, TN = WN / 32;
    constexpr int CPR = BK / 4, RP = 16 / CPR;                    // A chunks per row, rows per 256 bytes
    constexpr int CB = BN / 4, RB = 64 / CB;                      // B chunks per k row, k rows per direct load
    constexpr int A_STAGE_BYTES = BM * BK * 4, B_STAGE_BYTES = BK * BN * 4, STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
    constexpr int A_LOADS = A_STAGE_BYTES / 1024 / WAVES, B_LOADS = B_STAGE_BYTES / 1024 / WAVES, LOADS = A_LOADS + B_LOADS;
    // The two half-waves read k rows r and r + 4 of B at the same time.  In rows of 256 bytes or more those hit the
    // same banks unless rows with bit 2 set are shifted by 8 chunks (only TN == 1 reads as little as 128 bytes per
    // half-wave); 128-byte rows (BN == 32) have no room for that shift and are stored in the order 0 4 1 5 2 6 3 7
    // instead, so that r and r + 4 lie side by side.
    constexpr bool B_PAIRED_ROWS = BN == 32;
    constexpr int B_SHIFT = (TN == 1 && !B_PAIRED_ROWS) ? 8 : 0;  // chunk shift of k rows with bit 2 set
    static_assert(!B_PAIRED_ROWS || CHUNK_AHEAD, "paired rows are read by the small-tile loop only");
    static_assert(TM >= 1 && (TN == 1 || TN == 2 || TN == 4), "wave tile");
    static_assert(BK == 16 || BK == 32, "slab depth");     // an even number of 8-deep chunks: the fragments of a slab's last
                                                            // chunk and of the next slab's first one sit in different registers
    static_assert(CB <= 64 && 64 % CB == 0 && (B_SHIFT == 0 || CB >= 16), "B copy plan");
    static_assert(A_LOADS >= 1 && B_LOADS >= 1 && A_LOADS * WAVES * 1024 == A_STAGE_BYTES &&
                  B_LOADS * WAVES * 1024 == B_STAGE_BYTES, "copy plan must divide evenly");
    static_assert(STAGES >= 2 && STAGES * STAGE_BYTES <= 160 * 1024, "LDS budget");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
    static_assert(CHUNK_AHEAD || LOADS <= BK / 2 - 1, "one direct load per k step, the deferred last step excepted");
    
    __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE_BYTES];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)lds;

    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63;
    const int wave = __builtin_amdgcn_readfirstlane(t >> 6);      // uniform: LDS destinations stay in scalar registers
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l32 = lane & 31, h = lane >> 5;

    const unsigned char* __restrict__ A = (const unsigned char*)g.A;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B;
    const size_t lda_b = (size_t)g.lda * 4, ldb_b = (size_t)g.ldb * 4;

    // ---- copy plan.  A direct load I covers rows (64 / CPR) I ..: lane -> row I * 64 / CPR + lane / CPR,
    // slot lane % CPR, fetching chunk slot ^ ((row / RP) % CPR).  B direct load I covers k rows RB I ..:
    // lane -> row position RB I + lane / CB (= the k row, except for paired rows), slot lane % CB, fetching column
    // chunk slot ^ (B_SHIFT if k row & 4).
    // Rows beyond M and column chunks beyond N are replaced by the last valid ones.
    // CONV: the A operand is gathered from an image: the K elements of an output pixel are runs of conv_seg_bytes
    // contiguous bytes (one kernel row), conv_seg_stride apart.  Mode 1: a_src[i] walks along the patch of the
    // lane's pixel, a_seg[i] is its byte position inside the current run, and every slab issued moves it on by BK
    // floats, hopping to the next image row at the end of a run.  Mode 2 (runs are whole slabs): the lanes hop
    // together, so the walk is scalar, as in the plain GEMM.
    const unsigned char* a_src[A_LOADS];
    uint32_t b_voff[B_LOADS];
    int a_chunk[A_LOADS], b_krow[B_LOADS];
    uint32_t a_seg[CONV == 1 ? A_LOADS : 1];
    const uint32_t last_row = g.M - 1, last_col_chunk = (g.N - 1) / 4;
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int I = wave * A_LOADS + i;
        const int row = I * (64 / CPR) + lane / CPR;
        a_chunk[i] = (lane % CPR) ^ ((row / RP) % CPR);
        const uint32_t grow = (m0 + row) < last_row ? (m0 + row) : last_row;
        if constexpr (CONV != 0) {
            const uint32_t py = grow / g.conv_wout, px = grow % g.conv_wout;
            const uint32_t k_bytes = a_chunk[i] * 16;
            if constexpr (CONV == 1) a_seg[i] = k_bytes % g.conv_seg_bytes;
            a_src[i] = A + (size_t)py * g.conv_py_bytes + (size_t)px * g.conv_px_bytes +
                       (size_t)(k_bytes / g.conv_seg_bytes) * g.conv_seg_stride + k_bytes % g.conv_seg_bytes;
        } else {
            a_src[i] = A + (size_t)grow * lda_b + a_chunk[i] * 16;
        }
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int I = wave * B_LOADS + i;
        const int pos = I * RB + lane / CB;                // row position inside the stage
        b_krow[i] = B_PAIRED_ROWS ? (pos & ~7) + ((pos & 7) >> 1) + 4 * (pos & 1) : pos;
        const int chunk = (lane % CB) ^ ((b_krow[i] & 4) ? B_SHIFT : 0);
        const uint32_t gchunk = (n0 / 4 + chunk) < last_col_chunk ? (n0 / 4 + chunk) : last_col_chunk;
        b_voff[i] = (uint32_t)((size_t)b_krow[i] * ldb_b + (size_t)gchunk * 16);           // < BK * ldb_b + 4 N: the launcher checks
    }

    const uint32_t full_slabs = g.K / BK, k_tail = g.K % BK;
    const uint32_t slabs = full_slabs + (k_tail ? 1u : 0u);

    // Slabs are issued in ascending order.  A direct load takes its address as a scalar base (the tile's first
    // row of A, or the image; B's row k; running along K) plus a 32-bit lane offset that never changes, so that
    // advancing to the next slab is scalar arithmetic.  Only the per-lane image walk of CONV mode 1 keeps full
    // per-lane pointers for A, each left at the next slab by its load.
    const size_t b_step = (size_t)BK * ldb_b;
    uint32_t a_voff[CONV == 1 ? 1 : A_LOADS];
    const unsigned char* a_base = CONV ? A : A + (size_t)m0 * lda_b;
    const unsigned char* b_base = B;
    uint32_t run_pos = 0;                                  // CONV mode 2: bytes of the current run already issued
    if constexpr (CONV != 1) {
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) a_voff[i] = (uint32_t)(a_src[i] - a_base);       // < BM * lda_b / the image size: the launcher checks
    }
    auto a_ptr = [&](int i) { if constexpr (CONV == 1) return a_src[i]; else return a_base + a_voff[i]; };
    auto b_ptr = [&](int i) { return b_base + b_voff[i]; };
    auto issue_one = [&](uint32_t stage, auto ic) {        // direct load ic of a full slab: A first, then B
        constexpr int idx = decltype(ic)::value;
        const uint32_t stage_off = lds_base + stage * STAGE_BYTES;
        if constexpr (idx < A_LOADS) {
            constexpr int i = idx;
            const uint32_t dst = stage_off + (uint32_t)(wave * A_LOADS + i) * 1024u;
            if constexpr (CONV != 1) {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(dst), "v"(a_voff[i]), "s"(a_base) : "memory", "m0");
                if constexpr (i == A_LOADS - 1) {
                    a_base += BK * 4;
                    if constexpr (CONV == 2) {
                        run_pos += BK * 4;
                        if (run_pos == g.conv_seg_bytes) { run_pos = 0; a_base += g.conv_seg_stride - g.conv_seg_bytes; }
                    }
                }
            } else {
                asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(dst), "v"(a_src[i]) : "memory", "m0");
                a_src[i] += BK * 4;
                a_seg[i] += BK * 4;
                while (a_seg[i] >= g.conv_seg_bytes) {
                    a_seg[i] -= g.conv_seg_bytes;
                    a_src[i] += g.conv_seg_stride - g.conv_seg_bytes;
                }
            }
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
            const uint32_t k = k0 + a_chunk[i] * 4;
            floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
            if (k < g.K) {
                v = *(const floatx4*)a_ptr(i);             // inside the pitch: lda is a multiple of 4
#pragma unroll
                for (int e = 1; e < 4; ++e) if (k + e >= g.K) v[e] = 0.f;
            }
            *(floatx4*)(st + (wave * A_LOADS + i) * 1024 + lane * 16) = v;
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            floatx4 v = floatx4{0.f, 0.f, 0.f, 0.f};
            if (k0 + b_krow[i] < g.K) v = *(const floatx4*)b_ptr(i);
            *(floatx4*)(st + A_STAGE_BYTES + (wave * B_LOADS + i) * 1024 + lane * 16) = v;
        }
    };
    auto issue_loads = [&](uint32_t slab) {                // a whole slab in one burst
        if (slab < full_slabs) static_for<0, LOADS>([&](auto ic) { issue_one(slab % STAGES, ic); });
        else issue_tail(slab % STAGES);
    };

    // ---- fragment addressing inside a stage
    const int a_row = wm0 + l32;                       // + 32 i leaves (row / RP) % CPR unchanged
    const int a_sw = (a_row / RP) % CPR;
    int a_off[BK / 8];                                 // byte offset of chunk 2 c + h of this lane's row
#pragma unroll
    for (int c = 0; c < BK / 8; ++c) a_off[c] = a_row * (BK * 4) + (((2 * c + h) ^ a_sw) * 16);
    const int b_col = wn0 + TN * l32;
    const int b_off = A_STAGE_BYTES + (B_PAIRED_ROWS ? h : 4 * h) * BN * 4 + (((b_col / 4) ^ (h ? B_SHIFT : 0)) * 16) + (b_col % 4) * 4;
    constexpr int B_ROW_STEP = (B_PAIRED_ROWS ? 2 : 1) * BN * 4;  // from k row r to r + 1 (r % 8 < 3) inside a stage

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if ((uint32_t)p < slabs) issue_loads(p);

    // Split K on tiles of one 32 x 32 block per wave: the workgroup that finds itself the one to write the tile loads
    // its 16 values of C per lane together with the first slots, instead of a round trip to memory later, in the
    // epilogue (1000 x 1500 x 777 with C: 30.2 -> 28.0 us).  It is an instantiation of its own, launched when there is a
    // C: the 16 registers cost the same kernel WITHOUT C a microsecond (26.1 -> 27.0 us), as fetching C in front of
    // the K loop cost whole products (1024^3: 21.6 -> 23.0 us), which keep their late loads.  The whole tiles of a launch
    // with split ones are compiled with the 16 registers anyway and do fetch C in front of their first slab: the wait for
    // it is the wait for that slab (1000 x 1500 x 777 with C, 256 whole tiles of 384: 8.6 % -> 4.4 % above the same without C).
    constexpr bool C_EARLY = SPLIT_WITH_C;
    static_assert(!SPLIT_WITH_C || (SPLIT && TM * TN == 1 && CONV == 0), "early C: split K on 32 x 32 wave tiles");
    float c_early[C_EARLY ? 16 : 1];
    auto load_c_early = [&]() {
        const float* __restrict__ Cp = (const float*)g.C;
        if (!Cp) return;                                   // uniform: products without C pay a scalar branch
        const uint32_t col = n0 + b_col;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm0 + 8 * (r / 4) + 4 * h + (r % 4);
            c_early[r] = (row < g.M && col < g.N) ? Cp[(size_t)row * g.ldc + col] : 0.f;
        }
    };
    if constexpr (C_EARLY) { if (sb.splits == 1) load_c_early(); }      // a whole tile
    if (slabs >= (uint32_t)(STAGES - 1)) wait_loads_and_barrier<LOADS * (STAGES - 2)>();
    else wait_loads_and_barrier<0>();

    constexpr int STEPS = BK / 2, CHUNKS = BK / 8;
    typedef typename BFrag<TN>::type bfrag;

    if constexpr (!CHUNK_AHEAD) {
        // Large wave tiles: a k step is TM * TN MFMAs, long enough to hide an LDS read, so fragments
        // are fetched a few steps ahead, one or a few reads behind the first MFMA of each step (bursts
        // of reads, and reads only one step ahead, both measure slower: LDS reads are held up while
        // direct loads land).  af[c & 1] holds chunk c of A (4 k per lane), read during chunk c - 1, a
        // quarter of it per step; bf[step & 3] the B values of a k step, read 2 steps ahead.  The MFMAs of the last
        // step of a slab are issued after the slab barrier, behind the first fragment reads of the next
        // slab (before the first slab they multiply zeros).
        floatx4 af[2][TM];
        constexpr int BF_AHEAD = 2, BFM = 3;               // B fragments are read 2 k steps ahead into a ring of 4
        bfrag bf[BFM + 1];
#pragma unroll
        for (int i = 0; i < TM; ++i) af[(CHUNKS - 1) & 1][i] = floatx4{0.f, 0.f, 0.f, 0.f};
        bf[(STEPS - 1) & BFM] = bfrag{};

        // MFMAs FIRST .. LAST-1 (in i-major order) of a k step
        auto multiply_part = [&](auto stc, auto firstc, auto lastc) {
            constexpr int step = decltype(stc)::value;
            constexpr int c = step / 4, e = step % 4;
            static_for<decltype(firstc)::value, decltype(lastc)::value>([&](auto nc) {
                constexpr int i = decltype(nc)::value / TN, j = decltype(nc)::value % TN;
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c & 1][i][e], lane_of<TN>(bf[step & BFM], j), acc[i][j], 0, 0, 0);
            });
        };
        auto multiply = [&](auto stc) {
            multiply_part(stc, std::integral_constant<int, 0>{}, std::integral_constant<int, TM * TN>{});
        };
        auto read_b = [&](const unsigned char* st, auto stc) {
            constexpr int step = decltype(stc)::value;
            bf[step & BFM] = *(const bfrag*)(st + b_off + (8 * (step / 4) + step % 4) * BN * 4);
        };

        // One slab; STAGE >= 0: its stage is known at compile time and the slab asked for meanwhile is a whole one (see
        // the small-tile loop below for what that buys), STAGE < 0: the general form.
        auto slab_body = [&](uint32_t s, auto stage_c) {
            constexpr int STAGE = decltype(stage_c)::value;
            constexpr bool STEADY = STAGE >= 0;
            const unsigned char* st;
            if constexpr (STEADY) st = lds + STAGE * STAGE_BYTES; else st = lds + (s % STAGES) * STAGE_BYTES;
            const bool more = STEADY || s + STAGES - 1 < slabs;

#pragma unroll
            for (int i = 0; i < TM; ++i) af[0][i] = *(const floatx4*)(st + a_off[0] + i * 32 * BK * 4);
            static_for<0, BF_AHEAD>([&](auto stc) { read_b(st, stc); });
            multiply(std::integral_constant<int, STEPS - 1>{});
            __builtin_amdgcn_sched_group_barrier(0x100, TM + BF_AHEAD, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
            __builtin_amdgcn_sched_barrier(0);
            // The stage that held slab s-1 is free: every wave passed the barrier after reading it.
            const uint32_t nstage = STEADY ? (uint32_t)((STAGE + STAGES - 1) % STAGES) : (s + STAGES - 1) % STAGES;
            const bool direct = STEADY || s + STAGES - 1 < full_slabs;
            if constexpr (!STEADY) { if (more && !direct) issue_tail(nstage); }

            static_for<0, STEPS - 1>([&](auto stc) {
                constexpr int step = decltype(stc)::value;
                constexpr int c = step / 4, e = step % 4;
                constexpr bool next_b = step + BF_AHEAD < STEPS;
                constexpr int a_lo = (c + 1 < CHUNKS) ? (e * TM + 3) / 4 : 0, a_hi = (c + 1 < CHUNKS) ? ((e + 1) * TM + 3) / 4 : 0;
                constexpr int reads = (next_b ? 1 : 0) + (a_hi - a_lo);
                if constexpr (next_b) read_b(st, std::integral_constant<int, step + BF_AHEAD>{});
                static_for<a_lo, a_hi>([&](auto ic) {
                    constexpr int i = decltype(ic)::value;
                    af[(c + 1) & 1][i] = *(const floatx4*)(st + a_off[(c + 1) % CHUNKS] + i * 32 * BK * 4);
                });
                multiply_part(stc, std::integral_constant<int, 0>{}, std::integral_constant<int, 1>{});
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                if constexpr (reads > 0) __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (step < LOADS) {
                    if (direct) issue_one(nstage, std::integral_constant<int, step>{});
                    __builtin_amdgcn_sched_barrier(0);
                }
                multiply_part(stc, std::integral_constant<int, 1>{}, std::integral_constant<int, TM * TN>{});
                __builtin_amdgcn_sched_barrier(0);
            });

            // slab s+1 must have landed (ours: vmcnt; everyone's: barrier); the loads of the
            // STAGES-2 slabs behind it may stay in flight.
            if (more) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
        };
        const uint32_t steady = __builtin_amdgcn_readfirstlane(full_slabs > (uint32_t)(STAGES - 1) ? (full_slabs - (uint32_t)(STAGES - 1)) / STAGES * STAGES : 0u);
        uint32_t s = 0;
        for (; s < steady; s += STAGES) static_for<0, STAGES>([&](auto jc) { slab_body(s + decltype(jc)::value, jc); });
        for (; s < slabs; ++s) slab_body(s, std::integral_constant<int, -1>{});
        multiply(std::integral_constant<int, STEPS - 1>{});
    } else {
        // Small wave tiles: a k step is one or two MFMAs, shorter than an LDS read, so fragments are
        // fetched a whole 8-deep chunk (4 steps) ahead: fa[c & 1] / fb[c & 1] hold chunk c.  The last
        // chunk of a slab is multiplied after the slab barrier, behind the reads of the next slab's
        // first chunk.
        floatx4 fa[2][TM];
        bfrag fb[2][4];
#pragma unroll
        for (int i = 0; i < TM; ++i) fa[(CHUNKS - 1) & 1][i] = floatx4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int e = 0; e < 4; ++e) fb[(CHUNKS - 1) & 1][e] = bfrag{};

        auto read_chunk = [&](const unsigned char* st, auto cc) {
            constexpr int c = decltype(cc)::value;
#pragma unroll
            for (int i = 0; i < TM; ++i) fa[c & 1][i] = *(const floatx4*)(st + a_off[c] + i * 32 * BK * 4);
#pragma unroll
            for (int e = 0; e < 4; ++e) fb[c & 1][e] = *(const bfrag*)(st + b_off + 8 * c * BN * 4 + e * B_ROW_STEP);
        };
        auto multiply_chunk = [&](auto cc) {
            constexpr int c = decltype(cc)::value;
#pragma unroll
            for (int e = 0; e < 4; ++e)
#pragma unroll
                for (int i = 0; i < TM; ++i)
#pragma unroll
                    for (int j = 0; j < TN; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(fa[c & 1][i][e], lane_of<TN>(fb[c & 1][e], j), acc[i][j], 0, 0, 0);
        };
        constexpr int READS = TM + 4, MFMAS = 4 * TM * TN;

        // One slab.  STAGE >= 0: the stage it sits in is known at compile time, and the slab that is asked for while this
        // one multiplies is a whole one (direct loads, no questions asked); STAGE < 0: the general form.  A loop over
        // STAGES such slabs is one block of code without a branch inside and without a vector ALU instruction between its
        // MFMAs: every LDS address is a register that never changes plus an immediate.  A wavefront that has its SIMD
        // to itself (one workgroup per CU) needs that: a VALU instruction issued behind an MFMA holds up the next MFMA
        // of the same accumulator chain by about 20 cycles (measured on a bare chain of v_mfma_f32_32x32x2_f32: 64
        // cycles each, 74 with two integer adds per four of them), and a taken branch leaves the matrix pipe empty
        // (1024^3, one 64 x 64 tile per CU: 84 -> 70 cycles per MFMA, 21.5 -> 18.5 us).
        auto slab_body = [&](uint32_t s, auto stage_c) {
            constexpr int STAGE = decltype(stage_c)::value;
            constexpr bool STEADY = STAGE >= 0;
            const unsigned char* st;
            if constexpr (STEADY) st = lds + STAGE * STAGE_BYTES; else st = lds + (s % STAGES) * STAGE_BYTES;
            const bool more = STEADY || s + STAGES - 1 < slabs;

            read_chunk(st, std::integral_constant<int, 0>{});
            multiply_chunk(std::integral_constant<int, CHUNKS - 1>{});
            __builtin_amdgcn_sched_group_barrier(0x100, READS, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, MFMAS, 0);
            __builtin_amdgcn_sched_barrier(0);
            if constexpr (STEADY) {
                static_for<0, LOADS>([&](auto ic) { issue_one((uint32_t)((STAGE + STAGES - 1) % STAGES), ic); });
                __builtin_amdgcn_sched_barrier(0);             // the loads stay in front of the next chunk's reads
            } else if (more) issue_loads(s + STAGES - 1);

            static_for<0, CHUNKS - 1>([&](auto cc) {
                constexpr int c = decltype(cc)::value;
                read_chunk(st, std::integral_constant<int, c + 1>{});
                multiply_chunk(cc);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x100, READS, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, MFMAS - 1, 0);
                __builtin_amdgcn_sched_barrier(0);
            });

            if (more) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
        };
        // Slabs [0, steady): the slab STAGES - 1 ahead is a whole one; they are walked STAGES at a time in the tight form,
        // in launches of at most one round of workgroups (four 64 x 64 tiles to a CU).  With more rounds the tight form loses: the
        // wavefront that is oldest on its SIMD then wins every MFMA slot it is ready for, the workgroups of a round end
        // far apart (2048^3, four per CU: between 69 and 139 us, against 108 to 142) and the rounds no longer tile
        // (3072 x 2048 x 2048, six per CU: 207 us against 188; a VALU instruction per chunk put back on purpose mends
        // 8 per CU, 245 against 249 us, but neither 6 nor 9 per CU), so those launches keep the general form, whose
        // address arithmetic and branches happen to share the matrix pipe evenly.
        const uint32_t steady = __builtin_amdgcn_readfirstlane(full_slabs > (uint32_t)(STAGES - 1) ? (full_slabs - (uint32_t)(STAGES - 1)) / STAGES * STAGES : 0u);
        constexpr uint32_t FIT = BM * BN >= 128 * 128 ? 3u : 4u;                    // workgroups of this tile that share a CU
        const bool one_round = gridDim.x <= FIT * (g_in.cus ? g_in.cus : 256u);
        uint32_t s = 0;
        if (one_round)
            for (; s < steady; s += STAGES) static_for<0, STAGES>([&](auto jc) { slab_body(s + decltype(jc)::value, jc); });
        for (; s < slabs; ++s) slab_body(s, std::integral_constant<int, -1>{});
        multiply_chunk(std::integral_constant<int, CHUNKS - 1>{});
    }

    if constexpr (SPLIT) {
        // piece c of a lane: registers 4 (c % 4) .. + 3 of its 32 x 32 tile c / 4.  The ring is free: every LDS read
        // precedes the last slab barrier.
        const bool last = sb.splits == 1 || split_k_exchange<WAVES * 64, TM * TN * 4, floatx4>(g_in, sb, (uint32_t*)lds,
            [&](auto cc) {
                constexpr int c = decltype(cc)::value, tile = c / 4, q = c % 4;
                const floatx16& a = acc[tile / TN][tile % TN];
                return floatx4{a[4 * q], a[4 * q + 1], a[4 * q + 2], a[4 * q + 3]};
            },
            [&](auto cc, const floatx4& v, bool first) {
                constexpr int c = decltype(cc)::value, tile = c / 4, q = c % 4;
                floatx16& a = acc[tile / TN][tile % TN];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float old = a[4 * q + e], w = v[e];
                    a[4 * q + e] = first ? w : old + w;
                }
            },
            [&] { if constexpr (C_EARLY) load_c_early(); });
        if (!last) return;
    }

    // Epilogue: register r of lane (l32, h) is row 8*(r/4) + 4*h + r%4 of a 32x32 tile; the
    // lane's TN tiles are TN adjacent columns.
    const float* __restrict__ C = (const float*)g.C;
    float* __restrict__ D = (float*)g.D;
    const uint32_t col0 = n0 + b_col;
    const bool interior = (m0 + BM <= g.M) && (n0 + BN <= g.N);
    const auto row_of = [&](int i, int r) { return m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * h + (r % 4); };
    const auto d_row_of = [&](uint32_t row) {              // offset of the row's first element in D
        if constexpr (CONV != 0) return (size_t)(row / g.conv_wout) * g.conv_dst_row + (size_t)(row % g.conv_wout) * g.ldd;
        else return (size_t)row * g.ldd;
    };
    constexpr bool STRAIGHT = true;
    // (the 128 x 128 and 256 x 128 tiles take it with a C only: without one it gains nothing there, and edge shapes lose 2 %)
    if (STRAIGHT && interior && (TM * TN == 1 || (!C_EARLY && C != nullptr))) {
        // Straight-line code: with a C, the loads of a batch of rows are all asked for before the first is used (a load,
        // its wait, the fma and the store row by row made the C term cost 6 % at 2048^3 and 14 % at 65536 x 256 x 1024).
        // D is written once, read by whoever comes next, often larger than L2: the streaming hint (65536 x 256 x 1024
        // 244 -> 240 us, 2048^3 122.2 -> 120.6, 1024^3 18.65 -> 18.3, 8192^3 the same).  An address is a scalar base (the
        // row: tile, wavefront, register) plus one 32-bit lane offset for all rows, so no row costs a register pair.
        const bool with_c = !C_EARLY && C != nullptr;
        const uint32_t lane_d = (uint32_t)(4 * h) * g.ldd * 4u + (uint32_t)b_col * 4u;
        const uint32_t lane_c = (uint32_t)(4 * h) * g.ldc * 4u + (uint32_t)b_col * 4u;
        // The row offsets run from row to row (1, 1, 1, 5 rows on: registers 4 q .. 4 q + 3 are rows 8 q .. 8 q + 3) behind
        // an empty asm each, or the compiler computes the 16 TM offsets of a wavefront up front and they fill the register
        // file; with and without C are two copies of the code, or both are computed and one selected.
        size_t d_off = ((size_t)(m0 + (uint32_t)wm0) * g.ldd + n0) * 4, c_off = ((size_t)(m0 + (uint32_t)wm0) * g.ldc + n0) * 4;
        const size_t d_step = (size_t)g.ldd * 4, c_step = (size_t)g.ldc * 4;
        const auto d_ptr = [&](int i, int r) {
            if constexpr (CONV != 0) return (bfrag*)(D + d_row_of(row_of(i, r)) + col0);
            else {
                bfrag* const p = (bfrag*)((unsigned char*)D + d_off + lane_d);
                d_off += (r % 4 == 3 ? 5 : 1) * d_step;
                asm volatile("" : "+s"(d_off));
                return p;
            }
        };
        const auto c_ptr = [&](int r) {
            const bfrag* const p = (const bfrag*)((const unsigned char*)C + c_off + lane_c);
            c_off += (r % 4 == 3 ? 5 : 1) * c_step;
            asm volatile("" : "+s"(c_off));
            return p;
        };
        // rows per batch: few where the accumulators fill the register file
        constexpr int G = TM * TN >= 8 ? 4 : TM * TN >= 4 ? 8 : 16;
        const auto store_all = [&](auto with_c_t) {
            constexpr bool WITH_C = decltype(with_c_t)::value;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int r0 = 0; r0 < 16; r0 += G) {
                    bfrag cv[G];
                    if constexpr (WITH_C) {
#pragma unroll
                        for (int r = 0; r < G; ++r) cv[r] = *c_ptr(r0 + r);
                    }
#pragma unroll
                    for (int q = 0; q < G; ++q) {
                        const int r = r0 + q;
                        float v[TN];
#pragma unroll
                        for (int j = 0; j < TN; ++j) v[j] = acc[i][j][r];
                        if constexpr (C_EARLY) {
                            v[0] = __builtin_fmaf(c_early[r], g.beta, g.alpha * v[0]);     // (this instantiation runs with a C only)
                        }
                        if constexpr (WITH_C) {
#pragma unroll
                            for (int j = 0; j < TN; ++j) v[j] = __builtin_fmaf(lane_of<TN>(cv[q], j), g.beta, g.alpha * v[j]);
                        }
                        bfrag o;
                        if constexpr (TN == 1) o = v[0];
                        else {
#pragma unroll
                            for (int j = 0; j < TN; ++j) o[j] = v[j];
                        }
                        __builtin_nontemporal_store(o, d_ptr(i, r));
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (with_c) store_all(std::true_type{}); else store_all(std::false_type{});
        return;
    }
    if constexpr (STRAIGHT) {
        // edge tiles, element by element; the C values of a batch of rows are asked for together here too (1000 x 1500 x 777
        // on 64 x 64 tiles, 39 edge tiles of 384: the C term cost 14.8 %)
        constexpr int G = TM * TN >= 4 ? 8 : 16;
        const auto store_edge = [&](auto with_c_t) {
            constexpr bool WITH_C = decltype(with_c_t)::value;
#pragma unroll
            for (int i = 0; i < TM; ++i) {
#pragma unroll
                for (int r0 = 0; r0 < 16; r0 += G) {
                    float cv[G][TN];
                    if constexpr (WITH_C) {
#pragma unroll
                        for (int q = 0; q < G; ++q) {
                            const uint32_t row = row_of(i, r0 + q);
#pragma unroll
                            for (int j = 0; j < TN; ++j)
                                cv[q][j] = (row < g.M && col0 + j < g.N) ? C[(size_t)row * g.ldc + col0 + j] : 0.f;
                        }
                    }
#pragma unroll
                    for (int q = 0; q < G; ++q) {
                        const int r = r0 + q;
                        const uint32_t row = row_of(i, r);
                        if (row >= g.M) continue;
                        const size_t d_row = d_row_of(row);
#pragma unroll
                        for (int j = 0; j < TN; ++j) {
                            if (col0 + j < g.N) {
                                float o = acc[i][j][r];
                                if constexpr (C_EARLY) {
                                    if (j == 0) o = __builtin_fmaf(c_early[r], g.beta, g.alpha * o);
                                }
                                if constexpr (WITH_C) o = __builtin_fmaf(cv[q][j], g.beta, g.alpha * o);
                                D[d_row + col0 + j] = o;
                            }
                        }
                    }
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        if (!C_EARLY && C != nullptr) { store_edge(std::true_type{}); return; }
    }
    // without a C to fetch: the interior tiles of the two larger tiles row by row, edge tiles element by element
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = row_of(i, r);
            const size_t d_row = d_row_of(row);
            if ((!STRAIGHT || TM * TN > 1) && interior) {
                float v[TN];
#pragma unroll
                for (int j = 0; j < TN; ++j) v[j] = acc[i][j][r];
                if constexpr (!C_EARLY) {
                    if (C) {
                        const bfrag cv = *(const bfrag*)(C + (size_t)row * g.ldc + col0);
#pragma unroll
                        for (int j = 0; j < TN; ++j) v[j] = __builtin_fmaf(lane_of<TN>(cv, j), g.beta, g.alpha * v[j]);
                    }
                }
                bfrag o;
                if constexpr (TN == 1) o = v[0];
                else {
#pragma unroll
                    for (int j = 0; j < TN; ++j) o[j] = v[j];
                }
                __builtin_nontemporal_store(o, (bfrag*)(D + d_row + col0));
            } else if (row < g.M) {
#pragma unroll
                for (int j = 0; j < TN; ++j) {
                    if (col0 + j < g.N) {
                        float o = acc[i][j][r];
                        if constexpr (C_EARLY) {
                            if (j == 0) o = __builtin_fmaf(c_early[r], g.beta, g.alpha * o);
                        } else {
                            if (C) o = __builtin_fmaf(C[(size_t)row * g.ldc + col0 + j], g.beta, g.alpha * o);
                        }
                        D[d_row + col0 + j] = o;
                    }
                }
            }
        }
    }
}

namespace {

template <int BM, int BN, int WAVES_M, int WAVES_N, int BK, int STAGES, bool CHUNK_AHEAD, int CONV = 0>
int launch_dma(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    // 256 x 128 tiles, two independent workgroups per CU: patches two tile-rows high fetch least (8192^3: 5.5 GB through
    // L2 against 6.2 GB with four rows and 11.7 GB with eight, at the same speed)
    if constexpr (BM == 256 && BN == 128 && CONV == 0) g.group_m = 2;
    // The planner splits K on the smallest tiles only.  (On 128 x 128 tiles the exchange costs the kernel a workgroup per
    // CU -- 149 VGPRs beside the 64 accumulators, two workgroups where three fit -- and whole rounds in front of a split
    // last round then gain 1 % at 5120^3 and lose at 2560^3, 3072^3 and 3584^3.)
    if (g.split_len) {
        if constexpr (CONV == 0 && BM * BN == 64 * 64) {
            const uint32_t splits = g.split_count;
            if (g.C)
                hipLaunchKernelGGL((gemm_f32_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES, CHUNK_AHEAD, 0, true, true>),
                                   dim3(g.split_first + (nb - g.split_first) * splits), dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
            else
                hipLaunchKernelGGL((gemm_f32_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES, CHUNK_AHEAD, 0, true, false>),
                                   dim3(g.split_first + (nb - g.split_first) * splits), dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
            return (int)hipGetLastError();
        } else {
            return (int)hipErrorInvalidValue;
        }
    }
    hipLaunchKernelGGL((gemm_f32_dma_kernel<BM, BN, WAVES_M, WAVES_N, BK, STAGES, CHUNK_AHEAD, CONV>), dim3(nb),
                       dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
    return (int)hipGetLastError();
}

}  // namespace

// M, N, K >= 1; 16-byte aligned bases and pitches (the caller checks).  Measured on MI355X:
//   256 x 128 (TILE_LARGE, the largest tile): 4 wavefronts of 128 x 64, 16-deep slabs in a ring of 2, two workgroups
//     per CU, each with its own slab barrier: 149.3 TFLOP/s at 8192^3.  One 256 x 256 workgroup of 8 such wavefronts
//     per CU (ring of 4) reaches 147.7-148.4 and leaves more of the chip idle on grids that are no multiple of the
//     CU count (6144^3: 110 against 133); with 64 x 128 wave tiles, 16 wavefronts, 32-deep slabs or rings of 3 to
//     5 stages it lands between 138 and 144.
//   128 x 128 and 64 x 64: 4 wavefronts, chunk-ahead fragments, and a ring of only 2 stages (32 KB): what hides the
//     copy latency for these is not a deep ring but several workgroups per CU (4 fit), e.g. 128 x 128 at
//     6144^3 147 TFLOP/s against 130 with 4 stages, 64 x 64 at 3072^3 139 against 127; with a single workgroup per CU
//     (1024^3) both rings measure the same.  Deeper rings, 64-deep slabs, a second accumulator chain and splitting K
//     over two wavefront groups changed nothing or lost; so did 64 x 64 tiles of two wavefronts of 64 x 32 (a quarter
//     less LDS traffic per flop): 2048^3 128.6 against 126.2 us, 1024^3 36.7 against 21.5 (two of the four SIMDs idle).
int launch_gemm_f32_dma(int shape, const GemmArgs& args, hipStream_t stream)
{
    switch (shape) {
    case TILE_LARGE: return launch_dma<256, 128, 2, 2, 16, 2, false>(args, stream);
    case TILE_MEDIUM: return launch_dma<128, 128, 2, 2, 16, 2, true>(args, stream);
    case TILE_SMALL:                                           // outputs of at most 32 columns: 128 x 32 tiles, no idle half
        return args.N <= kNarrowN ? launch_dma<128, 32, 4, 1, 32, 2, true>(args, stream)
                                  : launch_dma< 64, 64, 2, 2, 32, 2, true>(args, stream);
    default:           return (int)hipErrorInvalidValue;
    }
}

// 2-D convolution as an implicit GEMM: M = output pixels, N = output channels, K = kernel rows x (kernel columns x
// channel pitch); B is the kernel set packed [K][N].  Replaces cu_im2col_*_fp32 + cu_im2col_GEMM_fp32
// (srcs/modules/NN/convolution/CUDA/fp32/im2col_fp32.cu, im2col_GEMM_fp32.cu:40-106) and their im2col buffer.
int launch_conv2d_f32_dma(int shape, const GemmArgs& args, hipStream_t stream)
{
    // runs that are a whole number of slabs (e.g. 3 x 112 channels: 21 slabs of 16 floats) let all copy lanes hop
    // together; image_bytes bounds the lanes' 32-bit offsets
    const uint32_t slab_bytes = (shape == TILE_SMALL ? 32u : 16u) * 4u;
    const bool uniform = args.conv_seg_bytes % slab_bytes == 0 && args.conv_image_bytes < (1ull << 31);
    switch (shape) {
    case TILE_LARGE: return uniform ? launch_dma<256, 256, 2, 4, 16, 4, false, 2>(args, stream)     // 137 TFLOP/s on the 3 x 3 x 112 workload; 256 x 128: 136
                                      : launch_dma<256, 256, 2, 4, 16, 4, false, 1>(args, stream);
    case TILE_MEDIUM: return uniform ? launch_dma<128, 128, 2, 2, 16, 2, true, 2>(args, stream)
                                      : launch_dma<128, 128, 2, 2, 16, 2, true, 1>(args, stream);
    case TILE_SMALL:
        if (args.N <= kNarrowN)                                // at most 32 kernels, all the reference's own path takes
            return uniform ? launch_dma<128, 32, 4, 1, 32, 2, true, 2>(args, stream)
                           : launch_dma<128, 32, 4, 1, 32, 2, true, 1>(args, stream);
        return uniform ? launch_dma< 64,  64, 2, 2, 32, 2, true, 2>(args, stream)
                       : launch_dma< 64,  64, 2, 2, 32, 2, true, 1>(args, stream);
    default:           return (int)hipErrorInvalidValue;
    }
}

}  // namespace decx_hip
