// fp32 GEMM, the full-tile fast path for gfx950: 256 x 256 block tile, 8 wavefronts of
// 64 x 128, K slabs of 16 copied global -> LDS by direct (LDS-DMA) 128-bit loads into a ring
// of STAGES stages.
//
// Same arithmetic and the same fragment scheme as gemm_f32_kernel (v_mfma_f32_32x32x2_f32,
// lower / upper half-waves take k and k+4 of each 8-deep chunk, interleaved column tiles);
// what changes is how the slabs reach LDS.  The register-staged kernel fetches one slab
// ahead and every wave then waits at the slab barrier for the slowest load of any wave;
// measured on 8192^3 that costs 8 % (152 TFLOP/s without the copy, 139 with it).  Here
//   * `global_load_lds_dwordx4` writes LDS directly: no staging registers, no ds_write,
//     so the ring can be STAGES - 1 slabs deep and late loads are absorbed;
//   * the A slab is stored unpadded, [256 rows][4 chunks of 16 bytes], with the chunks of a
//     row permuted (chunk c of row r sits in slot c ^ ((r >> 2) & 3)) on the global side of
//     the copy, which makes the 128-bit fragment reads of 16 consecutive rows hit 16
//     distinct bank groups; the B slab [16][256] is a straight copy as before;
//   * the direct loads are inline assembly and the barrier is a bare `s_barrier` with an
//     explicit vmcnt wait, because the compiler would otherwise wait for every outstanding
//     load in front of each LDS read and at each __syncthreads().
#include "gemm_common.hpp"
#include <type_traits>

namespace decx_hip {

namespace {

constexpr int BM = 256, BN = 256, BK = 16;
constexpr int WAVES_M = 4, WAVES_N = 2, NT = WAVES_M * WAVES_N * 64;
constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;       // 64 x 128
constexpr int TM = WM / 32, TN = WN / 32;                 // 2 x 4 MFMA tiles
constexpr int A_STAGE_BYTES = BM * BK * 4;                // 16 KB
constexpr int B_STAGE_BYTES = BK * BN * 4;                // 16 KB
constexpr int STAGE_BYTES = A_STAGE_BYTES + B_STAGE_BYTES;
constexpr int A_LOADS = A_STAGE_BYTES / 1024 / (NT / 64); // direct loads per wave per slab: 2
constexpr int B_LOADS = B_STAGE_BYTES / 1024 / (NT / 64); // 2
constexpr int LOADS = A_LOADS + B_LOADS;

typedef __attribute__((address_space(3))) void lds_void;

template <int I, int N, class F> __device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

template <int N> __device__ __forceinline__ void wait_loads_and_barrier()
{
    asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)\n\ts_barrier" :: "n"(N) : "memory");
}

}  // namespace

template <int STAGES>
__global__ void __launch_bounds__(NT)
gemm_f32_pipelined_kernel(const GemmArgs g)
{
    static_assert(STAGES >= 2 && STAGES * STAGE_BYTES <= 160 * 1024, "LDS budget");
    static_assert(LOADS * (STAGES - 1) < 64, "vmcnt is a 6-bit counter");
    __shared__ __attribute__((aligned(1024))) unsigned char lds[STAGES * STAGE_BYTES];
    const uint32_t lds_base = (uint32_t)(uintptr_t)(lds_void*)lds;

    uint32_t tile_m, tile_n;
    block_to_tile(g, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l32 = lane & 31, h = lane >> 5;

    const unsigned char* __restrict__ A = (const unsigned char*)g.A;
    const unsigned char* __restrict__ B = (const unsigned char*)g.B;
    const size_t lda_b = (size_t)g.lda * 4, ldb_b = (size_t)g.ldb * 4;

    // ---- copy plan.  A instruction I (0..15) covers rows 16 I .. 16 I + 15: lane -> row
    // 16 I + lane / 4, slot lane % 4, fetching chunk slot ^ ((row >> 2) & 3).  B instruction I
    // (0..15) is k-row I: lane -> 16 bytes at column 4 * lane.
    const unsigned char* a_src[A_LOADS];
    const unsigned char* b_src[B_LOADS];
#pragma unroll
    for (int i = 0; i < A_LOADS; ++i) {
        const int I = wave * A_LOADS + i;
        const int row = 16 * I + (lane >> 2);
        const int chunk = (lane & 3) ^ ((row >> 2) & 3);
        a_src[i] = A + (size_t)(m0 + row) * lda_b + chunk * 16;
    }
#pragma unroll
    for (int i = 0; i < B_LOADS; ++i) {
        const int I = wave * B_LOADS + i;
        b_src[i] = B + (size_t)I * ldb_b + (size_t)n0 * 4 + lane * 16;
    }

    auto issue_loads = [&](uint32_t slab) {
        const uint32_t stage_off = lds_base + (slab % STAGES) * STAGE_BYTES;
#pragma unroll
        for (int i = 0; i < A_LOADS; ++i) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(stage_off + (uint32_t)(wave * A_LOADS + i) * 1024u);
            const unsigned char* src = a_src[i] + (size_t)slab * (BK * 4);
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(dst), "v"(src) : "memory", "m0");
        }
#pragma unroll
        for (int i = 0; i < B_LOADS; ++i) {
            const uint32_t dst = __builtin_amdgcn_readfirstlane(stage_off + A_STAGE_BYTES +
                                                                (uint32_t)(wave * B_LOADS + i) * 1024u);
            const unsigned char* src = b_src[i] + (size_t)slab * BK * ldb_b;
            asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(dst), "v"(src) : "memory", "m0");
        }
    };

    // ---- fragment addressing inside a stage
    const int a_row = wm0 + l32;                       // + 32 i, which leaves (row >> 2) & 3 unchanged
    const int a_sw = (a_row >> 2) & 3;
    int a_off[BK / 8];                                 // byte offset of chunk 2 c + h of this lane's row
#pragma unroll
    for (int c = 0; c < BK / 8; ++c) a_off[c] = a_row * 64 + (((2 * c + h) ^ a_sw) * 16);
    const int b_off = A_STAGE_BYTES + ((4 * h) * BN + wn0 + TN * l32) * 4;

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const uint32_t slabs = g.K / BK;
#pragma unroll
    for (int p = 0; p < STAGES - 1; ++p)
        if ((uint32_t)p < slabs) issue_loads(p);
    if (slabs >= (uint32_t)(STAGES - 1)) wait_loads_and_barrier<LOADS * (STAGES - 2)>();
    else wait_loads_and_barrier<0>();

    // Fragment registers: af[c & 1] holds chunk c of A (4 k per lane), bf[step & 1] the B values
    // of a k step.  The MFMAs of the last step of a slab are issued after the slab barrier,
    // behind the first fragment reads of the next slab, so the matrix pipe has work while
    // those reads are in flight (before the first slab they multiply zeros).
    constexpr int STEPS = BK / 2, CHUNKS = BK / 8;
    floatx4 af[2][TM];
    floatx4 bf[2];
#pragma unroll
    for (int i = 0; i < TM; ++i) af[(CHUNKS - 1) & 1][i] = floatx4{0.f, 0.f, 0.f, 0.f};
    bf[(STEPS - 1) & 1] = floatx4{0.f, 0.f, 0.f, 0.f};

    auto multiply = [&](auto stc) {
        constexpr int step = decltype(stc)::value;
        constexpr int c = step / 4, e = step % 4;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c & 1][i][e], bf[step & 1][j], acc[i][j], 0, 0, 0);
    };

    for (uint32_t s = 0; s < slabs; ++s) {
        const unsigned char* st = lds + (s % STAGES) * STAGE_BYTES;
        const bool more = s + STAGES - 1 < slabs;

        // first fragments of this slab, then the deferred last step of the previous one
#pragma unroll
        for (int i = 0; i < TM; ++i) af[0][i] = *(const floatx4*)(st + a_off[0] + i * 32 * 64);
        bf[0] = *(const floatx4*)(st + b_off);
        multiply(std::integral_constant<int, STEPS - 1>{});
        __builtin_amdgcn_sched_group_barrier(0x100, TM + 1, 0);
        __builtin_amdgcn_sched_group_barrier(0x008, TM * TN, 0);
        __builtin_amdgcn_sched_barrier(0);
        // the stage that held slab s-1 is free: every wave passed the barrier after reading it
        if (more) issue_loads(s + STAGES - 1);

        // steps 0 .. STEPS-2: fragments fetched one step ahead, each LDS read pinned behind
        // the first MFMA of the step before the one that uses it
        static_for<0, STEPS - 1>([&](auto stc) {
            constexpr int step = decltype(stc)::value;
            constexpr int c = step / 4, e = step % 4;
            constexpr bool next_a = (e == 1) && (c + 1 < CHUNKS);
            constexpr int reads = 1 + (next_a ? TM : 0);
            bf[(step + 1) & 1] = *(const floatx4*)(st + b_off + (8 * ((step + 1) / 4) + (step + 1) % 4) * BN * 4);
            if constexpr (next_a) {
#pragma unroll
                for (int i = 0; i < TM; ++i) af[(c + 1) & 1][i] = *(const floatx4*)(st + a_off[c + 1] + i * 32 * 64);
            }
            multiply(stc);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
            __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1, 0);
            __builtin_amdgcn_sched_barrier(0);
        });

        // slab s+1 must have landed (ours: vmcnt; everyone's: barrier); the loads of the
        // STAGES-2 slabs behind it may stay in flight.  The fragments of the last step are in
        // registers (lgkmcnt(0)), so the stage is free once every wave is here.
        if (more) wait_loads_and_barrier<LOADS * (STAGES - 2)>(); else wait_loads_and_barrier<0>();
    }
    multiply(std::integral_constant<int, STEPS - 1>{});

    // Epilogue: register r of lane (l32, h) is row 8*(r/4) + 4*h + r%4 of a 32x32 tile; the
    // lane's TN tiles are TN adjacent columns.
    const float* __restrict__ C = (const float*)g.C;
    float* __restrict__ D = (float*)g.D;
    const uint32_t col0 = n0 + wn0 + TN * l32;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
            floatx4 v;
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] = acc[i][j][r];
            if (C) {
                const floatx4 cv = *(const floatx4*)(C + (size_t)row * g.ldc + col0);
#pragma unroll
                for (int j = 0; j < TN; ++j) v[j] = __builtin_fmaf(cv[j], g.beta, g.alpha * v[j]);
            }
            *(floatx4*)(D + (size_t)row * g.ldd + col0) = v;
        }
    }
}

// Full tiles only: M, N multiples of 256, K a positive multiple of 16, 16-byte aligned bases
// and pitches.  The caller checks.
int launch_gemm_f32_pipelined(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = g.M / BM;
    g.tiles_n = g.N / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    g.xcd_remap = (nb % kXcds == 0) ? 1u : 0u;
    // ring depth: 2, 3 and 4 stages measure the same, 5 is slower; 4 leaves slack for late loads
    hipLaunchKernelGGL((gemm_f32_pipelined_kernel<4>), dim3(nb), dim3(NT), 0, stream, g);
    return (int)hipGetLastError();
}

}  // namespace decx_hip
