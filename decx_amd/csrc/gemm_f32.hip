// fp32 GEMM for gfx950 on the fp32 matrix cores (v_mfma_f32_32x32x2_f32): the register-staged,
// fully predicated kernel.  It takes operands of any alignment (element loads where 128-bit
// ones would be misaligned; tiles that lie inside aligned matrices still take 128-bit loads)
// and K == 0.  16-byte aligned operands, the usual case (the reference's device pitch rule
// guarantees them), go to the direct-to-LDS kernels instead; launch_gemm_f32 below routes.
//
// Structure of one workgroup (BM x BN output tile, WAVES_M x WAVES_N wavefronts):
//   * K is walked in slabs of BK.  Slab s+1 travels global -> registers (128-bit loads)
//     while slab s is multiplied out of LDS; one barrier per slab, two LDS stages.
//   * A slab in LDS: [BM][BK + 4] floats.  A lane reads 4 consecutive k of one row with one
//     128-bit read; the +4 pad makes 16 consecutive rows start in 16 distinct 4-bank
//     groups, so the read is conflict-free.
//   * B slab in LDS: [BK][BN] floats, a straight copy of global.  A wave's TN column tiles
//     are interleaved (lane j owns columns TN*j .. TN*j+TN-1), so one 64/128-bit read
//     feeds all TN MFMAs of a k step and the epilogue stores TN contiguous floats per lane.
//   * MFMA 32x32x2: the lower 32 lanes supply k = kk, the upper 32 lanes k = kk + 4 of each
//     8-deep chunk (any pairing of k's is valid as long as A and B agree), which is what
//     lets A be fetched 4 k's at a time.
//   * Accumulators live in registers for the whole K loop: TM x TN tiles of 16 floats.
//
// Per-element arithmetic: products and sums in IEEE fp32 inside the MFMA unit, k ascending
// within a lane half; epilogue D = fma(C, beta, alpha * acc) as the reference's F kernels
// do (GEMM_fp32_B128_kernels.cu:725-744).
#include "gemm_common.hpp"
#include "split_k_exchange.hpp"

#include <type_traits>

namespace decx_hip {

template <int TN> struct BFrag;
template <> struct BFrag<1> { typedef float type; };
template <> struct BFrag<2> { typedef floatx2 type; };
template <> struct BFrag<4> { typedef floatx4 type; };

template <int TN> __device__ __forceinline__ float bfrag_get(const typename BFrag<TN>::type& v, int i)
{
    if constexpr (TN == 1) return v; else return v[i];
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_f32_kernel(const GemmArgs g)
{
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 32, TN = WN / 32;
    constexpr int A_STRIDE = BK + 4;
    constexpr int A_STAGE = BM * A_STRIDE, B_STAGE = BK * BN;
    constexpr int A_PER = BM * BK / 4 / NT, B_PER = BK * BN / 4 / NT;
    static_assert(A_PER >= 1 && B_PER >= 1, "tile too small for the workgroup");
    static_assert(BK % 8 == 0 && WM % 32 == 0 && WN % 32 == 0, "shape");
    typedef typename BFrag<TN>::type bvec;

    __shared__ __attribute__((aligned(16))) float lds[2 * (A_STAGE + B_STAGE)];
    float* const As = lds;
    float* const Bs = lds + 2 * A_STAGE;

    uint32_t tile_m, tile_n;
    block_to_tile(g, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l32 = lane & 31, h = lane >> 5;

    const float* __restrict__ A = (const float*)g.A;
    const float* __restrict__ B = (const float*)g.B;

    floatx4 ra[A_PER], rb[B_PER];

    // In the predicated variant most of the work is still interior: a tile that lies fully
    // inside M (or N) and a slab that lies fully inside K need no per-element guards.  These
    // tests are uniform over the workgroup, so they cost a scalar branch.
    const bool rows_inside = g.vec_ok && (m0 + BM <= g.M);
    const bool cols_inside = g.vec_ok && (n0 + BN <= g.N);

    auto load_slab = [&](uint32_t k0) {
        const bool k_inside = k0 + BK <= g.K;
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int q = t + i * NT;
            const uint32_t gm = m0 + q / (BK / 4), gk = k0 + (q % (BK / 4)) * 4;
            const float* p = A + (size_t)gm * g.lda + gk;
            if (rows_inside && k_inside) {
                ra[i] = *(const floatx4*)p;
            } else {
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (gm < g.M) {
                    if (g.vec_ok && gk + 3 < g.K) v = *(const floatx4*)p;
                    else {
                        if (gk     < g.K) v.x = p[0];
                        if (gk + 1 < g.K) v.y = p[1];
                        if (gk + 2 < g.K) v.z = p[2];
                        if (gk + 3 < g.K) v.w = p[3];
                    }
                }
                ra[i] = v;
            }
        }
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            const int q = t + i * NT;
            const uint32_t gk = k0 + q / (BN / 4), gn = n0 + (q % (BN / 4)) * 4;
            const float* p = B + (size_t)gk * g.ldb + gn;
            if (cols_inside && k_inside) {
                rb[i] = *(const floatx4*)p;
            } else {
                floatx4 v = {0.f, 0.f, 0.f, 0.f};
                if (gk < g.K) {
                    if (g.vec_ok && gn + 3 < g.N) v = *(const floatx4*)p;
                    else {
                        if (gn     < g.N) v.x = p[0];
                        if (gn + 1 < g.N) v.y = p[1];
                        if (gn + 2 < g.N) v.z = p[2];
                        if (gn + 3 < g.N) v.w = p[3];
                    }
                }
                rb[i] = v;
            }
        }
    };

    auto store_slab = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int q = t + i * NT;
            *(floatx4*)&As[buf * A_STAGE + (q / (BK / 4)) * A_STRIDE + (q % (BK / 4)) * 4] = ra[i];
        }
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            const int q = t + i * NT;
            *(floatx4*)&Bs[buf * B_STAGE + (q / (BN / 4)) * BN + (q % (BN / 4)) * 4] = rb[i];
        }
    };

    floatx16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

    const uint32_t slabs = (g.K + BK - 1) / BK;
    load_slab(0);
    store_slab(0);
    __syncthreads();

    for (uint32_t s = 0; s < slabs; ++s) {
        const int buf = s & 1;
        if (s + 1 < slabs) load_slab((s + 1) * BK);

        // The slab is walked in k steps of 2 (one MFMA per tile each).  Fragments are fetched
        // one step ahead into a second register set, and the group barriers keep every LDS
        // read directly behind the first MFMA of the step before it, so its latency is
        // covered by the remaining MFMAs instead of stalling the matrix pipe once per step.
        const float* a_base = As + buf * A_STAGE + (wm0 + l32) * A_STRIDE + 4 * h;
        const float* b_base = Bs + buf * B_STAGE + (4 * h) * BN + wn0 + TN * l32;
        constexpr int STEPS = BK / 2, CHUNKS = BK / 8;
        floatx4 af[2][TM];
        bvec bf[2];
#pragma unroll
        for (int i = 0; i < TM; ++i) af[0][i] = *(const floatx4*)(a_base + i * 32 * A_STRIDE);
        bf[0] = *(const bvec*)(b_base);
        __builtin_amdgcn_sched_barrier(0);
        static_for<0, STEPS>([&](auto stc) {
            constexpr int st = decltype(stc)::value;
            constexpr int c = st / 4, e = st % 4;
            constexpr bool next_b = st + 1 < STEPS;
            constexpr bool next_a = (e == 1) && (c + 1 < CHUNKS);
            constexpr int reads = (next_b ? 1 : 0) + (next_a ? TM : 0);
            if constexpr (next_b)
                bf[(st + 1) & 1] = *(const bvec*)(b_base + (8 * ((st + 1) / 4) + (st + 1) % 4) * BN);
            if constexpr (next_a) {
#pragma unroll
                for (int i = 0; i < TM; ++i)
                    af[(c + 1) & 1][i] = *(const floatx4*)(a_base + i * 32 * A_STRIDE + 8 * (c + 1));
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[c & 1][i][e], bfrag_get<TN>(bf[st & 1], j),
                                                                     acc[i][j], 0, 0, 0);
            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);                          // one MFMA
            if constexpr (reads > 0) __builtin_amdgcn_sched_group_barrier(0x100, reads, 0);   // this step's LDS reads
            if constexpr (TM * TN > 1) __builtin_amdgcn_sched_group_barrier(0x008, TM * TN - 1, 0);   // the other MFMAs
            __builtin_amdgcn_sched_barrier(0);                                          // steps stay in order
        });

        if (s + 1 < slabs) store_slab(buf ^ 1);
        __syncthreads();
    }

    // Epilogue.  MFMA 32x32 result layout: register r of lane (l32, h) is row
    // 8*(r/4) + 4*h + r%4, column l32 of the tile; column tiles are interleaved (see above).
    const float* __restrict__ C = (const float*)g.C;
    float* __restrict__ D = (float*)g.D;
    const uint32_t col0 = n0 + wn0 + TN * l32;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const uint32_t row = m0 + wm0 + i * 32 + 8 * (r / 4) + 4 * h + (r % 4);
            float v[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] = acc[i][j][r];
            if (rows_inside && cols_inside) {
                if (C) {
                    const bvec cv = *(const bvec*)(C + (size_t)row * g.ldc + col0);
#pragma unroll
                    for (int j = 0; j < TN; ++j) v[j] = __builtin_fmaf(bfrag_get<TN>(cv, j), g.beta, g.alpha * v[j]);
                }
                bvec out;
                if constexpr (TN == 1) out = v[0];
                else {
#pragma unroll
                    for (int j = 0; j < TN; ++j) out[j] = v[j];
                }
                *(bvec*)(D + (size_t)row * g.ldd + col0) = out;
            } else {
                if (row < g.M) {
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        if (col0 + j < g.N) {
                            float o = v[j];
                            if (C) o = __builtin_fmaf(C[(size_t)row * g.ldc + col0 + j], g.beta, g.alpha * o);
                            D[(size_t)row * g.ldd + col0 + j] = o;
                        }
                    }
                }
            }
        }
    }
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
static int launch_shape(const GemmArgs& args, hipStream_t stream)
{
    GemmArgs g = args;
    g.tiles_m = (g.M + BM - 1) / BM;
    g.tiles_n = (g.N + BN - 1) / BN;
    const uint32_t nb = g.tiles_m * g.tiles_n;
    hipLaunchKernelGGL((gemm_f32_kernel<BM, BN, BK, WAVES_M, WAVES_N>), dim3(nb), dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
    return (int)hipGetLastError();
}

int launch_gemm_f32(int shape, bool edge, const GemmArgs& args, hipStream_t stream)
{
    if (!edge && args.vec_ok && args.K > 0 && dma_offsets_fit(args, 4)) return launch_gemm_f32_dma(shape, args, stream);
    switch (shape) {
    case TILE_LARGE: return launch_shape<256, 256, 16, 4, 2>(args, stream);
    case TILE_MEDIUM: return launch_shape<128, 128, 16, 2, 2>(args, stream);
    case TILE_SMALL:   return launch_shape< 64,  64, 16, 2, 2>(args, stream);
    default:           return (int)hipErrorInvalidValue;
    }
}

}  // namespace decx_hip
