// fp16 GEMM for gfx950: half inputs, fp32 accumulation on the matrix cores
// (v_mfma_f32_16x16x32_f16, the same instruction and k order as the direct-to-LDS kernels), one round-to-nearest-even conversion to half at the end.  This is
// the register-staged, fully predicated kernel for operands of any alignment and K == 0;
// 16-byte aligned operands go to the direct-to-LDS kernels (launch_gemm_f16 below routes).
//
// Replaces the reference's cu_GEMM_fp16_[F_]kernel_* (srcs/modules/BLAS/GEMM/CUDA/
// large_squares/fp16/GEMM_fp16_B128_kernels.cu), which accumulate each K chunk in fp16 and
// store fp32 words into an fp16 destination; this kernel implements the documented
// contract instead: D(half) = round(alpha * sum_k A.B + beta * C), sums in fp32.
//
// Structure of one workgroup (BM x BN tile, WAVES_M x WAVES_N wavefronts, slab depth BK):
//   * Both operands sit in LDS k-contiguous: As[BM][BK + 8], Bs[BN][BK + 8] halves, because a
//     16x16x32 MFMA wants 8 consecutive k per lane for both A and B.  A is row-major already.
//     B (row-major K x N) is transposed on the way in: a thread fetches an 8(k) x 8(n) block
//     with eight 128-bit loads, transposes it in registers with byte permutes, and writes
//     eight 128-bit rows.  The +8-half pad puts 16 consecutive rows in 16 distinct 4-bank
//     groups, so the 128-bit fragment reads are conflict-free.
//   * The wave's TN column tiles are interleaved (lane j owns columns TN*j .. TN*j+TN-1): the
//     transposing store places column TN*j + t of a wave's strip in LDS row 16*t + j, so
//     the fragment reads stay unit-stride over lanes while the epilogue stores TN
//     contiguous halves per lane.
//   * Slab s+1 travels global -> registers while slab s is multiplied; two LDS stages, one
//     barrier per slab.  Accumulators (TM x TN x 16 floats) stay in registers.
#include "gemm_common.hpp"

namespace decx_hip {

__device__ __forceinline__ uint32_t pack_lo(uint32_t even_row, uint32_t odd_row)
{   // {odd.lo16, even.lo16}
    return __builtin_amdgcn_perm(odd_row, even_row, 0x05040100u);
}
__device__ __forceinline__ uint32_t pack_hi(uint32_t even_row, uint32_t odd_row)
{   // {odd.hi16, even.hi16}
    return __builtin_amdgcn_perm(odd_row, even_row, 0x07060302u);
}

template <int BM, int BN, int BK, int WAVES_M, int WAVES_N>
__global__ void __launch_bounds__(WAVES_M * WAVES_N * 64)
gemm_f16_kernel(const GemmArgs g)
{
    constexpr int NT = WAVES_M * WAVES_N * 64;
    constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
    constexpr int TM = WM / 16, TN = WN / 16;
    constexpr int STRIDE = BK + 8;                       // halves
    constexpr int A_STAGE = BM * STRIDE, B_STAGE = BN * STRIDE;
    constexpr int A_PER = BM * BK / 8 / NT;              // 16-byte chunks of A per thread
    constexpr int B_PER = (BK / 8) * (BN / 8) / NT;      // 8x8 blocks of B per thread
    static_assert(A_PER >= 1 && B_PER >= 1, "tile too small for the workgroup");
    static_assert(BK % 32 == 0 && WM % 16 == 0 && WN % 16 == 0 && (TN == 4 || TN == 8), "shape");

    __shared__ __attribute__((aligned(16))) _Float16 lds[2 * (A_STAGE + B_STAGE)];
    _Float16* const As = lds;
    _Float16* const Bs = lds + 2 * A_STAGE;

    uint32_t tile_m, tile_n;
    block_to_tile(g, tile_m, tile_n);
    const uint32_t m0 = tile_m * BM, n0 = tile_n * BN;

    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int wm0 = (wave / WAVES_N) * WM, wn0 = (wave % WAVES_N) * WN;
    const int l16 = lane & 15, kg = lane >> 4;          // row / column inside a 16 x 16 tile, group of 8 k

    const uint16_t* __restrict__ A = (const uint16_t*)g.A;
    const uint16_t* __restrict__ B = (const uint16_t*)g.B;

    uintx4 ra[A_PER];
    uintx4 rb[B_PER][8];

    auto load8 = [&](const uint16_t* p, uint32_t first, uint32_t limit) -> uintx4 {
        // 8 consecutive halves starting at index `first` of a row whose valid length is `limit`
        uintx4 v = {0u, 0u, 0u, 0u};
        if (g.vec_ok && first + 7 < limit) return *(const uintx4*)p;
#pragma unroll
        for (int e = 0; e < 8; ++e)
            if (first + e < limit) v[e / 2] |= (uint32_t)p[e] << (16 * (e & 1));
        return v;
    };

    // Interior tiles and interior slabs of the predicated variant skip the per-element guards
    // (uniform tests, scalar branches).
    const bool rows_inside = g.vec_ok && (m0 + BM <= g.M);
    const bool cols_inside = g.vec_ok && (n0 + BN <= g.N);

    auto load_slab = [&](uint32_t k0) {
        const bool k_inside = k0 + BK <= g.K;
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int q = t + i * NT;
            const uint32_t gm = m0 + q / (BK / 8), gk = k0 + (q % (BK / 8)) * 8;
            const uint16_t* p = A + (size_t)gm * g.lda + gk;
            if (rows_inside && k_inside) ra[i] = *(const uintx4*)p;
            else {
                uintx4 v = {0u, 0u, 0u, 0u};
                if (gm < g.M) v = load8(p, gk, g.K);
                ra[i] = v;
            }
        }
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            const int q = t + i * NT;
            const uint32_t gk = k0 + (q % (BK / 8)) * 8, gn = n0 + (q / (BK / 8)) * 8;
#pragma unroll
            for (int r = 0; r < 8; ++r) {
                const uint16_t* p = B + (size_t)(gk + r) * g.ldb + gn;
                if (cols_inside && k_inside) rb[i][r] = *(const uintx4*)p;
                else {
                    uintx4 v = {0u, 0u, 0u, 0u};
                    if (gk + r < g.K) v = load8(p, gn, g.N);
                    rb[i][r] = v;
                }
            }
        }
    };

    auto store_slab = [&](int buf) {
#pragma unroll
        for (int i = 0; i < A_PER; ++i) {
            const int q = t + i * NT;
            *(uintx4*)&As[buf * A_STAGE + (q / (BK / 8)) * STRIDE + (q % (BK / 8)) * 8] = ra[i];
        }
#pragma unroll
        for (int i = 0; i < B_PER; ++i) {
            const int q = t + i * NT;
            const int k8 = q % (BK / 8), n8 = q / (BK / 8);
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                // column c of the 8x8 block: halves of rows 0..7, two rows per word
                uintx4 col;
#pragma unroll
                for (int w = 0; w < 4; ++w)
                    col[w] = (c & 1) ? pack_hi(rb[i][2 * w][c / 2], rb[i][2 * w + 1][c / 2])
                                     : pack_lo(rb[i][2 * w][c / 2], rb[i][2 * w + 1][c / 2]);
                const int n = n8 * 8 + c;                 // column inside the block tile
                const int cw = n % WN;                    // column inside its wave strip
                const int row = (n / WN) * WN + 16 * (cw % TN) + cw / TN;
                *(uintx4*)&Bs[buf * B_STAGE + row * STRIDE + k8 * 8] = col;
            }
        }
    };

    floatx4 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) acc[i][j][r] = 0.f;

    const uint32_t slabs = (g.K + BK - 1) / BK;
    load_slab(0);
    store_slab(0);
    __syncthreads();

    for (uint32_t s = 0; s < slabs; ++s) {
        const int buf = s & 1;
        if (s + 1 < slabs) load_slab((s + 1) * BK);

        const _Float16* a_base = As + buf * A_STAGE + (wm0 + l16) * STRIDE + 8 * kg;
        const _Float16* b_base = Bs + buf * B_STAGE + (wn0 + l16) * STRIDE + 8 * kg;
#pragma unroll
        for (int ks = 0; ks < BK / 32; ++ks) {
            halfx8 af[TM], bf[TN];
#pragma unroll
            for (int i = 0; i < TM; ++i) af[i] = *(const halfx8*)(a_base + i * 16 * STRIDE + 32 * ks);
#pragma unroll
            for (int j = 0; j < TN; ++j) bf[j] = *(const halfx8*)(b_base + j * 16 * STRIDE + 32 * ks);
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af[i], bf[j], acc[i][j], 0, 0, 0);
        }

        if (s + 1 < slabs) store_slab(buf ^ 1);
        __syncthreads();
    }

    // Epilogue: register r of lane (kg, l16) is row 4 * kg + r, column l16 of a 16 x 16 tile;
    // the lane's TN tiles are TN adjacent columns.
    const _Float16* __restrict__ C = (const _Float16*)g.C;
    _Float16* __restrict__ D = (_Float16*)g.D;
    const uint32_t col0 = n0 + wn0 + TN * l16;
    typedef _Float16 hvec __attribute__((ext_vector_type(TN)));
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            const uint32_t row = m0 + wm0 + i * 16 + 4 * kg + r;
            float v[TN];
#pragma unroll
            for (int j = 0; j < TN; ++j) v[j] = acc[i][j][r];
            if (rows_inside && cols_inside) {
                if (C) {
                    const hvec cv = *(const hvec*)(C + (size_t)row * g.ldc + col0);
#pragma unroll
                    for (int j = 0; j < TN; ++j) v[j] = __builtin_fmaf((float)cv[j], g.beta, g.alpha * v[j]);
                }
                hvec out;
#pragma unroll
                for (int j = 0; j < TN; ++j) out[j] = (_Float16)v[j];
                *(hvec*)(D + (size_t)row * g.ldd + col0) = out;
            } else {
                if (row < g.M) {
#pragma unroll
                    for (int j = 0; j < TN; ++j) {
                        if (col0 + j < g.N) {
                            float o = v[j];
                            if (C) o = __builtin_fmaf((float)C[(size_t)row * g.ldc + col0 + j], g.beta, g.alpha * o);
                            D[(size_t)row * g.ldd + col0 + j] = (_Float16)o;
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
    hipLaunchKernelGGL((gemm_f16_kernel<BM, BN, BK, WAVES_M, WAVES_N>), dim3(nb), dim3(WAVES_M * WAVES_N * 64), 0, stream, g);
    return (int)hipGetLastError();
}

int launch_gemm_f16(int shape, bool edge, const GemmArgs& args, hipStream_t stream)
{
    if (!edge && args.vec_ok && args.K > 0 && dma_offsets_fit(args, 2)) return launch_gemm_f16_dma(shape, args, stream);
    switch (shape) {
    case TILE_F16_192x192: case TILE_F16_192x256: case TILE_F16_256x192:        // (classes of the direct-to-LDS family only)
    case TILE_LARGE: return launch_shape<256, 256, 64, 2, 2>(args, stream);
    case TILE_MEDIUM: return launch_shape<128, 128, 64, 2, 1>(args, stream);
    case TILE_SMALL:   return launch_shape< 64,  64, 64, 1, 1>(args, stream);
    default:           return (int)hipErrorInvalidValue;
    }
}

}  // namespace decx_hip
