// Direct 2-D convolution for shallow patches and few kernels (fp32), gfx950.
//
// The implicit GEMM of gemm_f32_dma.hip pays a workgroup's prologue, two slab barriers and an epilogue per
// 128 output pixels; with a patch of a few dozen values and at most 32 kernels (a 3 x 3 filter bank over an
// RGB image: K = 36) that is nearly all it does.  Here a lane owns one output pixel: it walks the KH runs of
// KW x channel-pitch contiguous floats of its patch with 128-bit loads (neighbouring lanes read neighbouring
// pixels, so the loads coalesce) and multiplies every value into one accumulator per kernel.  The weights of
// a patch element are the same for all lanes, so they come through scalar loads and cost no vector
// instruction; the vector pipe does one fma per (pixel, patch element, kernel), which is the arithmetic itself.
//
// What bounds it is the memory system's rate for traffic that is mostly writes (1920 x 1080 x 3, 8 kernels: 25 MB in,
// 66 MB out in 20.5-23 us; a copy kernel in the access order this part answers best moves 5.7-6.0 TB/s of reads plus
// writes, i.e. 15 us for these 91 MB, and a launch of next to nothing takes 4 us):
// the same arithmetic on the matrix cores (v_mfma_f32_4x4x1_16b_f32 with the weights of four kernels as one operand and
// the lane's own patch element as the other leaves every lane with its pixel's four outputs, bit for bit the same chain,
// in a sixteenth of the instructions) measured 23.2 us there and lost on smaller and larger images (640 x 480: 8.5
// against 6.9 us, 3840 x 2160: 143 against 126), so it is not in here; with the stores below and the weights in LDS it
// lost again (8 kernels 23.5 against 22.8 us, 16 kernels 46.8 against 34.5, 32 kernels at 1000 x 700: 40.7 against 24.3).
//
// Same operands and layouts as the GEMM form (image [row][column][channel pitch], kernels packed
// [patch element][kernel] with zero rows for padded channels, destination [row][column][channel pitch]), same
// k-ascending fma chain per output as the CPU oracle.  Replaces, for these sizes, the same reference path:
// cu_im2col_*_fp32 + cu_im2col_GEMM_fp32 (srcs/modules/NN/convolution/CUDA/fp32/im2col_fp32.cu,
// im2col_GEMM_fp32.cu:40-106).
#include "gemm_common.hpp"

namespace decx_hip {

namespace {

// Hardware deals consecutive workgroups to the 8 XCDs in turn, and each XCD has an L2 of its own.  An output row
// needs KH rows of the image, most of which the rows above and below need as well: workgroup b takes the b / 8-th tile
// of XCD b % 8's contiguous share of the pixels, so that an XCD works its way down a band of rows and finds the rows it
// fetched for the last output row in its L2 (1920 x 1080 x 3, 3 x 3: 67.9 MB fetched per launch before, the image is 24.9).
__device__ __forceinline__ uint32_t xcd_contiguous(uint32_t block, uint32_t blocks)
{
    const uint32_t per_xcd = blocks / kXcds;
    return block < per_xcd * kXcds ? (block % kXcds) * per_xcd + block / kXcds : block;
}

// NACC: accumulators per pixel = kernels rounded up to a multiple of 4 (never beyond the pitch of the packed kernels).
// REAL: channels of a 16-byte group that exist; below 4 only for a channel pitch of 4 with 1 to 3 channels (grey, RGB),
// whose padding channel meets zero weights and is left out of the arithmetic.
template <int NACC, int REAL>
__global__ void __launch_bounds__(256)
conv2d_direct_kernel(const float* __restrict__ image, const float* __restrict__ kmat, float* __restrict__ dst,
                     uint32_t out_w, uint32_t pixels, uint32_t out_c, uint32_t k_h, uint32_t seg_floats,
                     uint64_t row_floats, uint32_t px_floats, uint64_t py_floats, uint32_t kmat_pitch,
                     uint32_t dst_dpitch, uint32_t dst_wpitch)
{
    const uint32_t p = xcd_contiguous(blockIdx.x, gridDim.x) * 256 + threadIdx.x;
    const bool live = p < pixels;
    const uint32_t q = live ? p : pixels - 1;              // idle lanes of the last workgroup repeat the last pixel
    const uint32_t oy = q / out_w, ox = q % out_w;
    const float* patch = image + (size_t)oy * py_floats + (size_t)ox * px_floats;
    float acc[NACC];
#pragma unroll
    for (int o = 0; o < NACC; ++o) acc[o] = 0.f;

    const float* w = kmat;                             // row k of the packed kernels: the same for every lane
    for (uint32_t kh = 0; kh < k_h; ++kh) {
        const float* run = patch + (size_t)kh * row_floats;
        for (uint32_t e = 0; e < seg_floats; e += 4) {
            const floatx4 v = *(const floatx4*)(run + e);
#pragma unroll
            for (int c = 0; c < REAL; ++c) {
                const float* wr = w + (size_t)c * kmat_pitch;
#pragma unroll
                for (int o = 0; o < NACC; ++o) acc[o] = __builtin_fmaf(v[c], wr[o], acc[o]);
            }
            w += (size_t)4 * kmat_pitch;
        }
    }
    // The output is written once and is larger than L2: nontemporal stores, and whole cache lines per store instruction.
    // A lane's CHUNKS 16-byte pieces lie CHUNKS x 16 bytes from its neighbour's, so with two or more of them the wavefront
    // first lays its 64 pixels out in LDS as they lie in memory (no workgroup barrier: the region is the wavefront's own, a
    // wavefront's LDS operations complete in order, and a wavefront-scope fence keeps the compiler from reordering them) and lane l then stores piece 64 i + l of the wavefront in its i-th
    // store, at the offset that piece's pixel left in LDS.  1920 x 1080 x 3, 8 kernels of 3 x 3: 24.3 -> 22.9 us,
    // 3840 x 2160: 124.5 -> 84.2, 640 x 480: 7.0 -> 5.7; 16 kernels: 47.6 -> 37.3; 1000 x 700, 32 kernels: 39.1 -> 24.7.
    // (Nontemporal stores of the lanes' own pieces, half a line per instruction: 28.8 us for 8 kernels, 160 for 16.)
    const uint64_t my_off = ((uint64_t)oy * dst_wpitch + ox) * dst_dpitch;
    constexpr int CHUNKS = NACC / 4;
    if constexpr (CHUNKS >= 2) {
        if (out_c == (uint32_t)NACC) {
            __shared__ uint64_t offs[256];
            __shared__ __attribute__((aligned(16))) float tr[256 * NACC];
            const uint32_t lane = threadIdx.x & 63u, wave0 = threadIdx.x & ~63u;
            float* mine = tr + (size_t)threadIdx.x * NACC;
#pragma unroll
            for (int c = 0; c < CHUNKS; ++c) *(floatx4*)(mine + 4 * c) = floatx4{acc[4 * c], acc[4 * c + 1], acc[4 * c + 2], acc[4 * c + 3]};
            offs[threadIdx.x] = live ? my_off : ~0ull;
            // the other lanes of the wavefront read these back: writes first, for the compiler as well
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
#pragma unroll
            for (int i = 0; i < CHUNKS; ++i) {
                const uint32_t j = (uint32_t)i * 64u + lane, px = j / (uint32_t)CHUNKS, c = j % (uint32_t)CHUNKS;
                const floatx4 v = *(const floatx4*)(tr + (size_t)wave0 * NACC + (size_t)j * 4);
                const uint64_t off = offs[wave0 + px];
                if (off != ~0ull) __builtin_nontemporal_store(v, (floatx4*)(dst + off + 4 * c));
            }
            return;
        }
    }
    if (!live) return;
    float* out = dst + my_off;
#pragma unroll
    for (int o = 0; o < NACC; o += 4) {
        if ((uint32_t)o + 4 <= out_c) {
            __builtin_nontemporal_store(floatx4{acc[o], acc[o + 1], acc[o + 2], acc[o + 3]}, (floatx4*)(out + o));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if ((uint32_t)(o + e) < out_c) out[o + e] = acc[o + e];      // padding channels stay untouched
        }
    }
}

template <int NACC, int REAL>
int launch_direct(const GemmArgs& g, uint32_t k_h, hipStream_t stream)
{
    const uint32_t pixels = g.M;
    hipLaunchKernelGGL((conv2d_direct_kernel<NACC, REAL>), dim3((pixels + 255) / 256), dim3(256), 0, stream,
                       (const float*)g.A, (const float*)g.B, (float*)g.D, g.conv_wout, pixels, g.N, k_h,
                       g.conv_seg_bytes / 4u, g.conv_seg_stride / 4u, g.conv_px_bytes / 4u, g.conv_py_bytes / 4u, g.ldb, g.ldd,
                       g.conv_dst_row / g.ldd);
    return (int)hipGetLastError();
}

template <int NACC>
int launch_direct_real(const GemmArgs& g, uint32_t k_h, uint32_t real, hipStream_t stream)
{
    switch (real) {
    case 1:  return launch_direct<NACC, 1>(g, k_h, stream);
    case 2:  return launch_direct<NACC, 2>(g, k_h, stream);
    case 3:  return launch_direct<NACC, 3>(g, k_h, stream);
    default: return launch_direct<NACC, 4>(g, k_h, stream);
    }
}

}  // namespace

// One fma per (pixel, patch element, kernel) on the vector pipe against the implicit GEMM's fixed cost per 128
// pixels.  Measured on MI355X, picoseconds per output pixel: direct about 8 + 0.037 x patch elements x accumulators
// (640 x 480 x 3 image, 16 kernels of 3 x 3: 43, against 91 for the GEMM form; 1920 x 1080 x 3, 4 kernels: 10 against 73),
// the GEMM form about 70 + 0.55 x patch elements for any number of kernels up to 32.  The direct form also wants a
// short channel pitch: a lane reads 16 bytes per load, channel pitch x 4 bytes away from its neighbour's.
bool conv2d_direct_pays(uint32_t out_c, uint64_t patch_floats, uint32_t channel_pitch, uint32_t depth)
{
    if (out_c > 32 || channel_pitch > 8) return false;
    const double real = channel_pitch == 4 && depth < 4 ? depth / 4.0 : 1.0;      // share of the patch that is multiplied
    const double k = (double)patch_floats, nacc = (double)((out_c + 3) / 4 * 4);
    return 8.0 + 0.037 * k * real * nacc < 0.9 * (70.0 + 0.55 * k);
}

// g: the arguments of the GEMM form (M = pixels, N = kernels, conv_* set, ldb = pitch of the packed kernels);
// depth: channels that exist (<= the channel pitch).
int launch_conv2d_direct_f32(const GemmArgs& g, uint32_t channel_pitch, uint32_t depth, hipStream_t stream)
{
    const uint32_t k_h = g.K / (g.conv_seg_bytes / 4u);
    const uint32_t real = channel_pitch == 4 && depth >= 1 && depth < 4 ? depth : 4;
    switch ((g.N + 3) / 4) {
    case 1: return launch_direct_real<4>(g, k_h, real, stream);
    case 2: return launch_direct_real<8>(g, k_h, real, stream);
    case 3: return launch_direct_real<12>(g, k_h, real, stream);
    case 4: return launch_direct_real<16>(g, k_h, real, stream);
    case 5: return launch_direct_real<20>(g, k_h, real, stream);
    case 6: return launch_direct_real<24>(g, k_h, real, stream);
    case 7: return launch_direct_real<28>(g, k_h, real, stream);
    case 8: return launch_direct_real<32>(g, k_h, real, stream);
    default: return (int)hipErrorInvalidValue;
    }
}

}  // namespace decx_hip
