/* CPU oracle of the 2-D convolution path -- TEST INFRASTRUCTURE ONLY (tests, the smoke check and the
 * bench's CPU leg may use it; the product never does).
 *
 * Restates what de::nn::cuda::Conv2D computes for fp32 (srcs/modules/NN/convolution/CUDA/fp32/
 * Conv2D.cu:56-123): per output pixel and output channel the sum over the kernel window of
 * image x kernel, no flip (im2col_fp32.cu:36-100 reads image(y sy + kh, x sx + kw), the packed kernel
 * keeps its (kh, kw, ic) order, cuda_conv2D_fp32_im2col_planner.cu:40-88), accumulated with fmaf
 * (im2col_GEMM_fp32.cu:77-82), here k ascending in (kh, kw, ic) order from 0.
 * Output size (cuda_conv2D_fp32_im2col_planner.cu:225-241):
 *   no extension:        ((W - KW + 1) / sx) x ((H - KH + 1) / sy)      (integer division)
 *   constant extension:  (W / sx) x (H / sy), the image zero-extended by KW / 2 columns on the left and
 *                        KH / 2 rows on top (and whatever the window needs on the other sides)
 *                        (planner.cu:305-322: the copy into the extended buffer starts at column KW >> 1).
 *
 * Pinned by tests/test_conv_oracle.py: float64 brute force written independently in numpy (einsum over
 * strided windows), scipy.signal.correlate2d on single-channel cases, closed forms (box filter of ones,
 * identity kernel, shift kernel).  The reference has no CPU convolution and no test for this path:
 * parity with the reference itself is unpinned beyond these. */
#include <math.h>
#include <stddef.h>
#include <stdint.h>

void oracle_conv2d_out_dims(uint32_t W, uint32_t H, uint32_t KW, uint32_t KH, uint32_t sx, uint32_t sy, int extend,
                            uint32_t* out_w, uint32_t* out_h)
{
    if (extend) { *out_w = W / sx; *out_h = H / sy; }
    else { *out_w = (W >= KW) ? (W - KW + 1) / sx : 0; *out_h = (H >= KH) ? (H - KH + 1) / sy : 0; }
}

/* image [H][W][C] dense, kernels [OC][KH][KW][C] dense, out [OH][OW][OC] dense */
void oracle_conv2d_f32(const float* image, uint32_t W, uint32_t H, uint32_t C, const float* kernels, uint32_t OC,
                       uint32_t KW, uint32_t KH, uint32_t sx, uint32_t sy, int extend, float* out)
{
    uint32_t OW, OH;
    oracle_conv2d_out_dims(W, H, KW, KH, sx, sy, extend, &OW, &OH);
    const int64_t off_x = extend ? (int64_t)(KW / 2) : 0, off_y = extend ? (int64_t)(KH / 2) : 0;
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t oy = 0; oy < OH; ++oy)
        for (uint32_t ox = 0; ox < OW; ++ox)
            for (uint32_t oc = 0; oc < OC; ++oc) {
                float acc = 0.f;
                for (uint32_t kh = 0; kh < KH; ++kh)
                    for (uint32_t kw = 0; kw < KW; ++kw) {
                        const int64_t iy = (int64_t)oy * sy + kh - off_y, ix = (int64_t)ox * sx + kw - off_x;
                        const int inside = iy >= 0 && iy < (int64_t)H && ix >= 0 && ix < (int64_t)W;
                        for (uint32_t ic = 0; ic < C; ++ic) {
                            const float a = inside ? image[((size_t)iy * W + (size_t)ix) * C + ic] : 0.f;
                            acc = fmaf(a, kernels[(((size_t)oc * KH + kh) * KW + kw) * C + ic], acc);
                        }
                    }
                out[((size_t)oy * OW + ox) * OC + oc] = acc;
            }
}
