/*
 * decx_hip.h -- the C ABI of the MI355X (gfx950) dense-GEMM module.
 *
 * This is the whole surface through which host code reaches the GPU: plain pointers,
 * sizes and scalars, no C++ types.  The C++ objects and entry points of the DECX API
 * (include/DECX.h: de::GPU_Matrix, de::Memcpy, de::blas::cuda::GEMM) are implemented on
 * top of these functions and nothing else.
 *
 * Conventions
 *   - every function returns 0 on success; a positive value is a hipError_t, a negative
 *     value one of the DECX_HIP_E_* codes below; decx_hip_error_string() names either;
 *   - matrices are row-major; a pitch (lda, ldb, ...) is the distance between rows in
 *     ELEMENTS and must be >= the row width; padding beyond the width is never read and
 *     never written;
 *   - `stream` is a hipStream_t passed as void* (NULL = the null stream); launches are
 *     asynchronous with respect to the host;
 *   - fp16 payloads are IEEE binary16 bit patterns in uint16_t.
 */
#ifndef DECX_HIP_H_
#define DECX_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define DECX_HIP_API __attribute__((visibility("default")))

enum {
    DECX_HIP_OK            = 0,
    DECX_HIP_E_INVALID_ARG = -1,   /* null pointer, pitch smaller than width, unknown enum */
    DECX_HIP_E_NOT_INIT    = -2,   /* decx_hip_init() has not succeeded yet */
    DECX_HIP_E_NO_DEVICE   = -3,   /* no usable GPU */
    DECX_HIP_E_TOO_LARGE   = -4    /* decx_hip_gemm_f32_static: the shape wants more workspace than the static one */
};

typedef struct decx_hip_device_props {
    char     name[64];
    char     arch[32];             /* gcnArchName, e.g. "gfx950:sramecc+:xnack-" */
    int32_t  compute_units;
    int32_t  clock_khz;            /* peak engine clock */
    int32_t  memory_clock_khz;
    int32_t  memory_bus_bits;
    int32_t  lds_bytes_per_block;
    int32_t  wavefront_size;
    uint64_t global_mem_bytes;
} decx_hip_device_props;

/* Tile size classes the planner chooses between.  The block tile BM x BN a class stands for depends on the element
 * type: DECX_HIP_TILE_LARGE is 256 x 256 in fp16, 256 x 128 in fp32 on 16-byte aligned operands (256 x 256 otherwise)
 * and in fp64; DECX_HIP_TILE_MEDIUM is 128 x 128; DECX_HIP_TILE_SMALL is 64 x 64, or 128 x 32 for aligned fp32
 * outputs of at most 32 columns (all the kernel counts the reference's convolution takes).  decx_hip_gemm_plan
 * reports the actual BM x BN. */
enum {
    DECX_HIP_TILE_AUTO   = -1,
    DECX_HIP_TILE_LARGE  = 0,
    DECX_HIP_TILE_MEDIUM = 1,
    DECX_HIP_TILE_SMALL  = 2,
    /* fp16 on 16-byte aligned operands only: tiles between 128 x 128 and 256 x 256, for outputs that the largest tile
     * cuts into an awkward number of pieces (unaligned operands run these classes on the 256 x 256 register-staged kernel) */
    DECX_HIP_TILE_F16_192x192 = 3,
    DECX_HIP_TILE_F16_192x256 = 4,
    DECX_HIP_TILE_F16_256x192 = 5,
    DECX_HIP_PATH_GEMV   = 16,    /* N == 1: bandwidth-bound row-dot kernel */
    DECX_HIP_PATH_GEVM   = 17     /* M == 1: bandwidth-bound column-sum kernel */
};

typedef struct decx_hip_plan {
    int32_t  path;                 /* one of the enum above */
    int32_t  edge;                 /* 1: the predicated register-staged kernel runs (operands not 16-byte
                                      aligned, or K == 0); 0: a direct-to-LDS kernel */
    uint32_t tile_m, tile_n;       /* block tile */
    uint32_t grid;                 /* workgroups launched: whole_tiles + (tiles - whole_tiles) x k_splits */
    uint32_t k_splits;             /* ranges K is cut into when the *_ws entry point gets its workspace; 1: no split.
                                      With more than one, path / tile are those of the split (it may run on a smaller
                                      tile than the whole product takes without a workspace) */
    uint32_t whole_tiles;          /* with k_splits > 1: tiles that are multiplied whole all the same -- the full rounds
                                      of workgroups in front of a ragged last round, or one to three tiles per CU that
                                      share their CU with the workgroups of the split ones.  0: all are split */
} decx_hip_plan;

/* ---- device, memory, streams, events --------------------------------------------------
 * Replaces de::InitCuda (srcs/modules/core/configs/config.cu:35-40), the device pool
 * (srcs/modules/core/allocators, memory_management) and the stream / event pools
 * (srcs/modules/core/cudaStream_management) as far as the GEMM path uses them. */
DECX_HIP_API int decx_hip_init(int device);
DECX_HIP_API int decx_hip_get_device_props(decx_hip_device_props* out);
DECX_HIP_API const char* decx_hip_error_string(int code);

DECX_HIP_API int decx_hip_malloc(void** ptr, size_t bytes);
DECX_HIP_API int decx_hip_free(void* ptr);
DECX_HIP_API int decx_hip_host_malloc(void** ptr, size_t bytes);     /* pinned host memory */
DECX_HIP_API int decx_hip_host_free(void* ptr);
DECX_HIP_API int decx_hip_memset_async(void* ptr, int value, size_t bytes, void* stream);
/* free and total device memory in bytes (hipMemGetInfo) */
DECX_HIP_API int decx_hip_mem_info(size_t* free_bytes, size_t* total_bytes);

/* kind: 0 host->device, 1 device->host, 2 device->device.  Pitches and width in BYTES.
 * Replaces the cudaMemcpy2DAsync calls of de::Memcpy
 * (srcs/modules/core/data transmission/data_transmission.cu:139-170). */
DECX_HIP_API int decx_hip_memcpy2d_async(void* dst, size_t dst_pitch, const void* src, size_t src_pitch,
                                         size_t width_bytes, size_t height, int kind, void* stream);

DECX_HIP_API int decx_hip_stream_create(void** stream);
DECX_HIP_API int decx_hip_stream_destroy(void* stream);
DECX_HIP_API int decx_hip_stream_sync(void* stream);

DECX_HIP_API int decx_hip_event_create(void** event);
DECX_HIP_API int decx_hip_event_destroy(void* event);
DECX_HIP_API int decx_hip_event_record(void* event, void* stream);
DECX_HIP_API int decx_hip_event_sync(void* event);
/* work submitted to `stream` after this call starts only once `event` has completed */
DECX_HIP_API int decx_hip_stream_wait_event(void* stream, void* event);
DECX_HIP_API int decx_hip_event_elapsed_ms(void* start, void* stop, float* ms);

/* ---- the contraction -------------------------------------------------------------------
 * D (M x N) = A (M x K) . B (K x N)                      when C == NULL
 * D         = fma(C, beta, alpha * (A . B))              otherwise (C is M x N, may alias D)
 *
 * fp32: products and sums in fp32 on the matrix cores.  Replaces the kernels launched by
 * cuda_GEMM_LS_planner<float>::run (srcs/modules/BLAS/GEMM/CUDA/large_squares/fp32/
 * GEMM_fp32_callers.cu:56-122) behind de::blas::cuda::GEMM (GEMM_LS.cu:62-109,315-393).
 * N == 1 and M == 1 are routed to the bandwidth-bound vector kernels below. */
DECX_HIP_API int decx_hip_gemm_f32(const float* A, const float* B, const float* C, float* D,
                                   uint32_t M, uint32_t N, uint32_t K,
                                   uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                   float alpha, float beta, void* stream);

/* The same product with a device workspace the library may use to split K: when the tiles of the output would leave
 * CUs idle or unevenly loaded (e.g. 300 x 300 x 8192, 1280 x 1024 x 8192), several workgroups share a tile, each
 * multiplying a range of K and leaving its partial product in the workspace, and the one of them that finishes last
 * adds the partial products in a fixed order (results do not vary from run to run) and writes the tile: one launch.  decx_hip_gemm_f32_workspace returns the bytes that make the
 * split possible for a shape (0: the plain kernel is used anyway); a smaller or null workspace is never an
 * error.  The workspace must be 16-byte aligned and is free again when the call's work on `stream` is done.
 * For N == 1 (fp32, fp16) the workspace serves another purpose: B is then the single column of a pitched K x 1
 * matrix, every element in a cache line of its own, and with K * elem_bytes of workspace it is copied once into
 * a dense vector in front of the matrix-vector kernel (8192 x 8192: 46.9 -> 43.9 us); the query returns that
 * size where the copy pays.  For M == 1 with few columns and a long K (1 x 512 x 32768) ranges of K go to workgroups
 * of their own, their partial sums to the workspace, and the last of a column group adds them in range order (69 -> 23 us).
 * Plays the part of the scratch the reference's planner keeps for itself (cuda_GEMM_LS_planner: the transposed
 * A, srcs/modules/BLAS/GEMM/CUDA/large_squares/common/cuda_GEMM_LS_planner.cu:95-160).
 * Besides the workspace, a split launch uses a window of the library's own counter array (65 536 words per GPU, all
 * zero between launches).  Launches outside graphs go round the lower half: the library hands a window to a new launch
 * only when the launches that had it before are known to be over -- they went to the same stream, an event recorded
 * behind them has completed, or their stream is idle -- and otherwise runs the product unsplit, which is never an
 * error.  (Events are recorded only once launches have come from more than one stream; they are drawn from a pool of 32
 * that decx_hip_init makes, and more are created only while more windows than that are in flight at once.)  A split launch that is recorded into a HIP graph gets a window of the upper half and keeps it for the life
 * of the process (the graph may be replayed at any time; recording asks the runtime nothing but whether the stream is
 * recording); when that half is used up, later recordings run unsplit.  A graph's replays must not overlap each other.
 * Callers must not destroy a stream while split launches are in flight on it.  If a launch was cut short (a device fault, a reset), decx_hip_reset_split_counters() waits
 * for the device, puts every counter back to zero and forgets who owned what. */
DECX_HIP_API size_t decx_hip_gemm_f32_workspace(uint32_t M, uint32_t N, uint32_t K);
DECX_HIP_API int decx_hip_reset_split_counters(void);
DECX_HIP_API int decx_hip_gemm_f32_ws(const float* A, const float* B, const float* C, float* D,
                                      uint32_t M, uint32_t N, uint32_t K,
                                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                      float alpha, float beta, void* workspace, size_t workspace_bytes, void* stream);
/* decx_hip_gemm_f32_ws without the workspace arguments and without any allocation, by this call or by the library
 * on its behalf: the workspace is a device array of DECX_HIP_STATIC_WORKSPACE_BYTES that is part of the library's
 * code object (every GPU the library runs on holds its copy until the process ends; its address on a device is
 * looked up by decx_hip_init for that device).  It has no counterpart in the reference: it is for callers that
 * cannot allocate -- code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.  Same
 * results as decx_hip_gemm_f32_ws with a workspace of decx_hip_gemm_f32_workspace(M, N, K) bytes, bit for bit.
 * A product that decx_hip_gemm_f32_ws would split over more than DECX_HIP_STATIC_WORKSPACE_BYTES of partial
 * products returns DECX_HIP_E_TOO_LARGE and launches nothing (decx_hip_gemm_f32 still takes it, unsplit).  Operands
 * that the workspace form would not split anyway (not 16-byte aligned, K == 0) are not refused, and a column
 * operand too long for the array (N == 1, K x 4 bytes beyond it) is read in place, which changes no sum.  A split
 * launch also takes a window of the counter array described above: recorded into a graph, it keeps that window.
 * All calls on one GPU share the one array, which keeps
 * the last call's contents (every call writes what it reads, nothing needs clearing): calls that overlap on one
 * GPU -- two streams, two threads -- race; serialise them. */
#define DECX_HIP_STATIC_WORKSPACE_BYTES (16u << 20)
DECX_HIP_API int decx_hip_gemm_f32_static(const float* A, const float* B, const float* C, float* D,
                                          uint32_t M, uint32_t N, uint32_t K,
                                          uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                          float alpha, float beta, void* stream);
/* The same for the other two real types (elem_bytes 2, 4 or 8 in the query).  fp16 products keep their partial
 * products in fp32 and round once, after the sum. */
DECX_HIP_API size_t decx_hip_gemm_workspace(int elem_bytes, uint32_t M, uint32_t N, uint32_t K);
DECX_HIP_API int decx_hip_gemm_f16_ws(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                                      uint32_t M, uint32_t N, uint32_t K,
                                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                      float alpha, float beta, void* workspace, size_t workspace_bytes, void* stream);
DECX_HIP_API int decx_hip_gemm_f64_ws(const double* A, const double* B, const double* C, double* D,
                                      uint32_t M, uint32_t N, uint32_t K,
                                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                      double alpha, double beta, void* workspace, size_t workspace_bytes, void* stream);

/* fp16 in, fp32 accumulate, one rounding to fp16 out.  Replaces the kernels launched by
 * cuda_GEMM_LS_planner<de::Half>::run (large_squares/fp16/GEMM_fp16_callers.cu:57-124). */
DECX_HIP_API int decx_hip_gemm_f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                                   uint32_t M, uint32_t N, uint32_t K,
                                   uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                   float alpha, float beta, void* stream);

/* fp64: D = A.B or fma(C, beta, alpha * (A.B)) in double precision on the fp64 matrix cores.
 * Replaces the body of decx::blas::GEMM_fp64 (srcs/modules/BLAS/GEMM/CUDA/GEMM_LS.cu:164-211) and
 * cu_GEMM_fp64_*_16_64_64 (large_squares/GEMM_kernels.cuh:182-189).  Operands that are not 16-byte
 * aligned (base or pitch), and K == 0, take a plain one-thread-per-element kernel.  N == 1 and M == 1 run on the
 * bandwidth-bound vector kernels with sums in double (the reference has none for fp64: its
 * srcs/modules/BLAS/GEMM/CUDA/extreme_shapes/VMM_fp64.cu is empty and such shapes go through GEMM_fp64). */
DECX_HIP_API int decx_hip_gemm_f64(const double* A, const double* B, const double* C, double* D,
                                   uint32_t M, uint32_t N, uint32_t K,
                                   uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                   double alpha, double beta, void* stream);

/* Complex (interleaved re, im) single / double precision: D = alpha * (A . B) [+ beta * C], all pitches in
 * complex elements, C may alias D.  Replaces decx::blas::GEMM_cplxf / GEMM_cplxd (GEMM_LS.cu:214-312).  Runs as
 * one real GEMM on the matrix cores over the real expansion of alpha * B, which is written into `workspace`
 * (device memory, 16-byte aligned, at least decx_hip_gemm_complex_workspace(4 or 8, N, K) bytes; the library
 * never allocates). */
DECX_HIP_API size_t decx_hip_gemm_complex_workspace(int real_bytes, uint32_t N, uint32_t K);
DECX_HIP_API int decx_hip_gemm_c32(const float* A, const float* B, const float* C, float* D,
                                   uint32_t M, uint32_t N, uint32_t K,
                                   uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                   float alpha_re, float alpha_im, float beta_re, float beta_im,
                                   void* workspace, size_t workspace_bytes, void* stream);
DECX_HIP_API int decx_hip_gemm_c64(const double* A, const double* B, const double* C, double* D,
                                   uint32_t M, uint32_t N, uint32_t K,
                                   uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                   double alpha_re, double alpha_im, double beta_re, double beta_im,
                                   void* workspace, size_t workspace_bytes, void* stream);

/* The two vector corners, exported for callers that hold vectors (the GEMM entry points above
 * route N == 1 and M == 1 here themselves).  inc* are element strides (a K x 1 pitched matrix
 * has incx = its pitch); c == NULL -> no accumulate term.
 *   gemv:  y (M) = alpha * A (M x K) . x (K) + beta * c     replaces cu_mat_m_vec_fp32 / _fp16_L1..L3
 *   gevm:  y (N) = alpha * x (K) . B (K x N) + beta * c     replaces cu_vec_m_mat_fp32 / _fp16_L1..L3
 * (srcs/modules/BLAS/GEMM/CUDA/extreme_shapes/VMM_fp32.cu:35-146, VMM_fp16.cu) and their second
 * reduction pass.  fp16 inputs are accumulated in fp32; y is fp32 when y_is_f32 != 0 (the
 * reference's accuracy level 1) and fp16, rounded once, otherwise. */
DECX_HIP_API int decx_hip_gemv_f32(const float* A, const float* x, const float* c, float* y,
                                   uint32_t M, uint32_t K, uint32_t lda,
                                   uint32_t incx, uint32_t incc, uint32_t incy,
                                   float alpha, float beta, void* stream);
DECX_HIP_API int decx_hip_gemv_f16(const uint16_t* A, const uint16_t* x, const uint16_t* c, void* y,
                                   uint32_t M, uint32_t K, uint32_t lda,
                                   uint32_t incx, uint32_t incc, uint32_t incy,
                                   float alpha, float beta, int y_is_f32, void* stream);
DECX_HIP_API int decx_hip_gevm_f32(const float* x, const float* B, const float* c, float* y,
                                   uint32_t K, uint32_t N, uint32_t ldb,
                                   uint32_t incx, uint32_t incc, uint32_t incy,
                                   float alpha, float beta, void* stream);
DECX_HIP_API int decx_hip_gevm_f16(const uint16_t* x, const uint16_t* B, const uint16_t* c, void* y,
                                   uint32_t K, uint32_t N, uint32_t ldb,
                                   uint32_t incx, uint32_t incc, uint32_t incy,
                                   float alpha, float beta, int y_is_f32, void* stream);
/* Vector x matrix with a device workspace (decx_hip_gemm_workspace(elem_bytes, 1, N, K) bytes, 16-byte aligned): when
 * the matrix has few columns and a long K, ranges of K go to workgroups of their own and the last of a column group to
 * finish adds their partial sums in a fixed order -- the part of the reference's second pass reduce_sum2D_v_fp32_Async
 * behind cu_vec_m_mat_fp32 (srcs/modules/BLAS/GEMM/CUDA/extreme_shapes/VMM_callers.cuh:67-202), inside the one
 * kernel and taken only where whole columns per workgroup would leave most CUs idle.  With a smaller or null workspace
 * every workgroup sums its columns over all of K. */
DECX_HIP_API int decx_hip_gevm_f32_ws(const float* x, const float* B, const float* c, float* y,
                                      uint32_t K, uint32_t N, uint32_t ldb,
                                      uint32_t incx, uint32_t incc, uint32_t incy,
                                      float alpha, float beta, void* workspace, size_t workspace_bytes, void* stream);
DECX_HIP_API int decx_hip_gevm_f16_ws(const uint16_t* x, const uint16_t* B, const uint16_t* c, void* y,
                                      uint32_t K, uint32_t N, uint32_t ldb,
                                      uint32_t incx, uint32_t incc, uint32_t incy,
                                      float alpha, float beta, int y_is_f32,
                                      void* workspace, size_t workspace_bytes, void* stream);

/* ---- 2-D convolution as an implicit GEMM ---------------------------------------------------
 * Replaces the planner, the im2col kernels, the im2col buffer and cu_im2col_GEMM_fp32 behind
 * de::nn::cuda::Conv2D (srcs/modules/NN/convolution/CUDA/fp32/cuda_conv2D_fp32_im2col_planner.cu:
 * 212-552, im2col_fp32.cu, im2col_GEMM_fp32.cu:40-106).  Images are stored [row][column][channel]
 * with a channel pitch (multiple of 4 floats) and a row pitch in columns; all pointers 16-byte
 * aligned.
 *
 *   dst(y, x, oc) = sum over kh, kw, ic of image(y * stride_y + kh, x * stride_x + kw, ic) * kernel_oc(kh, kw, ic)
 *
 * (no flip: a cross-correlation, as the original computes).  `image` points at the pixel under
 * kernel element (0, 0) of output pixel (0, 0): for zero-extended borders pass a zero-padded copy.
 * The kernel set comes packed as kmat[(kh * k_w + kw) * img_dpitch + ic][oc] (row pitch kmat_pitch,
 * zero rows for ic >= depth); decx_hip_conv2d_pack_kernels_f32 builds it from out_c kernels stored
 * like images, tensor_stride floats apart.  Shallow patches with at most 32 kernels and a channel pitch of
 * 4 or 8 (a 3 x 3 filter bank over an RGB image) run a lane per output pixel on the vector pipe instead of the
 * matrix cores; same operands, same result. */
DECX_HIP_API int decx_hip_conv2d_pack_kernels_f32(const float* kernels, float* kmat, uint32_t k_w, uint32_t k_h,
                                                  uint32_t depth, uint32_t k_dpitch, uint32_t k_wpitch,
                                                  uint64_t tensor_stride, uint32_t out_c, uint32_t kmat_pitch,
                                                  uint32_t img_dpitch, void* stream);
DECX_HIP_API int decx_hip_conv2d_f32(const float* image, const float* kmat, float* dst,
                                     uint32_t out_w, uint32_t out_h, uint32_t out_c, uint32_t k_w, uint32_t k_h,
                                     uint32_t img_dpitch, uint32_t img_wpitch, uint32_t stride_x, uint32_t stride_y,
                                     uint32_t kmat_pitch, uint32_t dst_dpitch, uint32_t dst_wpitch, void* stream);
/* The same with the number of channels that exist (1 <= depth <= img_dpitch; the rest of the pitch is padding that
 * meets zero rows of kmat): the lane-per-pixel kernel then leaves the padding channel of grey and RGB images
 * (channel pitch 4) out of its arithmetic.  decx_hip_conv2d_f32 is this call with depth = img_dpitch. */
DECX_HIP_API int decx_hip_conv2d_f32_depth(const float* image, const float* kmat, float* dst,
                                           uint32_t out_w, uint32_t out_h, uint32_t out_c, uint32_t k_w, uint32_t k_h,
                                           uint32_t depth, uint32_t img_dpitch, uint32_t img_wpitch,
                                           uint32_t stride_x, uint32_t stride_y,
                                           uint32_t kmat_pitch, uint32_t dst_dpitch, uint32_t dst_wpitch, void* stream);

/* Same as decx_hip_gemm_f32 / _f16 with the planner's choice overridden (`tile` = one of
 * DECX_HIP_TILE_*; AUTO = planner) and, with force_edge != 0, the predicated kernel
 * variant forced even for shapes that are tile multiples.  For tests and tuning. */
DECX_HIP_API int decx_hip_gemm_f32_tile(const float* A, const float* B, const float* C, float* D,
                                        uint32_t M, uint32_t N, uint32_t K,
                                        uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                        float alpha, float beta, void* stream, int tile, int force_edge);
DECX_HIP_API int decx_hip_gemm_f16_tile(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D,
                                        uint32_t M, uint32_t N, uint32_t K,
                                        uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                        float alpha, float beta, void* stream, int tile, int force_edge);
/* fp64: DECX_HIP_TILE_LARGE selects the largest fp64 tile (256 x 128); force_plain != 0 forces the
 * one-thread-per-element kernel. */
DECX_HIP_API int decx_hip_gemm_f64_tile(const double* A, const double* B, const double* C, double* D,
                                        uint32_t M, uint32_t N, uint32_t K,
                                        uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                                        double alpha, double beta, void* stream, int tile, int force_plain);

/* What the planner would run for this problem (no GPU work).  elem_bytes: 4 = fp32, 2 = fp16, 8 = fp64.
 * `aligned` != 0 promises 16-byte aligned bases and pitches.  Replaces the scoring of
 * cuda_GEMM_LS_planner<T>::plan (large_squares/common/cuda_GEMM_LS_planner.cu:108-224).
 * Works without a GPU: before decx_hip_init() it assumes 256 compute units. */
DECX_HIP_API int decx_hip_gemm_plan(int elem_bytes, uint32_t M, uint32_t N, uint32_t K, int aligned,
                                    decx_hip_plan* out);

/* IEEE binary16 <-> binary32, round to nearest even; host-side helpers behind
 * de::Float2Half / de::Half2Float (srcs/common/FP16/float_half_convert.cu:35-46). */
DECX_HIP_API uint16_t decx_hip_float_to_half(float value);
DECX_HIP_API float decx_hip_half_to_float(uint16_t bits);

#ifdef __cplusplus
}
#endif
#endif  /* DECX_HIP_H_ */
