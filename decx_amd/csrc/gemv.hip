// The two vector corners of the GEMM entry point, both bound by HBM bandwidth (every
// element of the matrix is used once):
//
//   gemv:  y (M) = alpha * A (M x K) . x (K)  (+ beta * c)      -- N == 1
//   gevm:  y (N) = alpha * x (K) . B (K x N)  (+ beta * c)      -- M == 1
//
// They replace cu_mat_m_vec_fp32 / cu_vec_m_mat_fp32, their fp16 L1-L3 variants and the
// second reduction pass those need (srcs/modules/BLAS/GEMM/CUDA/extreme_shapes/
// VMM_fp32.cu:35-146, VMM_fp16.cu, VMM_callers.cuh:67-202): here a workgroup finishes its
// outputs itself, so there are no partial sums to reduce in another kernel.  fp16 inputs
// are always accumulated in fp32 (the reference's level 1); the result is written as fp32
// or rounded once to fp16, whichever the caller asks for.  fp64 matrices run on the same kernels
// with sums in double (the reference has no fp64 form of these: its VMM_fp64.cu is empty).
//
// gemv: 16 wavefronts per workgroup, two rows per wavefront (32 rows per workgroup: 8192
//   rows give one workgroup per CU with 64 KB of A in flight), one row per wavefront for
//   matrices of fewer than 8192 rows, and below 4096 rows 2, 4, 8 or all 16 wavefronts share a row
//   (they deal the steps of K among themselves), always the fewest that still give every CU a
//   workgroup (2048 x 8192: 24.3 -> 16.1 us with a dense x, 512 x 32768: 60.9 -> 23.8); x is staged in LDS once per
//   workgroup, as fp32, in chunks of 4096 (fp16: 8192) -- x may be strided (the single column of a
//   pitched K x 1 matrix puts every element in its own cache line), so staging it once per
//   32 rows keeps that gather small -- and a chunk of x is loaded into registers while the chunk
//   before is being multiplied, so that its latency hides behind the rows (8192 x 8192: fp32 43.1 -> 42.0 us,
//   fp16 26.1 -> 23.9; gevm the same way: 39.2 -> 37.8 and 24.3 -> 23.3); A is read with 128-bit loads; per
//   lane an fp32 fma chain, then a butterfly over the 64 lanes.
// gevm: a workgroup owns 128 bytes of columns (32 fp32 / 64 fp16); 8 lanes cover those with
//   one 128-bit load each, the other lane bits and the 16 wavefronts stride over k
//   (128 rows per sweep); partial sums meet in a shuffle over the row lanes and in LDS over
//   the wavefronts.  When that gives fewer workgroups than CUs, a workgroup owns 64 bytes
//   (4 lanes, 256 rows per sweep) and the two workgroups sharing a cache line share an XCD.
#include "gemm_common.hpp"
#include <type_traits>

namespace decx_hip {

namespace {

constexpr int GEMV_THREADS = 1024;
constexpr int GEMV_WAVES = GEMV_THREADS / 64;
constexpr int GEMV_ROWS_PER_BLOCK = 2 * GEMV_WAVES;
constexpr int GEMV_KC = 4096;            // elements of x staged per chunk (16 KB of LDS, 32 KB for fp64 and for gemv's fp16 chunks of twice as many)
constexpr int GEMV_XPT = GEMV_KC / GEMV_THREADS;   // of which a thread carries this many

typedef double doublex2 __attribute__((ext_vector_type(2)));

template <typename T> struct Per16 { static constexpr int n = 16 / sizeof(T); };

// the type sums are kept in: fp32 for fp32 and fp16 inputs, fp64 for fp64
template <typename T> struct Acc { typedef float type; };
template <> struct Acc<double> { typedef double type; };

__device__ __forceinline__ float to_acc(float v) { return v; }
__device__ __forceinline__ float to_acc(_Float16 v) { return (float)v; }
__device__ __forceinline__ double to_acc(double v) { return v; }
__device__ __forceinline__ float fma_acc(float a, float b, float c) { return __builtin_fmaf(a, b, c); }
__device__ __forceinline__ double fma_acc(double a, double b, double c) { return __builtin_fma(a, b, c); }

// 16 bytes of T at p, widened to the accumulation type
template <typename T> __device__ __forceinline__ void load16(const T* p, typename Acc<T>::type (&out)[Per16<T>::n])
{
    if constexpr (sizeof(T) == 8) {
        const doublex2 v = *(const doublex2*)p;
        out[0] = v[0]; out[1] = v[1];
    } else if constexpr (sizeof(T) == 4) {
        const floatx4 v = *(const floatx4*)p;
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = v[e];
    } else {
        const halfx8 v = *(const halfx8*)p;
#pragma unroll
        for (int e = 0; e < 8; ++e) out[e] = (float)v[e];
    }
}

// the same in two halves: the 16 bytes as they are (a load that nothing waits for yet), and their widening
template <typename T> struct Raw16 { typedef floatx4 type; };
template <> struct Raw16<_Float16> { typedef halfx8 type; };
template <> struct Raw16<double> { typedef doublex2 type; };
template <typename T> __device__ __forceinline__ void widen16(const typename Raw16<T>::type& v, typename Acc<T>::type (&out)[Per16<T>::n])
{
#pragma unroll
    for (int e = 0; e < Per16<T>::n; ++e) out[e] = (typename Acc<T>::type)v[e];
}

template <typename A> __device__ __forceinline__ A wave_sum(A v)
{
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// RPW rows per wavefront: 2, or 1 when two would leave CUs without a workgroup.  WPR wavefronts per
// row (RPW == 1 only): for matrices of few rows the wavefronts of a row deal the steps of K among
// themselves and their sums meet in LDS, in wavefront order, so that a workgroup holds 16 / WPR rows.
template <typename T, typename TO, int RPW, int WPR>
__global__ void __launch_bounds__(GEMV_THREADS)
gemv_kernel(const T* __restrict__ A, const T* __restrict__ x, const T* __restrict__ c, TO* __restrict__ y,
            uint32_t M, uint32_t K, uint32_t lda, uint32_t incx, uint32_t incc, uint32_t incy,
            typename Acc<T>::type alpha, typename Acc<T>::type beta, uint32_t vec_ok)
{
    typedef typename Acc<T>::type A_t;
    constexpr int N16 = Per16<T>::n;
    // fp16 rows are half as long in bytes: chunks of twice as many elements give a wavefront the same 16 KB of a row per
    // chunk as fp32 and, with 16 steps per chunk, every wavefront of the workgroup a start of its own (with 8 they
    // collided in pairs: 65536 x 8192 189 -> 177 us, 8192 x 16384 41.7 -> 40.8; fp32 gained nothing from the same, and
    // four times as many take the kernel beyond 64 VGPRs)
    constexpr int KC = sizeof(T) == 2 ? 2 * GEMV_KC : GEMV_KC, XPT = KC / GEMV_THREADS;
    __shared__ __attribute__((aligned(16))) A_t xs[KC];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    static_assert(WPR == 1 || RPW == 1, "rows are split over wavefronts only one at a time");
    __shared__ A_t wave_sums[GEMV_WAVES];
    const int sub = wave % WPR;                            // which share of the steps of K this wavefront takes
    const uint32_t row0 = blockIdx.x * (RPW * GEMV_WAVES / WPR) + (wave / WPR) * RPW;
    const bool has0 = row0 < M, has1 = RPW == 2 && row0 + 1 < M;
    const T* a0 = A + (size_t)(has0 ? row0 : 0) * lda;
    const T* a1 = A + (size_t)(has1 ? row0 + 1 : 0) * lda;
    A_t s0 = 0, s1 = 0;

    // Every workgroup walks the same K range of rows that lie a whole number of pitches apart; started
    // together at k = 0 they would all pull on the same memory channels at the same time.  So each
    // workgroup starts at another chunk and each wavefront at another step inside it (sums commute).
    const uint32_t chunks = (K + KC - 1) / KC;
    const uint32_t chunk0 = chunks ? (blockIdx.x * 3u) % chunks : 0u;
    // x travels one chunk ahead in registers, its loads dealt out among the steps of the chunk before: a strided x
    // (the column of a pitched K x 1 matrix) touches a cache line per element, and with one workgroup per CU the loads
    // of the rows queue behind whatever is issued in a burst.  (Asking for the first rows of A ahead of x as well, as
    // gevm_kernel does for B, takes this kernel beyond 64 VGPRs and with that from two workgroups per CU to one:
    // 16384 x 1024 13.2 -> 15.3 us, fp16 6.5 -> 9.9.)
    constexpr uint32_t STEP = 64 * N16;
    constexpr int PER = KC / (int)STEP / XPT;    // steps per load of x: fp32 4, fp16 2, fp64 8
    constexpr int XG = PER >= 4 ? 1 : 4 / PER;             // loads of x per group of at least 4 steps
    constexpr int GROUPS = XPT / XG;
    T xr[XPT];
    const auto fetch_x = [&](uint32_t kc, int j) {
        const uint32_t i = t + j * GEMV_THREADS;
        xr[j] = kc + i < K ? x[(size_t)(kc + i) * incx] : T(0);
    };
    if (chunks) {
#pragma unroll
        for (int j = 0; j < XPT; ++j) fetch_x(chunk0 * KC, j);
    }
    for (uint32_t ci = 0; ci < chunks; ++ci) {
        const uint32_t chunk = chunk0 + ci < chunks ? chunk0 + ci : chunk0 + ci - chunks;
        const uint32_t kc = chunk * KC;
        const uint32_t len = (K - kc) < (uint32_t)KC ? (K - kc) : (uint32_t)KC;
        __syncthreads();                                   // previous chunk fully consumed
#pragma unroll
        for (int j = 0; j < XPT; ++j) xs[t + j * GEMV_THREADS] = to_acc(xr[j]);
        __syncthreads();
        const bool more = ci + 1 < chunks;
        const uint32_t kc_next = (chunk + 1 < chunks ? chunk + 1 : 0u) * KC;
        const uint32_t lenv = vec_ok ? (len / N16) * N16 : 0u;   // part done with 128-bit loads
        const uint32_t steps = (lenv + STEP - 1) / STEP;
        const uint32_t mine = has0 && steps > (uint32_t)sub ? (steps - sub + WPR - 1) / WPR : 0u;   // steps of this wavefront
        const uint32_t step0 = steps ? ((blockIdx.x * GEMV_WAVES + wave - sub) * 5u) % steps : 0u;   // one start per row
#pragma unroll
        for (int g = 0; g < GROUPS; ++g) {
            if (more) {
#pragma unroll
                for (int j = 0; j < XG; ++j) fetch_x(kc_next, g * XG + j);
            }
            // the last chunk has no loads of x to make room for: its steps stay in one loop
            const uint32_t lo = more ? mine * g / GROUPS : (g == 0 ? 0u : mine), hi = more ? mine * (g + 1) / GROUPS : mine;
#pragma unroll 4
            for (uint32_t ii = lo; ii < hi; ++ii) {
                const uint32_t i = sub + ii * WPR;
                const uint32_t step = step0 + i < steps ? step0 + i : step0 + i - steps;
                const uint32_t k = step * STEP + lane * N16;
                if (k < lenv) {
                    A_t av[N16], bv[N16];
                    load16<T>(a0 + kc + k, av);
                    if (has1) load16<T>(a1 + kc + k, bv);
#pragma unroll
                    for (int e = 0; e < N16; ++e) {
                        const A_t xv = xs[k + e];
                        s0 = fma_acc(av[e], xv, s0);
                        if (has1) s1 = fma_acc(bv[e], xv, s1);
                    }
                }
            }
        }
        if (has0) {
            for (uint32_t k = lenv + lane + 64u * sub; k < len; k += 64u * WPR) {   // the tail, or a whole unaligned row
                s0 = fma_acc(to_acc(a0[kc + k]), xs[k], s0);
                if (has1) s1 = fma_acc(to_acc(a1[kc + k]), xs[k], s1);
            }
        }
    }
    s0 = wave_sum(s0);
    s1 = wave_sum(s1);
    if constexpr (WPR > 1) {
        if (lane == 0) wave_sums[wave] = s0;
        __syncthreads();
        if (sub != 0) return;
#pragma unroll
        for (int w = 1; w < WPR; ++w) s0 += wave_sums[wave + w];
    }
    if (lane == 0) {
        if (has0) {
            A_t o = s0;
            if (c) o = fma_acc(to_acc(c[(size_t)row0 * incc]), beta, alpha * o);
            y[(size_t)row0 * incy] = (TO)o;
        }
        if (has1) {
            A_t o = s1;
            if (c) o = fma_acc(to_acc(c[(size_t)(row0 + 1) * incc]), beta, alpha * o);
            y[(size_t)(row0 + 1) * incy] = (TO)o;
        }
    }
}

// CL lanes of 16 bytes cover a workgroup's columns (8: 128 bytes of a row, 4: 64 bytes), 64 / CL rows per wavefront.
template <typename T, typename TO, int CL>
__global__ void __launch_bounds__(GEMV_THREADS)
gevm_kernel(const T* __restrict__ x, const T* __restrict__ B, const T* __restrict__ c, TO* __restrict__ y,
            uint32_t K, uint32_t N, uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy,
            typename Acc<T>::type alpha, typename Acc<T>::type beta, uint32_t vec_ok, uint32_t split_len,
            typename Acc<T>::type* __restrict__ partial, uint32_t partial_stride, uint32_t* __restrict__ counters)
{
    typedef typename Acc<T>::type A_t;
    constexpr int N16 = Per16<T>::n;
    constexpr int CB = CL * N16;                           // columns per workgroup
    if (split_len) {                                       // blockIdx.y takes a range of K; its sums go to `partial`
        const uint32_t k0 = blockIdx.y * split_len;
        x += (size_t)k0 * incx;
        B += (size_t)k0 * ldb;
        K = K - k0 < split_len ? K - k0 : split_len;
    }
    constexpr int RL = 64 / CL;                            // rows per wavefront and sweep
    __shared__ __attribute__((aligned(16))) A_t xs[GEMV_KC];
    __shared__ A_t red[GEMV_WAVES][CB];
    const int t = threadIdx.x, lane = t & 63, wave = t >> 6;
    const int col_lane = lane % CL, row_lane = lane / CL;
    // Half-line column groups: the two workgroups that share every 128-byte line of B should share an L2,
    // so blocks b and b + 8 (dealt to the same XCD) take adjacent groups (the last grid % 16 blocks stay as they are).
    uint32_t group = blockIdx.x;
    if (CL == 4 && group < gridDim.x / 16 * 16) group = (group / 16) * 16 + (group % 8) * 2 + (group / 8) % 2;
    const uint32_t n0 = group * CB + col_lane * N16;
    const bool whole = vec_ok && (n0 + N16 <= N);
    A_t acc[N16];
#pragma unroll
    for (int e = 0; e < N16; ++e) acc[e] = 0;

    T xr[GEMV_XPT];                                        // x one chunk ahead, as in gemv_kernel
    const auto fetch_x = [&](uint32_t kc) {
#pragma unroll
        for (int j = 0; j < GEMV_XPT; ++j) {
            const uint32_t i = t + j * GEMV_THREADS;
            xr[j] = kc + i < K ? x[(size_t)(kc + i) * incx] : T(0);
        }
    };
    if (K) fetch_x(0);
    // The first rows of B are asked for before x is in LDS: the memory system has work from the first cycle on, not
    // only after the round trip of x and two barriers.
    constexpr int PRE = 4;
    typename Raw16<T>::type pre[PRE];
    const uint32_t len0 = K < (uint32_t)GEMV_KC ? K : (uint32_t)GEMV_KC;
    const bool pre_ok = whole && n0 < N;
    if (pre_ok) {
#pragma unroll
        for (int u = 0; u < PRE; ++u) {
            const uint32_t k = wave * RL + row_lane + u * (GEMV_WAVES * RL);
            if (k < len0) pre[u] = *(const typename Raw16<T>::type*)(B + (size_t)k * ldb + n0);
        }
    }
    for (uint32_t kc = 0; kc < K; kc += GEMV_KC) {
        const uint32_t len = (K - kc) < (uint32_t)GEMV_KC ? (K - kc) : (uint32_t)GEMV_KC;
        __syncthreads();
#pragma unroll
        for (int j = 0; j < GEMV_XPT; ++j) xs[t + j * GEMV_THREADS] = to_acc(xr[j]);
        __syncthreads();
        if (kc + GEMV_KC < K) fetch_x(kc + GEMV_KC);
        uint32_t k_first = wave * RL + row_lane;
        if (kc == 0 && pre_ok) {
#pragma unroll
            for (int u = 0; u < PRE; ++u) {
                const uint32_t k = wave * RL + row_lane + u * (GEMV_WAVES * RL);
                if (k < len) {
                    A_t bv[N16];
                    widen16<T>(pre[u], bv);
                    const A_t xv = xs[k];
#pragma unroll
                    for (int e = 0; e < N16; ++e) acc[e] = fma_acc(xv, bv[e], acc[e]);
                }
            }
            k_first += PRE * (GEMV_WAVES * RL);
        }
        if (n0 < N) {
#pragma unroll 4
            for (uint32_t k = k_first; k < len; k += GEMV_WAVES * RL) {
                const T* p = B + (size_t)(kc + k) * ldb + n0;
                const A_t xv = xs[k];
                if (whole) {
                    A_t bv[N16];
                    load16<T>(p, bv);
#pragma unroll
                    for (int e = 0; e < N16; ++e) acc[e] = fma_acc(xv, bv[e], acc[e]);
                } else {
#pragma unroll
                    for (int e = 0; e < N16; ++e)
                        if (n0 + e < N) acc[e] = fma_acc(xv, to_acc(p[e]), acc[e]);
                }
            }
        }
    }
#pragma unroll
    for (int e = 0; e < N16; ++e) {
        A_t v = acc[e];
        if (CL == 4) v += __shfl_xor(v, 4, 64);
        v += __shfl_xor(v, 8, 64);
        v += __shfl_xor(v, 16, 64);
        v += __shfl_xor(v, 32, 64);
        if (row_lane == 0) red[wave][col_lane * N16 + e] = v;
    }
    __syncthreads();
    const uint32_t n = group * CB + t;
    const bool mine = t < CB && n < N;
    A_t o = 0;
    if (mine) {
#pragma unroll
        for (int w = 0; w < GEMV_WAVES; ++w) o += red[w][t];
    }
    if (split_len) {
        // The workgroups of a column group (one per range of K) leave their sums in `partial` at device scope and count
        // themselves in; the last one to arrive adds the ranges in order and writes y.  Nobody waits for anybody.
        typedef typename std::conditional<sizeof(A_t) == 8, unsigned long long, uint32_t>::type bits_t;
        bits_t* const slots = (bits_t*)partial;
        if (mine) __hip_atomic_store(slots + (size_t)blockIdx.y * partial_stride + n, __builtin_bit_cast(bits_t, o), __ATOMIC_RELAXED,
                                     __HIP_MEMORY_SCOPE_AGENT);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __syncthreads();
        __shared__ uint32_t last;
        if (t == 0) {
            const uint32_t before = __hip_atomic_fetch_add(counters + blockIdx.x, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last = before + 1 == gridDim.y ? 1u : 0u;
        }
        __syncthreads();
        if (!last) return;
        if (t == 0) __hip_atomic_store(counters + blockIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        o = 0;
        if (mine) {
            for (uint32_t z = 0; z < gridDim.y; ++z) {
                const bits_t b = __hip_atomic_load(slots + (size_t)z * partial_stride + n, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                o += __builtin_bit_cast(A_t, b);
            }
        }
    }
    if (mine) {
        if (c) o = fma_acc(to_acc(c[(size_t)n * incc]), beta, alpha * o);
        y[(size_t)n * incy] = (TO)o;
    }
}

template <typename T> uint32_t rows_vectorisable(const void* base, uint32_t ld)
{
    return (((uintptr_t)base & 15u) == 0 && (ld * sizeof(T)) % 16 == 0) ? 1u : 0u;
}

}  // namespace

namespace {

template <typename T, typename TO>
void launch_gemv_as(const void* A, const void* x, const void* c, void* y, uint32_t M, uint32_t K, uint32_t lda,
                    uint32_t incx, uint32_t incc, uint32_t incy, typename Acc<T>::type alpha, typename Acc<T>::type beta,
                    hipStream_t stream)
{
    const uint32_t vec = rows_vectorisable<T>(A, lda);
    auto launch = [&](auto rpw_c, auto wpr_c) {
        constexpr int RPW = decltype(rpw_c)::value, WPR = decltype(wpr_c)::value;
        constexpr uint32_t ROWS = RPW * GEMV_WAVES / WPR;
        hipLaunchKernelGGL((gemv_kernel<T, TO, RPW, WPR>), dim3((M + ROWS - 1) / ROWS), dim3(GEMV_THREADS), 0, stream,
                           (const T*)A, (const T*)x, (const T*)c, (TO*)y, M, K, lda, incx, incc, incy, alpha, beta, vec);
    };
    using std::integral_constant;
    switch (gemv_rows_per_block(M)) {
    case 32: launch(integral_constant<int, 2>{}, integral_constant<int, 1>{}); break;
    case 16: launch(integral_constant<int, 1>{}, integral_constant<int, 1>{}); break;
    case 8:  launch(integral_constant<int, 1>{}, integral_constant<int, 2>{}); break;
    case 4:  launch(integral_constant<int, 1>{}, integral_constant<int, 4>{}); break;
    case 2:  launch(integral_constant<int, 1>{}, integral_constant<int, 8>{}); break;
    default: launch(integral_constant<int, 1>{}, integral_constant<int, 16>{}); break;
    }
}

// dst[i] = x[i * inc]: the dense copy of a strided vector
template <typename T>
__global__ void __launch_bounds__(256) gather_kernel(const T* __restrict__ x, T* __restrict__ dst, uint32_t K, uint32_t inc)
{
    const uint32_t i = blockIdx.x * 256 + threadIdx.x;
    if (i < K) dst[i] = x[(size_t)i * inc];
}

}  // namespace

// Rows per workgroup of gemv: 32 (two per wavefront) while that gives every CU a workgroup, else the largest
// power of two down to 1 (all 16 wavefronts on one row) that still does.
uint32_t gemv_rows_per_block(uint32_t M)
{
    uint32_t rows = 32;
    while (rows > 1 && (M + rows - 1) / rows < 256u) rows /= 2;
    return rows;
}

// A strided x (the single column of a pitched K x 1 matrix) costs every workgroup of gemv one cache
// line request per element; gathered once into a dense buffer it costs one per 32 (fp32) or 64.
// The copy is a launch of its own (about 4.5 us with its loads, all L2 misses): it pays from the sizes
// below (8192 x 8192: 45.4 -> 41.8 us, with a dense x 38.5; 512 x 32768: 44.7 -> 23.8, 256 x 8192: 10.8 -> 7.2,
// 4096 x 2048: 7.7 -> 7.9).
bool gemv_gather_pays(uint32_t M, uint32_t K, uint32_t incx)
{
    if (incx <= 1) return false;
    if (K >= 8192) return M >= 64;
    if (K >= 4096) return M >= 1024;
    return K >= 3072 && M >= 3072;
}

int launch_gather(int elem_bytes, const void* x, void* dst, uint32_t K, uint32_t inc, hipStream_t stream)
{
    if (K == 0) return 0;
    const dim3 grid((K + 255) / 256);
    if (elem_bytes == 2) hipLaunchKernelGGL(gather_kernel<_Float16>, grid, dim3(256), 0, stream, (const _Float16*)x, (_Float16*)dst, K, inc);
    else if (elem_bytes == 8) hipLaunchKernelGGL(gather_kernel<double>, grid, dim3(256), 0, stream, (const double*)x, (double*)dst, K, inc);
    else hipLaunchKernelGGL(gather_kernel<float>, grid, dim3(256), 0, stream, (const float*)x, (float*)dst, K, inc);
    return (int)hipGetLastError();
}

int launch_gemv_f64(const double* A, const double* x, const double* c, double* y, uint32_t M, uint32_t K, uint32_t lda,
                    uint32_t incx, uint32_t incc, uint32_t incy, double alpha, double beta, hipStream_t stream)
{
    launch_gemv_as<double, double>(A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, stream);
    return (int)hipGetLastError();
}

int launch_gemv(bool f16, bool out_f32, const void* A, const void* x, const void* c, void* y, uint32_t M, uint32_t K,
                uint32_t lda, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, hipStream_t stream)
{
    if (!f16) launch_gemv_as<float, float>(A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, stream);
    else if (out_f32) launch_gemv_as<_Float16, float>(A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, stream);
    else launch_gemv_as<_Float16, _Float16>(A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, stream);
    return (int)hipGetLastError();
}

namespace {

template <typename T, typename TO>
void launch_gevm_as(const void* x, const void* B, const void* c, void* y, uint32_t K, uint32_t N, uint32_t ldb,
                    uint32_t incx, uint32_t incc, uint32_t incy, typename Acc<T>::type alpha, typename Acc<T>::type beta,
                    hipStream_t stream, uint32_t split_len, typename Acc<T>::type* partial, uint32_t partial_stride, uint32_t* counters)
{
    // 128-byte column groups unless they leave CUs without a workgroup (fp16 at N = 8192: 128 groups for
    // 256 CUs); then 64-byte groups, two workgroups per cache line -- or, with a workspace for partial sums,
    // 128-byte groups and several workgroups per group, each on a range of K (split_len != 0)
    const uint32_t cb8 = 8u * Per16<T>::n;
    const uint32_t vec = rows_vectorisable<T>(B, ldb);
    const uint32_t splits = split_len ? (K + split_len - 1) / split_len : 1u;
    if (split_len || (N + cb8 - 1) / cb8 >= 256u)
        hipLaunchKernelGGL((gevm_kernel<T, TO, 8>), dim3((N + cb8 - 1) / cb8, splits), dim3(GEMV_THREADS), 0, stream, (const T*)x,
                           (const T*)B, (const T*)c, (TO*)y, K, N, ldb, incx, incc, incy, alpha, beta, vec, split_len, partial,
                           partial_stride, counters);
    else
        hipLaunchKernelGGL((gevm_kernel<T, TO, 4>), dim3((N + cb8 / 2 - 1) / (cb8 / 2)), dim3(GEMV_THREADS), 0, stream,
                           (const T*)x, (const T*)B, (const T*)c, (TO*)y, K, N, ldb, incx, incc, incy, alpha, beta, vec, 0u,
                           (typename Acc<T>::type*)nullptr, 0u, (uint32_t*)nullptr);
}

}  // namespace

// Few columns and a long K: 128-byte column groups alone would leave CUs without a workgroup.  With room for
// partial sums the groups are multiplied by ranges of K, aiming at two workgroups per CU.  The second kernel
// that adds the partial sums costs a launch, so this is for matrices that keep the first one busy long enough:
// 1 x 2048 x 8192 19.5 -> 16.5 us, 1 x 512 x 32768 69 -> 23, 1 x 64 x 65536 116 -> 23 (1 x 512 x 8192 would go from
// 9 to 14 and stays whole).  A range is a multiple of the 128 rows a workgroup sweeps at a time, at least 256 long.
SplitPlan plan_gevm_split(int elem_bytes, uint32_t N, uint32_t K, uint32_t cus)
{
    const uint32_t cb8 = 128u / (uint32_t)elem_bytes;
    const uint32_t groups = (N + cb8 - 1) / cb8;
    const uint64_t bytes = (uint64_t)K * N * (uint32_t)elem_bytes;
    if (groups == 0 || groups * 2 > cus || (K < 16384 && bytes < (32ull << 20))) return {1, 0};
    // two workgroups per CU; from a quarter of the CUs' worth of column groups upwards one per CU (fp16 1 x 8192 x 8192,
    // 128 groups: 2 ranges 23.6 us, 3 or 4 ranges 25.9-26.2, 64-byte groups without ranges 24.3)
    uint32_t splits = groups * 4 > cus ? cus / groups : (2 * cus + groups - 1) / groups;
    if (splits > K / 256) splits = K / 256;
    if (splits > 64) splits = 64;
    if (splits < 2) return {1, 0};
    const uint32_t len = ((K + splits - 1) / splits + 127) / 128 * 128;
    return {(K + len - 1) / len, len};
}

int launch_gevm(bool f16, bool out_f32, const void* x, const void* B, const void* c, void* y, uint32_t K, uint32_t N,
                uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, hipStream_t stream,
                uint32_t split_len, float* partial, uint32_t partial_stride, uint32_t* counters)
{
    if (!f16) launch_gevm_as<float, float>(x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, split_len, partial, partial_stride, counters);
    else if (out_f32) launch_gevm_as<_Float16, float>(x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, split_len, partial, partial_stride, counters);
    else launch_gevm_as<_Float16, _Float16>(x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, split_len, partial, partial_stride, counters);
    return (int)hipGetLastError();
}

int launch_gevm_f64(const double* x, const double* B, const double* c, double* y, uint32_t K, uint32_t N, uint32_t ldb,
                    uint32_t incx, uint32_t incc, uint32_t incy, double alpha, double beta, hipStream_t stream,
                    uint32_t split_len, double* partial, uint32_t partial_stride, uint32_t* counters)
{
    launch_gevm_as<double, double>(x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, split_len, partial, partial_stride, counters);
    return (int)hipGetLastError();
}

}  // namespace decx_hip
