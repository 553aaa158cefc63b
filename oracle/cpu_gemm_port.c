/*
 * TEST INFRASTRUCTURE ONLY -- never linked into, loaded by, or called from the
 * product library.  Used (a) by the tests as a second, structurally different
 * implementation that must agree bit-for-bit with the scalar fma chain, and
 * (b) by the benchmark's CPU-baseline leg, because the reference itself cannot
 * travel to the GPU host.
 *
 * A from-scratch restatement of the *algorithm* of the reference's multithreaded
 * fp32 CPU GEMM (de::blas::cpu::GEMM), not of its source text:
 *
 *   1. B is re-packed into column panels 16 floats wide; inside a panel the K rows
 *      are contiguous (16 floats per k).  A trailing panel that is only 8 wide is
 *      allowed (N rounded up to 8, the host pitch rule).
 *        srcs/modules/BLAS/GEMM/CPU/fp32/matrix_B_arrange_fp32.cxx:58-105,220-263
 *        srcs/modules/BLAS/GEMM/CPU/cpu_GEMM_config.cxx:46-85
 *   2. The output is split over a 2-D grid of T threads whose shape follows the
 *      aspect ratio N:M.
 *        srcs/common/FMGR/fragment_arangement.cxx:134-170
 *        srcs/modules/BLAS/GEMM/CPU/cpu_GEMM_config.cxx:92-141
 *   3. Each thread walks its tile as: panel (16 cols) -> block of 8 rows ->
 *      K slab of 128 -> row -> 1x16 micro-kernel.  The micro-kernel keeps two
 *      8-lane accumulators, runs one FMA per k in ascending order, and parks the
 *      partial sums in dst between slabs; the first slab starts from zero, or
 *      from C for the accumulate form.
 *        srcs/modules/BLAS/GEMM/CPU/cpu_GEMM_config.cxx:40-42 (BL=128, BW=2x8, BH=8)
 *        srcs/modules/BLAS/GEMM/CPU/fp32/x86/GEMM_fp32_kernels_x86_64.h:133-204,209-283
 *
 * Deliberate differences from the reference: the accumulate form seeds each row
 * with its own row of C (the reference hands every row of an 8-row block the
 * block's first C row, GEMM_fp32_kernels_x86_64.h:231-232, which its fp64 twin does
 * not), and the partitioning is plain ceil-division so every (shape, thread count)
 * pair is covered.  Per-element arithmetic is identical: a k-ascending fma chain.
 *
 * Layout contract (the reference's host rule, srcs/modules/core/classes/Matrix.cxx:35-64):
 * every pitch is a multiple of 8 floats, every base pointer 32-byte aligned, and
 * the padding columns of dst may be overwritten.
 */
#include <immintrin.h>
#include <math.h>
#include <omp.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>

enum { SLAB_K = 128, BLOCK_ROWS = 8, PANEL_W = 16 };

/* number of threads the reference would ever use (its pool has 16 slots:
   srcs/modules/core/thread_management/thread_pool.h:40) */
uint32_t cpu_port_max_threads(void) { return 16; }

/* ---- step 1: pack B ------------------------------------------------------ */

static void pack_panels(const float* B, float* packed, uint32_t K, uint32_t N8, uint32_t ldb,
                        uint32_t threads)
{
    const uint32_t panels = (N8 + PANEL_W - 1) / PANEL_W;
#pragma omp parallel for num_threads(threads) schedule(static)
    for (uint32_t p = 0; p < panels; ++p) {
        const uint32_t col = p * PANEL_W;
        const int wide = (col + PANEL_W <= N8);
        float* out = packed + (size_t)p * K * PANEL_W;
        for (uint32_t k = 0; k < K; ++k) {
            const float* src = B + (size_t)k * ldb + col;
            _mm256_store_ps(out + (size_t)k * PANEL_W, _mm256_load_ps(src));
            _mm256_store_ps(out + (size_t)k * PANEL_W + 8,
                            wide ? _mm256_load_ps(src + 8) : _mm256_setzero_ps());
        }
    }
}

/* ---- step 3: micro-kernels ------------------------------------------------ */

static inline void row_x16(const float* a, const float* panel, float* d, const float* seed,
                           uint32_t klen, int first)
{
    __m256 acc0, acc1;
    if (!first)      { acc0 = _mm256_load_ps(d);    acc1 = _mm256_load_ps(d + 8); }
    else if (seed)   { acc0 = _mm256_load_ps(seed); acc1 = _mm256_load_ps(seed + 8); }
    else             { acc0 = _mm256_setzero_ps();  acc1 = _mm256_setzero_ps(); }
    uint32_t k = 0;
    for (; k + 4 <= klen; k += 4) {
        const float* b = panel + (size_t)k * PANEL_W;
        __m256 av;
        av = _mm256_broadcast_ss(a + k);
        acc0 = _mm256_fmadd_ps(av, _mm256_load_ps(b), acc0);
        acc1 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 8), acc1);
        av = _mm256_broadcast_ss(a + k + 1);
        acc0 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 16), acc0);
        acc1 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 24), acc1);
        av = _mm256_broadcast_ss(a + k + 2);
        acc0 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 32), acc0);
        acc1 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 40), acc1);
        av = _mm256_broadcast_ss(a + k + 3);
        acc0 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 48), acc0);
        acc1 = _mm256_fmadd_ps(av, _mm256_load_ps(b + 56), acc1);
    }
    for (; k < klen; ++k) {
        const __m256 av = _mm256_broadcast_ss(a + k);
        acc0 = _mm256_fmadd_ps(av, _mm256_load_ps(panel + (size_t)k * PANEL_W), acc0);
        acc1 = _mm256_fmadd_ps(av, _mm256_load_ps(panel + (size_t)k * PANEL_W + 8), acc1);
    }
    _mm256_store_ps(d, acc0);
    _mm256_store_ps(d + 8, acc1);
}

static inline void row_x8(const float* a, const float* panel, float* d, const float* seed,
                          uint32_t klen, int first)
{
    __m256 acc;
    if (!first)      acc = _mm256_load_ps(d);
    else if (seed)   acc = _mm256_load_ps(seed);
    else             acc = _mm256_setzero_ps();
    for (uint32_t k = 0; k < klen; ++k)
        acc = _mm256_fmadd_ps(_mm256_broadcast_ss(a + k),
                              _mm256_load_ps(panel + (size_t)k * PANEL_W), acc);
    _mm256_store_ps(d, acc);
}

/* one thread's tile: rows [r0,r1), panels [p0,p1) */
static void thread_tile(const float* A, const float* packed, const float* C, float* D,
                        uint32_t K, uint32_t N8, uint32_t lda, uint32_t ldc, uint32_t ldd,
                        uint32_t r0, uint32_t r1, uint32_t p0, uint32_t p1)
{
    for (uint32_t p = p0; p < p1; ++p) {
        const uint32_t col = p * PANEL_W;
        const int wide = (col + PANEL_W <= N8);
        const float* panel = packed + (size_t)p * K * PANEL_W;
        for (uint32_t rb = r0; rb < r1; rb += BLOCK_ROWS) {
            const uint32_t rend = rb + BLOCK_ROWS < r1 ? rb + BLOCK_ROWS : r1;
            for (uint32_t ks = 0; ks < K; ks += SLAB_K) {
                const uint32_t klen = ks + SLAB_K < K ? SLAB_K : K - ks;
                for (uint32_t r = rb; r < rend; ++r) {
                    const float* a = A + (size_t)r * lda + ks;
                    float* d = D + (size_t)r * ldd + col;
                    const float* seed = C ? C + (size_t)r * ldc + col : NULL;
                    if (wide) row_x16(a, panel + (size_t)ks * PANEL_W, d, seed, klen, ks == 0);
                    else      row_x8 (a, panel + (size_t)ks * PANEL_W, d, seed, klen, ks == 0);
                }
            }
        }
    }
}

/* ---- step 2: thread grid --------------------------------------------------- */

static void thread_grid(uint32_t T, uint32_t N, uint32_t M, uint32_t* tx, uint32_t* ty)
{
    /* ty ~ sqrt(T * M / N), snapped to the nearest divisor of T */
    if (T <= 1) { *tx = *ty = 1; return; }
    const float ratio = (float)N / (float)M;
    uint32_t base = (uint32_t)lroundf(sqrtf((float)T / ratio));
    if (base < 2)      { *tx = T; *ty = 1; return; }
    if (base > T)      { *tx = 1; *ty = T; return; }
    uint32_t up = base, down = base;
    while (T % up) ++up;
    while (T % down) --down;
    const uint32_t pick = (up - base) > (base - down) ? down : up;
    *ty = pick;
    *tx = T / pick;
}

/*
 * D = A.B (C == NULL) or D = A.B + C.  `scratch` must hold cpu_port_scratch_floats(K, N)
 * floats, 32-byte aligned.  Returns 0, or -1 on a layout-contract violation.
 */
size_t cpu_port_scratch_floats(uint32_t K, uint32_t N)
{
    const uint32_t N8 = (N + 7u) & ~7u;
    return (size_t)((N8 + PANEL_W - 1) / PANEL_W) * K * PANEL_W;
}

int cpu_port_gemm_f32(const float* A, const float* B, const float* C, float* D,
                      uint32_t M, uint32_t N, uint32_t K,
                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                      float* scratch, uint32_t threads)
{
    if ((lda | ldb | ldd | (C ? ldc : 0)) & 7u) return -1;
    if (((uintptr_t)A | (uintptr_t)B | (uintptr_t)D | (uintptr_t)C | (uintptr_t)scratch) & 31u) return -1;
    if (threads < 1) threads = 1;
    if (threads > cpu_port_max_threads()) threads = cpu_port_max_threads();
    const uint32_t N8 = (N + 7u) & ~7u;
    if (N8 > ldb || N8 > ldd || (C && N8 > ldc)) return -1;
    const uint32_t panels = (N8 + PANEL_W - 1) / PANEL_W;

    pack_panels(B, scratch, K, N8, ldb, threads);

    uint32_t tx, ty;
    thread_grid(threads, N, M, &tx, &ty);
    const uint32_t panels_per = (panels + tx - 1) / tx;
    uint32_t rows_per = (M + ty - 1) / ty;
    rows_per = (rows_per + BLOCK_ROWS - 1) / BLOCK_ROWS * BLOCK_ROWS;

#pragma omp parallel num_threads(tx * ty)
    {
        /* one tile per thread when the runtime grants tx*ty threads; a stride loop
           keeps every tile covered when it grants fewer */
        const uint32_t granted = (uint32_t)omp_get_num_threads();
        for (uint32_t t = (uint32_t)omp_get_thread_num(); t < tx * ty; t += granted) {
            const uint32_t gx = t % tx, gy = t / tx;
            uint32_t p0 = gx * panels_per, p1 = p0 + panels_per;
            uint32_t r0 = gy * rows_per, r1 = r0 + rows_per;
            if (p1 > panels) p1 = panels;
            if (r1 > M) r1 = M;
            if (p0 < p1 && r0 < r1)
                thread_tile(A, scratch, C, D, K, N8, lda, ldc, ldd, r0, r1, p0, p1);
        }
    }
    return 0;
}
