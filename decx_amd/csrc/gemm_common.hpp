// Shared declarations of the gfx950 GEMM kernels: argument block, tile-shape table,
// block -> tile mapping.  Device code here is written for CDNA4 only (wave64, MFMA,
// 160 KB LDS per CU, 8 XCDs with one L2 each).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

namespace decx_hip {

typedef float    floatx4  __attribute__((ext_vector_type(4)));
typedef float    floatx2  __attribute__((ext_vector_type(2)));
typedef float    floatx16 __attribute__((ext_vector_type(16)));
typedef _Float16 halfx8   __attribute__((ext_vector_type(8)));
typedef _Float16 halfx4   __attribute__((ext_vector_type(4)));
typedef uint32_t uintx4   __attribute__((ext_vector_type(4)));
typedef uint32_t uintx2   __attribute__((ext_vector_type(2)));

// One GEMM problem: D = A.B  (C == nullptr)  or  D = fma(C, beta, alpha * (A.B)).
// All matrices row-major; ld* are row pitches in elements.
struct GemmArgs {
    const void* A;
    const void* B;
    const void* C;
    void*       D;
    uint32_t M, N, K;
    uint32_t lda, ldb, ldc, ldd;
    float alpha, beta;
    double alpha64, beta64;      // the same two scalars for the fp64 kernels
    uint32_t tiles_m, tiles_n;   // number of block tiles along M and N
    uint32_t vec_ok;             // 1: every base pointer is 16-byte aligned and every pitch a multiple of 16 bytes
    uint32_t cus;                // compute units of the device (0: not given, the kernels take 256)
    // Split K (direct-load kernels; a 1-D grid of split_first whole tiles, then split 0 of every split tile, split 1 of
    // every split tile, ...): split z multiplies k in [z * split_len, (z + 1) * split_len), the last one up to K (its range may be longer or shorter than the others').  Every workgroup stores its accumulators (fp32, or fp64 for fp64 operands) to its
    // slot of split_ws and counts itself in at split_counters[tile]; the one that arrives last adds all slots of the
    // tile in split order (its own included, so the result does not depend on who is last), writes D and puts the
    // counter back to zero (split_k_exchange.hpp).
    uint32_t group_m;            // tile-rows per L2 patch of the block -> tile map (0: the default, kGroupM)
    uint32_t split_len;          // 0: no split
    uint32_t split_count;        // splits per split tile
    uint32_t split_first;        // tiles below this index are multiplied whole, by one workgroup each (full rounds of
                                 // workgroups, or one to three per CU that share their CU with the split ones)
    uint32_t split_urgent;       // 1: the workgroups of split tiles raise their wave priority (set where whole tiles
                                 // share the CUs with them and K is short: the split ones then finish first and meet
                                 // in the workspace while the whole ones still multiply)
    void*    split_ws;
    uint32_t* split_counters;    // one per tile, zero before and after every launch
    // Convolution as an implicit GEMM (used by the CONV instantiations only): row p of the A operand is the
    // patch under output pixel (p / conv_wout, p % conv_wout) of an image stored [row][column][channel]; its K
    // elements are KH runs of conv_seg_bytes contiguous bytes (KW columns x channel pitch), conv_seg_stride bytes
    // apart (one image row).  D row p lands at pixel pitch ldd inside image rows of conv_dst_row floats.
    uint32_t conv_wout;
    uint32_t conv_seg_bytes;
    uint32_t conv_px_bytes;      // bytes between patches of horizontally adjacent output pixels
    uint32_t conv_dst_row;       // floats per output image row
    uint64_t conv_seg_stride;
    uint64_t conv_py_bytes;      // bytes between patches of vertically adjacent output pixels
    uint64_t conv_image_bytes;   // size of the image the patches lie in
};

constexpr uint32_t kNarrowN = 32;   // fp32 outputs of at most this many columns run the smallest tile class as 128 x 32
constexpr int kXcds = 8;        // MI355X: 8 accelerator complex dies, blocks are dealt to them round-robin
constexpr int kGroupM = 4;      // tile-rows per L2 patch (4 x 8 tiles run together on one XCD's 32 CUs)

// Maps the hardware block index to a tile.  Hardware deals consecutive block ids to
// consecutive XCDs; each XCD has a private L2.  Step 1 gives every XCD a contiguous
// range of logical ids (the first 8 * (nb / 8) blocks; the up to 7 that remain keep their
// ids, at the end of the last range), step 2 walks logical ids in groups of kGroupM tile-rows so the
// 32 tiles resident on one XCD form a compact patch that shares A rows and B columns.
// `id`: the block's index among the `nb` blocks dealt to the XCDs in turn that it belongs to (all tiles of a whole
// product; the whole tiles, or one split of the split tiles, of a split one), `first`: the tile the first of them takes.
__device__ __forceinline__ void block_to_tile(const GemmArgs& g, uint32_t id, uint32_t nb, uint32_t first, uint32_t& tile_m, uint32_t& tile_n)
{
    const uint32_t per_xcd = nb / kXcds;
    if (id < per_xcd * kXcds) id = (id % kXcds) * per_xcd + id / kXcds;
    id += first;
    const uint32_t group_m = g.group_m ? g.group_m : (uint32_t)kGroupM;
    const uint32_t per_group = group_m * g.tiles_n;
    const uint32_t group = id / per_group;
    const uint32_t first_m = group * group_m;
    const uint32_t rows = (g.tiles_m - first_m) < group_m ? (g.tiles_m - first_m) : group_m;
    const uint32_t in_group = id % per_group;
    tile_m = first_m + in_group % rows;
    tile_n = in_group / rows;
}
__device__ __forceinline__ void block_to_tile(const GemmArgs& g, uint32_t& tile_m, uint32_t& tile_n)
{
    block_to_tile(g, blockIdx.x, g.tiles_m * g.tiles_n, 0, tile_m, tile_n);
}

// Where a block of a split-K launch works: its tile's index, its split and the number of splits of its tile (1 for the
// whole tiles in front).
struct SplitBlock { uint32_t tile, z, splits; };
__device__ __forceinline__ SplitBlock split_block(const GemmArgs& g, uint32_t& tile_m, uint32_t& tile_n)
{
    const uint32_t tiles = g.tiles_m * g.tiles_n;
    if (blockIdx.x < g.split_first) {
        block_to_tile(g, blockIdx.x, g.split_first, 0, tile_m, tile_n);
        return {0u, 0u, 1u};                               // (whole tiles have no slot)
    }
    const uint32_t r = blockIdx.x - g.split_first, rest = tiles - g.split_first;
    block_to_tile(g, r % rest, rest, g.split_first, tile_m, tile_n);
    return {r % rest, r / rest, g.split_count};
}

// ---- tile-shape table shared by the planner and the launchers -----------------

// Size classes; the block tile each stands for depends on the element type and the kernel family (tile_info_*):
// LARGE 256 x 256 (fp16, and the register-staged fp32 kernels) or 256 x 128 (fp32 and fp64 direct-to-LDS),
// MEDIUM 128 x 128, SMALL 64 x 64 (128 x 32 for fp32 outputs of at most kNarrowN columns).
enum TileShape : int {
    TILE_LARGE  = 0,
    TILE_MEDIUM = 1,
    TILE_SMALL  = 2,
    TILE_COUNT  = 3,                // the classes every element type has
    // fp16 on 16-byte aligned operands only: tiles between the two largest classes
    TILE_F16_192x192 = 3,
    TILE_F16_192x256 = 4,
    TILE_F16_256x192 = 5,
    TILE_F16_COUNT = 6,
};

// per_cu: workgroups of the shape that fit a CU together.  full: throughput of a CU filled with them, alone: of
// a workgroup that has its CU to itself (or, for the largest tile, of a chip no more than half occupied: fp16
// runs under the power cap, so a CU does more when its neighbours idle), both relative to the largest tile on
// a full chip.  Smaller tiles fetch more operand bytes per flop and lean on co-resident workgroups to hide the
// latency of their copies.
struct TileInfo { int bm, bn, threads, per_cu; float full, alone; };

// Time (in units of tile area over rate) of `tiles` workgroups on `cus` CUs: whole rounds of cus * per_cu
// workgroups at the full rate, then the remainder, whose busiest CU holds m workgroups and runs at a rate
// between the lone-workgroup one (m = 1) and the full one (m = per_cu).
__host__ inline double tile_cost(const TileInfo& ti, uint64_t tiles, uint32_t cus)
{
    const double area = (double)ti.bm * ti.bn;
    const uint64_t slots = (uint64_t)cus * ti.per_cu;
    const uint64_t rounds = tiles / slots, rest = tiles % slots;
    double t = (double)rounds * ti.per_cu * area / ti.full;
    if (rest > 0) {
        const uint64_t m = (rest + cus - 1) / cus;
        double rate = ti.alone;
        if (ti.per_cu > 1) rate += (ti.full - ti.alone) * (double)(m - 1) / (double)(ti.per_cu - 1);
        else if (rest > cus / 2)                           // between half and all CUs busy: towards the full-chip rate
            rate += (ti.full - ti.alone) * (double)(rest - cus / 2) / (double)(cus - cus / 2);
        t += (double)m * area / rate;
    }
    return t;
}

// fp32, measured on MI355X (direct-to-LDS kernels; nanoseconds per k and workgroup with m workgroups on the CU, slopes
// of time against K): 256 x 128 (the largest tile; 256 x 256 in the register-staged family) 108.9 alone, 109.6 two per
// CU (the matrix pipe alone would take 106.7); 128 x 128 55.8 / 55.1 / 56.3 for one to three per CU (53.3), 58.4 in a
// second round; 64 x 64 15.8 / 15.1 / 15.0 / 15.0 for one to four per CU (13.3), 15.5 per workgroup in launches of
// several rounds.  The predicated register-staged kernels (operands that are not 16-byte aligned) run at about
// 1 : 0.8 : 0.7 of the largest tile, two workgroups per CU.
// N: columns of the output; at most kNarrowN of them turn the smallest aligned tile into 128 x 32 (the same area, no
// idle half: 65536 x 32 x 1024 46.8 us against 81.9 us for 64 columns on 64 x 64 tiles).
__host__ inline TileInfo tile_info_f32(int shape, bool aligned = true, uint32_t N = 0xffffffffu)
{
    switch (shape) {
    case TILE_LARGE: return aligned ? TileInfo{256, 128, 256, 2, 1.00f, 1.00f} : TileInfo{256, 256, 512, 1, 1.00f, 1.00f};
    case TILE_MEDIUM: return {128, 128, 256, aligned ? 3 : 2, aligned ? 0.97f : 0.80f, aligned ? 0.98f : 0.72f};
    default:
        if (aligned && N <= kNarrowN) return {128, 32, 256, 4, 0.90f, 0.70f};
        return { 64,  64, 256, aligned ? 4 : 2, aligned ? 0.90f : 0.70f, aligned ? 0.865f : 0.49f};
    }
}
// fp16 (TFLOP/s per CU; TILE_F16_*: tiles between the two largest classes, one workgroup per CU, chosen where they cut
// the output into a number of pieces that suits the CUs better -- 3000^3: 256 tiles of 192 x 192, 52.7 us, against 144 of
// 256 x 256, 56.5 us; 4608^3: 432 of 256 x 192, 174 us, against 324, 186 us): 256 x 256 4.64 on a full chip, 6.4 with at most half the CUs busy; 128 x 128 3.1 alone,
// 3.9 two per CU; 64 x 64 1.27 alone, 2.4 four per CU.  Predicated register-staged kernels about 1 : 0.6 : 0.25.
__host__ inline TileInfo tile_info_f16(int shape, bool aligned = true)
{
    switch (shape) {
    // per flop these read a third more from LDS than 256 x 256 (wave tiles of 48 x 96 and 96 x 64): measured 0.80 /
    // 0.89 / 0.88 of its rate on a full chip (6144^3: 1132 / 1242 / 1227 TFLOP/s against 1400) and 0.65 / 0.74 / 0.74
    // of it on a chip at most half busy, where the largest tile runs 1.38 times its full-chip rate
    case TILE_F16_192x192: return {192, 192, 512, 1, 0.80f, 0.90f};
    case TILE_F16_192x256: return {192, 256, 512, 1, 0.89f, 1.02f};
    case TILE_F16_256x192: return {256, 192, 512, 1, 0.88f, 1.02f};
    case TILE_LARGE: return {256, 256, aligned ? 512 : 256, 1, 1.00f, aligned ? 1.38f : 1.00f};
    case TILE_MEDIUM: return {128, 128, aligned ? 512 : 128, 2, aligned ? 0.84f : 0.60f, aligned ? 0.70f : 0.50f};
    default:           return { 64,  64, aligned ? 256 :  64, aligned ? 4 : 2, aligned ? 0.55f : 0.25f, aligned ? 0.27f : 0.12f};
    }
}

// fp64 (nanoseconds per k and workgroup): 256 x 128 (what TILE_LARGE stands for) 218.6 alone (the matrix pipe alone:
// 213.4); 128 x 128 109.4 alone or two per CU; 64 x 64 28.2 alone, 28.8 two per CU.  All three run 8 wavefronts per
// workgroup: with 4, the two smaller tiles are a tenth slower (their accumulators leave no room for the four workgroups
// per CU that the fp32 tiles use).
__host__ inline TileInfo tile_info_f64(int shape)
{
    switch (shape) {
    case TILE_LARGE: return {256, 128, 512, 1, 1.00f, 1.00f};
    case TILE_MEDIUM: return {128, 128, 512, 2, 1.00f, 1.00f};
    default:           return { 64,  64, 512, 2, 0.95f, 0.97f};
    }
}

int launch_gemm_f32(int shape, bool edge, const GemmArgs& args, hipStream_t stream);
// fp64: direct-to-LDS kernels on 16-byte aligned operands, else (or with `plain`) a one-thread-per-element kernel
// The direct-load kernels address a slab as scalar base + 32-bit lane offset: 256 rows of A and 64 rows
// of B must span less than 2 GiB (any realistic pitch does; otherwise the register-staged kernels run).  The fp32
// epilogue addresses D and C the same way, with a lane offset of up to 4 rows and a row of the tile.
inline bool dma_offsets_fit(const GemmArgs& g, uint32_t elem_bytes)
{
    return 256ull * g.lda * elem_bytes < (1ull << 31) && 64ull * g.ldb * elem_bytes + 16ull < (1ull << 31) &&
           8ull * g.ldd * elem_bytes < (1ull << 31) && (!g.C || 8ull * g.ldc * elem_bytes < (1ull << 31));
}

int launch_gemm_f64(int shape, bool plain, const GemmArgs& args, hipStream_t stream);
// direct-to-LDS fp32 kernel for any M, N, K >= 1 on 16-byte aligned bases and pitches, in the three tile shapes
int launch_gemm_f32_dma(int shape, const GemmArgs& args, hipStream_t stream);

struct SplitPlan { uint32_t splits, len; };     // ranges of K and their length
// the same kernels with the A operand gathered from an image (GemmArgs::conv_*): 2-D convolution without an im2col buffer
int launch_conv2d_f32_dma(int shape, const GemmArgs& args, hipStream_t stream);
// shallow patches and at most 32 kernels: a lane per output pixel on the vector pipe (conv_direct.hip)
bool conv2d_direct_pays(uint32_t out_c, uint64_t patch_floats, uint32_t channel_pitch, uint32_t depth);
int launch_conv2d_direct_f32(const GemmArgs& args, uint32_t channel_pitch, uint32_t depth, hipStream_t stream);
int launch_gemm_f16(int shape, bool edge, const GemmArgs& args, hipStream_t stream);
// direct-to-LDS fp16 kernel for any M, N, K >= 1 on 16-byte aligned bases and pitches, in the three tile shapes
int launch_gemm_f16_dma(int shape, const GemmArgs& args, hipStream_t stream);
// complex GEMM helpers: B -> the real 2K x 2N expansion of alpha * B; D = beta * C (interleaved complex)
template <typename T>
int launch_complex_expand_b(const T* B, T* Bx, uint32_t K, uint32_t N, uint32_t ldb, uint32_t ldx, T ar, T ai, hipStream_t stream);
template <typename T>
int launch_complex_scale(const T* C, T* D, uint32_t M, uint32_t N, uint32_t ldc, uint32_t ldd, T br, T bi, hipStream_t stream);

// y = alpha * A.x (+ beta * c) and y = alpha * x.B (+ beta * c); f16 inputs accumulate in fp32 and write
// fp32 (out_f32) or fp16.  inc* are element strides.
uint32_t gemv_rows_per_block(uint32_t M);
bool gemv_gather_pays(uint32_t M, uint32_t K, uint32_t incx);
int launch_gather(int elem_bytes, const void* x, void* dst, uint32_t K, uint32_t inc, hipStream_t stream);
int launch_gemv(bool f16, bool out_f32, const void* A, const void* x, const void* c, void* y, uint32_t M, uint32_t K,
                uint32_t lda, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, hipStream_t stream);
int launch_gevm(bool f16, bool out_f32, const void* x, const void* B, const void* c, void* y, uint32_t K, uint32_t N,
                uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, hipStream_t stream,
                uint32_t split_len = 0, float* partial = nullptr, uint32_t partial_stride = 0, uint32_t* counters = nullptr);
SplitPlan plan_gevm_split(int elem_bytes, uint32_t N, uint32_t K, uint32_t cus);
int launch_gemv_f64(const double* A, const double* x, const double* c, double* y, uint32_t M, uint32_t K, uint32_t lda,
                    uint32_t incx, uint32_t incc, uint32_t incy, double alpha, double beta, hipStream_t stream);
int launch_gevm_f64(const double* x, const double* B, const double* c, double* y, uint32_t K, uint32_t N, uint32_t ldb,
                    uint32_t incx, uint32_t incc, uint32_t incy, double alpha, double beta, hipStream_t stream,
                    uint32_t split_len = 0, double* partial = nullptr, uint32_t partial_stride = 0, uint32_t* counters = nullptr);

}  // namespace decx_hip
