// The C ABI declared in include/decx_hip.h: argument checking, the tile planner, and
// thin wrappers over the HIP runtime.  No C++ type crosses this boundary.
#include "../../include/decx_hip.h"
#include "../../include/decx_hip_profiling.h"
#include "gemm_common.hpp"
#include "split_k_exchange.hpp"
#include "split_counter_ring.hpp"

#include <chrono>
#include <cstring>
#include <functional>
#include <mutex>
#include <thread>
#include <vector>

using namespace decx_hip;

namespace {

struct DeviceState {
    bool ready = false;
    int device = -1;
    int compute_units = 256;       // MI355X; used by the planner before init
    hipDeviceProp_t prop;
};
DeviceState g_dev;

// Workspace of decx_hip_gemm_f32_static: a device array that exists from the moment the code object is loaded, so the
// entry point never allocates.  Each GPU holds its own copy at its own address; g_scratch[d] is the address on device d,
// looked up once by decx_hip_init(d).  The array's name is only a host-side handle: kernels, copies and fills get the
// looked-up pointer.
constexpr size_t kScratchBytes = (size_t)DECX_HIP_STATIC_WORKSPACE_BYTES;
constexpr int kMaxDevices = 16;
static __device__ __align__(256) unsigned char scratch[kScratchBytes];
void* g_scratch[kMaxDevices] = {};

// Counters of the split-K kernels (per tile, or per column group of a vector x matrix product: one, plus one per group
// of ranges when there are many; the workgroups of a tile count themselves in, the last one sums the tile and puts
// the counter back to zero, so the array is all zero between launches).  Every launch takes the next window of the
// array; a window only goes to a new launch once the launches that had it before are known to be over
// (split_counter_ring.hpp: same stream, a completed event, or an idle stream), and a launch that cannot have one
// runs unsplit.
constexpr uint32_t kSplitCounters = 1u << 16;
static __device__ uint32_t split_counters[kSplitCounters];
uint32_t* g_split_counters[kMaxDevices] = {};
std::mutex g_counter_mutex;

struct HipRingRuntime final : CounterRingRuntime {
    // Events that are not in use, per device (an event belongs to the device it was created on).  decx_hip_init() puts
    // kEventsAtInit of them here, so that launches from several streams do not create events in the middle of a
    // caller's loop; more are made only when that many windows are in flight at once.
    static constexpr int kEventsAtInit = 32;
    std::vector<hipEvent_t> pools[kMaxDevices];
    std::vector<hipEvent_t>& pool() { return pools[g_dev.device >= 0 && g_dev.device < kMaxDevices ? g_dev.device : 0]; }
    void prefill()
    {
        std::vector<hipEvent_t>& p = pool();
        while ((int)p.size() < kEventsAtInit) {
            hipEvent_t ev = nullptr;
            if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) { (void)hipGetLastError(); return; }
            p.push_back(ev);
        }
    }
    void* record_event(void* stream) override
    {
        std::vector<hipEvent_t>& p = pool();
        hipEvent_t ev = nullptr;
        if (!p.empty()) { ev = p.back(); p.pop_back(); }
        else if (hipEventCreateWithFlags(&ev, hipEventDisableTiming) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
        if (hipEventRecord(ev, (hipStream_t)stream) != hipSuccess) { (void)hipGetLastError(); p.push_back(ev); return nullptr; }
        return ev;
    }
    bool event_done(void* event) override
    {
        const hipError_t e = hipEventQuery((hipEvent_t)event);
        if (e != hipSuccess) (void)hipGetLastError();              // "not ready" is no error of the caller's
        return e == hipSuccess;
    }
    void release_event(void* event) override { pool().push_back((hipEvent_t)event); }
    bool stream_idle_or_gone(void* stream) override
    {
        const auto gone = [](hipError_t e) {
            return e == hipErrorContextIsDestroyed || e == hipErrorInvalidHandle || e == hipErrorInvalidResourceHandle;
        };
        // (a stream that is recording a graph must not be queried: the query would end the recording with an error)
        hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
        hipError_t e = hipStreamIsCapturing((hipStream_t)stream, &st);
        if (e != hipSuccess) { (void)hipGetLastError(); return gone(e); }
        if (st != hipStreamCaptureStatusNone) return false;
        e = hipStreamQuery((hipStream_t)stream);
        if (e != hipSuccess) (void)hipGetLastError();
        return e == hipSuccess || gone(e);
    }
};
HipRingRuntime g_ring_runtime;
CounterRing* g_rings[kMaxDevices] = {};

// A window of `n` counters for a launch on `stream`, or nullptr (run unsplit).  `ticket` goes to commit_split_counters()
// right behind the launch.
uint32_t* take_split_counters(uint32_t n, hipStream_t stream, uint64_t& ticket)
{
    ticket = 0;
    const int d = g_dev.device;
    if (d < 0 || d >= kMaxDevices || !g_split_counters[d] || !g_rings[d]) return nullptr;
    hipStreamCaptureStatus st = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &st) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    uint64_t key = (uint64_t)(uintptr_t)stream;
    if (stream == hipStreamPerThread) key ^= (uint64_t)std::hash<std::thread::id>{}(std::this_thread::get_id()) << 8;
    std::lock_guard<std::mutex> lock(g_counter_mutex);
    const uint32_t at = g_rings[d]->take(g_ring_runtime, (void*)stream, key, n, st != hipStreamCaptureStatusNone, &ticket);
    return at == CounterRing::kNone ? nullptr : g_split_counters[d] + at;
}

void commit_split_counters(uint64_t ticket)
{
    if (!ticket) return;
    const int d = g_dev.device;
    std::lock_guard<std::mutex> lock(g_counter_mutex);
    if (d >= 0 && d < kMaxDevices && g_rings[d]) g_rings[d]->commit(g_ring_runtime, ticket);
}

inline int hip_rc(hipError_t e) { return (int)e; }
inline hipStream_t as_stream(void* s) { return (hipStream_t)s; }

inline bool aligned16(const void* p) { return ((uintptr_t)p & 15u) == 0; }

// Picks the block tile by the time estimate of tile_cost().  Big tiles win once they fill the chip;
// small tiles win while the grid would otherwise leave CUs idle.  Ties go to the larger tile.
int choose_tile_f64(uint32_t M, uint32_t N)
{
    int best = TILE_SMALL;
    double best_cost = 1e300;
    for (int s = TILE_COUNT - 1; s >= 0; --s) {
        const TileInfo ti = tile_info_f64(s);
        const uint64_t tiles = (uint64_t)((M + ti.bm - 1) / ti.bm) * ((N + ti.bn - 1) / ti.bn);
        const double cost = tile_cost(ti, tiles, g_dev.compute_units);
        if (cost <= best_cost) { best_cost = cost; best = s; }
    }
    return best;
}

int choose_tile(bool f16, uint32_t M, uint32_t N, bool aligned)
{
    // candidates from the smallest to the largest tile: ties go to the larger one
    static const int kBasic[] = {TILE_SMALL, TILE_MEDIUM, TILE_LARGE};
    static const int kF16Aligned[] = {TILE_SMALL, TILE_MEDIUM, TILE_F16_192x192, TILE_F16_192x256, TILE_F16_256x192, TILE_LARGE};
    const int* const shapes = f16 && aligned ? kF16Aligned : kBasic;
    const int count = f16 && aligned ? 6 : 3;
    int best = TILE_SMALL;
    double best_cost = 1e300;
    for (int c = 0; c < count; ++c) {
        const int s = shapes[c];
        const TileInfo ti = f16 ? tile_info_f16(s, aligned) : tile_info_f32(s, aligned, N);
        const uint64_t tiles = (uint64_t)((M + ti.bm - 1) / ti.bm) * ((N + ti.bn - 1) / ti.bn);
        const double cost = tile_cost(ti, tiles, g_dev.compute_units);
        if (cost <= best_cost) { best_cost = cost; best = s; }
    }
    return best;
}

int check_gemm(const void* A, const void* B, const void* C, const void* D, uint32_t M, uint32_t N, uint32_t K,
               uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd)
{
    if (M == 0 || N == 0) return DECX_HIP_OK;
    if (!A || !B || !D) return DECX_HIP_E_INVALID_ARG;
    if (lda < K || ldb < N || ldd < N || (C && ldc < N)) return DECX_HIP_E_INVALID_ARG;
    return DECX_HIP_OK;
}

// Split K is planned for products on 16-byte aligned operands whose tiles would leave CUs idle or unevenly loaded.
// The ranges are added inside the kernel (split_k_exchange), so a split costs no second launch, and it runs on one of
// the smaller tiles whatever the whole product would take.  Tile and number of ranges are the pair that a small model
// of the kernel's time likes best, in microseconds:
//   workgroups = tiles x ranges, each as long as its range.  `fit` of them share a CU: whole rounds of fit x CUs
//   workgroups run at the full-CU rate and the remainder, m on the busiest CU, at the measured rate of m co-resident
//   workgroups (ns_per_k[m], per workgroup; slopes of time against K at exactly m tiles per CU);
//   fp32: a remainder of more than half a workgroup per CU right after ONE full round lands unevenly (the CUs that
//   finish first take several) and counts as two;
//   fp16 on 128 x 128 tiles: a workgroup that has its CU to itself runs faster the fewer CUs are busy (the power cap);
//   every range costs a trip of the output through the workspace (us_per_mb) and the last workgroup a round trip to
//   memory per 16 pieces a lane loads (us_per_trip: where several workgroups share a CU the others hide most of it).
// fp32 fitted to 20 output shapes x K = 777 ... 16384 x 1 ... 8 ranges, fp16 and fp64 to 12 and 9 shapes x 2 ... 32
// ranges: the estimate is within 4 % of the measurement on most, the pick within 1 % (fp16: 2.5 %) of the best on
// average.  The whole product is kept unless the split promises 3 % (4 % left a launch-bound fp16 shape of the held-out sweep 10 % off its best plan).
struct SplitChoice { int shape; uint32_t splits, len, first, urgent; };     // first: tiles in front that stay whole; urgent: GemmArgs::split_urgent
struct SplitTile {
    int shape, fit, pieces;          // size class, workgroups per CU, 16-byte pieces of accumulators per lane
    double ns_per_k[5];              // per workgroup with m = 1 .. fit of them on the CU
    double ns_per_k_one_round[5];    // the same in a launch of at most fit x CUs workgroups, where the kernel has a tighter loop (0: none)
};
struct SplitModel {
    SplitTile tiles[3]; int n_tiles;
    uint32_t len_align, acc_bytes;   // ranges are multiples of the deepest slab; bytes of an accumulator
    double us_fixed, us_per_trip, us_per_mb, whole_flop_per_us;      // the last: the largest tile, per CU of a full chip
    bool uneven_second_round;
    // Whole tiles that share their CUs with split ones (on tiles[shared_tile]; rate 0: not planned): microseconds of a
    // launch beside its k steps, nanoseconds per k step of a CU (plus shared_ns_busy x the share of the CUs that hold
    // a split workgroup: fp16 runs into the power cap), and the longest K at which the split workgroups run at a
    // raised priority
    int shared_tile;
    double shared_us_fixed, shared_ns_per_k, shared_ns_busy;
    uint32_t urgent_max_k;
};
// 64 x 64 tiles of 32 KB LDS: four fit a CU (160 KB would hold five, but time against the number of tiles steps as for four)
static const SplitModel kSplitF32 = {{{TILE_SMALL, 4, 4, {0, 17.72, 15.51, 15.07, 14.77}, {0, 15.8, 15.1, 15.0, 14.96}}, {}, {}}, 1, 32, 4, 1.0, 0.4, 0.15, 0.600e6, true,
                                     0, 6.2, 14.0, 0, 2048};
static const SplitModel kSplitF16 = {{{TILE_SMALL, 4, 4, {0, 3.4, 3.3, 3.15, 3.1}}, {TILE_MEDIUM, 2, 8, {0, 7.4, 7.0}}, {TILE_LARGE, 1, 32, {0, 22.7}}}, 3,
                                     64, 4, 2.0, 2.0, 0.15, 5.4e6, false, 1, 4.3, 6.5, 1.6, 0};     // (fixed: 2.0 us; with 0.5, 4096 x 512 x 2048 went on two ranges, 15.8 us, where whole takes 14.0)
static const SplitModel kSplitF64 = {{{TILE_SMALL, 2, 4, {0, 28.2, 28.8}}, {}, {}}, 1, 32, 8, 0.5, 2.0, 0.30, 0.300e6, false,
                                     0, 5.7, 27.8, 0, 1u << 30};

TileInfo dma_tile_info(int elem_bytes, int shape, uint32_t N);

// K on about p ranges whose starts are multiples of `align` (the deepest slab): `len` for all but the last, which takes
// what is left.  Rounding K / p up makes the last range the shortest, rounding it down the longest; the one whose
// longest range is shorter wins (K = 777 on two: 416 + 361 or 384 + 393).
struct RangeLen { uint32_t len, ranges, longest; };
RangeLen range_len(uint32_t K, uint32_t p, uint32_t align)
{
    const uint32_t up = ((K + p - 1) / p + align - 1) / align * align, n_up = (K + up - 1) / up;
    const uint32_t down = K / p / align * align;
    if (down && (uint64_t)down * p < K && n_up == p) {
        const uint32_t last = K - (p - 1) * down;
        if (last < up) return {down, p, last};
    }
    return {up, n_up, up};
}

SplitChoice split_plan_model(int elem_bytes, uint32_t M, uint32_t N, uint32_t K, int whole_shape, const TileInfo& whole)
{
    const SplitModel& md = elem_bytes == 8 ? kSplitF64 : elem_bytes == 2 ? kSplitF16 : kSplitF32;
    const uint32_t cus = g_dev.compute_units;
    constexpr double kLaunch = 4.0;                             // launch to launch
    if (K < 512) return {whole_shape, 1, 0, 0};
    const double out_mb = (double)M * N * md.acc_bytes / 1e6;
    const auto tiles_of = [&](int shape) {
        const TileInfo ti = dma_tile_info(elem_bytes, shape, N);
        return (uint64_t)((M + ti.bm - 1) / ti.bm) * ((N + ti.bn - 1) / ti.bn);
    };
    // `whole` tiles in front run unsplit (full rounds of workgroups: whole is a multiple of fit x CUs), the other
    // t - whole on `ranges` ranges of `len`
    const auto estimate = [&](const SplitTile& st, uint64_t t, uint32_t len, uint32_t ranges, uint64_t whole = 0) {
        const uint64_t wgs = (t - whole) * ranges, slots = (uint64_t)st.fit * cus;
        const uint64_t full = wgs / slots, rem = wgs % slots;
        uint64_t m = (rem + cus - 1) / cus;
        if (md.uneven_second_round && full == 1 && rem > cus / 2 && rem <= cus) m = 2;
        const double* rate = (whole + wgs <= slots && st.ns_per_k_one_round[1] > 0) ? st.ns_per_k_one_round : st.ns_per_k;
        double lone = rate[1];
        if (elem_bytes == 2 && st.shape == TILE_MEDIUM)        // 5.4 ns with half the CUs busy, 7.4 with all
            lone = wgs <= cus / 2 ? 5.4 : 5.4 + 2.0 * (double)(wgs - cus / 2) / (double)(cus - cus / 2);
        const uint32_t k_whole = (K + md.len_align - 1) / md.len_align * md.len_align;
        double last = m == 1 ? lone : (double)m * rate[m];          // the remainder's round, per k step
        if (elem_bytes == 2 && st.shape == TILE_MEDIUM && full == 0 && m == 2)      // two on some CUs, one on the others: 5.8 ns with a
            last = 2.0 * (5.6 + 1.4 * (double)(rem - cus) / (double)cus);           // quarter of the CUs doubly loaded, 6.0 with half, 7.0 with all
        const double ns = (double)len * ((double)full * st.fit * rate[st.fit] + last) +
                          (double)k_whole * (double)(whole / slots) * st.fit * rate[st.fit];
        double us = ns * 1e-3 + kLaunch;
        if (ranges > 1) {
            const uint32_t group = st.pieces < 16 ? st.pieces : 16, batch = 16 / group, per_slot = st.pieces / group;
            uint32_t trips = (ranges + batch - 1) / batch * per_slot;
            if (ranges > kSplitFlat)                           // two levels: a group of kSplitGroup, the group sums, and a second store and count
                trips = ((kSplitGroup + batch - 1) / batch + ((ranges + kSplitGroup - 1) / kSplitGroup + batch - 1) / batch) * per_slot + 1;
            us += md.us_fixed + md.us_per_trip * trips + md.us_per_mb * ranges * out_mb * (double)(t - whole) / (double)t;
        }
        return us;
    };
    const uint64_t whole_tiles = (uint64_t)((M + whole.bm - 1) / whole.bm) * ((N + whole.bn - 1) / whole.bn);
    double whole_us = tile_cost(whole, whole_tiles, cus) * 2.0 * K / md.whole_flop_per_us + kLaunch;
    const double whole_us_by_cost = whole_us;
    for (int i = 0; i < md.n_tiles; ++i)                        // the model's own figure where the whole product runs on one of its tiles
        if (md.tiles[i].shape == whole_shape && whole_shape != TILE_LARGE)
            whole_us = estimate(md.tiles[i], tiles_of(whole_shape), (K + md.len_align - 1) / md.len_align * md.len_align, 1);
    SplitChoice best = {whole_shape, 1, 0, 0};
    double best_us = whole_us / 1.03;
    const uint32_t max_p = K / 256 < 64u ? K / 256 : 64u;
    for (int i = 0; i < md.n_tiles; ++i) {
        const SplitTile& st = md.tiles[i];
        const uint64_t t = tiles_of(st.shape), slots = (uint64_t)st.fit * cus;
        if (st.shape == TILE_LARGE) continue;                  // (planned below)
        if (t > 16ull * cus) continue;
        const uint32_t tile_max_p = st.shape == TILE_SMALL ? max_p : (max_p < kSplitFlat ? max_p : kSplitFlat);     // only the smallest tiles sum on two levels
        // all tiles split, or only those of the ragged last round (the full rounds in front stay whole)
        for (uint64_t whole = 0; whole <= t / slots * slots; whole += (t / slots * slots ? t / slots * slots : 1)) {
            if (whole == t || (whole == 0 && t > 4ull * cus)) continue;
            // fp16: the rates above are those of launches of some tens of microseconds; full rounds of 128 x 128 tiles
            // run for longer than that, into the power cap, and then 15 % slower (3072^3: estimate 55 us, measured
            // 66.7, whole on 256 x 256 tiles 60.4): full rounds in front only where the whole product takes the same tile
            if (elem_bytes == 2 && whole > 0 && st.shape != whole_shape) continue;
            for (uint32_t p = 2; p <= tile_max_p && (t - whole) * p <= 4096; ++p) {
                const RangeLen rl = range_len(K, p, md.len_align);
                if (rl.ranges < 2) continue;
                const double us = estimate(st, t, rl.longest, rl.ranges, whole);
                if (us < best_us) { best_us = us; best = {st.shape, rl.ranges, rl.len, (uint32_t)whole}; }
            }
        }
        // Or the CUs hold j whole tiles each (the first j x CUs workgroups of the grid: the hardware deals them out evenly)
        // and the other tiles on so many ranges that every workgroup of the launch is resident from the start, m split ones
        // on the busiest CU.  A CU then multiplies j K + m len steps, and does so at a better rate than in any launch of
        // equal workgroups: the whole ones, which are older, take the matrix pipe whenever they are ready and the split
        // ones the slots they leave (fp32, 1 + 1: 1280 x 1024 x 8192 163 -> 150 us, 1536^3 62.0 -> 55.1 with 2 + 1,
        // 1000 x 1500 x 777 25.5 -> 23.4; fp64 1000 x 1500 x 777 48.2 -> 39.4, 1280 x 1024 x 2048 87.1 -> 77.3).  Where K is
        // short the split ones run at a raised wave priority instead, finish first, and meet in the workspace behind the
        // whole ones' last steps; where K is long that costs more than it hides, because the whole ones are then alone
        // on their CU for most of the launch (fp32 K = 777: 24.2 -> 23.4 us, K = 1536 the same, K = 3072 71.1 -> 73.5).
        // fp16 on 128 x 128 tiles, one whole and at most one split workgroup per CU: 2304 x 2304 x 4096 59.4 -> 50.3 us,
        // 2560 x 2048 x 4096 58.4 -> 50.6, 3072 x 2048 x 8192 116.3 -> 104.2; the more CUs hold two, the slower each step.
        if (i == md.shared_tile && md.shared_ns_per_k > 0) {
            const uint32_t k_whole = (K + md.len_align - 1) / md.len_align * md.len_align;
            for (uint64_t j = 1; j < (uint64_t)st.fit && j * cus < t; ++j) {
                const uint64_t rest = t - j * cus, room = ((uint64_t)st.fit - j) * cus;
                for (uint32_t p = 2; p <= max_p && rest * p <= room && (elem_bytes != 2 || (K >= 4096 && K < 8192)); ++p) {     // (fp16: no gain measured below 4096, nor from 8192 on, where all tiles on 3 ranges do as well)
                    const RangeLen rl = range_len(K, p, md.len_align);
                    const uint32_t len = rl.longest, ranges = rl.ranges;
                    if (ranges < 2 || ranges > kSplitFlat || rest * ranges > room) continue;
                    const uint64_t m = (rest * ranges + cus - 1) / cus;
                    const uint32_t group = st.pieces < 16 ? st.pieces : 16, batch = 16 / group, per_slot = st.pieces / group;
                    const double us = md.shared_us_fixed + md.us_per_trip * ((ranges + batch - 1) / batch * per_slot) +
                                      (md.shared_ns_per_k + md.shared_ns_busy * (double)(rest * ranges) / (double)room) * 1e-3 *
                                          ((double)j * k_whole + (double)m * len);
                    if (us < best_us) { best_us = us; best = {st.shape, ranges, rl.len, (uint32_t)(j * cus), K <= md.urgent_max_k ? 1u : 0u}; }
                }
            }
        }
    }
    // fp16, more 256 x 256 tiles than CUs: the full rounds stay whole and the few tiles of the last round go on 2 to 8 ranges
    // each (one workgroup per CU, so a last round of R tiles otherwise leaves all but R CUs idle for a whole tile's time).
    // 22.7 ns per k step of a round on a full chip, 17.4 where at most half the CUs are busy (the power cap); the last
    // workgroup of a tile reads its 32 pieces per lane and slot in two trips of about 2 us.  Measured: 7000^3 (784 tiles:
    // 768 + 16 on 7 ranges) 602 -> 533 us, 4352 x 4352 x 8192 (256 + 33 on 4) 313 -> 249, 6948 x 4688 x 5282 (512 + 20 on 5)
    // 315 -> 291, 4098 x 7824 x 5104 302 -> 281, 2023 x 8829 x 4246 153 -> 142.  Held against the whole product as the
    // tile cost model prices it (for full rounds of 128 x 128 tiles the rates above are too kind).
    if (elem_bytes == 2 && md.n_tiles > 2 && md.tiles[2].shape == TILE_LARGE) {
        const SplitTile& st = md.tiles[2];
        const uint64_t t = tiles_of(TILE_LARGE), rounds = t / cus, rest = t % cus;
        const uint32_t k_whole = (K + md.len_align - 1) / md.len_align * md.len_align;
        // What it must beat: the best plan so far, and by 4 % (not 3) a whole product on these same tiles -- both estimates
        // then rest on the same rate for the full rounds, and a promise smaller than that did not show in the measurements.
        double bar = best.splits > 1 ? best_us : whole_us_by_cost / 1.03;
        if (whole_us / 1.04 < bar && whole_shape == TILE_LARGE) bar = whole_us / 1.04;
        for (uint32_t p = 2; rounds >= 1 && rest > 0 && p <= kSplitFlat && p <= max_p && rest * p <= cus; ++p) {
            const RangeLen rl = range_len(K, p, md.len_align);
            if (rl.ranges < 2) continue;
            const uint64_t wgs = rest * rl.ranges;
            const double lone = wgs <= cus / 2 ? 17.4 : 17.4 + (st.ns_per_k[1] - 17.4) * (double)(wgs - cus / 2) / (double)(cus - cus / 2);
            const double us = kLaunch + ((double)rounds * k_whole * st.ns_per_k[1] + (double)rl.longest * lone) * 1e-3 + md.us_fixed +
                              md.us_per_trip * rl.ranges * (st.pieces / 16) + md.us_per_mb * rl.ranges * out_mb * (double)rest / (double)t;
            if (us < bar) { bar = us; best_us = us; best = {TILE_LARGE, rl.ranges, rl.len, (uint32_t)(rounds * cus), 0}; }
        }
    }
    return best;
}

// elem_bytes: 2, 4 or 8.  `shape` of the result is the tile the split runs on (it may differ from the one the whole
// product takes).
SplitChoice split_plan(int elem_bytes, uint32_t M, uint32_t N, uint32_t K)
{
    if (M == 0 || N == 0) return {0, 1, 0, 0};
    if (M == 1 || N == 1) return {0, 1, 0, 0};                      // the vector corners have their own kernels
    const int shape = elem_bytes == 8 ? choose_tile_f64(M, N) : choose_tile(elem_bytes == 2, M, N, true);
    return split_plan_model(elem_bytes, M, N, K, shape, dma_tile_info(elem_bytes, shape, N));
}

// Block tile of a size class in the direct-to-LDS family of an element type.
TileInfo dma_tile_info(int elem_bytes, int shape, uint32_t N)
{
    return elem_bytes == 8 ? tile_info_f64(shape) : elem_bytes == 2 ? tile_info_f16(shape, true) : tile_info_f32(shape, true, N);
}

// Bytes of workspace a split of `splits` ranges needs: one slot of BM x BN accumulators (fp32; fp64 for fp64 operands)
// per workgroup, the tiles being those of the shape the split runs on.
size_t split_workspace_bytes(int elem_bytes, const SplitChoice& sp, uint32_t M, uint32_t N)
{
    const TileInfo ti = dma_tile_info(elem_bytes, sp.shape, N);
    const uint64_t tiles = (uint64_t)((M + ti.bm - 1) / ti.bm) * ((N + ti.bn - 1) / ti.bn);
    return (size_t)((tiles - sp.first) * sp.splits * (uint64_t)(ti.bm * ti.bn) * (elem_bytes == 8 ? 8u : 4u));
}

// Fills the split fields of g when the plan says so, the workspace is large enough and the tiles have counters; returns
// the number of splits and, with more than one, the tile shape they run on.
uint32_t arm_split(GemmArgs& g, int elem_bytes, void* workspace, size_t workspace_bytes, int& shape, hipStream_t stream,
                   uint64_t& ticket)
{
    ticket = 0;
    if (!workspace || !aligned16(workspace)) return 1;
    const SplitChoice sp = split_plan(elem_bytes, g.M, g.N, g.K);
    if (sp.splits <= 1 || workspace_bytes < split_workspace_bytes(elem_bytes, sp, g.M, g.N)) return 1;
    const TileInfo ti = dma_tile_info(elem_bytes, sp.shape, g.N);
    const uint64_t tiles = (uint64_t)((g.M + ti.bm - 1) / ti.bm) * ((g.N + ti.bn - 1) / ti.bn);
    const uint64_t n_counters = (tiles - sp.first) * split_counters_per_tile(sp.splits);
    uint32_t* const counters = n_counters <= kSplitCounters ? take_split_counters((uint32_t)n_counters, stream, ticket) : nullptr;
    if (!counters) return 1;
    g.split_counters = counters;
    g.split_len = sp.len; g.split_count = sp.splits; g.split_first = sp.first; g.split_ws = workspace;
    g.split_urgent = sp.urgent;
    shape = sp.shape;
    return sp.splits;
}

// The same with the plan given by the caller (a measurement aid: the planner's pick is held against every other plan):
// `splits` ranges on tile class `shape`, the first `first` tiles whole.  Returns false when that plan cannot run.
bool arm_split_forced(GemmArgs& g, int elem_bytes, void* workspace, size_t workspace_bytes, int shape, uint32_t splits, uint32_t first,
                      hipStream_t stream, uint64_t& ticket)
{
    ticket = 0;
    const SplitModel& md = elem_bytes == 8 ? kSplitF64 : elem_bytes == 2 ? kSplitF16 : kSplitF32;
    bool has_kernel = false;
    for (int i = 0; i < md.n_tiles; ++i) has_kernel |= md.tiles[i].shape == shape;
    if (!has_kernel || splits < 2 || splits > 64 || !workspace || !aligned16(workspace)) return false;
    const RangeLen rl = range_len(g.K, splits, md.len_align);
    if (rl.ranges != splits || (shape != TILE_SMALL && splits > kSplitFlat)) return false;
    const TileInfo ti = dma_tile_info(elem_bytes, shape, g.N);
    const uint64_t tiles = (uint64_t)((g.M + ti.bm - 1) / ti.bm) * ((g.N + ti.bn - 1) / ti.bn);
    if (first >= tiles) return false;
    const SplitChoice sp = {shape, splits, rl.len, first, 0};
    if (workspace_bytes < split_workspace_bytes(elem_bytes, sp, g.M, g.N)) return false;
    const uint64_t n_counters = (tiles - first) * split_counters_per_tile(splits);
    uint32_t* const counters = n_counters <= kSplitCounters ? take_split_counters((uint32_t)n_counters, stream, ticket) : nullptr;
    if (!counters) return false;
    g.split_counters = counters;
    g.split_len = sp.len; g.split_count = splits; g.split_first = first; g.split_ws = workspace;
    g.split_urgent = 0;
    return true;
}

// y = alpha * x.B (+ beta * c).  Few columns and a long K: with a workspace, ranges of K go to workgroups of their
// own, and the last of a column group to finish adds their partial sums in range order.
int gevm_maybe_split(bool f16, bool out_f32, const void* x, const void* B, const void* c, void* y, uint32_t K, uint32_t N,
                     uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, void* workspace,
                     size_t workspace_bytes, hipStream_t stream)
{
    const SplitPlan sp = plan_gevm_split(f16 ? 2 : 4, N, K, g_dev.compute_units);
    const uint32_t ldw = (N + 3) / 4 * 4;
    if (sp.splits > 1 && workspace && aligned16(workspace) && workspace_bytes >= (size_t)sp.splits * ldw * 4) {
        const uint32_t groups = (N + (f16 ? 64u : 32u) - 1) / (f16 ? 64u : 32u);
        uint64_t ticket;
        uint32_t* const counters = take_split_counters(groups, stream, ticket);     // the last workgroup of a column group adds its ranges
        if (counters) {
            const int rc = launch_gevm(f16, out_f32, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, sp.len, (float*)workspace, ldw,
                                       counters);
            commit_split_counters(ticket);
            return rc;
        }
    }
    return launch_gevm(f16, out_f32, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream);
}

template <bool F16>
int run_gemm(const void* A, const void* B, const void* C, void* D, uint32_t M, uint32_t N, uint32_t K,
             uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta, void* stream,
             int tile, int force_edge, void* workspace = nullptr, size_t workspace_bytes = 0)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    const int rc = check_gemm(A, B, C, D, M, N, K, lda, ldb, ldc, ldd);
    if (rc != DECX_HIP_OK || M == 0 || N == 0) return rc;
    if (tile != DECX_HIP_TILE_AUTO && (tile < 0 || tile >= (F16 ? TILE_F16_COUNT : TILE_COUNT))) return DECX_HIP_E_INVALID_ARG;

    // the two vector corners are bandwidth-bound and have kernels of their own
    if (N == 1 && tile == DECX_HIP_TILE_AUTO && K > 0) {
        // x is the single column of a pitched K x 1 matrix: with a workspace it is gathered once into a dense vector
        if (workspace && workspace_bytes >= (size_t)K * (F16 ? 2 : 4) && gemv_gather_pays(M, K, ldb)) {
            const int rg = launch_gather(F16 ? 2 : 4, B, workspace, K, ldb, as_stream(stream));
            return rg != 0 ? rg : launch_gemv(F16, false, A, workspace, C, D, M, K, lda, 1, ldc, ldd, alpha, beta, as_stream(stream));
        }
        return launch_gemv(F16, false, A, B, C, D, M, K, lda, ldb, ldc, ldd, alpha, beta, as_stream(stream));
    }
    if (M == 1 && tile == DECX_HIP_TILE_AUTO && K > 0)
        return gevm_maybe_split(F16, false, A, B, C, D, K, N, ldb, 1, 1, 1, alpha, beta, workspace, workspace_bytes,
                                as_stream(stream));

    constexpr uint32_t per16 = F16 ? 8u : 4u;          // elements per 16 bytes
    GemmArgs g;
    std::memset(&g, 0, sizeof g);
    g.cus = (uint32_t)g_dev.compute_units;
    g.A = A; g.B = B; g.C = C; g.D = D;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldd = ldd;
    g.alpha = alpha; g.beta = beta;
    g.vec_ok = (aligned16(A) && aligned16(B) && aligned16(D) && (!C || aligned16(C)) &&
                lda % per16 == 0 && ldb % per16 == 0 && ldd % per16 == 0 && (!C || ldc % per16 == 0)) ? 1u : 0u;
    int shape = (tile == DECX_HIP_TILE_AUTO) ? choose_tile(F16, M, N, g.vec_ok != 0) : tile;
    const bool edge = force_edge != 0 || K == 0;
    uint64_t ticket = 0;
    if (workspace && tile == DECX_HIP_TILE_AUTO && !edge && g.vec_ok && dma_offsets_fit(g, F16 ? 2 : 4)) {
        arm_split(g, F16 ? 2 : 4, workspace, workspace_bytes, shape, as_stream(stream), ticket);    // with ranges, the last workgroup of a tile sums them
    }
    const int launched = F16 ? launch_gemm_f16(shape, edge, g, as_stream(stream))
                             : launch_gemm_f32(shape, edge, g, as_stream(stream));
    commit_split_counters(ticket);
    return launched;
}

__global__ void __launch_bounds__(256) calibration_copy_kernel(uintx4* __restrict__ dst,
                                                              const uintx4* __restrict__ src, size_t n16)
{
    for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (size_t)gridDim.x * 256) dst[i] = src[i];
}

// A read-only pass in the pattern the matrix x vector kernel reads its rows in, which is the one HBM answers best of those
// tried (2 GiB: a grid-stride loop 5.5 TB/s, a contiguous region per wavefront or per workgroup 6.0-6.3, this 6.6-6.7): the
// buffer as rows of 64 KB, a workgroup of 16 wavefronts on 32 of them, a wavefront on two, 1 KB of each a step, every
// wavefront starting at another step.  Every 16-byte piece is loaded once and folded into a word per lane that is stored
// only if it comes out as a value the fold cannot produce from a buffer filled with one byte value: nothing is written.
constexpr uint32_t kReadRow16 = 65536 / 16;        // 16-byte pieces per row
__global__ void __launch_bounds__(1024) calibration_read_kernel(const uintx4* __restrict__ src, uint32_t* __restrict__ sink, uint32_t never)
{
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const uintx4* a = src + ((size_t)blockIdx.x * 32 + wave * 2) * kReadRow16 + lane;
    const uintx4* b = a + kReadRow16;
    constexpr uint32_t steps = kReadRow16 / 64;
    const uint32_t s0 = ((blockIdx.x * 16 + wave) * 5u) % steps;
    uint32_t fold = 0;
    for (uint32_t s = 0; s < steps; s += 4) {
        uintx4 v[4], w[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            const uint32_t at = (s0 + s + u) % steps;
            v[u] = a[(size_t)at * 64]; w[u] = b[(size_t)at * 64];
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) fold ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3] ^ w[u][0] ^ w[u][1] ^ w[u][2] ^ w[u][3];
    }
    if (fold == never) sink[(size_t)blockIdx.x * 1024 + threadIdx.x] = fold;
}

// The copy in the same order (whole blocks of 2 MiB; what is left over goes through calibration_copy_kernel), with
// streaming stores.  1 GiB: 5.7-5.9 TB/s of reads plus writes, where the grid-stride loop above moves 4.6-4.8 and the
// runtime's own device-to-device copy 5.0.
__global__ void __launch_bounds__(1024) calibration_copy_rows_kernel(uintx4* __restrict__ dst, const uintx4* __restrict__ src)
{
    const uint32_t lane = threadIdx.x & 63u, wave = threadIdx.x >> 6;
    const size_t a = ((size_t)blockIdx.x * 32 + wave * 2) * kReadRow16 + lane, b = a + kReadRow16;
    constexpr uint32_t steps = kReadRow16 / 64;
    const uint32_t s0 = ((blockIdx.x * 16 + wave) * 5u) % steps;
    for (uint32_t s = 0; s < steps; s += 4) {
        uintx4 v[4], w[4];
        size_t at[4];
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            at[u] = (size_t)((s0 + s + u) % steps) * 64;
            v[u] = src[a + at[u]]; w[u] = src[b + at[u]];
        }
#pragma unroll
        for (uint32_t u = 0; u < 4; ++u) {
            __builtin_nontemporal_store(v[u], dst + a + at[u]);
            __builtin_nontemporal_store(w[u], dst + b + at[u]);
        }
    }
}

// Register-only matrix-core loops: what the matrix pipe sustains on this board with nothing else to do -- no loads,
// no LDS, no barriers -- on operands of the caller's choosing (their values set the power drawn, and with it the
// clock the board's power management allows).  8 wavefronts per CU, two per SIMD, the accumulator layouts of the
// largest GEMM tiles: F16 sixteen 16x16x32 tiles (a 64 x 64 wave tile, 4 x 4 operand fragments), fp32 eight 32x32x2
// tiles (128 x 64, 4 x 2 fragments that change every step as in a k loop).
template <bool F16>
__global__ void __launch_bounds__(512) calibration_mfma_kernel(const uintx4* __restrict__ operands, size_t n16, float* __restrict__ sink,
                                                              uint32_t iters)
{
    const size_t at = ((size_t)blockIdx.x * 512 + threadIdx.x) * 8;
    uintx4 raw[8];
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[i] = operands[(at + i) % n16];
    float s = 0.f;
    if constexpr (F16) {
        halfx8 a[4], b[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) { a[i] = __builtin_bit_cast(halfx8, raw[i]); b[i] = __builtin_bit_cast(halfx8, raw[4 + i]); }
        floatx4 acc[4][4] = {};
        for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
            for (int j = 0; j < 4; ++j)
#pragma unroll
                for (int i = 0; i < 4; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(b[j], a[i], acc[j][i], 0, 0, 0);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int i = 0; i < 4; ++i) s += acc[j][i][0] + acc[j][i][1] + acc[j][i][2] + acc[j][i][3];
    } else {
        float v[32];
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const floatx4 f = __builtin_bit_cast(floatx4, raw[i]);
            v[4 * i] = f[0]; v[4 * i + 1] = f[1]; v[4 * i + 2] = f[2]; v[4 * i + 3] = f[3];
        }
        floatx16 acc[4][2] = {};
        for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
            for (int k = 0; k < 4; ++k)
#pragma unroll
                for (int i = 0; i < 4; ++i)
#pragma unroll
                    for (int j = 0; j < 2; ++j)
                        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(v[8 * k + i], v[8 * k + 4 + j], acc[i][j], 0, 0, 0);
        }
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
#pragma unroll
                for (int r = 0; r < 16; ++r) s += acc[i][j][r];
    }
    sink[(size_t)blockIdx.x * 512 + threadIdx.x] = s;
}

// kmat[(kh * k_w + kw) * img_dpitch + ic][oc] = kernel oc at (kh, kw, ic); zero where ic >= depth or oc >= out_c
__global__ void __launch_bounds__(256) conv2d_pack_kernels_kernel(const float* __restrict__ kernels, float* __restrict__ kmat,
                                                                  uint32_t k_w, uint32_t k_h, uint32_t depth,
                                                                  uint32_t k_dpitch, uint32_t k_wpitch, uint64_t tensor_stride,
                                                                  uint32_t out_c, uint32_t kmat_pitch, uint32_t img_dpitch)
{
    const uint64_t total = (uint64_t)k_h * k_w * img_dpitch * kmat_pitch;
    for (uint64_t i = (uint64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (uint64_t)gridDim.x * 256) {
        const uint32_t oc = (uint32_t)(i % kmat_pitch);
        const uint64_t k = i / kmat_pitch;
        const uint32_t ic = (uint32_t)(k % img_dpitch);
        const uint32_t kw = (uint32_t)((k / img_dpitch) % k_w), kh = (uint32_t)(k / img_dpitch / k_w);
        float v = 0.f;
        if (oc < out_c && ic < depth) v = kernels[oc * tensor_stride + ((uint64_t)kh * k_wpitch + kw) * k_dpitch + ic];
        kmat[i] = v;
    }
}

}  // namespace

extern "C" {

int decx_hip_calibration_copy(void* dst, const void* src, size_t bytes, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (!bytes) return DECX_HIP_OK;
    if (!dst || !src || (bytes & 15u) || !aligned16(dst) || !aligned16(src)) return DECX_HIP_E_INVALID_ARG;
    constexpr size_t kBlockBytes = (size_t)32 * kReadRow16 * 16;           // 2 MiB per workgroup of the fast form
    const size_t blocks = bytes / kBlockBytes < 0x7fffffffu ? bytes / kBlockBytes : 0;
    if (blocks)
        hipLaunchKernelGGL(calibration_copy_rows_kernel, dim3((unsigned)blocks), dim3(1024), 0, as_stream(stream), (uintx4*)dst, (const uintx4*)src);
    const size_t done16 = blocks * kBlockBytes / 16, n16 = bytes / 16 - done16;
    if (n16) {
        const size_t want = (n16 + 255) / 256;
        const dim3 grid((unsigned)(want < 16384 ? want : 16384)), block(256);
        hipLaunchKernelGGL(calibration_copy_kernel, grid, block, 0, as_stream(stream), (uintx4*)dst + done16, (const uintx4*)src + done16, n16);
    }
    return (int)hipGetLastError();
}

int decx_hip_calibration_read(const void* src, size_t bytes, uint32_t* sink, size_t sink_words, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (!bytes) return DECX_HIP_OK;
    constexpr size_t kBlockBytes = (size_t)32 * kReadRow16 * 16;           // 2 MiB per workgroup
    const size_t blocks = bytes / kBlockBytes;
    if (!src || bytes % kBlockBytes || blocks > 0x7fffffffu || !aligned16(src) || !sink || sink_words < blocks * 1024) return DECX_HIP_E_INVALID_ARG;
    hipLaunchKernelGGL(calibration_read_kernel, dim3((unsigned)blocks), dim3(1024), 0, as_stream(stream), (const uintx4*)src, sink,
                       0x5a5a5a5bu);                           // (a buffer filled with one byte value folds to a word of four equal bytes)
    return (int)hipGetLastError();
}

int decx_hip_calibration_mfma(int elem_bytes, const void* operands, size_t operand_bytes, float* sink, size_t sink_floats,
                              uint32_t iters, double* flops, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    const uint32_t blocks = (uint32_t)g_dev.compute_units;
    if ((elem_bytes != 2 && elem_bytes != 4) || !operands || operand_bytes < 16 || !aligned16(operands) || !sink ||
        sink_floats < (size_t)blocks * 512)
        return DECX_HIP_E_INVALID_ARG;
    // per wavefront and iteration: 16 tiles of 16 x 16 x 32, or 4 steps of 8 tiles of 32 x 32 x 2
    const double per_wave = elem_bytes == 2 ? 16.0 * 2 * 16 * 16 * 32 : 32.0 * 2 * 32 * 32 * 2;
    if (flops) *flops = (double)blocks * 8.0 * (double)iters * per_wave;
    if (elem_bytes == 2)
        hipLaunchKernelGGL(calibration_mfma_kernel<true>, dim3(blocks), dim3(512), 0, as_stream(stream), (const uintx4*)operands,
                           operand_bytes / 16, sink, iters);
    else
        hipLaunchKernelGGL(calibration_mfma_kernel<false>, dim3(blocks), dim3(512), 0, as_stream(stream), (const uintx4*)operands,
                           operand_bytes / 16, sink, iters);
    return (int)hipGetLastError();
}

int decx_hip_init(int device)
{
    int count = 0;
    hipError_t e = hipGetDeviceCount(&count);
    if (e != hipSuccess) return hip_rc(e);
    if (count <= 0 || device < 0 || device >= count) return DECX_HIP_E_NO_DEVICE;
    if ((e = hipSetDevice(device)) != hipSuccess) return hip_rc(e);
    if ((e = hipGetDeviceProperties(&g_dev.prop, device)) != hipSuccess) return hip_rc(e);
    if (device < kMaxDevices && !g_scratch[device]) {              // this device's copy of the static workspace
        void* p = nullptr;
        if ((e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch))) != hipSuccess) return hip_rc(e);
        g_scratch[device] = p;
    }
    if (device < kMaxDevices && !g_split_counters[device]) {
        void* p = nullptr;
        if ((e = hipGetSymbolAddress(&p, HIP_SYMBOL(split_counters))) != hipSuccess) return hip_rc(e);
        g_split_counters[device] = (uint32_t*)p;
        std::lock_guard<std::mutex> lock(g_counter_mutex);
        if (!g_rings[device]) g_rings[device] = new CounterRing(kSplitCounters);
    }
    g_dev.device = device;
    if (device < kMaxDevices) {
        std::lock_guard<std::mutex> lock(g_counter_mutex);
        g_ring_runtime.prefill();
    }
    g_dev.compute_units = g_dev.prop.multiProcessorCount > 0 ? g_dev.prop.multiProcessorCount : 256;
    g_dev.ready = true;
    return DECX_HIP_OK;
}

int decx_hip_get_device_props(decx_hip_device_props* out)
{
    if (!out) return DECX_HIP_E_INVALID_ARG;
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    std::memset(out, 0, sizeof *out);
    std::strncpy(out->name, g_dev.prop.name, sizeof out->name - 1);
    std::strncpy(out->arch, g_dev.prop.gcnArchName, sizeof out->arch - 1);
    out->compute_units = g_dev.prop.multiProcessorCount;
    out->clock_khz = g_dev.prop.clockRate;
    out->memory_clock_khz = g_dev.prop.memoryClockRate;
    out->memory_bus_bits = g_dev.prop.memoryBusWidth;
    out->lds_bytes_per_block = (int32_t)g_dev.prop.sharedMemPerBlock;
    out->wavefront_size = g_dev.prop.warpSize;
    out->global_mem_bytes = g_dev.prop.totalGlobalMem;
    return DECX_HIP_OK;
}

const char* decx_hip_error_string(int code)
{
    switch (code) {
    case DECX_HIP_OK:            return "success";
    case DECX_HIP_E_INVALID_ARG: return "invalid argument (null pointer, pitch smaller than width, or unknown enum)";
    case DECX_HIP_E_NOT_INIT:    return "decx_hip_init() has not been called";
    case DECX_HIP_E_NO_DEVICE:   return "no usable GPU";
    case DECX_HIP_E_TOO_LARGE:   return "the product needs more workspace than the static one holds";
    default:                     return code > 0 ? hipGetErrorString((hipError_t)code) : "unknown error";
    }
}

int decx_hip_malloc(void** ptr, size_t bytes)
{
    if (!ptr) return DECX_HIP_E_INVALID_ARG;
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    return hip_rc(hipMalloc(ptr, bytes ? bytes : 1));
}
int decx_hip_free(void* ptr) { return ptr ? hip_rc(hipFree(ptr)) : DECX_HIP_OK; }

int decx_hip_host_malloc(void** ptr, size_t bytes)
{
    if (!ptr) return DECX_HIP_E_INVALID_ARG;
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    return hip_rc(hipHostMalloc(ptr, bytes ? bytes : 1, hipHostMallocDefault));
}
int decx_hip_host_free(void* ptr) { return ptr ? hip_rc(hipHostFree(ptr)) : DECX_HIP_OK; }

int decx_hip_memset_async(void* ptr, int value, size_t bytes, void* stream)
{
    if (!ptr && bytes) return DECX_HIP_E_INVALID_ARG;
    if (!bytes) return DECX_HIP_OK;
    return hip_rc(hipMemsetAsync(ptr, value, bytes, as_stream(stream)));
}

int decx_hip_mem_info(size_t* free_bytes, size_t* total_bytes)
{
    if (!free_bytes || !total_bytes) return DECX_HIP_E_INVALID_ARG;
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    return hip_rc(hipMemGetInfo(free_bytes, total_bytes));
}

int decx_hip_memcpy2d_async(void* dst, size_t dst_pitch, const void* src, size_t src_pitch,
                            size_t width_bytes, size_t height, int kind, void* stream)
{
    if (!width_bytes || !height) return DECX_HIP_OK;
    if (!dst || !src || dst_pitch < width_bytes || src_pitch < width_bytes || kind < 0 || kind > 2)
        return DECX_HIP_E_INVALID_ARG;
    static const hipMemcpyKind kinds[3] = {hipMemcpyHostToDevice, hipMemcpyDeviceToHost, hipMemcpyDeviceToDevice};
    return hip_rc(hipMemcpy2DAsync(dst, dst_pitch, src, src_pitch, width_bytes, height, kinds[kind], as_stream(stream)));
}

int decx_hip_stream_create(void** stream)
{
    if (!stream) return DECX_HIP_E_INVALID_ARG;
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    hipStream_t s;
    const hipError_t e = hipStreamCreateWithFlags(&s, hipStreamNonBlocking);   // default priority
    *stream = (e == hipSuccess) ? (void*)s : nullptr;
    return hip_rc(e);
}
int decx_hip_stream_destroy(void* stream) { return stream ? hip_rc(hipStreamDestroy(as_stream(stream))) : DECX_HIP_OK; }
// Polls for a quarter of a millisecond before it blocks: a blocking wait is woken by an interrupt, some 10 us after the
// work is done, which is a tenth of an fp16 4096^3 product.
int decx_hip_stream_sync(void* stream)
{
    const auto t0 = std::chrono::steady_clock::now();
    do {
        const hipError_t e = hipStreamQuery(as_stream(stream));
        if (e != hipErrorNotReady) return hip_rc(e);
    } while (std::chrono::steady_clock::now() - t0 < std::chrono::microseconds(250));
    return hip_rc(hipStreamSynchronize(as_stream(stream)));
}

int decx_hip_event_create(void** event)
{
    if (!event) return DECX_HIP_E_INVALID_ARG;
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    hipEvent_t ev;
    const hipError_t e = hipEventCreate(&ev);
    *event = (e == hipSuccess) ? (void*)ev : nullptr;
    return hip_rc(e);
}
int decx_hip_event_destroy(void* event) { return event ? hip_rc(hipEventDestroy((hipEvent_t)event)) : DECX_HIP_OK; }
int decx_hip_event_record(void* event, void* stream)
{
    return event ? hip_rc(hipEventRecord((hipEvent_t)event, as_stream(stream))) : DECX_HIP_E_INVALID_ARG;
}
int decx_hip_stream_wait_event(void* stream, void* event)
{
    return event ? hip_rc(hipStreamWaitEvent(as_stream(stream), (hipEvent_t)event, 0)) : DECX_HIP_E_INVALID_ARG;
}
int decx_hip_event_sync(void* event)
{
    return event ? hip_rc(hipEventSynchronize((hipEvent_t)event)) : DECX_HIP_E_INVALID_ARG;
}
int decx_hip_event_elapsed_ms(void* start, void* stop, float* ms)
{
    if (!start || !stop || !ms) return DECX_HIP_E_INVALID_ARG;
    return hip_rc(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
}

int decx_hip_gemm_f32(const float* A, const float* B, const float* C, float* D, uint32_t M, uint32_t N, uint32_t K,
                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta, void* stream)
{
    return run_gemm<false>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0);
}

size_t decx_hip_gemm_workspace(int elem_bytes, uint32_t M, uint32_t N, uint32_t K)
{
    if (!g_dev.ready || (elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8)) return 0;
    if (N == 1 && M > 0)                                           // room for a dense copy of x
        return gemv_gather_pays(M, K, 2) ? ((size_t)K * elem_bytes + 15) / 16 * 16 : 0;
    if (M == 1 && N > 0) {                                         // room for the partial sums of ranges of K
        const SplitPlan sp = plan_gevm_split(elem_bytes, N, K, g_dev.compute_units);
        return sp.splits > 1 ? (size_t)sp.splits * ((N + 3) / 4 * 4) * (elem_bytes == 8 ? 8 : 4) : 0;
    }
    const SplitChoice sp = split_plan(elem_bytes, M, N, K);
    return sp.splits > 1 ? split_workspace_bytes(elem_bytes, sp, M, N) : 0;
}

size_t decx_hip_gemm_f32_workspace(uint32_t M, uint32_t N, uint32_t K) { return decx_hip_gemm_workspace(4, M, N, K); }

int decx_hip_gemm_f32_ws(const float* A, const float* B, const float* C, float* D, uint32_t M, uint32_t N, uint32_t K,
                         uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta,
                         void* workspace, size_t workspace_bytes, void* stream)
{
    return run_gemm<false>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0, workspace,
                           workspace_bytes);
}

int decx_hip_gemm_f32_static(const float* A, const float* B, const float* C, float* D, uint32_t M, uint32_t N, uint32_t K,
                             uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    void* ws = g_dev.device < kMaxDevices ? g_scratch[g_dev.device] : nullptr;
    if (!ws) return DECX_HIP_E_NOT_INIT;
    // What the workspace form would use for THESE operands.  A column operand that does not fit is read in place (the
    // dense copy changes no sum); a split that does not fit is refused (unsplit, the sums would come in another order).
    if (decx_hip_gemm_workspace(4, M, N, K) > kScratchBytes) {
        GemmArgs g;
        std::memset(&g, 0, sizeof g);
        g.C = C; g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldd = ldd;
        const bool can_split = K > 0 && aligned16(A) && aligned16(B) && aligned16(D) && (!C || aligned16(C)) && lda % 4 == 0 &&
                               ldb % 4 == 0 && ldd % 4 == 0 && (!C || ldc % 4 == 0) && dma_offsets_fit(g, 4);
        if (N != 1 && (M == 1 || can_split)) return DECX_HIP_E_TOO_LARGE;
        ws = nullptr;
    }
    return run_gemm<false>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0, ws, ws ? kScratchBytes : 0);
}

int decx_hip_gemm_forced_plan(int elem_bytes, const void* A, const void* B, const void* C, void* D, uint32_t M, uint32_t N, uint32_t K,
                              uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha, double beta, int tile,
                              uint32_t k_splits, uint32_t whole_tiles, void* workspace, size_t workspace_bytes, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (elem_bytes != 2 && elem_bytes != 4 && elem_bytes != 8) return DECX_HIP_E_INVALID_ARG;
    const int rc = check_gemm(A, B, C, D, M, N, K, lda, ldb, ldc, ldd);
    if (rc != DECX_HIP_OK) return rc;
    if (M == 0 || N == 0 || K == 0) return DECX_HIP_E_INVALID_ARG;
    if (tile < 0 || tile >= (elem_bytes == 2 ? TILE_F16_COUNT : TILE_COUNT)) return DECX_HIP_E_INVALID_ARG;
    const uint32_t per16 = 16u / (uint32_t)elem_bytes;
    GemmArgs g;
    std::memset(&g, 0, sizeof g);
    g.cus = (uint32_t)g_dev.compute_units;
    g.A = A; g.B = B; g.C = C; g.D = D;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldd = ldd;
    g.alpha = (float)alpha; g.beta = (float)beta; g.alpha64 = alpha; g.beta64 = beta;
    g.vec_ok = (aligned16(A) && aligned16(B) && aligned16(D) && (!C || aligned16(C)) && lda % per16 == 0 && ldb % per16 == 0 &&
                ldd % per16 == 0 && (!C || ldc % per16 == 0)) ? 1u : 0u;
    if (!g.vec_ok || !dma_offsets_fit(g, (uint32_t)elem_bytes)) return DECX_HIP_E_INVALID_ARG;      // the direct-to-LDS kernels only
    uint64_t ticket = 0;
    if (k_splits > 1 && !arm_split_forced(g, elem_bytes, workspace, workspace_bytes, tile, k_splits, whole_tiles, as_stream(stream), ticket))
        return DECX_HIP_E_INVALID_ARG;
    const int launched = elem_bytes == 8 ? launch_gemm_f64(tile, false, g, as_stream(stream))
                       : elem_bytes == 2 ? launch_gemm_f16(tile, false, g, as_stream(stream))
                                         : launch_gemm_f32(tile, false, g, as_stream(stream));
    commit_split_counters(ticket);
    return launched;
}

int decx_hip_reset_split_counters(void)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    const int d = g_dev.device;
    if (d < 0 || d >= kMaxDevices || !g_split_counters[d]) return DECX_HIP_E_NOT_INIT;
    hipError_t e = hipDeviceSynchronize();
    if (e != hipSuccess) return hip_rc(e);
    if ((e = hipMemset(g_split_counters[d], 0, sizeof(uint32_t) * kSplitCounters)) != hipSuccess) return hip_rc(e);
    std::lock_guard<std::mutex> lock(g_counter_mutex);
    if (g_rings[d]) g_rings[d]->reset(g_ring_runtime);
    return DECX_HIP_OK;
}

int decx_hip_split_counter_stats(uint64_t out[6])
{
    if (!out) return DECX_HIP_E_INVALID_ARG;
    const int d = g_dev.device;
    std::lock_guard<std::mutex> lock(g_counter_mutex);
    if (!g_dev.ready || d < 0 || d >= kMaxDevices || !g_rings[d]) return DECX_HIP_E_NOT_INIT;
    const CounterRing::Stats& st = g_rings[d]->stats();
    out[0] = st.taken; out[1] = st.wraps; out[2] = st.refused; out[3] = st.events; out[4] = st.reserved;
    out[5] = g_rings[d]->ring_size();
    return DECX_HIP_OK;
}

int decx_hip_gemm_f16_ws(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, uint32_t M, uint32_t N,
                         uint32_t K, uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta,
                         void* workspace, size_t workspace_bytes, void* stream)
{
    return run_gemm<true>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0, workspace,
                          workspace_bytes);
}

int decx_hip_gemm_f16(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, uint32_t M, uint32_t N,
                      uint32_t K, uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha, float beta,
                      void* stream)
{
    return run_gemm<true>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0);
}

static int run_gemm_f64(const double* A, const double* B, const double* C, double* D, uint32_t M, uint32_t N, uint32_t K,
                        uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha, double beta, void* stream,
                        int tile, int force_plain, void* workspace = nullptr, size_t workspace_bytes = 0)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    const int rc = check_gemm(A, B, C, D, M, N, K, lda, ldb, ldc, ldd);
    if (rc != DECX_HIP_OK || M == 0 || N == 0) return rc;
    if (tile != DECX_HIP_TILE_AUTO && (tile < 0 || tile >= TILE_COUNT)) return DECX_HIP_E_INVALID_ARG;

    // the two vector corners: the bandwidth-bound kernels, as for the other real types
    if (N == 1 && tile == DECX_HIP_TILE_AUTO && !force_plain && K > 0) {
        if (workspace && workspace_bytes >= (size_t)K * 8 && gemv_gather_pays(M, K, ldb)) {
            const int rg = launch_gather(8, B, workspace, K, ldb, as_stream(stream));
            return rg != 0 ? rg : launch_gemv_f64(A, (const double*)workspace, C, D, M, K, lda, 1, ldc, ldd, alpha, beta, as_stream(stream));
        }
        return launch_gemv_f64(A, B, C, D, M, K, lda, ldb, ldc, ldd, alpha, beta, as_stream(stream));
    }
    if (M == 1 && tile == DECX_HIP_TILE_AUTO && !force_plain && K > 0) {
        const SplitPlan sp = plan_gevm_split(8, N, K, g_dev.compute_units);
        const uint32_t ldw = (N + 3) / 4 * 4;
        if (sp.splits > 1 && workspace && aligned16(workspace) && workspace_bytes >= (size_t)sp.splits * ldw * 8) {
            uint64_t ticket;
            uint32_t* const counters = take_split_counters((N + 15) / 16, as_stream(stream), ticket);
            if (counters) {
                const int rc = launch_gevm_f64(A, B, C, D, K, N, ldb, 1, 1, 1, alpha, beta, as_stream(stream), sp.len, (double*)workspace, ldw,
                                               counters);
                commit_split_counters(ticket);
                return rc;
            }
        }
        return launch_gevm_f64(A, B, C, D, K, N, ldb, 1, 1, 1, alpha, beta, as_stream(stream));
    }

    GemmArgs g;
    std::memset(&g, 0, sizeof g);
    g.cus = (uint32_t)g_dev.compute_units;
    g.A = A; g.B = B; g.C = C; g.D = D;
    g.M = M; g.N = N; g.K = K;
    g.lda = lda; g.ldb = ldb; g.ldc = ldc; g.ldd = ldd;
    g.alpha = (float)alpha; g.beta = (float)beta;
    g.alpha64 = alpha; g.beta64 = beta;
    g.vec_ok = (aligned16(A) && aligned16(B) && aligned16(D) && (!C || aligned16(C)) &&
                lda % 2 == 0 && ldb % 2 == 0 && ldd % 2 == 0 && (!C || ldc % 2 == 0)) ? 1u : 0u;
    int shape = (tile == DECX_HIP_TILE_AUTO) ? choose_tile_f64(M, N) : tile;
    uint64_t ticket = 0;
    if (workspace && tile == DECX_HIP_TILE_AUTO && !force_plain && K > 0 && g.vec_ok && dma_offsets_fit(g, 8)) {
        arm_split(g, 8, workspace, workspace_bytes, shape, as_stream(stream), ticket);
    }
    const int launched = launch_gemm_f64(shape, force_plain != 0, g, as_stream(stream));
    commit_split_counters(ticket);
    return launched;
}

int decx_hip_gemm_f64(const double* A, const double* B, const double* C, double* D, uint32_t M, uint32_t N, uint32_t K,
                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha, double beta, void* stream)
{
    return run_gemm_f64(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0);
}

int decx_hip_gemm_f64_ws(const double* A, const double* B, const double* C, double* D, uint32_t M, uint32_t N, uint32_t K,
                         uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha, double beta,
                         void* workspace, size_t workspace_bytes, void* stream)
{
    return run_gemm_f64(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, DECX_HIP_TILE_AUTO, 0, workspace,
                        workspace_bytes);
}

int decx_hip_gemm_f64_tile(const double* A, const double* B, const double* C, double* D, uint32_t M, uint32_t N,
                           uint32_t K, uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha,
                           double beta, void* stream, int tile, int force_plain)
{
    return run_gemm_f64(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, tile, force_plain);
}

size_t decx_hip_gemm_complex_workspace(int real_bytes, uint32_t N, uint32_t K)
{
    if (real_bytes != 4 && real_bytes != 8) return 0;
    const size_t ldx = ((size_t)2 * N + 15) / 16 * 16;           // 64 / 128 bytes per row at least
    return (size_t)2 * K * ldx * (size_t)real_bytes;
}

extern "C++" {
template <typename T>
static int run_gemm_complex(const T* A, const T* B, const T* C, T* D, uint32_t M, uint32_t N, uint32_t K, uint32_t lda,
                            uint32_t ldb, uint32_t ldc, uint32_t ldd, T ar, T ai, T br, T bi, void* workspace,
                            size_t workspace_bytes, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    const int rc0 = check_gemm(A, B, C, D, M, N, K, lda, ldb, ldc, ldd);
    if (rc0 != DECX_HIP_OK || M == 0 || N == 0) return rc0;
    if (N > 0x7fffffffu || K > 0x7fffffffu || lda > 0x7fffffffu || ldd > 0x7fffffffu) return DECX_HIP_E_INVALID_ARG;
    const size_t need = decx_hip_gemm_complex_workspace((int)sizeof(T), N, K);
    if (K > 0 && (!workspace || workspace_bytes < need || !aligned16(workspace))) return DECX_HIP_E_INVALID_ARG;
    hipStream_t S = as_stream(stream);
    int rc = DECX_HIP_OK;
    if (C) rc = launch_complex_scale<T>(C, D, M, N, ldc, ldd, br, bi, S);
    const uint32_t ldx = (uint32_t)(((size_t)2 * N + 15) / 16 * 16);
    if (rc == DECX_HIP_OK && K > 0) rc = launch_complex_expand_b<T>(B, (T*)workspace, K, N, ldb, ldx, ar, ai, S);
    if (rc != DECX_HIP_OK) return rc;
    // real GEMM M x 2N x 2K accumulating onto D when C was given (K == 0 leaves D = beta * C, or zero; no element of
    // B' is read then and the caller may have passed no workspace: any non-null pointer stands in)
    if (K == 0 && !workspace) workspace = D;
    if constexpr (sizeof(T) == 4)
        return run_gemm<false>(A, workspace, C ? D : nullptr, D, M, 2 * N, 2 * K, 2 * lda, ldx, 2 * ldd, 2 * ldd, 1.f, 1.f, stream,
                               DECX_HIP_TILE_AUTO, 0);
    else
        return run_gemm_f64((const double*)A, (const double*)workspace, C ? (const double*)D : nullptr, (double*)D, M, 2 * N, 2 * K,
                            2 * lda, ldx, 2 * ldd, 2 * ldd, 1.0, 1.0, stream, DECX_HIP_TILE_AUTO, 0);
}
}  // extern "C++"

int decx_hip_gemm_c32(const float* A, const float* B, const float* C, float* D, uint32_t M, uint32_t N, uint32_t K,
                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha_re, float alpha_im, float beta_re,
                      float beta_im, void* workspace, size_t workspace_bytes, void* stream)
{
    return run_gemm_complex<float>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha_re, alpha_im, beta_re, beta_im, workspace,
                                   workspace_bytes, stream);
}

int decx_hip_gemm_c64(const double* A, const double* B, const double* C, double* D, uint32_t M, uint32_t N, uint32_t K,
                      uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, double alpha_re, double alpha_im, double beta_re,
                      double beta_im, void* workspace, size_t workspace_bytes, void* stream)
{
    return run_gemm_complex<double>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha_re, alpha_im, beta_re, beta_im, workspace,
                                    workspace_bytes, stream);
}

int decx_hip_gemm_f32_tile(const float* A, const float* B, const float* C, float* D, uint32_t M, uint32_t N,
                           uint32_t K, uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd, float alpha,
                           float beta, void* stream, int tile, int force_edge)
{
    return run_gemm<false>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, tile, force_edge);
}

int decx_hip_gemm_f16_tile(const uint16_t* A, const uint16_t* B, const uint16_t* C, uint16_t* D, uint32_t M,
                           uint32_t N, uint32_t K, uint32_t lda, uint32_t ldb, uint32_t ldc, uint32_t ldd,
                           float alpha, float beta, void* stream, int tile, int force_edge)
{
    return run_gemm<true>(A, B, C, D, M, N, K, lda, ldb, ldc, ldd, alpha, beta, stream, tile, force_edge);
}

static int run_gemv(bool f16, bool out_f32, const void* A, const void* x, const void* c, void* y, uint32_t M,
                    uint32_t K, uint32_t lda, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta,
                    void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (M == 0) return DECX_HIP_OK;
    if (!A || !x || !y || lda < K || incx == 0 || incy == 0 || (c && incc == 0)) return DECX_HIP_E_INVALID_ARG;
    return launch_gemv(f16, out_f32, A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, as_stream(stream));
}

static int run_gevm(bool f16, bool out_f32, const void* x, const void* B, const void* c, void* y, uint32_t K,
                    uint32_t N, uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta,
                    void* stream, void* workspace = nullptr, size_t workspace_bytes = 0)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (N == 0) return DECX_HIP_OK;
    if (!x || !B || !y || ldb < N || incx == 0 || incy == 0 || (c && incc == 0)) return DECX_HIP_E_INVALID_ARG;
    return gevm_maybe_split(f16, out_f32, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, workspace, workspace_bytes,
                            as_stream(stream));
}

int decx_hip_gemv_f32(const float* A, const float* x, const float* c, float* y, uint32_t M, uint32_t K, uint32_t lda,
                      uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, void* stream)
{
    return run_gemv(false, true, A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, stream);
}
int decx_hip_gemv_f16(const uint16_t* A, const uint16_t* x, const uint16_t* c, void* y, uint32_t M, uint32_t K,
                      uint32_t lda, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, int y_is_f32,
                      void* stream)
{
    return run_gemv(true, y_is_f32 != 0, A, x, c, y, M, K, lda, incx, incc, incy, alpha, beta, stream);
}
int decx_hip_gevm_f32(const float* x, const float* B, const float* c, float* y, uint32_t K, uint32_t N, uint32_t ldb,
                      uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, void* stream)
{
    return run_gevm(false, true, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream);
}
int decx_hip_gevm_f16(const uint16_t* x, const uint16_t* B, const uint16_t* c, void* y, uint32_t K, uint32_t N,
                      uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, int y_is_f32,
                      void* stream)
{
    return run_gevm(true, y_is_f32 != 0, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream);
}

int decx_hip_gevm_f32_ws(const float* x, const float* B, const float* c, float* y, uint32_t K, uint32_t N, uint32_t ldb,
                         uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, void* workspace,
                         size_t workspace_bytes, void* stream)
{
    return run_gevm(false, true, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, workspace, workspace_bytes);
}
int decx_hip_gevm_f16_ws(const uint16_t* x, const uint16_t* B, const uint16_t* c, void* y, uint32_t K, uint32_t N,
                         uint32_t ldb, uint32_t incx, uint32_t incc, uint32_t incy, float alpha, float beta, int y_is_f32,
                         void* workspace, size_t workspace_bytes, void* stream)
{
    return run_gevm(true, y_is_f32 != 0, x, B, c, y, K, N, ldb, incx, incc, incy, alpha, beta, stream, workspace,
                    workspace_bytes);
}

int decx_hip_conv2d_pack_kernels_f32(const float* kernels, float* kmat, uint32_t k_w, uint32_t k_h, uint32_t depth,
                                     uint32_t k_dpitch, uint32_t k_wpitch, uint64_t tensor_stride, uint32_t out_c,
                                     uint32_t kmat_pitch, uint32_t img_dpitch, void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (!kernels || !kmat || !k_w || !k_h || !depth || !out_c || k_dpitch < depth || k_wpitch < k_w ||
        img_dpitch < depth || kmat_pitch < out_c || tensor_stride < (uint64_t)k_dpitch * k_wpitch * (k_h - 1) + (uint64_t)k_dpitch * (k_w - 1) + depth)
        return DECX_HIP_E_INVALID_ARG;
    const uint64_t total = (uint64_t)k_h * k_w * img_dpitch * kmat_pitch;
    const uint64_t want = (total + 255) / 256;
    hipLaunchKernelGGL(conv2d_pack_kernels_kernel, dim3((unsigned)(want < 4096 ? want : 4096)), dim3(256), 0, as_stream(stream),
                       kernels, kmat, k_w, k_h, depth, k_dpitch, k_wpitch, tensor_stride, out_c, kmat_pitch, img_dpitch);
    return (int)hipGetLastError();
}

int decx_hip_conv2d_f32(const float* image, const float* kmat, float* dst, uint32_t out_w, uint32_t out_h, uint32_t out_c,
                        uint32_t k_w, uint32_t k_h, uint32_t img_dpitch, uint32_t img_wpitch, uint32_t stride_x,
                        uint32_t stride_y, uint32_t kmat_pitch, uint32_t dst_dpitch, uint32_t dst_wpitch, void* stream)
{
    return decx_hip_conv2d_f32_depth(image, kmat, dst, out_w, out_h, out_c, k_w, k_h, img_dpitch, img_dpitch, img_wpitch, stride_x,
                                     stride_y, kmat_pitch, dst_dpitch, dst_wpitch, stream);
}

int decx_hip_conv2d_f32_depth(const float* image, const float* kmat, float* dst, uint32_t out_w, uint32_t out_h, uint32_t out_c,
                              uint32_t k_w, uint32_t k_h, uint32_t depth, uint32_t img_dpitch, uint32_t img_wpitch,
                              uint32_t stride_x, uint32_t stride_y, uint32_t kmat_pitch, uint32_t dst_dpitch, uint32_t dst_wpitch,
                              void* stream)
{
    if (!g_dev.ready) return DECX_HIP_E_NOT_INIT;
    if (!out_w || !out_h || !out_c) return DECX_HIP_OK;
    if (!image || !kmat || !dst || !k_w || !k_h || !stride_x || !stride_y || !img_dpitch || img_dpitch % 4 || kmat_pitch % 4 ||
        !depth || depth > img_dpitch ||
        dst_dpitch % 4 || kmat_pitch < out_c || dst_dpitch < out_c || dst_wpitch < out_w ||
        img_wpitch < (uint64_t)(out_w - 1) * stride_x + k_w || !aligned16(image) || !aligned16(kmat) || !aligned16(dst) ||
        (uint64_t)out_w * out_h > 0xffffffffull || (uint64_t)k_w * img_dpitch * 4 > 0xffffffffull ||
        (uint64_t)k_h * k_w * img_dpitch > 0xffffffffull || (uint64_t)kmat_pitch * 256 >= (1ull << 31))
        return DECX_HIP_E_INVALID_ARG;
    GemmArgs g;
    std::memset(&g, 0, sizeof g);
    g.cus = (uint32_t)g_dev.compute_units;
    g.A = image; g.B = kmat; g.C = nullptr; g.D = dst;
    g.M = out_w * out_h; g.N = out_c; g.K = k_h * k_w * img_dpitch;
    g.lda = g.K; g.ldb = kmat_pitch; g.ldc = 0; g.ldd = dst_dpitch;
    g.alpha = 1.f; g.beta = 1.f;
    g.vec_ok = 1;
    g.conv_wout = out_w;
    g.conv_seg_bytes = k_w * img_dpitch * 4u;
    g.conv_px_bytes = stride_x * img_dpitch * 4u;
    g.conv_dst_row = dst_wpitch * dst_dpitch;
    g.conv_seg_stride = (uint64_t)img_wpitch * img_dpitch * 4u;
    g.conv_py_bytes = (uint64_t)stride_y * img_wpitch * img_dpitch * 4u;
    g.conv_image_bytes = ((uint64_t)(out_h - 1) * stride_y + k_h) * img_wpitch * img_dpitch * 4u;
    if (conv2d_direct_pays(g.N, g.K, img_dpitch, depth)) return launch_conv2d_direct_f32(g, img_dpitch, depth, as_stream(stream));
    return launch_conv2d_f32_dma(choose_tile(false, g.M, g.N, true), g, as_stream(stream));
}

int decx_hip_gemm_plan(int elem_bytes, uint32_t M, uint32_t N, uint32_t K, int aligned, decx_hip_plan* out)
{
    if (!out || (elem_bytes != 4 && elem_bytes != 2 && elem_bytes != 8)) return DECX_HIP_E_INVALID_ARG;
    std::memset(out, 0, sizeof *out);
    out->k_splits = 1;
    if (M == 0 || N == 0) return DECX_HIP_OK;
    if (elem_bytes == 8 && !((N == 1 || M == 1) && K > 0)) {
        const int shape = choose_tile_f64(M, N);
        const TileInfo ti = tile_info_f64(shape);
        out->path = shape;
        out->tile_m = ti.bm; out->tile_n = ti.bn;
        out->grid = ((M + ti.bm - 1) / ti.bm) * ((N + ti.bn - 1) / ti.bn);
        out->edge = (K == 0 || !aligned) ? 1 : 0;
        if (out->edge) { out->tile_m = out->tile_n = 16; out->grid = ((M + 15) / 16) * ((N + 15) / 16); }
        else {
            const SplitChoice sc = split_plan(8, M, N, K);
            if (sc.splits > 1 && sc.shape != shape) {               // the split runs on another tile than the whole product
                const TileInfo ts = tile_info_f64(sc.shape);
                out->path = sc.shape; out->tile_m = ts.bm; out->tile_n = ts.bn;
                out->grid = ((M + ts.bm - 1) / ts.bm) * ((N + ts.bn - 1) / ts.bn);
            }
            out->k_splits = sc.splits; out->whole_tiles = sc.first;
            out->grid = sc.first + (out->grid - sc.first) * sc.splits;
        }
        return DECX_HIP_OK;
    }
    const bool f16 = elem_bytes == 2;
    if (N == 1 && K > 0) {
        out->path = DECX_HIP_PATH_GEMV;
        out->tile_m = gemv_rows_per_block(M);                  // 32 (two rows per wavefront) down to 1 (16 wavefronts per row)
        out->tile_n = 1;
        out->grid = (M + out->tile_m - 1) / out->tile_m;
        return DECX_HIP_OK;
    }
    if (M == 1 && K > 0) {
        out->path = DECX_HIP_PATH_GEVM;
        out->tile_m = 1; out->tile_n = 128u / (uint32_t)elem_bytes; // 128 bytes of a row, or 64 when that leaves CUs idle
        const SplitPlan sp = plan_gevm_split(elem_bytes, N, K, g_dev.compute_units);
        if (sp.splits > 1) {                                        // with a workspace: whole lines, several ranges of K
            out->k_splits = sp.splits;
            out->grid = (N + out->tile_n - 1) / out->tile_n * sp.splits;
            return DECX_HIP_OK;
        }
        if ((N + out->tile_n - 1) / out->tile_n < 256u) out->tile_n /= 2;
        out->grid = (N + out->tile_n - 1) / out->tile_n;
        return DECX_HIP_OK;
    }
    const int shape = choose_tile(f16, M, N, aligned != 0);
    const TileInfo ti = f16 ? tile_info_f16(shape, aligned != 0) : tile_info_f32(shape, aligned != 0, N);
    out->path = shape;
    out->tile_m = ti.bm; out->tile_n = ti.bn;
    out->grid = ((M + ti.bm - 1) / ti.bm) * ((N + ti.bn - 1) / ti.bn);
    // the direct-to-LDS kernels take every aligned shape
    out->edge = (K == 0 || !aligned) ? 1 : 0;
    if (!out->edge) {
        const SplitChoice sc = split_plan(elem_bytes, M, N, K);
        if (sc.splits > 1 && sc.shape != shape) {                   // the split runs on another tile than the whole product
            const TileInfo ts = f16 ? tile_info_f16(sc.shape, true) : tile_info_f32(sc.shape, true, N);
            out->path = sc.shape; out->tile_m = ts.bm; out->tile_n = ts.bn;
            out->grid = ((M + ts.bm - 1) / ts.bm) * ((N + ts.bn - 1) / ts.bn);
        }
        out->k_splits = sc.splits; out->whole_tiles = sc.first;
        out->grid = sc.first + (out->grid - sc.first) * sc.splits;
    }
    return DECX_HIP_OK;
}

uint16_t decx_hip_float_to_half(float value)
{
    uint32_t f;
    std::memcpy(&f, &value, 4);
    const uint32_t sign = (f >> 16) & 0x8000u;
    const uint32_t mag = f & 0x7fffffffu;
    if (mag > 0x7f800000u) return (uint16_t)(sign | 0x7e00u | ((mag >> 13) & 0x1ffu));    // NaN
    if (mag >= 0x47800000u) return (uint16_t)(sign | 0x7c00u);                            // >= 2^16: inf
    uint32_t bits;
    if (mag >= 0x38800000u) {                 // normal half: drop 13 mantissa bits, rebias by 112
        const uint32_t base = mag - 0x38000000u;
        bits = base >> 13;
        const uint32_t rest = base & 0x1fffu;
        if (rest > 0x1000u || (rest == 0x1000u && (bits & 1u))) ++bits;   // carry may reach 0x7c00 = inf
    } else if (mag >= 0x33000000u) {          // subnormal half
        const uint32_t exp = mag >> 23;       // 102 .. 112
        const uint32_t sig = (mag & 0x7fffffu) | 0x800000u;
        const uint32_t shift = 126u - exp;    // 14 .. 24
        bits = sig >> shift;
        const uint32_t rest = sig & ((1u << shift) - 1u), half = 1u << (shift - 1);
        if (rest > half || (rest == half && (bits & 1u))) ++bits;
    } else {
        bits = 0;
    }
    return (uint16_t)(sign | bits);
}

float decx_hip_half_to_float(uint16_t h)
{
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t e = (h >> 10) & 0x1fu, m = h & 0x3ffu;
    uint32_t f;
    if (e == 0x1fu)      f = sign | 0x7f800000u | (m << 13);
    else if (e)          f = sign | ((e + 112u) << 23) | (m << 13);
    else if (!m)         f = sign;
    else {
        // subnormal: value = m * 2^-24; let the FPU normalise it
        float v = (float)m * 5.9604644775390625e-08f;
        std::memcpy(&f, &v, 4);
        f |= sign;
    }
    float out;
    std::memcpy(&out, &f, 4);
    return out;
}

}  // extern "C"
