// Where the workgroups that share a split-K tile meet: partial products through a workspace, added in a fixed order
// by the workgroup that finishes last, inside the GEMM kernel itself (no second launch, nobody waits for anybody).
// Device code for gfx950.
#pragma once
#include "gemm_common.hpp"

namespace decx_hip {

// Compile-time loop: f(std::integral_constant<int, I>{}) for I in [I, N).
template <int I, int N, class F> __device__ __forceinline__ void static_for(F&& f)
{
    if constexpr (I < N) {
        f(std::integral_constant<int, I>{});
        static_for<I + 1, N>(f);
    }
}

constexpr uint32_t kSplitFlat = 8;      // up to this many splits the last workgroup of a tile adds them all itself
constexpr uint32_t kSplitGroup = 4;     // beyond: groups of this many consecutive splits are added first

// Counters a launch of `tiles` tiles on `splits` splits needs (all zero before and after the launch).
__host__ __device__ inline uint32_t split_counters_per_tile(uint32_t splits)
{
    return splits <= kSplitFlat ? 1u : 1u + (splits + kSplitGroup - 1) / kSplitGroup;
}

// sb: the block's split tile (counted from the first split tile), split and number of splits; NT threads per workgroup.
// A lane's accumulators are PIECES 16-byte pieces, piece c read by
// get(c) and given back by put(c, value, first): put stores `value` when `first`, else adds it.  Every workgroup
// writes its pieces to its slot of the workspace, [piece][thread] so that a wave writes whole lines, and counts itself
// in on the tile's counter; the function returns false in all but the workgroup that arrives last, and in that one
// after it has summed every slot in split order (its own included: the sum does not depend on who is last) into the
// accumulators and put the counter back to zero.
// With more than kSplitFlat splits the sum has two levels, so that its chain of round trips to memory stays short (one
// workgroup adding 64 slots makes 16 of them, 2 us each when it has its CU to itself): the last of every group of
// kSplitGroup consecutive splits adds the group in split order, leaves the sum in the group's first slot and counts
// the group in; the last group to do so adds the group sums in group order.  Still a fixed order of additions.
// Slots are written and read with device-scope accesses (`sc1`: they pass the XCD's own L2, which is not coherent with
// the other seven), so no cache-wide write-back or invalidation is needed around the count -- those would throw out the
// operand lines that workgroups still multiplying live on.
// A sum runs GROUP pieces at a time (16 registers of loads in flight next to the accumulators), and tiles with few
// pieces per lane fetch the same pieces of BATCH slots together (one slot at a time costs a round trip to memory per
// split).  `flag`: a word of LDS that no wave still reads for anything else.  on_last() runs in the workgroup that will
// write the tile, before it loads the last level's first slot.
// TWO_LEVEL false: one level whatever the number of splits (a kernel whose registers the second copy of the sum would
// cost a workgroup per CU, and which the planner gives few splits anyway).
template <int NT, int PIECES, typename V, bool TWO_LEVEL = true, class Get, class Put, class OnLast>
__device__ __forceinline__ bool split_k_exchange(const GemmArgs& g, const SplitBlock& sb, uint32_t* flag, Get&& get, Put&& put, OnLast&& on_last)
{
    static_assert(sizeof(V) == 16, "pieces are 16 bytes");
    constexpr int GROUP = PIECES <= 16 ? PIECES : 16, BATCH = 16 / GROUP;
    static_assert(PIECES % GROUP == 0 && GROUP * BATCH == 16, "pieces per lane: 1, 2, 4, 8, or a multiple of 16");
    const int t = threadIdx.x;
    const uint32_t splits = sb.splits, z = sb.z;
    constexpr size_t SLOT = (size_t)NT * PIECES;           // pieces per slot
    V* const slots = (V*)g.split_ws + (size_t)sb.tile * splits * SLOT;
    uint32_t* const counters = g.split_counters + (size_t)sb.tile * split_counters_per_tile(splits);

    // this lane's pieces -> slot `s`
    const auto store_slot = [&](uint32_t s) {
        V* const mine = slots + (size_t)s * SLOT;
        static_for<0, PIECES>([&](auto cc) {
            constexpr int c = decltype(cc)::value;
            const V v = get(cc);
            V* const dst = mine + (size_t)c * NT + t;
            // s_nop: a store of more than 64 bits reads its data registers up to two cycles after it issues, and the
            // compiler, which inserts that gap for its own stores, does not know that this is one
            asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" :: "v"(dst), "v"(v) : "memory");
        });
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");   // this lane's stores have arrived
        __syncthreads();                                   // everyone's have
    };
    // counts this workgroup in; true in the one that makes the count `expected` (it puts the counter back to zero)
    const auto arrive = [&](uint32_t* counter, uint32_t expected) {
        if (t == 0) {
            const uint32_t before = __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool last = before + 1 == expected;
            if (last) __hip_atomic_store(counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            *flag = last ? 1u : 0u;
        }
        __syncthreads();
        const bool last = __builtin_amdgcn_readfirstlane(*flag) != 0;
        __syncthreads();                                   // the flag may be written again
        return last;
    };
    // accumulators = slot first + slot (first + step) + ... (count of them), in that order.  The loads are buffer loads
    // the compiler knows as loads (it places the waits, and no copy of a destination register can slip in between a
    // load and its wait, as it could with loads written as inline assembly): the tile's slots are the buffer, a lane's
    // offset is its own 16 bytes and the slot and piece go into the scalar offset.
    const __amdgpu_buffer_rsrc_t slot_buffer = __builtin_amdgcn_make_buffer_rsrc((void*)slots, 0, 0x7fffffff, 0x00020000);
    constexpr int kDeviceScope = 16;                       // the sc1 bit of a gfx950 load
    const auto sum_slots = [&](uint32_t first, uint32_t count, uint32_t step) {
        static_for<0, PIECES / GROUP>([&](auto gc) {
            constexpr int c0 = decltype(gc)::value * GROUP;
            for (uint32_t i0 = 0; i0 < count; i0 += BATCH) {
                V v[BATCH][GROUP];
#pragma unroll
                for (int ib = 0; ib < BATCH; ++ib) {
                    if (ib == 0 || i0 + ib < count) {      // slots beyond the last are neither loaded nor added
                        const uint32_t slot_bytes = (first + (i0 + ib) * step) * (uint32_t)(SLOT * 16);
#pragma unroll
                        for (int c = 0; c < GROUP; ++c)
                            v[ib][c] = __builtin_bit_cast(V, __builtin_amdgcn_raw_buffer_load_b128(
                                slot_buffer, (uint32_t)t * 16u, slot_bytes + (uint32_t)((c0 + c) * NT * 16), kDeviceScope));
                    }
                }
#pragma unroll
                for (int ib = 0; ib < BATCH; ++ib) {
                    if (ib == 0 || i0 + ib < count) {
                        static_for<0, GROUP>([&](auto cc) {
                            constexpr int c = decltype(cc)::value;
                            put(std::integral_constant<int, c0 + c>{}, v[ib][c], i0 + ib == 0);
                        });
                    }
                }
            }
        });
    };

    // The stores are inline asm, and the compiler does not count the wait states an MFMA needs before its result
    // registers may be read for an instruction it cannot see into (accumulators that live in VGPRs go to the stores
    // without a copy in between): every MFMA stays in front of the fence and has drained behind it.
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_nop 15\n\ts_nop 15" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
    // one pass with few splits; with many, a pass over this workgroup's group first and, for the last of every group,
    // the pass over the group sums
    const bool flat = !TWO_LEVEL || splits <= kSplitFlat;
    uint32_t slot = z;
    if (TWO_LEVEL && !flat) {
        const uint32_t grp = z / kSplitGroup, first = grp * kSplitGroup;
        const uint32_t members = splits - first < kSplitGroup ? splits - first : kSplitGroup;
        store_slot(slot);
        if (!arrive(counters + 1 + grp, members)) return false;
        sum_slots(first, members, 1);
        slot = first;                                      // its partial product is in the sum: the slot is free
    }
    const uint32_t count = flat ? splits : (splits + kSplitGroup - 1) / kSplitGroup;
    store_slot(slot);
    if (!arrive(counters, count)) return false;
    on_last();
    sum_slots(0, count, flat ? 1u : kSplitGroup);
    return true;
}

}  // namespace decx_hip
