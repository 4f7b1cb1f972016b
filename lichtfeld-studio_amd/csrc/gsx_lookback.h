// gsx_lookback.h - chained prefix across the workgroups of ONE launch (decoupled look-back), device side.
//
// A workgroup that needs "the sum of what all workgroups in front of me contribute" publishes its own contribution
// in a status word and walks back over its predecessors' words until it meets one that already holds a full prefix.
// Value and state share one 32-bit word (2 state bits + 30 value bits), written and read with relaxed device-scope
// atomics, so no fence is needed: a word is either empty or complete.
//
// Forward progress: a workgroup's place p is its index in a one-dimensional grid.  The dispatcher of each XCD starts
// the workgroups it is given in ascending index order, so the unfinished workgroup with the smallest index never
// waits for anyone and is either running or next in line on an XCD whose running workgroups all have smaller
// indices - i.e. are finished: it always gets to run.  (A ticket counter would make the order explicit, but one
// returning atomic on a single address per workgroup costs ~20 ns each, serialised: 80 us for 4000 workgroups.)
// The wait is bounded all the same: after kLbSpinLimit empty reads a lane gives up, reports it, and returns the
// partial sum it has - which only ever under-counts, so positions derived from it stay inside the output.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gsx {

static constexpr uint32_t kLbEmpty = 0u, kLbAggregate = 1u, kLbPrefix = 2u;
static constexpr uint32_t kLbValueBits = 30u, kLbValueMask = (1u << kLbValueBits) - 1u;
static constexpr uint32_t kLbSpinLimit = 1u << 16; // about a tenth of a second: far beyond any wait that ends

__device__ __forceinline__ void lb_publish(uint32_t* slot, uint32_t state, uint32_t value) {
    __hip_atomic_store(slot, (state << kLbValueBits) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Whether a waiting lane should give up: the bounded wait ran out here, or somewhere else already (then every lane
// still waiting ends too, so a launch that cannot make progress ends after about one wait, not one per workgroup).
// (`limit`: kLbSpinLimit, or what a test set through gsx_debug_set_lookback_spin_limit to see the give-up path)
__device__ __forceinline__ bool lb_give_up(uint32_t spins, uint32_t* error, uint32_t limit) {
    if (spins > limit ||
        ((spins & 255u) == 0 && (__hip_atomic_load(error, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) & 2u) != 0)) {
        atomicOr(error, 2u);
        return true;
    }
    return false;
}

// Sum of the values of places p-1, p-2, ... down to and including the first one in state PREFIX, for one column of a
// table with `stride` words per place (place q's word is status[q * stride + column]); every lane walks its own
// column.  Eight predecessors are requested at a time: a status word that another XCD wrote comes from memory, not
// from this XCD's L2, and the walk is as long as the prefixes have not caught up with the aggregates.
// When the bounded wait runs out, bit 1 of *error is set and the partial sum returned.
__device__ __forceinline__ uint32_t lb_exclusive(const uint32_t* status, uint32_t p, uint32_t stride,
                                                 uint32_t column, uint32_t* error,
                                                 uint32_t limit = kLbSpinLimit) {
    constexpr int kWindow = 8;
    uint32_t sum = 0, spins = 0;
    int64_t q = (int64_t)p - 1;
    while (q >= 0) {
        uint32_t word[kWindow];
#pragma unroll
        for (int j = 0; j < kWindow; ++j)
            word[j] = q - j >= 0 ? __hip_atomic_load(status + (size_t)(q - j) * stride + column, __ATOMIC_RELAXED,
                                                     __HIP_MEMORY_SCOPE_AGENT)
                                 : (kLbPrefix << kLbValueBits);
        int used = 0;
        bool done = false;
#pragma unroll
        for (int j = 0; j < kWindow; ++j) {
            const uint32_t state = word[j] >> kLbValueBits;
            if (!done && used == j && state != kLbEmpty) {
                sum += word[j] & kLbValueMask;
                ++used;
                done = state == kLbPrefix;
            }
        }
        if (done)
            break;
        q -= used;
        if (used == 0) {
            if (lb_give_up(++spins, error, limit))
                break;
            __builtin_amdgcn_s_sleep(1);
        }
    }
    return sum;
}

// The same sum for a table with one word per place, formed by a whole wave (all 64 lanes must call; all receive the
// sum): lane l looks at place p - 1 - l, so 64 predecessors are inspected per round.
__device__ __forceinline__ uint32_t lb_exclusive_wave(const uint32_t* status, uint32_t p, uint32_t* error,
                                                      uint32_t limit = kLbSpinLimit) {
    const uint32_t lane = threadIdx.x & 63u;
    uint32_t sum = 0, spins = 0;
    int64_t top = (int64_t)p - 1; // the nearest place not yet added
    while (top >= 0) {
        const int64_t q = top - (int64_t)lane;
        const uint32_t word = q >= 0 ? __hip_atomic_load(status + q, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
                                     : (kLbPrefix << kLbValueBits);
        const uint32_t state = word >> kLbValueBits;
        const uint64_t prefixes = __ballot(state == kLbPrefix), empties = __ballot(state == kLbEmpty);
        const uint32_t first_prefix = prefixes ? (uint32_t)__builtin_ctzll(prefixes) : 64u;
        const uint32_t first_empty = empties ? (uint32_t)__builtin_ctzll(empties) : 64u;
        // the lanes in front of the first empty word can be added now; the walk ends at a prefix among them
        const uint32_t usable = first_empty < first_prefix ? first_empty : (first_prefix < 64u ? first_prefix + 1u : 64u);
        uint32_t v = lane < usable ? (word & kLbValueMask) : 0u;
#pragma unroll
        for (int m = 32; m >= 1; m >>= 1)
            v += (uint32_t)__shfl_xor((int)v, m, 64);
        sum += v;
        if (first_prefix < first_empty)
            break;
        top -= usable;
        if (usable == 0) {
            bool stop = false;
            if (lane == 0)
                stop = lb_give_up(++spins, error, limit);
            if (__ballot(stop))
                break;
            __builtin_amdgcn_s_sleep(1);
        }
    }
    return sum;
}

} // namespace gsx
