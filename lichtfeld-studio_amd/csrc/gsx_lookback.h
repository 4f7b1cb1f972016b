// gsx_lookback.h - chained prefix across the workgroups of ONE launch (decoupled look-back), device side.
//
// A workgroup that needs "the sum of what all workgroups in front of me contribute" publishes its own contribution
// in a status word and walks back over its predecessors' words until it meets one that already holds a full prefix.
// Value and state share one 32-bit word (2 state bits + 30 value bits), written and read with relaxed device-scope
// atomics, so no fence is needed: a word is either empty or complete.
//
// Forward progress: workgroups take their place p from a ticket counter when they start running, so every
// predecessor of a running workgroup is itself running or finished, and a running wave is never starved by a
// spinning one (the look-back only waits for work that is already resident).  The wait is bounded all the same: after
// kLbSpinLimit empty reads a lane gives up, reports it, and returns the partial sum it has - which only ever
// under-counts, so positions derived from it stay inside the output.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gsx {

static constexpr uint32_t kLbEmpty = 0u, kLbAggregate = 1u, kLbPrefix = 2u;
static constexpr uint32_t kLbValueBits = 30u, kLbValueMask = (1u << kLbValueBits) - 1u;
static constexpr uint32_t kLbSpinLimit = 1u << 22;

__device__ __forceinline__ void lb_publish(uint32_t* slot, uint32_t state, uint32_t value) {
    __hip_atomic_store(slot, (state << kLbValueBits) | value, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// Sum of the values of places p-1, p-2, ... down to and including the first one in state PREFIX.  Place q's word is
// status[q * stride + column].  *gave_up is set (never cleared) when the bounded wait ran out.
__device__ __forceinline__ uint32_t lb_exclusive(const uint32_t* status, uint32_t p, uint32_t stride,
                                                 uint32_t column, uint32_t* gave_up) {
    uint32_t sum = 0;
    for (int64_t q = (int64_t)p - 1; q >= 0; --q) {
        const uint32_t* slot = status + (size_t)q * stride + column;
        uint32_t word = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        uint32_t spins = 0;
        while ((word >> kLbValueBits) == kLbEmpty) {
            if (++spins > kLbSpinLimit) {
                *gave_up = 1u;
                return sum;
            }
            __builtin_amdgcn_s_sleep(1);
            word = __hip_atomic_load(slot, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        sum += word & kLbValueMask;
        if ((word >> kLbValueBits) == kLbPrefix)
            break;
    }
    return sum;
}

// the place of this workgroup in the chain (one ticket per workgroup; all lanes get the value)
__device__ __forceinline__ uint32_t lb_take_ticket(uint32_t* ticket, uint32_t* lds_slot) {
    if (threadIdx.x == 0)
        *lds_slot = atomicAdd(ticket, 1u);
    __syncthreads();
    return *lds_slot;
}

} // namespace gsx
