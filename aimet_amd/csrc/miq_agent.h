// Publishing results from many workgroups to the one that finishes last ("ticket" pattern), shared by the calibration
// and histogram-observer kernels.
//
// The invariant, in one place:
//   * Everything a workgroup PUBLISHES for the last workgroup goes through agent_store() or a device-scope atomic
//     (atomicAdd and friends).  These are performed at the device's point of coherence, not in a per-XCD cache.
//   * A workgroup draws its ticket only after every wavefront has seen its own publications acknowledged
//     ("s_waitcnt vmcnt(0)") and the workgroup has passed a barrier; the ticket itself is a relaxed device-scope
//     fetch-add.  The ticket is therefore performed after all of the workgroup's publications.
//   * The workgroup that draws the last ticket passes last_ticket_acquire() and then READS what the others published
//     through agent_load() only.
// A plain store on the publishing side, or a plain load on the reading side, breaks this silently: the L2 caches of
// different XCDs are not coherent for plain accesses.  The reason for not using release / acquire fences on the
// publishing side: a device-scope release per wavefront writes the L2 back every time (measured 65 us for 1024
// workgroups); one acquire in the single last workgroup costs nothing measurable and is kept as a backstop.
#ifndef MIQ_AGENT_H
#define MIQ_AGENT_H

#include "miq_common.h"

namespace miq
{
template <typename T>
__device__ __forceinline__ T agent_load(const T* p)
{
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// written through: also leaves no modified line behind in a cache for the launch's end-of-kernel release to write back
template <typename T>
__device__ __forceinline__ void agent_store(T* p, T v)
{
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// every wavefront of a workgroup, before the barrier that precedes the ticket
__device__ __forceinline__ void publications_acknowledged()
{
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}
// the workgroup that drew the last ticket, before its first agent_load()
__device__ __forceinline__ void last_ticket_acquire()
{
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "agent");
}
}   // namespace miq
#endif
