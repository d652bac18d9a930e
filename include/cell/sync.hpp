// Copy-completion fences. Same names as the reference's include/cell/sync.hpp:8-23
// (wait_group<N>, commit_copy_group, __copy_async). On gfx950 a global->LDS copy is a
// vector-memory load followed by an LDS write (or a direct-to-LDS load), both tracked by
// the wavefront's vmcnt / lgkmcnt counters, so "wait for my copies" is s_waitcnt; making
// the data visible to the other wavefronts still takes the __syncthreads() that follows in
// user code, exactly as with cp.async.
#pragma once

#include "config.hpp"

namespace tiledcuda::cell {

/// Wait until at most N of this wavefront's vector-memory loads are outstanding.
template <int N>
DEVICE void wait_group() {
    __builtin_amdgcn_s_waitcnt(/*vmcnt(N) lgkmcnt(0)*/ 0x0070 | (N & 0xF) | ((N >> 4) << 14));
}

/// Copies are issued in program order; nothing to commit explicitly.
DEVICE void commit_copy_group() { __builtin_amdgcn_sched_barrier(0); }

/// Wait for every outstanding copy of this wavefront.
DEVICE void __copy_async() {
    commit_copy_group();
    __builtin_amdgcn_s_waitcnt(0);
}

/// Wait until at most N of this wavefront's copies are outstanding, then a workgroup barrier that orders LDS accesses
/// only: the hand-over of a stage of a SharedRing filled by GlobalToSharedDirectLoader. __syncthreads() would also
/// wait for every copy still in flight (its fence covers the LDS writes of direct-to-LDS loads), which empties the
/// pipeline at every hand-over.
template <int N = 0>
DEVICE void wait_group_and_barrier() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | (N & 0xF) | ((N >> 4) << 14));  // vmcnt(N) lgkmcnt(0)
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

/// wait_group_and_barrier for a kernel that keeps LDS fragment reads in flight across the hand-over (requested with
/// copy::SharedToRegPieces for the matrix instructions that follow the barrier): only the vector-memory counter is
/// waited for. Correct when the reads in flight address stages that are not being handed over - the caller's
/// business, like the reads' own waits (copy::wait_shared_reads).
template <int N = 0>
DEVICE void wait_group_and_barrier_keep_reads() {
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_waitcnt(0x0070 | 0x0f00 | (N & 0xF) | ((N >> 4) << 14));  // vmcnt(N) only
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

}  // namespace tiledcuda::cell
