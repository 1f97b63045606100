// Sum of the blocks of partial sums of the workgroups that share an XCD, formed inside the launch that wrote them, through that XCD's L2.
//
// A kernel whose workgroups each leave a block of `count` partial sums (partial + id * count) would otherwise hand all of them to the
// launch that adds them up: for a grid of 256 that is 256 blocks written to memory and read back. Workgroups are handed to the eight XCDs
// round robin by their index, so the workgroups id = x, x + 8, x + 16, .. run on XCD x and share its L2: each of them, after its block is
// written, announces it, waits for the others of its XCD, and adds up a slice of the elements over the group's blocks, in the order of the
// members, into block x of `out`. What leaves the XCD is one block per XCD: 8 instead of the grid size, in an order that does not depend on
// scheduling. Nothing here needs the caches written back or invalidated: stores are in the L2 once the wavefront's s_waitcnt has passed,
// and the loads of other members' data do not allocate in this compute unit's cache.
//
// The wait is bounded (the device handle's wait limit): the members of a group must be resident together, which the host only asks for
// where the grid has at most one workgroup per compute unit. A member that gives up sets *fault and skips its slice.
// Announcements: member m stores epoch + 1 in flags[m]; `epoch` is the group's own word, which member 0 advances after its wait, when every
// member has read it (each reads it before it announces). The words only ever grow, so nothing has to be cleared between launches.
#pragma once
#include "common.h"
#include "optim.h"

constexpr int RLT_XCD_GROUPS = 8, RLT_XCD_MAX_MEMBERS = 32, RLT_XCD_GROUP_WORDS = 40;      // per group: 32 flags, the epoch word, padding
constexpr int RLT_XCD_WORDS_OFFSET = 1024;      // where the groups' words lie in the device handle's counters block (uint32 index); room for 16 groups

struct rlt_xcd_reduce_args {
    int enabled;
    unsigned max_poll;
    uint32_t* words;        // group g's words at words + g * RLT_XCD_GROUP_WORDS
    unsigned* fault;
};

// Called by every thread of the workgroup after its last store to its block. `group`: which group's words (the caller numbers its groups,
// one per XCD and network), member / n_members: this workgroup's place among the group's, blocks: the group's first block, whose
// members' blocks are member * 8 * count apart; out: the group's block of sums. lds_word: one LDS word of the workgroup.
// epoch0: the group's epoch word as read at the start of the kernel (rlt_xcd_epoch).
__device__ __forceinline__ uint32_t rlt_xcd_epoch(const rlt_xcd_reduce_args& X, int group) {
    return __hip_atomic_load(X.words + group * RLT_XCD_GROUP_WORDS + RLT_XCD_MAX_MEMBERS, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <int THREADS>
__device__ __forceinline__ void rlt_xcd_group_reduce(const rlt_xcd_reduce_args& X, int group, int member, int n_members, uint32_t epoch0, const float* blocks, int count, float* out,
                                                     __attribute__((address_space(3))) int* lds_word) {
    uint32_t* const flags = X.words + group * RLT_XCD_GROUP_WORDS;
    const uint32_t target = epoch0 + 1u;
    __builtin_amdgcn_s_waitcnt(0);        // this wavefront's stores are in the L2
    __syncthreads();
    if (threadIdx.x < 64) {
        if (threadIdx.x == 0) flags[member] = target;
        int ok = 1;
        unsigned tries = 0;
        for (;;) {
            const uint32_t f = __hip_atomic_load(flags + min((int)threadIdx.x, n_members - 1), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (__all((int32_t)(f - target) >= 0)) break;
            if (++tries >= X.max_poll || ((tries & 63u) == 0u && __hip_atomic_load(X.fault, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))) {
                if (threadIdx.x == 0) __hip_atomic_store(X.fault, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                ok = 0;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        if (threadIdx.x == 0) {
            *lds_word = ok;
            if (ok && member == 0) __hip_atomic_store(flags + RLT_XCD_MAX_MEMBERS, target, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    __syncthreads();
    if (!*lds_word) return;
    // this member's slice of the elements, summed over the members' blocks in member order
    const int chunk = (count + n_members - 1) / n_members, begin = member * chunk, end = min(count, begin + chunk);
    const size_t stride = (size_t)RLT_XCD_GROUPS * count;
    for (int e = begin + (int)threadIdx.x; e < end; e += THREADS) {
        float v[RLT_XCD_MAX_MEMBERS];
#pragma unroll
        for (int m = 0; m < RLT_XCD_MAX_MEMBERS; m++) v[m] = m < n_members ? rlt_load_shared<1>(blocks + (size_t)m * stride + e) : 0.f;
        float s = v[0];
#pragma unroll
        for (int m = 1; m < RLT_XCD_MAX_MEMBERS; m++) s += m < n_members ? v[m] : 0.f;
        out[e] = s;
    }
}
