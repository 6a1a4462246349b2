// Shared pieces of the device-side "roles".
//
// A role is the body of one kernel of the path (tzgemm, stencil, lbm, mri-q, cp)
// written as a __device__ function that is told where it lives inside the
// launch: which of the role's persistent workgroups it is (role_block of
// role_blocks) and which of the role's threads the caller is (tid of
// role_threads).  The same role function is the body of the plain GPTB kernel
// (role = whole launch) and of every fused kernel (role = a subset of the
// workgroups, or a subset of the waves of each workgroup).
//
// Reference: the GPTB trailer and the blockIdx/threadIdx reconstruction of
// src/gptb_kernel/*.cu (block_pos = blockIdx.x + ptb_start_block_pos, stepping by
// ptb_iter_block_step until ptb_end_block_pos; thread = threadIdx.x - thread_base).
#pragma once
#include <hip/hip_runtime.h>
#include "../header/pets_common.h"

namespace tk {

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef unsigned uint4_t __attribute__((ext_vector_type(4)));

// Barrier among all threads of a workgroup: usable when the role owns every wave
// of the workgroup (plain GPTB kernels and workgroup-split fused kernels).
// Only LDS traffic is ordered (s_waitcnt lgkmcnt(0)); global loads in flight are
// deliberately left in flight -- the GEMM role keeps several chunks of
// LDS-direct loads outstanding across its barriers and tracks them itself.
struct WorkgroupSync {
    __device__ __forceinline__ void sync()
    {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
};

// Barrier among the waves of ONE role inside a workgroup that also hosts
// another role (wave-split fused kernels).  gfx950 has a single hardware
// barrier per workgroup and no named barriers, so a role-local barrier is an
// LDS arrival counter: lane 0 of each wave adds 1, everybody polls until the
// count reaches the number of arrivals expected so far.  All waves of a
// workgroup are resident at the same time, so polling cannot starve a wave that
// has yet to arrive.  The poll is bounded: after spin_limit polls the wave gives
// up, raises *fail (a global word the host checks) and carries on, so a logic
// error ends in a wrong answer plus a flag, never in waves that do not finish.
struct RoleSpinSync {
    unsigned *counter;       // LDS word, zero when the role starts
    unsigned waves;          // waves taking part
    unsigned expected;       // arrivals that complete the current barrier
    unsigned *fail;          // global flag, may be nullptr
    unsigned spin_limit;
    __device__ __forceinline__ RoleSpinSync(unsigned *c, unsigned w, unsigned *f,
                                            unsigned limit = (1u << 22))
        : counter(c), waves(w), expected(0), fail(f), spin_limit(limit) {}
    __device__ __forceinline__ void sync()
    {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");   // LDS reads/writes of this wave are done
        expected += waves;
        if ((threadIdx.x & (TK_WAVE_SIZE - 1)) == 0)
            __hip_atomic_fetch_add(counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        unsigned polls = 0;
        while ((int)(__hip_atomic_load(counter, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP) -
                     expected) < 0) {
            __builtin_amdgcn_s_sleep(1);
            if (++polls > spin_limit) {
                if (fail) *fail = 1u;
                break;
            }
        }
        asm volatile("" ::: "memory");
    }
};

// Where a workgroup of a workgroup-split fused launch belongs.
// The launch has gridDim.x = groups * (a + b) workgroups.  Hardware hands
// consecutive workgroup ids to the 8 XCDs round-robin, so roles are assigned by
// (blockIdx / 8): every XCD receives the same a : b mix, and role-local ids keep
// blockIdx % 8 so that id % 8 still names the XCD.
struct WgSplit {
    int role;         // 0 = first role (a workgroups per group), 1 = second role
    int role_block;   // id among the role's workgroups
    int role_blocks;  // workgroups of this role in the launch
};

__device__ __forceinline__ WgSplit wg_split(int block, int blocks, int a, int b)
{
    WgSplit s;
    const int xcd = block % TK_XCD_NUM;
    const int slot = block / TK_XCD_NUM;
    const int group = slot / (a + b);
    const int in_group = slot % (a + b);
    const int slots = blocks / TK_XCD_NUM;            // host guarantees divisibility
    const int groups = slots / (a + b);
    if (in_group < a) {
        s.role = 0;
        s.role_block = (group * a + in_group) * TK_XCD_NUM + xcd;
        s.role_blocks = groups * a * TK_XCD_NUM;
    } else {
        s.role = 1;
        s.role_block = (group * b + (in_group - a)) * TK_XCD_NUM + xcd;
        s.role_blocks = groups * b * TK_XCD_NUM;
    }
    return s;
}

}  // namespace tk
