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

// Raised by device code that has to give up (bits TK_FAIL_*), read and cleared by the host.
__device__ unsigned tk_spin_fail = 0u;

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
    __device__ __forceinline__ void wait()
    {
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
    __device__ __forceinline__ void sync()
    {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait();
    }
    __device__ __forceinline__ void finish() {}
};

// Barrier among the waves of ONE role inside a workgroup that also hosts another role (wave-split
// fused kernels).  gfx950 has a single hardware barrier per workgroup and no named barriers, so a
// role-local barrier is an LDS arrival counter: lane 0 of each wave adds 1, everybody polls until
// the count reaches the number of arrivals expected so far.  All waves of a workgroup are resident
// at the same time, so polling cannot starve a wave that has yet to arrive.  The poll is bounded:
// after spin_limit polls the wave gives up, raises *fail (a global word the host checks) and
// carries on, so a logic error ends in a wrong answer plus a flag, never in waves that do not
// finish.  The counter hands over to the hardware barrier once the waves of the other role have ended:
//
// The hardware barrier counts the waves of the workgroup that have not terminated.  While waves of
// the other role run it cannot serve one role; once they have all ended it serves the waves that are
// left, and it costs nothing where the arrival counter costs an LDS atomic and a poll per barrier (the
// GEMM role's K loop runs a fifth slower on the counter).  Three LDS words: the arrival counter,
// `alive` = waves of the other role that have not finished (each subtracts 1 when its work is done,
// role_wave_done), and `switch_at`.  The role's first wave is the decider: when it has seen alive == 0
// it writes the index of the barrier it is about to arrive at into switch_at, then arrives.  Every wave
// reads switch_at after each barrier it passes on the counter and takes the hardware barrier for all
// barriers behind index switch_at.  The write precedes the decider's arrival and LDS serves a wave's
// operations in order, so every wave that passes barrier switch_at reads it, and waves that read it
// earlier still take that barrier on the counter: all waves change over at the same barrier.  A wave
// whose poll runs into its limit changes over too (and raises the failure word): from then on it can
// only hold the others up at the hardware barrier until they give up as well, never spin on.
struct RoleHandoverSync {
    unsigned counter_addr;   // LDS byte address of the three words
    unsigned waves;
    unsigned expected;       // arrivals that complete the current barrier = its index
    unsigned gave_up;
    unsigned *fail;
    unsigned spin_limit;
    // wave-uniform state, kept in scalar registers (every value below comes out of a readfirstlane):
    unsigned hw;             // 1 = hardware barrier from now on
    unsigned announce;       // decider has seen the other role's waves gone
    unsigned decider;        // this is the role's first wave
    // role_tid: the caller's thread index within the role (its first 64 threads are the decider wave)
    __device__ __forceinline__ RoleHandoverSync(unsigned *words, unsigned w, int role_tid, unsigned *f,
                                                unsigned limit = (1u << 24))
        : counter_addr((unsigned)(size_t)(__attribute__((address_space(3))) unsigned *)words), waves(w), expected(0),
          gave_up(0), fail(f), spin_limit(limit), hw(0), announce(0),
          decider(__builtin_amdgcn_readfirstlane(role_tid) < 64 ? 1u : 0u) {}

    // what thread 0 of the workgroup stores before the roles part ways: no arrival, other_waves
    // waves of the other role at work, no change-over in sight
    static __device__ __forceinline__ void init(unsigned *words, unsigned other_waves)
    {
        words[0] = 0u;
        words[1] = other_waves;
        words[2] = 0x7fffffffu;
    }

    // The hardware barrier is the path the K loop falls through; the counter's code sits out of its
    // way.  (Every instruction at the barrier is a gap in the wave's MFMA stream: with the change-over
    // test and the counter's code in line the loop ran 12 % slower than with the bare s_barrier.)
    __device__ __forceinline__ void wait()
    {
        if (__builtin_expect(hw != 0u, 1)) {
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        } else {
            on_the_counter();
        }
    }
    // arrive, poll until every wave of the role has, then look whether this was the barrier to change over at
    __device__ __forceinline__ void on_the_counter()
    {
        expected += waves;
        unsigned now, at, alive, left, hw_lanes, announce_lanes;
        unsigned long long saved_exec;
        asm volatile("s_mov_b32 %[left], %[limit]\n\t"
                     "s_mov_b64 %[saved], exec\n\t"
                     "s_mov_b64 exec, 1\n\t"
                     "s_cmp_eq_u32 %[announce_in], 0\n\t"
                     "s_cbranch_scc1 8f\n\t"
                     "ds_write_b32 %[addr], %[index] offset:8\n"
                     "8:\n\t"
                     "ds_add_u32 %[addr], %[one]\n\t"
                     "s_mov_b64 exec, %[saved]\n"
                     "4:\n\t"                              // poll
                     "ds_read_b32 %[now], %[addr]\n\t"
                     "s_waitcnt lgkmcnt(0)\n\t"
                     "v_sub_u32 %[now], %[now], %[index]\n\t"
                     "v_cmp_gt_i32 vcc, 0, %[now]\n\t"
                     "s_cbranch_vccz 2f\n\t"
                     "s_sub_u32 %[left], %[left], 1\n\t"
                     "s_cmp_lg_u32 %[left], 0\n\t"
                     "s_cbranch_scc1 4b\n"
                     "2:\n\t"                              // passed (or gave up): change over from here?
                     "ds_read_b32 %[at], %[addr] offset:8\n\t"
                     "ds_read_b32 %[alive], %[addr] offset:4\n\t"
                     "s_waitcnt lgkmcnt(0)\n\t"
                     "v_sub_u32 %[at], %[index], %[at]\n\t"
                     "v_cmp_le_i32 vcc, 0, %[at]\n\t"
                     "v_cndmask_b32_e64 %[hw], 0, 1, vcc\n\t"
                     "v_cmp_eq_u32 vcc, 0, %[alive]\n\t"
                     "v_cndmask_b32_e64 %[announce_out], 0, 1, vcc"
                     : [now] "=&v"(now), [at] "=&v"(at), [alive] "=&v"(alive), [left] "=&s"(left),
                       [saved] "=&s"(saved_exec), [hw] "=&v"(hw_lanes), [announce_out] "=&v"(announce_lanes)
                     : [addr] "v"(counter_addr), [index] "v"(expected), [one] "v"(1u), [limit] "s"(spin_limit),
                       [announce_in] "s"(announce)
                     : "vcc", "scc", "memory");
        announce = __builtin_amdgcn_readfirstlane(announce_lanes) & decider;
        const unsigned out_of_polls = (left == 0u);
        gave_up |= out_of_polls;
        hw = __builtin_amdgcn_readfirstlane(hw_lanes) | out_of_polls;
    }
    __device__ __forceinline__ void sync()
    {
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        wait();
    }
    __device__ __forceinline__ void finish()
    {
        if (gave_up && fail) __hip_atomic_fetch_or(fail, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
};

// What a wave of the other role calls when its work is done (every wave of it, on every path): one
// less to wait for before the hardware barrier can serve the role that synchronises.
__device__ __forceinline__ void role_wave_done(unsigned *words)
{
    const int lane = (int)__builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
    if (lane == 0) __hip_atomic_fetch_sub(words + 1, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
}

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
