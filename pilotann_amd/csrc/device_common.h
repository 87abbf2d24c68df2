// Wavefront-level helpers shared by the traversal and router kernels (gfx950,
// 64-lane wavefronts).
#ifndef PILOTANN_DEVICE_COMMON_H
#define PILOTANN_DEVICE_COMMON_H

#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

namespace pa {

constexpr int kWave = 64;

__device__ __forceinline__ int uni(int x) {
    return __builtin_amdgcn_readfirstlane(x);
}
__device__ __forceinline__ float uni(float x) {
    return __int_as_float(__builtin_amdgcn_readfirstlane(__float_as_int(x)));
}
// Orders LDS traffic between the lanes of this wavefront (the hardware keeps a
// wavefront's LDS operations in issue order; this keeps the compiler from
// moving them).
__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}
__device__ __forceinline__ int lane_rank(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi(
        (unsigned)(mask >> 32),
        __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0u));
}

template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_f(float x) {
    return __int_as_float(__builtin_amdgcn_update_dpp(
        __float_as_int(x), __float_as_int(x), CTRL, ROW_MASK, 0xF, false));
}

// Maximum over the wavefront, returned in every lane.
__device__ __forceinline__ float wave_max(float x) {
    x = fmaxf(x, dpp_f<0xB1, 0xF>(x));   // quad_perm [1,0,3,2]
    x = fmaxf(x, dpp_f<0x4E, 0xF>(x));   // quad_perm [2,3,0,1]
    x = fmaxf(x, dpp_f<0x141, 0xF>(x));  // row_half_mirror
    x = fmaxf(x, dpp_f<0x140, 0xF>(x));  // row_mirror: rows of 16 done
    x = fmaxf(x, dpp_f<0x142, 0xA>(x));  // row_bcast15 into rows 1 and 3
    x = fmaxf(x, dpp_f<0x143, 0xC>(x));  // row_bcast31 into rows 2 and 3
    return __int_as_float(
        __builtin_amdgcn_readlane(__float_as_int(x), kWave - 1));
}


// Maximum of a signed integer over the wavefront, in every lane: six DPP
// steps (rows of 16 by quad_perm and mirrors, then row_bcast15 / row_bcast31
// into the upper rows) and a read of lane 63.  Written as v_max_i32_dpp so
// that each step is one instruction; the s_nop covers the two wait states a
// DPP read needs after a vector write of the same register.
__device__ __forceinline__ int wave_max_key(int x) {
#ifdef PA_WAVE_MAX_ASM
    asm("s_nop 1\n\t"
        "v_max_i32_dpp %0, %0, %0 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_i32_dpp %0, %0, %0 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_i32_dpp %0, %0, %0 row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_i32_dpp %0, %0, %0 row_mirror row_mask:0xf bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_i32_dpp %0, %0, %0 row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
        "s_nop 1\n\t"
        "v_max_i32_dpp %0, %0, %0 row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
        "s_nop 1"
        : "+v"(x));
#else
    constexpr int kLow = (int)0x80000000;
    x = max(x, __builtin_amdgcn_update_dpp(kLow, x, 0xB1, 0xF, 0xF, false));
    x = max(x, __builtin_amdgcn_update_dpp(kLow, x, 0x4E, 0xF, 0xF, false));
    x = max(x, __builtin_amdgcn_update_dpp(kLow, x, 0x141, 0xF, 0xF, false));
    x = max(x, __builtin_amdgcn_update_dpp(kLow, x, 0x140, 0xF, 0xF, false));
    x = max(x, __builtin_amdgcn_update_dpp(kLow, x, 0x142, 0xA, 0xF, false));
    x = max(x, __builtin_amdgcn_update_dpp(kLow, x, 0x143, 0xC, 0xF, false));
#endif
    return __builtin_amdgcn_readlane(x, kWave - 1);
}

// Squared L2 between a query held in LDS and one plain row (the router's leaf
// vectors, which stay as the caller passes them), in the order of
// the reference's host code (extension/inc/distance.h:31-55): element j of
// every group of eight goes to accumulator j with one FMA, the eight
// accumulators are then added left to right.  Four adjacent lanes (a quad)
// share a row: lane a of the quad owns accumulators 2a and 2a + 1 and streams
// its 8 bytes of every 32-byte group, so all loads of a row are in flight at
// once in 2 * dp / 8 registers.  `row` points at the lane's pair of the first
// group, `qv` at the lane's run of the query in LDS (query_slot layout).  Lane 0
// of the quad returns the distance; every
// lane of the wavefront must call this (the exchange inside the quad is a DPP
// move), lanes without a row pass active = false.
constexpr int kLanesPerRow = 4;
constexpr int kRowsPerPass = kWave / kLanesPerRow;

// Where element i of a query goes in LDS: the 8-byte pairs one lane of a quad
// needs (pair a of every group of eight) lie next to each other, so that two
// groups are one 16-byte read; two pairs of padding after each lane's run keep
// the four runs on different banks.  `groups` = dp / 8.
__host__ __device__ constexpr int query_run(int groups) { return groups + 2; }
__host__ __device__ constexpr int query_floats(int dp) { return 8 * query_run(dp >> 3); }
__device__ __forceinline__ int query_slot(int i, int groups) {
    return 2 * (((i >> 1) & 3) * query_run(groups) + (i >> 3)) + (i & 1);
}

// The eight accumulators of a row, added left to right (distance.h:50-54):
// lane a of the quad holds accumulators 2a and 2a + 1; lane 0 of the quad
// returns the sum.  One v_add_f32_dpp per term (the other lanes' accumulators come in as
// the swizzled operand); the s_nop covers the two wait states a DPP read needs
// after the last FMA wrote a0 / a1.
__device__ __forceinline__ float quad_reduce(float a0, float a1) {
    float s;
    asm("s_nop 1\n\t"
        "v_add_f32 %0, %1, %2\n\t"
        "v_add_f32_dpp %0, %1, %0 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %0, %2, %0 quad_perm:[1,1,1,1] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %0, %1, %0 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %0, %2, %0 quad_perm:[2,2,2,2] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %0, %1, %0 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf\n\t"
        "v_add_f32_dpp %0, %2, %0 quad_perm:[3,3,3,3] row_mask:0xf bank_mask:0xf"
        : "=&v"(s)
        : "v"(a0), "v"(a1));
    return s;
}

template <int DP8>
__device__ __forceinline__ float quad_square_dist(const float2 *row,
                                                  const float2 *qv, int groups,
                                                  bool active) {
    float a0 = 0.f, a1 = 0.f;
    if (active) {
        if (DP8 > 0 && DP8 % 2 == 0) {
            // All loads of the row first, then the query from LDS, 16 bytes
            // (two groups) per read, four groups at a time (the fences keep
            // the compiler from hoisting those reads, which would double the
            // live registers).
            constexpr int kPairs = DP8 > 0 ? DP8 : 2;
            float2 x[kPairs];
#pragma unroll
            for (int t = 0; t < kPairs; ++t) x[t] = row[4 * t];
            __builtin_amdgcn_sched_barrier(0);
            const float4 *q4 = reinterpret_cast<const float4 *>(qv);
#pragma unroll
            for (int t = 0; t < kPairs; t += 2) {
                const float4 y = q4[t >> 1];
                const float d0 = y.x - x[t].x, d1 = y.y - x[t].y;
                a0 = fmaf(d0, d0, a0);
                a1 = fmaf(d1, d1, a1);
                const float d2 = y.z - x[t + 1].x, d3 = y.w - x[t + 1].y;
                a0 = fmaf(d2, d2, a0);
                a1 = fmaf(d3, d3, a1);
                if ((t & 2) == 2) __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_sched_barrier(0);
        } else {
#pragma unroll 4
            for (int t = 0; t < groups; ++t) {
                const float2 x = row[4 * t];
                const float2 y = qv[t];
                const float d0 = y.x - x.x, d1 = y.y - x.y;
                a0 = fmaf(d0, d0, a0);
                a1 = fmaf(d1, d1, a1);
            }
        }
    }
    return quad_reduce(a0, a1);
}

// Long rows (the full-dimension refine) are kept in device memory with the
// two groups of every 64-byte block interleaved by lane: the 16 bytes lane a
// of a quad needs of groups 2b and 2b + 1 (its pair of each) are adjacent, at
// floats 16b + 4a .. 16b + 4a + 3, so a lane streams a row with 16-byte loads
// and a quad covers 64 contiguous bytes per instruction — half the memory
// instructions of the plain layout, which is what bounds a kernel that streams
// 3 KB rows.  A last group without a partner (d / 8 odd) stays plain.
// Position of lane a's pair of group g in a row of `groups` groups:
__host__ __device__ constexpr int row_pair_slot(int g, int a, int groups) {
    return (g == groups - 1 && (groups & 1)) ? 8 * g + 2 * a
                                             : 16 * (g >> 1) + 4 * a + 2 * (g & 1);
}

// Squared L2 over groups [first, groups) of such a row (the accumulators start
// at zero at `first`), in the host's order as above: the FMAs of a group
// follow those of the group before it.  `row` is the row's start, `qrun` the
// lane's run of the query in LDS (query_slot layout), `part` the lane's place
// in its quad.  Eight blocks (16 groups) of loads are in flight at once.
// Lane 0 of the quad returns the sum; every lane must call this.
#ifndef PA_LONG_CHUNK
#define PA_LONG_CHUNK 8
#endif
__device__ __forceinline__ float quad_square_dist_long(const float *row,
                                                       const float2 *qrun,
                                                       int groups, int first,
                                                       int part, bool active) {
    float a0 = 0.f, a1 = 0.f;
    if (active) {
        auto one_group = [&](int g) {
            const float2 x = *reinterpret_cast<const float2 *>(
                row + row_pair_slot(g, part, groups));
            const float2 y = qrun[g];
            const float d0 = y.x - x.x, d1 = y.y - x.y;
            a0 = fmaf(d0, d0, a0);
            a1 = fmaf(d1, d1, a1);
        };
        int g = first;
        // the query is read 16 bytes at a time: the run must start 16-byte
        // aligned, which it does when the number of groups is even
        if ((groups & 1) == 0) {
            if (g & 1) one_group(g++);
            constexpr int kChunk = PA_LONG_CHUNK;  // blocks per batch of loads
            const float4 *r4 = reinterpret_cast<const float4 *>(row) + part;
            const float4 *q4 = reinterpret_cast<const float4 *>(qrun);
            for (; g + 2 * kChunk <= groups; g += 2 * kChunk) {
                float4 x[kChunk];
#pragma unroll
                for (int u = 0; u < kChunk; ++u) x[u] = r4[4 * ((g >> 1) + u)];
                __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                for (int u = 0; u < kChunk; ++u) {
                    const float4 y = q4[(g >> 1) + u];
                    const float d0 = y.x - x[u].x, d1 = y.y - x[u].y;
                    a0 = fmaf(d0, d0, a0);
                    a1 = fmaf(d1, d1, a1);
                    const float d2 = y.z - x[u].z, d3 = y.w - x[u].w;
                    a0 = fmaf(d2, d2, a0);
                    a1 = fmaf(d3, d3, a1);
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
        for (; g < groups; ++g) one_group(g);
    }
    return quad_reduce(a0, a1);
}

// The whole row, for the traversal's reduced rows (same interleaved layout):
// with a length known at compile time (DP8 groups, even) all loads of the row
// are in flight at once, DP8 / 2 of 16 bytes per lane.
template <int DP8>
__device__ __forceinline__ float quad_square_dist_rows(const float *row,
                                                       const float2 *qrun,
                                                       int groups, int part,
                                                       bool active) {
    if (DP8 > 0 && DP8 % 2 == 0) {
        float a0 = 0.f, a1 = 0.f;
        if (active) {
            constexpr int kBlocks = DP8 > 0 ? DP8 / 2 : 1;
            const float4 *r4 = reinterpret_cast<const float4 *>(row) + part;
            float4 x[kBlocks];
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) x[b] = r4[4 * b];
            __builtin_amdgcn_sched_barrier(0);
            const float4 *q4 = reinterpret_cast<const float4 *>(qrun);
#pragma unroll
            for (int b = 0; b < kBlocks; ++b) {
                const float4 y = q4[b];
                const float d0 = y.x - x[b].x, d1 = y.y - x[b].y;
                a0 = fmaf(d0, d0, a0);
                a1 = fmaf(d1, d1, a1);
                const float d2 = y.z - x[b].z, d3 = y.w - x[b].w;
                a0 = fmaf(d2, d2, a0);
                a1 = fmaf(d3, d3, a1);
                if ((b & 1) == 1) __builtin_amdgcn_sched_barrier(0);
            }
            __builtin_amdgcn_sched_barrier(0);
        }
        return quad_reduce(a0, a1);
    }
    return quad_square_dist_long(row, qrun, groups, 0, part, active);
}

}  // namespace pa

#endif
