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


// Squared L2 between a query held in LDS and one storage row, in the order of
// the reference's host code (extension/inc/distance.h:31-55): element j of
// every group of eight goes to accumulator j with one FMA, the eight
// accumulators are then added left to right.  Two adjacent lanes share a row:
// the even lane (half 0) owns accumulators 0..3, the odd lane (half 1) 4..7;
// `row` and `qv` already point at the lane's half of the first group.  The
// even lane returns the distance; every lane of the wavefront must call this
// (the exchange between the two lanes is a DPP move), lanes without a row
// pass active = false.
template <int DP8>
__device__ __forceinline__ float pair_square_dist(const float4 *row,
                                                  const float4 *qv, int groups,
                                                  bool active) {
    float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
    if (active) {
        const int n = DP8 ? DP8 : groups;
#pragma unroll 8
        for (int t = 0; t < n; ++t) {
            const float4 x = row[2 * t];
            const float4 y = qv[2 * t];
            const float d0 = y.x - x.x, d1 = y.y - x.y;
            const float d2 = y.z - x.z, d3 = y.w - x.w;
            acc.x = fmaf(d0, d0, acc.x);
            acc.y = fmaf(d1, d1, acc.y);
            acc.z = fmaf(d2, d2, acc.z);
            acc.w = fmaf(d3, d3, acc.w);
        }
    }
    float s = ((acc.x + acc.y) + acc.z) + acc.w;
    const float o0 = dpp_f<0xF5, 0xF>(acc.x);  // quad_perm [1,1,3,3]
    const float o1 = dpp_f<0xF5, 0xF>(acc.y);
    const float o2 = dpp_f<0xF5, 0xF>(acc.z);
    const float o3 = dpp_f<0xF5, 0xF>(acc.w);
    return (((s + o0) + o1) + o2) + o3;
}

}  // namespace pa

#endif
