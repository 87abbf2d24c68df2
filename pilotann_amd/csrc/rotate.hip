// Query rotation for gfx950: out = query . VT^T, first n_out columns.
//
// The reference rotates a batch of queries onto the index's SVD basis with a
// host matmul and then slices off the first d_principle coordinates for the
// device stage (pilot_ann/layers/staged.py:198-201).  That is a plain dense
// contraction, queries x basis vectors, so it runs on the matrix cores: a
// workgroup of four wavefronts owns a 64 x 64 tile of the output, each
// wavefront a 32 x 32 quarter of it, accumulated over the whole row length
// with v_mfma_f32_32x32x2_f32 in float32.  Both operands are row major with
// the contraction along the row (out[b][j] = sum_k query[b][k] * VT[j][k]), so
// every lane streams 16 contiguous bytes of one query row and of one basis
// row per group of eight elements, the same operand layout as the router's
// scoring kernel; the four wavefronts of a workgroup read each row twice, the
// second time from cache.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_common.h"
#include "pilotann.h"

using namespace pa;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 32;

// MFMA operands as in route_score_kernel: lane l supplies A[i = l % 32][k] and
// B[k][j = l % 32] with k = l / 32 of the instruction's two; lanes 0..31 take
// elements 8c..8c+3 of every group of eight, lanes 32..63 elements 8c+4..8c+7
// (the contraction index is a free relabelling).  Its 16 results are
// D[i = 8 * (r / 4) + 4 * (l / 32) + r % 4][j = l % 32].  Two accumulators
// take alternate instructions, so that no instruction waits for the result
// of the one before it.
__global__ __launch_bounds__(256) void rotate_kernel(
    const float *__restrict__ query, const float *__restrict__ basis,
    float *__restrict__ out, int batch, int d, int n_out) {
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int col = lane & 31, half = lane >> 5;
    const int q0 = blockIdx.x * 2 * kTile + kTile * (wave & 1);
    const int j0 = blockIdx.y * 2 * kTile + kTile * (wave >> 1);
    if (q0 >= batch || j0 >= n_out) return;
    const int qi = q0 + col, ji = j0 + col;
    const bool q_ok = qi < batch, j_ok = ji < n_out;
    const float4 *a_row =
        reinterpret_cast<const float4 *>(query + (size_t)(q_ok ? qi : 0) * d) + half;
    const float4 *b_row =
        reinterpret_cast<const float4 *>(basis + (size_t)(j_ok ? ji : 0) * d) + half;
    floatx16 acc0, acc1;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc0[r] = 0.f, acc1[r] = 0.f;
    const int groups = d >> 3;
    int c = 0;
    for (; c + 2 <= groups; c += 2) {
        float4 a0 = a_row[2 * c], a1 = a_row[2 * c + 2];
        float4 b0 = b_row[2 * c], b1 = b_row[2 * c + 2];
        if (!q_ok) a0 = a1 = make_float4(0.f, 0.f, 0.f, 0.f);
        if (!j_ok) b0 = b1 = make_float4(0.f, 0.f, 0.f, 0.f);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.x, b0.x, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.y, b0.y, acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.z, b0.z, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a0.w, b0.w, acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.x, b1.x, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.y, b1.y, acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.z, b1.z, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a1.w, b1.w, acc1, 0, 0, 0);
    }
    for (; c < groups; ++c) {
        float4 a = a_row[2 * c], b = b_row[2 * c];
        if (!q_ok) a = make_float4(0.f, 0.f, 0.f, 0.f);
        if (!j_ok) b = make_float4(0.f, 0.f, 0.f, 0.f);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc1, 0, 0, 0);
        acc0 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc1, 0, 0, 0);
    }
    if (!j_ok) return;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
        const int i = q0 + 8 * (r >> 2) + 4 * half + (r & 3);
        if (i < batch) out[(size_t)i * n_out + ji] = acc0[r] + acc1[r];
    }
}

}  // namespace

extern "C" int pa_rotate(float *out, const float *query, const float *basis,
                         int64_t batch, int d, int n_out, void *stream_) {
    if (batch < 0 || n_out < 1 || n_out > d) return PA_E_SHAPE;
    if (batch >= (1ll << 31)) return PA_E_RANGE;
    if (d <= 0 || d % 8) return PA_E_DIM;
    if (batch == 0) return PA_OK;
    if (!out || !query || !basis) return PA_E_NULL;
    const dim3 grid((unsigned)((batch + 2 * kTile - 1) / (2 * kTile)),
                    (unsigned)((n_out + 2 * kTile - 1) / (2 * kTile)));
    rotate_kernel<<<grid, 256, 0, (hipStream_t)stream_>>>(
        query, basis, out, (int)batch, d, n_out);
    return (int)hipGetLastError();
}
