// Entry router (FES) for gfx950.
//
// The reference picks, per query, the nearest of n_routers route vectors with
// a library cdist + argmin and then computes the squared distances to that
// route's n_leaves entry vectors (extension/routing_cuda.cu:70-113).
//
// Here the route choice is a dense contraction on the matrix cores: a
// wavefront takes 32 queries and scores them against 32 route vectors at a
// time with v_mfma_f32_32x32x2_f32, score(i, r) = |route_r|^2 - 2 q_i.route_r
// (|q_i|^2 is the same for every r), followed by a row-wise argmin.  The leaf
// distances are direct sums of squared differences (routing_cuda.cu:53-61) in
// the same summation order as the traversal's distances, so an entry's
// distance is bit-identical to what the traversal would compute for that row.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "device_common.h"
#include "pilotann.h"

using namespace pa;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kTile = 32;

// One wavefront per 32 queries.  MFMA operands: lane l supplies
// A[i = l % 32][k = l / 32] and B[k = l / 32][j = l % 32]; its 16 results are
// D[i = 8 * (r / 4) + 4 * (l / 32) + r % 4][j = l % 32].  The k index is a
// free relabelling: lanes 0..31 take elements 8c..8c+3 of every group of eight
// and lanes 32..63 elements 8c+4..8c+7, so every lane reads 16 contiguous
// bytes per group and four MFMAs consume them.
__global__ __launch_bounds__(kWave) void route_score_kernel(
    const float *__restrict__ query, const float *__restrict__ routes,
    int64_t *__restrict__ router, int batch, int n_routers, int dp) {
    __shared__ float score[kTile][kTile + 1];
    const int lane = threadIdx.x;
    const int col = lane & 31, half = lane >> 5;
    const int q0 = blockIdx.x * kTile;
    const int qi = q0 + col;
    const bool q_ok = qi < batch;
    const float4 *qrow =
        reinterpret_cast<const float4 *>(query + (size_t)(q_ok ? qi : 0) * dp) + half;
    const int groups = dp >> 3;

    float best = INFINITY;
    int best_r = 0;
    for (int r0 = 0; r0 < n_routers; r0 += kTile) {
        const int rj = r0 + col;
        const bool r_ok = rj < n_routers;
        const float4 *rrow =
            reinterpret_cast<const float4 *>(routes + (size_t)(r_ok ? rj : 0) * dp) + half;
        // two accumulators take alternate instructions: none waits for the
        // result of the one before it
        floatx16 acc, acc_odd;
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] = 0.f, acc_odd[r] = 0.f;
        float norm = 0.f;
        for (int c = 0; c < groups; ++c) {
            float4 a = qrow[2 * c];
            float4 b = rrow[2 * c];
            if (!q_ok) a = make_float4(0.f, 0.f, 0.f, 0.f);
            if (!r_ok) b = make_float4(0.f, 0.f, 0.f, 0.f);
            norm = fmaf(b.x, b.x, norm);
            norm = fmaf(b.y, b.y, norm);
            norm = fmaf(b.z, b.z, norm);
            norm = fmaf(b.w, b.w, norm);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.x, b.x, acc, 0, 0, 0);
            acc_odd = __builtin_amdgcn_mfma_f32_32x32x2f32(a.y, b.y, acc_odd, 0, 0, 0);
            acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.z, b.z, acc, 0, 0, 0);
            acc_odd = __builtin_amdgcn_mfma_f32_32x32x2f32(a.w, b.w, acc_odd, 0, 0, 0);
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) acc[r] += acc_odd[r];
        norm += __shfl_xor(norm, 32);
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int i = 8 * (r >> 2) + 4 * half + (r & 3);
            score[i][col] = r_ok ? fmaf(-2.f, acc[r], norm) : INFINITY;
        }
        __syncthreads();
        // lane (col, half) scans 16 columns of query row `col`
        float m = INFINITY;
        int mi = 0;
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            const float s = score[col][half * 16 + j];
            if (s < m) m = s, mi = r0 + half * 16 + j;
        }
        const float om = __shfl_xor(m, 32);
        const int oi = __shfl_xor(mi, 32);
        if (om < m || (om == m && oi < mi)) m = om, mi = oi;
        if (m < best) best = m, best_r = mi;
        __syncthreads();
    }
    if (half == 0 && q_ok) router[qi] = best_r;
}

// One wavefront per query: squared distances to the n_leaves vectors of the
// query's group, 16 leaves per pass, four lanes per leaf.
template <int DP8>
__global__ __launch_bounds__(256) void leaf_dist_kernel(
    const float *__restrict__ query, const float *__restrict__ entry_vectors,
    const int64_t *__restrict__ router, float *__restrict__ dist,
    const int64_t *__restrict__ entry_nodes, int64_t *__restrict__ entry_ids,
    int batch, int n_leaves, int dp) {
    extern __shared__ __align__(16) float qv_all[];
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    const int q = blockIdx.x * (blockDim.x / kWave) + wave;
    float *qv = qv_all + wave * query_floats(dp);
    if (q < batch)
        for (int i = lane; i < dp; i += kWave)
            qv[query_slot(i, dp >> 3)] = query[(size_t)q * dp + i];
    __syncthreads();
    if (q >= batch) return;
    const int64_t group = router ? router[q] : 0;
    const float *leaves = entry_vectors + (size_t)group * n_leaves * dp;
    // layers/entry.py:86: the ids of the chosen group's leaves
    if (entry_ids)
        for (int l = lane; l < n_leaves; l += kWave)
            entry_ids[(size_t)q * n_leaves + l] =
                entry_nodes[(size_t)group * n_leaves + l];
    const int quad = lane >> 2, part = lane & 3;
    const float2 *qq = reinterpret_cast<const float2 *>(qv) + part * query_run(dp >> 3);
    for (int base = 0; base < n_leaves; base += kRowsPerPass) {
        const int l = base + quad;
        const bool active = l < n_leaves;
        const float2 *row =
            reinterpret_cast<const float2 *>(leaves + (size_t)(active ? l : 0) * dp) + part;
        const float s = quad_square_dist<DP8>(row, qq, dp >> 3, active);
        if (active && part == 0) dist[(size_t)q * n_leaves + l] = s;
    }
}

}  // namespace

extern "C" int pa_route(int64_t *router, float *dist, const float *query,
                        const float *route_vectors, const float *entry_vectors,
                        int64_t batch, int n_routers, int n_leaves, int dp,
                        const int64_t *entry_nodes, int64_t *entry_ids,
                        void *stream_) {
    if (batch < 0 || n_routers < 0 || n_leaves < 1) return PA_E_SHAPE;
    if (batch >= (1ll << 31)) return PA_E_RANGE;
    if (dp <= 0 || dp % 8) return PA_E_DIM;
    if (n_routers > 0 && n_leaves % 32) return PA_E_LEAVES;
    if (batch == 0) return PA_OK;
    if (!dist || !query || !entry_vectors) return PA_E_NULL;
    if (n_routers > 0 && (!router || !route_vectors)) return PA_E_NULL;
    if (entry_ids && !entry_nodes) return PA_E_NULL;
    hipStream_t stream = (hipStream_t)stream_;
    if (n_routers > 0) {
        const unsigned blocks = (unsigned)((batch + kTile - 1) / kTile);
        route_score_kernel<<<blocks, kWave, 0, stream>>>(
            query, route_vectors, router, (int)batch, n_routers, dp);
    }
    const int waves = 4;
    const unsigned blocks = (unsigned)((batch + waves - 1) / waves);
    const size_t lds = (size_t)waves * query_floats(dp) * sizeof(float);
    const int64_t *group = n_routers > 0 ? router : nullptr;
    switch (dp) {
        case 32:
            leaf_dist_kernel<4><<<blocks, waves * kWave, lds, stream>>>(
                query, entry_vectors, group, dist, entry_nodes, entry_ids, (int)batch,
                n_leaves, dp);
            break;
        case 64:
            leaf_dist_kernel<8><<<blocks, waves * kWave, lds, stream>>>(
                query, entry_vectors, group, dist, entry_nodes, entry_ids, (int)batch,
                n_leaves, dp);
            break;
        case 128:
            leaf_dist_kernel<16><<<blocks, waves * kWave, lds, stream>>>(
                query, entry_vectors, group, dist, entry_nodes, entry_ids, (int)batch,
                n_leaves, dp);
            break;
        default:
            leaf_dist_kernel<0><<<blocks, waves * kWave, lds, stream>>>(
                query, entry_vectors, group, dist, entry_nodes, entry_ids, (int)batch,
                n_leaves, dp);
    }
    return (int)hipGetLastError();
}
