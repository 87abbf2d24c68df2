// Subgraph traversal for gfx950: graph preparation and the per-query search.
//
// One wavefront (64 lanes, one workgroup) runs one query and reproduces, step
// for step, what the reference's host search does for that query
// (extension/traverse_cpu.cpp:12-163):
//   * the open list is the same array heap, with the same sift rules
//     (extension/inc/heapq.cuh:13-88), kept in LDS and advanced by the whole
//     wavefront in lock step (uniform control flow, lane 0 stores);
//   * the result list is the exact set of the H best distances seen so far —
//     what the reference's result heap holds — spread over registers,
//     ceil(H/64) entries per lane;
//   * the visited set is exact: one bit per storage row in a per-wavefront
//     slice of a pooled HBM bitmask, tested and set with one atomic OR per
//     neighbour;
//   * a distance is the reference's eight-accumulator FMA sum
//     (extension/inc/distance.h:31-55) bit for bit: two lanes share a row,
//     the even lane owns accumulators 0..3 and the odd lane 4..7, each lane
//     streams its half of every 8-float group with 16-byte loads.
// Expansion of a node therefore costs one coalesced row of neighbour ids, one
// atomic per neighbour and one coalesced 4*dp-byte row per unvisited
// neighbour, 32 rows in flight per pass.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "device_common.h"
#include "pilotann.h"

using namespace pa;

namespace {

constexpr int kSlotAlignWords = 256;   // bitmask slice: multiple of 1 KiB
constexpr int kWorkCounterBytes = 256; // head of the workspace

// ---- open list: heapq.cuh on LDS -------------------------------------------

__device__ __forceinline__ void open_put(float *key, int *val, int at, float k,
                                         int v, int lane) {
    if (lane == 0) {
        key[at] = k;
        val[at] = v;
    }
}

// heapq.cuh:37-45 with the sift of :13-29: the root leaves, (inf, -1) sinks
// along the smaller child (left on ties) until it is not larger than it.
__device__ __forceinline__ void open_pop(float *key, int *val, int size,
                                         int lane, float &out_k, int &out_v) {
    out_k = uni(key[0]);
    out_v = uni(val[0]);
    int at = 0;
    for (;;) {
        int c = 2 * at + 1;
        if (c >= size) break;
        float ck = uni(key[c]);
        int cv = uni(val[c]);
        if (c + 1 < size) {
            float rk = uni(key[c + 1]);
            int rv = uni(val[c + 1]);
            if (rk < ck) ck = rk, cv = rv, c += 1;
        }
        if (INFINITY <= ck) break;
        open_put(key, val, at, ck, cv, lane);
        at = c;
    }
    open_put(key, val, at, INFINITY, -1, lane);
    wave_sync();
}

// heapq.cuh:47-77: walk to a leaf through the larger child (left on ties),
// overwrite it when the new key is strictly smaller, let the new entry rise.
__device__ __forceinline__ void open_replace(float *key, int *val, int size,
                                             float k, int v, int lane) {
    int at = 0;
    float leaf = uni(key[0]);
    for (;;) {
        int c = 2 * at + 1;
        if (c >= size) break;
        float ck = uni(key[c]);
        if (c + 1 < size) {
            float rk = uni(key[c + 1]);
            if (rk > ck) ck = rk, c += 1;
        }
        at = c;
        leaf = ck;
    }
    if (k >= leaf) return;
    while (at > 0) {
        int up = (at - 1) >> 1;
        float pk = uni(key[up]);
        if (pk <= k) break;
        int pv = uni(val[up]);
        open_put(key, val, at, pk, pv, lane);
        at = up;
    }
    open_put(key, val, at, k, v, lane);
    wave_sync();
}

// ---- result list: the H smallest distances, S entries per lane --------------
//
// The reference keeps them in a heap of negated keys whose root is the worst
// kept (traverse_cpu.cpp:21-39): a candidate enters iff its distance is
// strictly below that root, and replaces it.  Which array cell holds what has
// no effect on the search; only the set and its maximum do.  Empty cells hold
// +inf (so the maximum is +inf until H candidates came), cells beyond H hold
// -inf and never win.

template <int S>
struct Results {
    float key[S];
    int val[S];
    float lane_max;
    float worst;  // uniform

    __device__ __forceinline__ void init(int H, int lane) {
        lane_max = -INFINITY;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            key[s] = (s * kWave + lane < H) ? INFINITY : -INFINITY;
            val[s] = -1;
            lane_max = fmaxf(lane_max, key[s]);
        }
        worst = INFINITY;
    }
    // Caller has checked !(d >= worst).
    __device__ __forceinline__ void insert(float d, int v, int lane) {
        unsigned long long holders = __ballot(lane_max == worst);
        int owner = __builtin_ctzll(holders);
        if (lane == owner) {
            bool done = false;
            float m = -INFINITY;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (!done && key[s] == worst) {
                    key[s] = d;
                    val[s] = v;
                    done = true;
                }
                m = fmaxf(m, key[s]);
            }
            lane_max = m;
        }
        worst = wave_max(lane_max);
    }
};

// ---- distances ---------------------------------------------------------------

// Squared L2 from the query (LDS) to the storage rows listed in cand_id[0..n),
// written to cand_key.  Lane 2p and 2p+1 share row p of each group of 32.
template <int DP8>
__device__ __forceinline__ void eval_rows(const float *__restrict__ storage,
                                          const float *qv, const int *cand_id,
                                          float *cand_key, int n, int dp,
                                          int lane) {
    const int pair = lane >> 1, half = lane & 1;
    const float4 *qq = reinterpret_cast<const float4 *>(qv) + half;
    for (int base = 0; base < n; base += 32) {
        const int c = base + pair;
        const bool active = c < n;
        const float4 *row = reinterpret_cast<const float4 *>(storage);
        if (active)
            row = reinterpret_cast<const float4 *>(
                      storage + (size_t)cand_id[c] * (size_t)dp) + half;
        const float s = pair_square_dist<DP8>(row, qq, dp >> 3, active);
        if (active && half == 0) cand_key[c] = s;
    }
}

// ---- the search ---------------------------------------------------------------

struct TraverseArgs {
    int64_t *out_I;
    float *out_D;
    const int32_t *adj;
    const int32_t *gid;
    const int64_t *mapping;
    const float *storage;
    const float *query;
    const int64_t *init_I;
    const float *init_D;
    uint32_t *seen;
    int *work_counter;
    unsigned long long *counters;
    int batch, n_nodes, n_storage, dp, n_init, k, H, deg, max_iter;
    int words_per_slot, sort_n;
};

__global__ void reset_work_counter(int *counter) { *counter = 0; }

template <int S, int DP8>
__global__ __launch_bounds__(kWave) void traverse_kernel(TraverseArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int lane = threadIdx.x;
    const int H = a.H, O = 2 * a.H;
    const int heap_cells = O > a.sort_n ? O : a.sort_n;
    float *okey = reinterpret_cast<float *>(smem);
    int *oval = reinterpret_cast<int *>(okey + heap_cells);
    int *cand_id = oval + heap_cells;
    float *cand_key = reinterpret_cast<float *>(cand_id + kWave);
    float *qv = cand_key + kWave;
    const int dp = DP8 ? DP8 * 8 : a.dp;
    const int deg = a.deg;
    uint32_t *seen = a.seen + (size_t)blockIdx.x * (size_t)a.words_per_slot;

    for (;;) {
        int q = 0;
        if (lane == 0) q = atomicAdd(a.work_counter, 1);
        q = uni(q);
        if (q >= a.batch) break;

        unsigned long long n_expand = 0, n_adj = 0, n_dist = 0, n_admit = 0;

        // fresh visited slice, query to LDS, empty lists
        for (int w = lane * 4; w < a.words_per_slot; w += kWave * 4)
            *reinterpret_cast<uint4 *>(seen + w) = make_uint4(0, 0, 0, 0);
        for (int i = lane; i < dp; i += kWave)
            qv[i] = a.query[(size_t)q * dp + i];
        for (int i = lane; i < O; i += kWave) okey[i] = INFINITY, oval[i] = -1;
        Results<S> res;
        res.init(H, lane);
        __threadfence();
        wave_sync();

        // traverse_cpu.cpp:69-79: entries are marked and pushed on the open
        // list, in order.  An entry without a storage row has no adjacency
        // here; it is kept under the code -2-i (i = its position) so that it
        // is popped, and costs a step, like any other.
        const int64_t *eI = a.init_I + (size_t)q * a.n_init;
        const float *eD = a.init_D + (size_t)q * a.n_init;
        for (int base = 0; base < a.n_init; base += kWave) {
            const int i = base + lane;
            int u = -1, row = -1;
            float d = INFINITY;
            if (i < a.n_init) {
                const int64_t g = eI[i];
                d = eD[i];
                if (g >= 0 && g < a.n_nodes) {
                    u = (int)g;
                    row = (int)a.mapping[g];
                    if (row >= 0)
                        atomicOr(&seen[row >> 5], 1u << (row & 31));
                }
            }
            const int cnt = min(kWave, a.n_init - base);
            for (int j = 0; j < cnt; ++j) {
                const int uj = __builtin_amdgcn_readlane(u, j);
                if (uj < 0) continue;
                const int rj = __builtin_amdgcn_readlane(row, j);
                const float dj =
                    __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d), j));
                open_replace(okey, oval, O, dj, rj >= 0 ? rj : -2 - (base + j),
                             lane);
            }
        }

        // traverse_cpu.cpp:82-136
        for (int step = 0; step < a.max_iter; ++step) {
            float uk;
            int u;
            open_pop(okey, oval, O, lane, uk, u);
            if (u == -1 || uk >= res.worst) break;
            n_expand += 1;
            if (u < 0) continue;

            int v = -1;
            if (lane < deg) v = a.adj[(size_t)u * deg + lane];
            n_adj += deg;
            bool fresh = false;
            if (v >= 0) {
                const uint32_t bit = 1u << (v & 31);
                fresh = !(atomicOr(&seen[v >> 5], bit) & bit);
            }
            const unsigned long long mask = __ballot(fresh);
            const int n = __popcll(mask);
            if (n == 0) continue;
            if (fresh) cand_id[lane_rank(mask)] = v;
            wave_sync();
            eval_rows<DP8>(a.storage, qv, cand_id, cand_key, n, dp, lane);
            n_dist += n;
            wave_sync();

            // heap_update, traverse_cpu.cpp:25-39, in adjacency order
            const float d = lane < n ? cand_key[lane] : INFINITY;
            const int id = lane < n ? cand_id[lane] : -1;
            unsigned long long todo = __ballot(!(d >= res.worst));
            while (todo) {
                const int j = __builtin_ctzll(todo);
                todo &= todo - 1;
                const float dj =
                    __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d), j));
                if (dj >= res.worst) continue;
                const int vj = __builtin_amdgcn_readlane(id, j);
                res.insert(dj, vj, lane);
                open_replace(okey, oval, O, dj, vj, lane);
                n_admit += 1;
            }
        }

        // traverse_cpu.cpp:138-148: storage rows -> global ids, then the
        // entries compete for a result slot.
#pragma unroll
        for (int s = 0; s < S; ++s)
            if (res.val[s] >= 0) res.val[s] = a.gid[res.val[s]];
        for (int base = 0; base < a.n_init; base += kWave) {
            const int i = base + lane;
            int u = -1;
            float d = INFINITY;
            if (i < a.n_init) {
                const int64_t g = eI[i];
                d = eD[i];
                if (g >= 0 && g < a.n_nodes) u = (int)g;
            }
            unsigned long long todo = __ballot(u >= 0 && !(d >= res.worst));
            while (todo) {
                const int j = __builtin_ctzll(todo);
                todo &= todo - 1;
                const float dj =
                    __int_as_float(__builtin_amdgcn_readlane(__float_as_int(d), j));
                if (dj >= res.worst) continue;
                res.insert(dj, __builtin_amdgcn_readlane(u, j), lane);
            }
        }

        // traverse_cpu.cpp:150-162: best first.  Sort the H cells (padded to
        // a power of two with +inf) in the LDS the open list no longer needs.
        wave_sync();
        for (int i = lane; i < a.sort_n; i += kWave)
            okey[i] = INFINITY, oval[i] = -1;
        wave_sync();
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int e = s * kWave + lane;
            if (e < H) okey[e] = res.key[s], oval[e] = res.val[s];
        }
        wave_sync();
        for (int size = 2; size <= a.sort_n; size <<= 1) {
            for (int stride = size >> 1; stride > 0; stride >>= 1) {
                for (int t = lane; t < (a.sort_n >> 1); t += kWave) {
                    const int i = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
                    const int j = i | stride;
                    const float ki = okey[i], kj = okey[j];
                    const int vi = oval[i], vj = oval[j];
                    const bool gt = ki > kj || (ki == kj && vi > vj);
                    const bool lt = ki < kj || (ki == kj && vi < vj);
                    if ((i & size) == 0 ? gt : lt) {
                        okey[i] = kj, oval[i] = vj;
                        okey[j] = ki, oval[j] = vi;
                    }
                }
                wave_sync();
            }
        }
        int64_t *oI = a.out_I + (size_t)q * a.k;
        float *oD = a.out_D + (size_t)q * a.k;
        for (int i = lane; i < a.k; i += kWave) {
            oI[i] = (int64_t)oval[i];
            oD[i] = okey[i];
        }
        wave_sync();

        if (a.counters && lane == 0) {
            atomicAdd(&a.counters[0], n_expand);
            atomicAdd(&a.counters[1], n_adj);
            atomicAdd(&a.counters[2], n_dist);
            atomicAdd(&a.counters[3], n_admit);
            atomicAdd(&a.counters[4], (unsigned long long)a.k);
        }
    }
}

// ---- graph preparation ----------------------------------------------------------

__global__ void fill_i32(int32_t *p, int64_t n, int32_t value) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = value;
}

__global__ void invert_mapping(const int64_t *mapping, int64_t n_nodes,
                               int64_t n_storage, int32_t *gid,
                               int32_t *status) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_nodes) return;
    const int64_t row = mapping[g];
    if (row < 0) return;
    if (row >= n_storage) {
        atomicOr(status, 1);
        return;
    }
    if (atomicExch(&gid[row], (int32_t)g) != -1) atomicOr(status, 1);
}

// One wavefront per storage row; lane i looks at entry i of the node's row.
__global__ __launch_bounds__(256) void build_rows(
    const int64_t *indptr, const int64_t *indices, const int64_t *mapping,
    int64_t n_nodes, int64_t n_storage, int deg, const int32_t *gid,
    int32_t *adj, int32_t *status) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t r = (int64_t)blockIdx.x * (blockDim.x / kWave) +
                      (threadIdx.x / kWave);
    if (r >= n_storage) return;
    const int g = gid[r];
    int keep_row = -1;
    int n_valid = 0;
    if (g < 0) {
        if (lane == 0) atomicOr(status, 1);
    } else {
        const int64_t lo = indptr[g];
        int64_t len = indptr[g + 1] - lo;
        if (len > deg) {
            if (lane == 0) atomicOr(status, 2);
            len = deg;
        }
        if (len < 0) len = 0;
        int64_t e = -1;
        if (lane < len) e = indices[lo + lane];
        const unsigned long long neg = __ballot(lane < len && e < 0);
        n_valid = neg ? __builtin_ctzll(neg) : (int)len;
        bool ok = lane < n_valid;
        if (ok && e >= n_nodes) {
            atomicOr(status, 4);
            ok = false;
        }
        int row = ok ? (int)mapping[e] : -1;
        if (row >= n_storage) row = -1;
        if (row == r) row = -1;
        // an entry equal to an earlier one of the row is dropped
        for (int j = 0; j < n_valid; ++j) {
            const int other = __builtin_amdgcn_readlane(row, j);
            if (j < lane && other == row) row = -1;
        }
        keep_row = row;
    }
    const unsigned long long kept = __ballot(keep_row >= 0);
    const int n_kept = __popcll(kept);
    int32_t *out = adj + r * deg;
    if (keep_row >= 0) out[lane_rank(kept)] = keep_row;
    if (lane >= n_kept && lane < deg) out[lane] = -1;
}

// ---- host side --------------------------------------------------------------------

int round_up(int64_t x, int64_t m) { return (int)(((x + m - 1) / m) * m); }

int next_pow2(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

typedef void (*TraverseFn)(TraverseArgs);

template <int S>
TraverseFn pick_dp(int dp) {
    switch (dp) {
        case 32: return traverse_kernel<S, 4>;
        case 64: return traverse_kernel<S, 8>;
        case 128: return traverse_kernel<S, 16>;
        default: return traverse_kernel<S, 0>;
    }
}

TraverseFn pick_kernel(int H, int dp) {
    const int S = (H + kWave - 1) / kWave;
    switch (S) {
        case 1: return pick_dp<1>(dp);
        case 2: return pick_dp<2>(dp);
        case 3: return pick_dp<3>(dp);
        case 4: return pick_dp<4>(dp);
        case 6: return pick_dp<6>(dp);
        case 8: return pick_dp<8>(dp);
        case 16: return pick_dp<16>(dp);
        case 32: return pick_dp<32>(dp);
        default: return nullptr;
    }
}

struct Plan {
    int H, sort_n, lds_bytes, n_slots, words_per_slot;
    size_t workspace_bytes;
    TraverseFn fn;
};

int make_plan(int64_t n_storage, int64_t batch, int dp, int ef_total, Plan *p) {
    if (n_storage <= 0 || batch < 0) return PA_E_SHAPE;
    if (n_storage >= (1ll << 31)) return PA_E_RANGE;
    if (dp <= 0 || dp % 8) return PA_E_DIM;
    if (ef_total < 1 || ef_total > PA_MAX_EF_TOTAL) return PA_E_EF;
    p->H = pa_heap_size(ef_total);
    p->sort_n = next_pow2(p->H < kWave ? kWave : p->H);
    const int cells = 2 * p->H > p->sort_n ? 2 * p->H : p->sort_n;
    p->lds_bytes = cells * 8 + kWave * 8 + dp * 4;
    p->fn = pick_kernel(p->H, dp);
    if (!p->fn) return PA_E_EF;
    int dev = 0, cus = 0, per_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e == hipSuccess)
        e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    if (e == hipSuccess)
        e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
            &per_cu, reinterpret_cast<const void *>(p->fn), kWave, p->lds_bytes);
    if (e != hipSuccess) return (int)e;
    if (per_cu < 1) per_cu = 1;
    int64_t slots = (int64_t)per_cu * cus;
    if (slots > batch) slots = batch;
    if (slots < 1) slots = 1;
    p->n_slots = (int)slots;
    p->words_per_slot = round_up((n_storage + 31) / 32, kSlotAlignWords);
    p->workspace_bytes =
        kWorkCounterBytes + (size_t)p->n_slots * p->words_per_slot * 4;
    return PA_OK;
}

}  // namespace

extern "C" int pa_heap_size(int ef_search) {
    static const int ladder[] = {16,  32,  48,  64,  96,   128,
                                 192, 256, 384, 512, 1024, 2048};
    for (int h : ladder)
        if (ef_search <= h) return h;
    return -1;
}

extern "C" const char *pa_error_string(int code) {
    if (code > 0) return hipGetErrorString((hipError_t)code);
    switch (code) {
        case PA_OK: return "ok";
        case PA_E_NULL: return "a required pointer is null";
        case PA_E_SHAPE: return "a size is negative or inconsistent";
        case PA_E_DIM: return "vector length must be a multiple of 8";
        case PA_E_NEIGHBORS: return "n_neighbors must be in 1..64";
        case PA_E_EF: return "beam * ef must be in 1..2048";
        case PA_E_WORKSPACE: return "workspace too small";
        case PA_E_GRAPH: return "malformed graph (see status word)";
        case PA_E_LEAVES: return "n_leaves must be a multiple of 32";
        case PA_E_CHUNK: return "batch must be a multiple of chunk_size";
        case PA_E_RANGE: return "an id does not fit 31 bits";
        default: return "unknown error";
    }
}

extern "C" int pa_graph_prepare(const int64_t *indptr, const int64_t *indices,
                                const int64_t *mapping, int64_t n_nodes,
                                int64_t n_storage, int n_neighbors,
                                int32_t *adj, int32_t *gid, int32_t *status,
                                void *stream_) {
    if (!indptr || !indices || !mapping || !adj || !gid || !status)
        return PA_E_NULL;
    if (n_nodes <= 0 || n_storage <= 0 || n_storage > n_nodes) return PA_E_SHAPE;
    if (n_nodes >= (1ll << 31)) return PA_E_RANGE;
    if (n_neighbors < 1 || n_neighbors > PA_MAX_NEIGHBORS) return PA_E_NEIGHBORS;
    hipStream_t stream = (hipStream_t)stream_;
    const int T = 256;
    fill_i32<<<1, 1, 0, stream>>>(status, 1, 0);
    fill_i32<<<(unsigned)((n_storage + T - 1) / T), T, 0, stream>>>(gid, n_storage, -1);
    invert_mapping<<<(unsigned)((n_nodes + T - 1) / T), T, 0, stream>>>(
        mapping, n_nodes, n_storage, gid, status);
    const int rows_per_block = T / kWave;
    build_rows<<<(unsigned)((n_storage + rows_per_block - 1) / rows_per_block), T,
                 0, stream>>>(indptr, indices, mapping, n_nodes, n_storage,
                              n_neighbors, gid, adj, status);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return (int)e;
    int32_t host_status = 0;
    e = hipMemcpyAsync(&host_status, status, sizeof(int32_t),
                       hipMemcpyDeviceToHost, stream);
    if (e == hipSuccess) e = hipStreamSynchronize(stream);
    if (e != hipSuccess) return (int)e;
    return host_status ? PA_E_GRAPH : PA_OK;
}

extern "C" int pa_traverse_plan(int64_t n_storage, int64_t batch, int dp,
                                int ef_total, int *n_slots,
                                size_t *workspace_bytes) {
    Plan p;
    const int rc = make_plan(n_storage, batch, dp, ef_total, &p);
    if (rc != PA_OK) return rc;
    if (n_slots) *n_slots = p.n_slots;
    if (workspace_bytes) *workspace_bytes = p.workspace_bytes;
    return PA_OK;
}

extern "C" int pa_traverse(int64_t *out_I, float *out_D, const int32_t *adj,
                           const int32_t *gid, const int64_t *mapping,
                           const float *storage, const float *query,
                           const int64_t *init_I, const float *init_D,
                           int64_t batch, int64_t n_nodes, int64_t n_storage,
                           int dp, int n_init, int beam, int ef,
                           int n_neighbors, void *workspace,
                           size_t workspace_bytes, uint64_t *counters,
                           void *stream_) {
    if (batch < 0 || n_nodes <= 0 || n_init < 0 || beam < 1 || ef < 1)
        return PA_E_SHAPE;
    if (n_nodes >= (1ll << 31)) return PA_E_RANGE;
    if (n_neighbors < 1 || n_neighbors > PA_MAX_NEIGHBORS) return PA_E_NEIGHBORS;
    if ((int64_t)beam * ef > PA_MAX_EF_TOTAL) return PA_E_EF;
    Plan p;
    const int rc = make_plan(n_storage, batch, dp, beam * ef, &p);
    if (rc != PA_OK) return rc;
    if (batch == 0) return PA_OK;
    if (!out_I || !out_D || !adj || !gid || !mapping || !storage || !query ||
        !workspace || (n_init > 0 && (!init_I || !init_D)))
        return PA_E_NULL;
    if (workspace_bytes < p.workspace_bytes) return PA_E_WORKSPACE;

    TraverseArgs a;
    a.out_I = out_I, a.out_D = out_D;
    a.adj = adj, a.gid = gid, a.mapping = mapping;
    a.storage = storage, a.query = query;
    a.init_I = init_I, a.init_D = init_D;
    a.work_counter = reinterpret_cast<int *>(workspace);
    a.seen = reinterpret_cast<uint32_t *>(
        reinterpret_cast<unsigned char *>(workspace) + kWorkCounterBytes);
    a.counters = reinterpret_cast<unsigned long long *>(counters);
    a.batch = (int)batch, a.n_nodes = (int)n_nodes, a.n_storage = (int)n_storage;
    a.dp = dp, a.n_init = n_init, a.k = beam * ef, a.H = p.H;
    a.deg = n_neighbors;
    // traverse_cpu.cpp:18,82
    a.max_iter = 2 * beam * ef < 1024 ? 2 * beam * ef : 1024;
    a.words_per_slot = p.words_per_slot, a.sort_n = p.sort_n;

    hipStream_t stream = (hipStream_t)stream_;
    reset_work_counter<<<1, 1, 0, stream>>>(a.work_counter);
    p.fn<<<p.n_slots, kWave, p.lds_bytes, stream>>>(a);
    return (int)hipGetLastError();
}
