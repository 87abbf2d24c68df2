// Full-dimension refine on the device, for gfx950.
//
// The reference refines the device stage's candidates on the host
// (extension/traverse_cpu.cpp:261-369): per query two searches of
// traverse_cpu_kernel (:12-163) that share one visited set — first on the
// sampled subgraph, two expansions at most, from the candidates, whose
// distances over the first d_principle coordinates are completed to the full
// dimension in place (:42-62); then on the full graph from what the first one
// kept.  Here one wavefront runs both searches of a query, with the lists of
// the subgraph traversal (search_lists.h): the same array heap cell for cell,
// the same exact visited set (one bit per node in the wavefront's slice of a
// pooled bitmask, kept across the two searches), the same eight-accumulator
// distances bit for bit.  Rows are d_model floats; a quad of lanes streams a
// row sixteen 32-byte groups at a time.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include <map>
#include <mutex>
#include <tuple>

#include "device_common.h"
#include "pilotann.h"
#include "search_lists.h"

using namespace pa;

namespace {

struct RefineArgs {
    int64_t *out_I;          // [batch, k]
    float *out_D;
    int64_t *buf_I;          // [batch, n_buffers]
    float *buf_D;
    const int64_t *init_I;   // [batch, n_init]
    float *init_D;           // completed in place
    const int32_t *sub_adj;  // prepared subgraph: rows of sampled-node ranks
    const int32_t *sub_gid;  // rank -> node
    const int64_t *sub_mapping;  // node -> rank or -1
    const int32_t *full_adj; // prepared full graph: rows of nodes
    const float *storage;    // [n_nodes, d]
    const float *query;      // [batch, d]
    uint32_t *seen;
    int *work_counter;
    unsigned long long *counters;
    int batch, n_nodes, d, dp, n_init, n_buffers, k, H;
    int sub_deg, full_deg, sub_iter, full_iter;
    int words_per_slot, slot_stride, sort_n;
};

__global__ void reset_refine_counter(int *counter) { *counter = 0; }

// Optional per-phase cycle tally for tuning builds (-DPA_PHASE_TIMERS): adds
// eight words after the six work counters.
#ifdef PA_PHASE_TIMERS
#define PA_TIMER_BEGIN() unsigned long long t_mark_ = __builtin_readcyclecounter()
#define PA_TIMER(i)                                                  \
    do {                                                             \
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory"); \
        unsigned long long t_now_ = __builtin_readcyclecounter();    \
        phase[i] += t_now_ - t_mark_;                                \
        t_mark_ = t_now_;                                            \
    } while (0)
#else
#define PA_TIMER_BEGIN() do {} while (0)
#define PA_TIMER(i) do {} while (0)
#endif

// Squared L2 over the coordinates [from, d) between the query (LDS) and the
// rows listed in cand_id[0..n), written to cand_key: 16 rows per pass, four
// lanes per row; the accumulators start at zero at `from`
// (extension/inc/distance.h:31-55 called with an offset, traverse_cpu.cpp:56-59).
// Rows are in the interleaved layout of pa_rows_prepare.
__device__ __forceinline__ void eval_rows_from(const float *__restrict__ storage,
                                               const float *qv, const int *cand_id,
                                               float *cand_key, int n, int d,
                                               int from, int lane) {
    const int quad = lane >> 2, part = lane & 3;
    const int groups = d >> 3;
    const float2 *qrun =
        reinterpret_cast<const float2 *>(qv) + part * query_run(groups);
    for (int base = 0; base < n; base += kRowsPerPass) {
        const int c = base + quad;
        const bool active = c < n;
        const float *row = storage;
        if (active) row = storage + (size_t)cand_id[c] * (size_t)d;
        const float s =
            quad_square_dist_long(row, qrun, groups, from >> 3, part, active);
        if (active && part == 0) cand_key[c] = s;
    }
}

// Plain rows -> the interleaved layout (row_pair_slot); one thread per pair.
__global__ void interleave_rows(const float *__restrict__ src,
                                float *__restrict__ dst, int64_t n_pairs,
                                int groups) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n_pairs) return;
    const int per_row = groups * 4;
    const int64_t r = i / per_row;
    const int p = (int)(i - r * per_row);  // pair p of the row: group p / 4, lane p % 4
    const float2 v = reinterpret_cast<const float2 *>(src)[i];
    *reinterpret_cast<float2 *>(dst + r * (int64_t)groups * 8 +
                                row_pair_slot(p >> 2, p & 3, groups)) = v;
}

// The LDS visited table: 512 buckets of 8 nodes, 8 KB.  A query of the
// headline configuration marks about a thousand nodes: next to no bucket fills
// up, so most queries never touch the bitmask.  Measured per 10 000 queries:
// 1024 x 4 5.76 ms, 2048 x 4 5.77 ms, 1024 x 8 5.52 ms, 512 x 8 5.36 ms.
#ifndef PA_REFINE_SEEN_LOG2
#define PA_REFINE_SEEN_LOG2 9
#endif
#ifndef PA_REFINE_SEEN_WAYS
#define PA_REFINE_SEEN_WAYS 8
#endif
typedef Visited<PA_REFINE_SEEN_LOG2, PA_REFINE_SEEN_WAYS> RefineVisited;

#define PA_REFINE_OCCUPANCY(H) \
    __attribute__((amdgpu_waves_per_eu((H) <= 256 ? 4 : (H) <= 384 ? 3 : (H) <= 1024 ? 2 : 1, 8)))

template <int H>
__global__ __launch_bounds__(kWave) PA_REFINE_OCCUPANCY(H) void refine_kernel(RefineArgs a) {
    constexpr int S = (H + kWave - 1) / kWave;
    constexpr int kSortN = H <= kWave ? kWave : 1 << (floor_log2(H - 1) + 1);
    constexpr int kHeapCells =
        OpenList<H>::kLdsCells > kSortN ? OpenList<H>::kLdsCells : kSortN;
    struct Lds {
        uint32_t seen_table[RefineVisited::kWords];
        int cand_id[kWave];
        float cand_key[kWave];
        int2 heap[kHeapCells];   // open list tail; the sorts reuse it
        int res_key[Results<S>::kLdsKeys];  // result list: keys, unless in registers
                                            // (values: the slot's memory)
    };
    __shared__ __align__(16) Lds lds;
    extern __shared__ __align__(16) float qv[];  // the query, query_slot layout
    const int lane = threadIdx.x;
    float *okey = reinterpret_cast<float *>(lds.heap);
    int *oval = reinterpret_cast<int *>(okey + kHeapCells);
    OpenList<H> open;
    open.cells = lds.heap;
    open.deep = nullptr;  // the whole list in registers and LDS
    int *cand_id = lds.cand_id;
    float *cand_key = lds.cand_key;
    const int d = a.d;
    uint32_t *seen = a.seen + (size_t)blockIdx.x * (size_t)a.slot_stride;
    RefineVisited visited;
    visited.init(lds.seen_table, seen, a.n_nodes);
    // the wavefront's slice of the bitmask starts at zero and is put back to
    // zero after every query that used it
    visited.dirty = true;
    visited.clean(a.words_per_slot, lane);

    for (;;) {
        int q = 0;
        if (lane == 0) q = atomicAdd(a.work_counter, 1);
        q = uni(q);
        if (q >= a.batch) break;

        unsigned n_expand0 = 0, n_expand1 = 0, n_dist = 0, n_admit = 0, n_tail = 0, n_adj = 0;
#ifdef PA_PHASE_TIMERS
        unsigned long long phase[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#endif
        PA_TIMER_BEGIN();

        // empty visited set (it serves both searches), query to LDS
        visited.reset(lane);
        for (int i = lane; i < d; i += kWave)
            qv[query_slot(i, d >> 3)] = a.query[(size_t)q * d + i];
        wave_sync();

        // stage 0: subgraph from the candidates (traverse_cpu.cpp:317-326);
        // stage 1: full graph from the buffer (:327-336)
        for (int stage = 0; stage < 2; ++stage) {
            const int64_t *eI = stage == 0 ? a.init_I + (size_t)q * a.n_init
                                           : a.buf_I + (size_t)q * a.n_buffers;
            float *eD = stage == 0 ? a.init_D + (size_t)q * a.n_init
                                   : a.buf_D + (size_t)q * a.n_buffers;
            const int n_ent = stage == 0 ? a.n_init : a.n_buffers;
            const int tail_from = stage == 0 ? a.dp : d;  // == d: nothing to add
            const int deg = stage == 0 ? a.sub_deg : a.full_deg;
            const int max_iter = stage == 0 ? a.sub_iter : a.full_iter;
            int64_t *oI = stage == 0 ? a.buf_I + (size_t)q * a.n_buffers
                                     : a.out_I + (size_t)q * a.k;
            float *oD = stage == 0 ? a.buf_D + (size_t)q * a.n_buffers
                                   : a.out_D + (size_t)q * a.k;
            const int n_out = stage == 0 ? a.n_buffers : a.k;

            PA_TIMER(0);
            open.reset(lane);
            Results<S> res;
            res.rk = lds.res_key;
            res.rv = reinterpret_cast<int *>(seen + a.words_per_slot);
            res.init(H, lane);
            wave_sync();

            // traverse_cpu.cpp:42-79: complete the entries' distances, mark
            // the entries, push them on the open list in order
            for (int base = 0; base < n_ent; base += kWave) {
                const int i = base + lane;
                int u = -1;
                float dist = INFINITY;
                if (i < n_ent) {
                    const int64_t g = eI[i];
                    dist = eD[i];
                    if (g >= 0 && g < a.n_nodes) u = (int)g;
                }
                if (tail_from < d) {
                    const unsigned long long mask = __ballot(u >= 0);
                    const int n = __popcll(mask);
                    const int rank = lane_rank(mask);
                    if (u >= 0) cand_id[rank] = u;
                    wave_sync();
                    eval_rows_from(a.storage, qv, cand_id, cand_key, n, d,
                                   tail_from, lane);
                    n_tail += n;
                    wave_sync();
                    PA_TIMER(1);
                    if (u >= 0) {
                        dist += cand_key[rank];
                        eD[i] = dist;
                    }
                    wave_sync();
                }
                if (u >= 0) visited.mark(u);
                const int cnt = min(kWave, n_ent - base);
                for (int j = 0; j < cnt; ++j) {
                    const int uj = __builtin_amdgcn_readlane(u, j);
                    if (uj < 0) continue;
                    const float dj = __int_as_float(
                        __builtin_amdgcn_readlane(__float_as_int(dist), j));
                    open.template replace<true>(float_to_key(dj), uj, lane);
                }
                PA_TIMER(2);
            }

            // traverse_cpu.cpp:82-136
            for (int step = 0; step < max_iter; ++step) {
                int uk, u;
                open.pop(lane, uk, u);
                PA_TIMER(3);
                if (u < 0 || uk >= res.worst) break;
                n_expand0 += stage == 0, n_expand1 += stage != 0;
                int v = -1;
                if (stage == 0) {
                    const int64_t r = a.sub_mapping[u];
                    if (r >= 0 && lane < deg) {
                        const int w = a.sub_adj[(size_t)r * deg + lane];
                        if (w >= 0) v = a.sub_gid[w];
                    }
                } else if (lane < deg) {
                    v = a.full_adj[(size_t)u * deg + lane];
                }
                n_adj += deg;
                const bool fresh = v >= 0 && visited.mark(v);
                const unsigned long long mask = __ballot(fresh);
                const int n = __popcll(mask);
                PA_TIMER(4);
                if (n == 0) continue;
                if (fresh) cand_id[lane_rank(mask)] = v;
                wave_sync();
                eval_rows_from(a.storage, qv, cand_id, cand_key, n, d, 0, lane);
                n_dist += n;
                wave_sync();
                PA_TIMER(5);
                const int dk = float_to_key(lane < n ? cand_key[lane] : INFINITY);
                const int id = lane < n ? cand_id[lane] : -1;
                wave_sync();
                // heap_update, traverse_cpu.cpp:25-39, in adjacency order
                unsigned long long todo = __ballot(dk < res.worst);
                while (todo) {
                    const int j = __builtin_ctzll(todo);
                    todo &= todo - 1;
                    const int dj = __builtin_amdgcn_readlane(dk, j);
                    if (dj >= res.worst) continue;
                    const int vj = __builtin_amdgcn_readlane(id, j);
                    int mine[S];
                    res.begin_insert(dj, vj, lane, mine);
                    const typename OpenList<H>::Leaf leaf = open.walk_to_large_leaf();
                    res.finish_insert(lane, mine);
                    open.replace_leaf(leaf, dj, vj, lane);
                    n_admit += 1;
                }
                PA_TIMER(6);
            }

            // traverse_cpu.cpp:138-148: now the entries compete for a slot
            wave_sync();
            for (int base = 0; base < n_ent; base += kWave) {
                const int i = base + lane;
                int u = -1;
                float dist = INFINITY;
                if (i < n_ent) {
                    const int64_t g = eI[i];
                    dist = eD[i];
                    if (g >= 0 && g < a.n_nodes) u = (int)g;
                }
                const int dk = float_to_key(dist);
                unsigned long long todo = __ballot(u >= 0 && dk < res.worst);
                while (todo) {
                    const int j = __builtin_ctzll(todo);
                    todo &= todo - 1;
                    const int dj = __builtin_amdgcn_readlane(dk, j);
                    if (dj >= res.worst) continue;
                    res.insert(dj, __builtin_amdgcn_readlane(u, j), lane);
                }
            }

            // traverse_cpu.cpp:150-162: best first; with more output slots
            // than heap cells the surplus comes first, as (-1, -inf).  Sorted
            // in the LDS the open list no longer needs.
            wave_sync();
            for (int i = lane; i < a.sort_n; i += kWave)
                okey[i] = INFINITY, oval[i] = -1;
            wave_sync();
#pragma unroll
            for (int s = 0; s < S; ++s) {
                const int e = lane * S + s;
                if (e < H) okey[e] = key_to_float(res.cell_key(lane, s)), oval[e] = res.rv[e];
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
            const int surplus = n_out > H ? n_out - H : 0;
            for (int i = lane; i < n_out; i += kWave) {
                const int e = i - surplus;
                oI[i] = e < 0 ? (int64_t)-1 : (int64_t)oval[e];
                oD[i] = e < 0 ? -INFINITY : okey[e];
            }
            // the buffer is read back as the next search's entries, by other
            // lanes than those that wrote it
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
            wave_sync();
            PA_TIMER(7);
        }

        visited.clean(a.words_per_slot, lane);

        if (a.counters && lane == 0) {
            atomicAdd(&a.counters[0], (unsigned long long)n_expand0);
            atomicAdd(&a.counters[1], (unsigned long long)n_expand1);
            atomicAdd(&a.counters[2], (unsigned long long)n_dist);
            atomicAdd(&a.counters[3], (unsigned long long)n_admit);
            atomicAdd(&a.counters[4], (unsigned long long)n_tail);
            atomicAdd(&a.counters[5], (unsigned long long)n_adj);
#ifdef PA_PHASE_TIMERS
            for (int i = 0; i < 8; ++i) atomicAdd(&a.counters[6 + i], phase[i]);
#endif
        }
    }
}

typedef void (*RefineFn)(RefineArgs);

RefineFn pick_kernel(int H) {
    switch (H) {
        case 16: return refine_kernel<16>;
        case 32: return refine_kernel<32>;
        case 48: return refine_kernel<48>;
        case 64: return refine_kernel<64>;
        case 96: return refine_kernel<96>;
        case 128: return refine_kernel<128>;
        case 192: return refine_kernel<192>;
        case 256: return refine_kernel<256>;
        case 384: return refine_kernel<384>;
        case 512: return refine_kernel<512>;
        case 1024: return refine_kernel<1024>;
        case 2048: return refine_kernel<2048>;
        default: return nullptr;
    }
}

int round_up(int64_t x, int64_t m) { return (int)(((x + m - 1) / m) * m); }

struct Plan {
    int H, sort_n, lds_bytes, n_slots, words_per_slot, slot_stride;
    size_t workspace_bytes;
    RefineFn fn;
};

#ifndef PA_REFINE_MAX_WAVES
#define PA_REFINE_MAX_WAVES 20
#endif
constexpr int kMaxWavesPerCu = PA_REFINE_MAX_WAVES;

int make_plan(int64_t n_nodes, int64_t batch, int d, int ef_search, Plan *p) {
    if (n_nodes <= 0 || batch < 0) return PA_E_SHAPE;
    if (n_nodes >= (1ll << 31)) return PA_E_RANGE;
    if (d <= 0 || d % 8) return PA_E_DIM;
    if (ef_search < 1 || ef_search > PA_MAX_EF_TOTAL) return PA_E_EF;
    p->H = pa_heap_size(ef_search);
    p->sort_n = kWave;
    while (p->sort_n < p->H) p->sort_n <<= 1;
    p->lds_bytes = query_floats(d) * 4;
    p->fn = pick_kernel(p->H);
    if (!p->fn) return PA_E_EF;
    int dev = 0, cus = 0, per_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    {
        static std::mutex mutex;
        static std::map<std::tuple<int, const void *, int>, std::pair<int, int>> known;
        std::lock_guard<std::mutex> guard(mutex);
        const auto key = std::make_tuple(
            dev, reinterpret_cast<const void *>(p->fn), p->lds_bytes);
        auto it = known.find(key);
        if (it == known.end()) {
            e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e == hipSuccess)
                e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &per_cu, reinterpret_cast<const void *>(p->fn), kWave,
                    p->lds_bytes);
            if (e != hipSuccess) return (int)e;
            it = known.emplace(key, std::make_pair(cus, per_cu)).first;
        }
        cus = it->second.first, per_cu = it->second.second;
    }
    if (per_cu < 1) per_cu = 1;
    if (per_cu > kMaxWavesPerCu) per_cu = kMaxWavesPerCu;
    int64_t slots = (int64_t)per_cu * cus;
    if (slots > batch) slots = batch;
    if (slots < 1) slots = 1;
    p->n_slots = (int)slots;
    p->words_per_slot = round_up((n_nodes + 31) / 32, kSlotAlignWords);
    // a slot: the visited slice, then the values of the result list
    p->slot_stride = p->words_per_slot + round_up(p->H, kWave);
    p->workspace_bytes =
        kWorkCounterBytes + (size_t)p->n_slots * p->slot_stride * 4;
    return PA_OK;
}

}  // namespace

extern "C" int pa_rows_prepare(float *dst, const float *src, int64_t n_rows,
                               int d_model, void *stream_) {
    if (n_rows < 0) return PA_E_SHAPE;
    if (d_model <= 0 || d_model % 8) return PA_E_DIM;
    if (n_rows == 0) return PA_OK;
    if (!dst || !src || dst == src) return PA_E_NULL;
    const int64_t n_pairs = n_rows * (d_model / 2);
    if ((n_pairs + 255) / 256 >= (1ll << 31)) return PA_E_RANGE;
    interleave_rows<<<(unsigned)((n_pairs + 255) / 256), 256, 0,
                      (hipStream_t)stream_>>>(src, dst, n_pairs, d_model / 8);
    return (int)hipGetLastError();
}

extern "C" int pa_refine_plan(int64_t n_nodes, int64_t batch, int d_model,
                              int ef_search, int *n_slots,
                              size_t *workspace_bytes) {
    Plan p;
    const int rc = make_plan(n_nodes, batch, d_model, ef_search, &p);
    if (rc != PA_OK) return rc;
    if (n_slots) *n_slots = p.n_slots;
    if (workspace_bytes) *workspace_bytes = p.workspace_bytes;
    return PA_OK;
}

extern "C" int pa_refine(int64_t *out_I, float *out_D, int64_t *buf_I,
                         float *buf_D, const int64_t *init_I, float *init_D,
                         const int32_t *sub_adj, const int32_t *sub_gid,
                         const int64_t *sub_mapping, const int32_t *full_adj,
                         const float *storage, const float *query,
                         int64_t batch, int64_t n_nodes, int d_model,
                         int d_principle, int n_init, int n_buffers, int k,
                         int ef_search, int sub_neighbors, int full_neighbors,
                         void *workspace, size_t workspace_bytes,
                         uint64_t *counters, void *stream_) {
    if (batch < 0 || n_nodes <= 0 || n_init < 0 || n_buffers < 0 || k < 0)
        return PA_E_SHAPE;
    if (n_nodes >= (1ll << 31) || batch >= (1ll << 31)) return PA_E_RANGE;
    if (sub_neighbors < 1 || sub_neighbors > PA_MAX_NEIGHBORS ||
        full_neighbors < 1 || full_neighbors > PA_MAX_NEIGHBORS)
        return PA_E_NEIGHBORS;
    if (d_principle <= 0 || d_principle > d_model || d_principle % 8)
        return PA_E_DIM;
    Plan p;
    const int rc = make_plan(n_nodes, batch, d_model, ef_search, &p);
    if (rc != PA_OK) return rc;
    if (batch == 0) return PA_OK;
    if (!out_I || !out_D || !buf_I || !buf_D || !sub_adj || !sub_gid ||
        !sub_mapping || !full_adj || !storage || !query || !workspace ||
        (n_init > 0 && (!init_I || !init_D)))
        return PA_E_NULL;
    if (workspace_bytes < p.workspace_bytes) return PA_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return PA_E_WORKSPACE;

    RefineArgs a;
    a.out_I = out_I, a.out_D = out_D, a.buf_I = buf_I, a.buf_D = buf_D;
    a.init_I = init_I, a.init_D = init_D;
    a.sub_adj = sub_adj, a.sub_gid = sub_gid, a.sub_mapping = sub_mapping;
    a.full_adj = full_adj, a.storage = storage, a.query = query;
    a.work_counter = reinterpret_cast<int *>(workspace);
    a.seen = reinterpret_cast<uint32_t *>(
        reinterpret_cast<unsigned char *>(workspace) + kWorkCounterBytes);
    a.counters = reinterpret_cast<unsigned long long *>(counters);
    a.batch = (int)batch, a.n_nodes = (int)n_nodes;
    a.d = d_model, a.dp = d_principle;
    a.n_init = n_init, a.n_buffers = n_buffers, a.k = k, a.H = p.H;
    a.sub_deg = sub_neighbors, a.full_deg = full_neighbors;
    // traverse_cpu.cpp:82 with the limits of :325 (REFINE_STEP) and :18 (1024)
    a.sub_iter = 2 * ef_search < 2 ? 2 * ef_search : 2;
    a.full_iter = 2 * ef_search < 1024 ? 2 * ef_search : 1024;
    a.words_per_slot = p.words_per_slot, a.slot_stride = p.slot_stride;
    a.sort_n = p.sort_n;

    hipStream_t stream = (hipStream_t)stream_;
    reset_refine_counter<<<1, 1, 0, stream>>>(a.work_counter);
    p.fn<<<p.n_slots, kWave, p.lds_bytes, stream>>>(a);
    return (int)hipGetLastError();
}
