// Subgraph traversal for gfx950: graph preparation and the per-query search.
//
// One wavefront (64 lanes, one workgroup) runs one query and reproduces, step
// for step, what the reference's host search does for that query
// (extension/traverse_cpu.cpp:12-163):
//   * the open list is the same array heap, with the same sift rules
//     (extension/inc/heapq.cuh:13-88): its top eight levels sit in registers
//     (one node per lane, read with v_readlane), the rest in LDS, and the
//     whole wavefront advances it in lock step (uniform control flow, walks
//     unrolled by level, scalar integer compares);
//   * the result list is the exact set of the H best distances seen so far —
//     what the reference's result heap holds — as a flat LDS array of which
//     the registers track the maximum and where it sits;
//   * the visited set is exact: one bit per storage row in a per-wavefront
//     slice of a pooled HBM bitmask (atomic OR), behind a small LDS table of
//     rows already known to be marked;
//   * a distance is the reference's eight-accumulator FMA sum
//     (extension/inc/distance.h:31-55) bit for bit: four lanes share a row,
//     lane a of the quad owns accumulators 2a and 2a+1 and streams its 16
//     bytes of every 64-byte block of the row (rows are in the layout of
//     pa_rows_prepare: the pairs of two groups of eight interleaved by lane).
// Expansion of a node therefore costs one coalesced row of neighbour ids, an
// atomic for each neighbour the LDS table does not know and one coalesced
// 4*dp-byte row per unvisited neighbour, 16 rows in flight per pass.
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
    int words_per_slot, slot_stride, sort_n;
};

__global__ void reset_work_counter(int *counter) { *counter = 0; }

// Optional per-phase cycle tally for tuning builds (-DPA_PHASE_TIMERS): adds
// seven words after the five work counters.
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

// Wavefronts per SIMD the register allocator must fit.  A budget a few
// registers under what the code needs costs more (spills, serialised loads)
// than the extra wavefront brings — measured: H = 256 with 128-float rows
// needs 113 registers and is 4 % faster at four wavefronts (128) than squeezed
// into the 96 of five, while three wavefronts are 11 % slower than four.  So
// only a floor is given, under which no instance has to be squeezed (the
// largest heaps are bounded by their LDS anyway), and the allocator's own
// count decides the residency above it: 8 for the smallest instances, 4 for
// H = 256 with 128-float rows.
#ifdef PA_WAVES_PER_EU
#define PA_OCCUPANCY(H) __attribute__((amdgpu_waves_per_eu(PA_WAVES_PER_EU, PA_WAVES_PER_EU)))
#else
#define PA_OCCUPANCY(H) __attribute__((amdgpu_waves_per_eu((H) <= 256 ? 4 : (H) <= 384 ? 3 : (H) <= 1024 ? 2 : 1, 8)))
#endif

// The longest open list (4096 cells) keeps its last two levels in the
// wavefront's region of device memory instead of LDS (search_lists.h): first
// level kept there, 0 = the whole list in registers and LDS.  Measured on
// 10 000 queries over 500 000 rows of 128 floats: lists of 4096 cells run in
// 50.0 instead of 69.7 ms with level 11 on in device memory (7 instead of 4
// wavefronts per compute unit) and in 60.4 ms with level 10 on; lists of 2048
// cells take 23.1 ms with level 10 on in device memory against 23.4 ms
// without (11 instead of 8 wavefronts, each as much slower) and 29.6 ms with
// level 9 on, so they stay in LDS.
#ifndef PA_DEEP_512
#define PA_DEEP_512 0
#endif
#ifndef PA_DEEP_1024
#define PA_DEEP_1024 0
#endif
#ifndef PA_DEEP_2048
#define PA_DEEP_2048 11
#endif
constexpr int deep_from(int H) {
    return H == 2048 ? PA_DEEP_2048 : H == 1024 ? PA_DEEP_1024 : H == 512 ? PA_DEEP_512 : 0;
}

template <int H, int DP8>
__global__ __launch_bounds__(kWave) PA_OCCUPANCY(H) void traverse_kernel(TraverseArgs a) {
    // One static block, in this order: the compiler then knows every LDS
    // address, and a heap cell [j - 256] is the scalar j * 8 plus a positive
    // constant that fits the instruction's offset field.
    using Open = OpenList<H, deep_from(H)>;
    constexpr int S = (H + kWave - 1) / kWave;
    // cells of the final sort: all of them, and those sorted in LDS at once
    constexpr int kSortAll = H <= kWave ? kWave : 1 << (floor_log2(H - 1) + 1);
    constexpr int kSortLds = kSortAll > 1024 ? 1024 : kSortAll;
    constexpr int kHeapCells =
        Open::kLdsCells > kSortLds ? Open::kLdsCells : kSortLds;
    // The table of recently marked rows in front of the bitmask: half the
    // size for the long lists, whose residency is bound by LDS (lists of 2048
    // and 4096 cells: 9 instead of 8 wavefronts per compute unit, 5 % faster
    // on 10 000 queries over 500 000 rows of 128 floats although the table
    // answers fewer tests; a quarter of the size is slower again, and
    // where LDS does not bound the residency the smaller table only costs).
    constexpr int kSeenLog2 =
        H >= 1024 && kSeenCacheLog2 > 0 ? kSeenCacheLog2 - 1 : kSeenCacheLog2;
    constexpr int kSeen = 1 << kSeenLog2;
    struct Lds {
        uint32_t seen_cache[kSeen];
        int cand_id[kWave];
        float cand_key[kWave];
        float query[DP8 ? query_floats(8 * DP8) : 4];
        int2 heap[kHeapCells];  // open list tail; the final sort reuses it
    };
    __shared__ __align__(16) Lds lds;
    extern __shared__ __align__(16) float query_any_length[];  // DP8 == 0 only
    const int lane = threadIdx.x;
    float *okey = reinterpret_cast<float *>(lds.heap);
    int *oval = reinterpret_cast<int *>(okey + kHeapCells);
    Open open;
    open.cells = lds.heap;
    int *cand_id = lds.cand_id;
    float *cand_key = lds.cand_key;
    float *qv = DP8 ? lds.query : query_any_length;
    const int dp = DP8 ? DP8 * 8 : a.dp;
    uint32_t *seen_cache = lds.seen_cache;
    const bool use_cache = a.n_storage <= (0xffff << kSeenLog2);
    const int deg = a.deg;
    uint32_t *seen = a.seen + (size_t)blockIdx.x * (size_t)a.slot_stride;
    // after the visited slice: the log of admitted candidates, then the
    // levels of the open list kept in device memory
    ResultLog log;
    log.entry = reinterpret_cast<int2 *>(seen + a.words_per_slot);
    log.capacity = ResultLog::capacity_for(H);
    open.deep = log.entry + ResultLog::capacity_for(H);

    for (;;) {
        int q = 0;
        if (lane == 0) q = atomicAdd(a.work_counter, 1);
        q = uni(q);
        if (q >= a.batch) break;

        unsigned n_expand = 0, n_adj = 0, n_dist = 0, n_admit = 0;
#ifdef PA_PHASE_TIMERS
        unsigned long long phase[7] = {0, 0, 0, 0, 0, 0, 0};
#endif
        PA_TIMER_BEGIN();

        // fresh visited slice, query to LDS, empty lists
#ifndef PA_CLEAR_REPS  // tuning builds: the clearing repeated, to time it
#define PA_CLEAR_REPS 1
#endif
        for (int rep = 0; rep < PA_CLEAR_REPS; ++rep)
            for (int w = lane * 4; w < a.words_per_slot; w += kWave * 4)
                *reinterpret_cast<uint4 *>(seen + w) = make_uint4(0, 0, 0, 0);
        for (int i = lane; i < dp; i += kWave)
            qv[query_slot(i, dp >> 3)] = a.query[(size_t)q * dp + i];
        for (int i = lane; i < kSeen; i += kWave) seen_cache[i] = 0xffffffffu;
        open.reset(lane);
        ResultKeys<S> res;
        res.init(H, lane);
        log.n = 0;
        // The clearing stores must have reached the cache level where the
        // atomic ORs are performed before the first OR is issued.  Only this
        // wavefront touches the slice, so waiting for its own stores is
        // enough; a device-scope fence here would write back and invalidate
        // caches once per query.
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
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
                open.template replace<true>(float_to_key(dj), rj >= 0 ? rj : -2 - (base + j), lane);
            }
        }

        PA_TIMER(5);
        // traverse_cpu.cpp:82-136, software-pipelined.  The node a pop will
        // return is the root of the open list as it stands after the last
        // insert, so once a step's inserts are done the next step's node is
        // certain: its neighbours' visited bits are tested and set *before*
        // the pop (the atomics are in flight while the pop sifts).  If the
        // search ends at the next pop instead, the marks set for a node that
        // is never expanded are harmless: the slice is cleared per query.
        // (Requesting that node's row of neighbour ids even earlier, before
        // the inserts, for the most likely next root, measured the same.)
        auto load_row = [&](int r) -> int {
            int row = -1;
            if (r >= 0 && lane < deg) row = a.adj[(size_t)r * deg + lane];
            return row;
        };
        // Returns the bitmask word before the OR; it is looked at only after
        // the pop.  Most neighbours of a node were seen a few steps ago: a
        // two-way LDS table of rows whose bit is known to be set answers for
        // them without going to memory.  Word r mod 1024 holds the 16-bit
        // tags r / 1024 of the two rows seen last (newest in the low half).
        // A row enters the table only after its atomic has been issued, so a
        // hit is always right; a miss (never seen, or displaced) asks the
        // bitmask, which is exact.
        auto test_and_set = [&](int v) -> uint32_t {
            uint32_t before = 0xffffffffu;
            if (v >= 0) {
                const int cell = v & (kSeen - 1);
                const uint32_t tag = (uint32_t)v >> kSeenLog2;
                const uint32_t ways = use_cache ? seen_cache[cell] : 0xffffffffu;
                if (!use_cache || ((ways & 0xffffu) != tag && (ways >> 16) != tag)) {
                    before = atomicOr(&seen[v >> 5], 1u << (v & 31));
                    if (use_cache) seen_cache[cell] = (ways << 16) | tag;
                }
            }
            return before;
        };
        int v = load_row(Open::rl(open.Av, 1));
        uint32_t before = test_and_set(v);
        for (int step = 0; step < a.max_iter; ++step) {
            int uk, u;
            open.pop(lane, uk, u);
            PA_TIMER(0);
            if (u == -1 || uk >= res.worst) break;
            n_expand += 1;
            bool popped = false;  // the pop has been finished
            if (u >= 0) {
                n_adj += deg;
                const bool fresh = !((before >> (v & 31)) & 1u);
                const unsigned long long mask = __ballot(fresh);
                const int n = __popcll(mask);
                PA_TIMER(2);
                if (n > 0) {
                    if (fresh) cand_id[lane_rank(mask)] = v;
                    wave_sync();
                    eval_rows<DP8>(a.storage, qv, cand_id, cand_key, n, dp, lane);
                    n_dist += n;
                    wave_sync();
                    PA_TIMER(3);
                    // levels of the open list in device memory: their pair
                    // was requested by the pop and has arrived with the rows
                    open.pop_finish(lane);
                    popped = true;

                    const int d = float_to_key(lane < n ? cand_key[lane] : INFINITY);
                    const int id = lane < n ? cand_id[lane] : -1;
                    // heap_update, traverse_cpu.cpp:25-39, in adjacency order
                    unsigned long long todo = __ballot(d < res.worst);
                    unsigned long long admitted = 0;
                    while (todo) {
                        const int j = __builtin_ctzll(todo);
                        todo &= todo - 1;
                        const int dj = __builtin_amdgcn_readlane(d, j);
                        if (dj >= res.worst) continue;
                        const int vj = __builtin_amdgcn_readlane(id, j);
                        typename Open::Leaf leaf;
                        if (Open::kFusedTop) {
                            // the result list's new maximum and the top of
                            // the open list's walk in one instruction stream
                            const typename Open::Choice ch = open.template choices<true>();
                            int first = res.replace_worst(dj, lane);
                            const int j7 = Open::top_levels_and_wave_max(ch, first);
                            res.set_worst(first);
                            leaf = open.walk_below(ch, 7, j7);
                        } else {
                            leaf = open.walk_to_large_leaf();
                            res.insert(dj, lane);
                        }
                        open.replace_leaf(leaf, dj, vj, lane);
                        admitted |= 1ull << j;
                    }
                    if (admitted) {
                        n_admit += __popcll(admitted);
                        log.append(admitted, d, id, lane);
                        if (log.nearly_full()) log.cut(res.worst, lane);
                    }
                    PA_TIMER(4);
                }
            }
            if (!popped) open.pop_finish(lane);
            v = load_row(Open::rl(open.Av, 1));
            before = test_and_set(v);
            PA_TIMER(1);
        }

        // traverse_cpu.cpp:138-148: the entries compete for a result slot.  A
        // log value below -1 is the global id -2 - value of an entry, the
        // others are storage rows.
        for (int base = 0; base < a.n_init; base += kWave) {
            const int i = base + lane;
            int u = -1;
            float d = INFINITY;
            if (i < a.n_init) {
                const int64_t g = eI[i];
                d = eD[i];
                if (g >= 0 && g < a.n_nodes) u = (int)g;
            }
            const int dk = float_to_key(d);
            unsigned long long todo = __ballot(u >= 0 && dk < res.worst);
            unsigned long long admitted = 0;
            while (todo) {
                const int j = __builtin_ctzll(todo);
                todo &= todo - 1;
                const int dj = __builtin_amdgcn_readlane(dk, j);
                if (dj >= res.worst) continue;
                res.insert(dj, lane);
                admitted |= 1ull << j;
            }
            if (admitted) {
                log.append(admitted, dk, -2 - u, lane);
                if (log.nearly_full()) log.cut(res.worst, lane);
            }
        }

        // traverse_cpu.cpp:150-162: best first.  The set is read back from
        // the log — every entry below the maximum, and of those at the
        // maximum as many as make H — into the LDS the open list no longer
        // needs, padded to a power of two with +inf, and sorted there.
        wave_sync();
        ResultLog::settle();
        int n_below = 0;
        for (int base = 0; base < log.n; base += kWave) {
            const int i = base + lane;
            n_below += __popcll(__ballot(i < log.n && log.entry[i].x < res.worst));
        }
        // Stages of a bitonic network over okey / oval [0, n): merges of
        // `first_size` cells and up (2: a full sort; n: the last merge alone,
        // for cells that are bitonic already); `desc`: largest first.
        auto lds_sort = [&](int n, int first_size, bool desc) {
            for (int size = first_size; size <= n; size <<= 1) {
                for (int stride = size >> 1; stride > 0; stride >>= 1) {
                    for (int t = lane; t < (n >> 1); t += kWave) {
                        const int i = ((t & ~(stride - 1)) << 1) | (t & (stride - 1));
                        const int j = i | stride;
                        const float ki = okey[i], kj = okey[j];
                        const int vi = oval[i], vj = oval[j];
                        const bool gt = ki > kj || (ki == kj && vi > vj);
                        const bool lt = ki < kj || (ki == kj && vi < vj);
                        if ((((i & size) == 0) != desc) ? gt : lt) {
                            okey[i] = kj, oval[i] = vj;
                            okey[j] = ki, oval[j] = vi;
                        }
                    }
                    wave_sync();
                }
            }
        };
        int64_t *oI = a.out_I + (size_t)q * a.k;
        float *oD = a.out_D + (size_t)q * a.k;
        if constexpr (kSortAll <= kSortLds) {
            for (int i = lane; i < a.sort_n; i += kWave)
                okey[i] = INFINITY, oval[i] = -1;
            wave_sync();
            int at_below = 0, at_worst = n_below;
            for (int base = 0; base < log.n; base += kWave) {
                const int i = base + lane;
                int2 e = make_int2(0x7fffffff, -1);
                if (i < log.n) e = log.entry[i];
                const bool below = i < log.n && e.x < res.worst;
                const bool tie = i < log.n && e.x == res.worst;
                const unsigned long long mb = __ballot(below), mt = __ballot(tie);
                int place = -1;
                if (below) place = at_below + lane_rank(mb);
                if (tie) place = at_worst + lane_rank(mt);
                if (place >= 0 && place < H) {
                    okey[place] = key_to_float(e.x);
                    oval[place] = e.y < -1 ? -2 - e.y : a.gid[e.y];
                }
                at_below += __popcll(mb);
                at_worst += __popcll(mt);
            }
            wave_sync();
            lds_sort(a.sort_n, 2, false);
            for (int i = lane; i < a.k; i += kWave) {
                oI[i] = (int64_t)oval[i];
                oD[i] = okey[i];
            }
        } else {
            // The longest lists sort in two halves of kSortLds cells, so that
            // the sort does not decide the size of the LDS block (and with it
            // how many wavefronts a compute unit holds).  The set is
            // compacted at the head of the log (in log order: a write lands
            // on an entry already read), as (distance, id); the first half is
            // sorted ascending and the second descending through LDS; one
            // exchange between the halves in the log leaves every cell of the
            // first below every cell of the second and both bitonic; each is
            // then merged in LDS and written out.
            static_assert(kSortAll == 2 * kSortLds, "two halves");
            static_assert(ResultLog::capacity_for(H) >= kSortAll, "the log holds them");
            int m = 0, ties_left = H - n_below;
            for (int base = 0; base < log.n; base += kWave) {
                const int i = base + lane;
                int2 e = make_int2(0x7fffffff, -1);
                if (i < log.n) e = log.entry[i];
                const bool below = i < log.n && e.x < res.worst;
                const bool tie = i < log.n && e.x == res.worst;
                const unsigned long long mt = __ballot(tie);
                const bool keep = below || (tie && lane_rank(mt) < ties_left);
                const unsigned long long mk = __ballot(keep);
                if (keep) {
                    const int id = e.y < -1 ? -2 - e.y : a.gid[e.y];
                    log.entry[m + lane_rank(mk)] =
                        make_int2(__float_as_int(key_to_float(e.x)), id);
                }
                m += __popcll(mk);
                ties_left -= min(ties_left, (int)__popcll(mt));
            }
            ResultLog::settle();
            auto load_half = [&](int half) {
                for (int i = lane; i < kSortLds; i += kWave) {
                    const int at = half * kSortLds + i;
                    int2 e = make_int2(__float_as_int(INFINITY), -1);
                    if (at < m) e = log.entry[at];
                    okey[i] = __int_as_float(e.x), oval[i] = e.y;
                }
                wave_sync();
            };
            for (int half = 0; half < 2; ++half) {
                load_half(half);
                lds_sort(kSortLds, 2, half == 1);
                for (int i = lane; i < kSortLds; i += kWave)
                    log.entry[half * kSortLds + i] =
                        make_int2(__float_as_int(okey[i]), oval[i]);
                wave_sync();
            }
            ResultLog::settle();
            m = kSortAll;  // both halves are whole now, +inf cells included
            for (int i = lane; i < kSortLds; i += kWave) {
                const int2 x = log.entry[i], y = log.entry[kSortLds + i];
                const float kx = __int_as_float(x.x), ky = __int_as_float(y.x);
                if (kx > ky || (kx == ky && x.y > y.y)) {
                    log.entry[i] = y;
                    log.entry[kSortLds + i] = x;
                }
            }
            ResultLog::settle();
            for (int half = 0; half < 2; ++half) {
                load_half(half);
                lds_sort(kSortLds, kSortLds, false);
                for (int i = lane; i < kSortLds; i += kWave) {
                    const int r = half * kSortLds + i;
                    if (r < a.k) {
                        oI[r] = (int64_t)oval[i];
                        oD[r] = okey[i];
                    }
                }
                wave_sync();
            }
        }
        wave_sync();

        if (a.counters && lane == 0) {
            atomicAdd(&a.counters[0], (unsigned long long)n_expand);
            atomicAdd(&a.counters[1], (unsigned long long)n_adj);
            atomicAdd(&a.counters[2], (unsigned long long)n_dist);
            atomicAdd(&a.counters[3], (unsigned long long)n_admit);
            atomicAdd(&a.counters[4], (unsigned long long)a.k);
#ifdef PA_PHASE_TIMERS
            PA_TIMER(6);
            for (int i = 0; i < 7; ++i) atomicAdd(&a.counters[5 + i], phase[i]);
#endif
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
    int64_t n_nodes, int64_t n_storage, int64_t nnz, int deg,
    const int32_t *gid, int32_t *adj, int32_t *status) {
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
        // a row that does not lie inside `indices` is reported and read as
        // empty: nothing outside the array is ever touched
        if (lo < 0 || lo > nnz || len > nnz - lo) {
            if (lane == 0) atomicOr(status, 8);
            len = 0;
        }
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

// ---- scratch for callers that cannot allocate -----------------------------------
//
// pa_traverse_static runs the search in this array instead of a caller's
// workspace.  Every GPU the library is used on holds its own copy at its own
// address; host code never uses the array's name as a pointer, only the
// address hipGetSymbolAddress returns for the current device.
static __device__ __align__(256) unsigned char scratch[PA_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;

// Device address of `scratch` on the current device, looked up once per device.
int static_scratch(unsigned char **out) {
    static std::mutex mutex;
    static unsigned char *known[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    if (dev < 0 || dev >= kMaxDevices) return PA_E_RANGE;
    std::lock_guard<std::mutex> guard(mutex);
    if (!known[dev]) {
        void *ptr = nullptr;
        e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
        if (e != hipSuccess) return (int)e;
        if (!ptr) return PA_E_NULL;
        known[dev] = static_cast<unsigned char *>(ptr);
    }
    *out = known[dev];
    return PA_OK;
}

// ---- host side --------------------------------------------------------------------

int round_up(int64_t x, int64_t m) { return (int)(((x + m - 1) / m) * m); }

int next_pow2(int x) {
    int p = 1;
    while (p < x) p <<= 1;
    return p;
}

typedef void (*TraverseFn)(TraverseArgs);

template <int H>
TraverseFn pick_dp(int dp) {
    switch (dp) {
        case 32: return traverse_kernel<H, 4>;
        case 64: return traverse_kernel<H, 8>;
        case 128: return traverse_kernel<H, 16>;
        default: return traverse_kernel<H, 0>;
    }
}

TraverseFn pick_kernel(int H, int dp) {
    switch (H) {
        case 16: return pick_dp<16>(dp);
        case 32: return pick_dp<32>(dp);
        case 48: return pick_dp<48>(dp);
        case 64: return pick_dp<64>(dp);
        case 96: return pick_dp<96>(dp);
        case 128: return pick_dp<128>(dp);
        case 192: return pick_dp<192>(dp);
        case 256: return pick_dp<256>(dp);
        case 384: return pick_dp<384>(dp);
        case 512: return pick_dp<512>(dp);
        case 1024: return pick_dp<1024>(dp);
        case 2048: return pick_dp<2048>(dp);
        default: return nullptr;
    }
}

struct Plan {
    int H, sort_n, lds_bytes, n_slots, words_per_slot, slot_stride;
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
    // dynamic LDS: the query when its length has no specialised kernel (the
    // rest is static in the kernel)
    p->lds_bytes = (dp == 32 || dp == 64 || dp == 128) ? 0 : query_floats(dp) * 4;
#ifdef PA_EXTRA_LDS  // tuning builds: lower the residency without touching code
    p->lds_bytes += PA_EXTRA_LDS;
#endif
    p->fn = pick_kernel(p->H, dp);
    if (!p->fn) return PA_E_EF;
    int dev = 0, cus = 0, per_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    {
        // the residency of a (device, kernel, LDS size) never changes
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
    // more than five wavefronts per SIMD have measured slower on every
    // instance that fits them (the SIMDs' issue slots are the bound)
#ifndef PA_MAX_WAVES_PER_CU
#define PA_MAX_WAVES_PER_CU 20
#endif
    if (per_cu > PA_MAX_WAVES_PER_CU) per_cu = PA_MAX_WAVES_PER_CU;
    int64_t slots = (int64_t)per_cu * cus;
    if (slots < 1) slots = 1;
    if (slots > batch) slots = batch;
    if (slots < 1) slots = 1;
    p->n_slots = (int)slots;
    p->words_per_slot = round_up((n_storage + 31) / 32, kSlotAlignWords);
    // a slot: the visited slice, the log of admitted candidates, the levels
    // of the open list that are kept in device memory (8 bytes an entry or cell)
    p->slot_stride = p->words_per_slot + 2 * ResultLog::capacity_for(p->H) +
                     round_up(2 * open_list_deep_cells(p->H, deep_from(p->H)), kWave);
    p->workspace_bytes =
        kWorkCounterBytes + (size_t)p->n_slots * p->slot_stride * 4;
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
        case PA_E_WORKSPACE: return "workspace too small or not 256-byte aligned";
        case PA_E_GRAPH: return "malformed graph (see status word)";
        case PA_E_LEAVES: return "n_leaves must be a multiple of 32";
        case PA_E_CHUNK: return "batch must be a multiple of chunk_size";
        case PA_E_RANGE: return "an id does not fit 31 bits";
        case PA_E_STATIC:
            return "index too large for the static scratch of pa_traverse_static";
        default: return "unknown error";
    }
}

extern "C" int pa_graph_prepare(const int64_t *indptr, const int64_t *indices,
                                const int64_t *mapping, int64_t n_nodes,
                                int64_t n_storage, int64_t nnz,
                                int n_neighbors, int32_t *adj, int32_t *gid,
                                int32_t *status, void *stream_) {
    if (n_nodes <= 0 || n_storage <= 0 || n_storage > n_nodes || nnz < 0)
        return PA_E_SHAPE;
    if (!indptr || !indices || !mapping || !adj || !gid || !status)
        return PA_E_NULL;
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
                              nnz, n_neighbors, gid, adj, status);
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

namespace {

// Checks and launch shared by pa_traverse and pa_traverse_static.  With
// `fit_slots` the number of wavefronts is lowered to what the workspace holds
// (at least min(batch, kMinStaticSlots), else PA_E_STATIC); without it a
// workspace smaller than the plan's is an error.
constexpr int kMinStaticSlots = 256;

int launch_traverse(int64_t *out_I, float *out_D, const int32_t *adj,
                    const int32_t *gid, const int64_t *mapping,
                    const float *storage, const float *query,
                    const int64_t *init_I, const float *init_D, int64_t batch,
                    int64_t n_nodes, int64_t n_storage, int dp, int n_init,
                    int beam, int ef, int n_neighbors, void *workspace,
                    size_t workspace_bytes, bool fit_slots, uint64_t *counters,
                    void *stream_) {
    if (batch < 0 || n_nodes <= 0 || n_init < 0 || beam < 1 || ef < 1)
        return PA_E_SHAPE;
    if (n_nodes >= (1ll << 31) || batch >= (1ll << 31)) return PA_E_RANGE;
    if (n_neighbors < 1 || n_neighbors > PA_MAX_NEIGHBORS) return PA_E_NEIGHBORS;
    if ((int64_t)beam * ef > PA_MAX_EF_TOTAL) return PA_E_EF;
    Plan p;
    const int rc = make_plan(n_storage, batch, dp, beam * ef, &p);
    if (rc != PA_OK) return rc;
    if (batch == 0) return PA_OK;
    if (!out_I || !out_D || !adj || !gid || !mapping || !storage || !query ||
        !workspace || (n_init > 0 && (!init_I || !init_D)))
        return PA_E_NULL;
    if (fit_slots) {
        const size_t slot_bytes = (size_t)p.slot_stride * 4;
        const size_t fit = workspace_bytes < kWorkCounterBytes
                               ? 0
                               : (workspace_bytes - kWorkCounterBytes) / slot_bytes;
        const int64_t need = batch < kMinStaticSlots ? batch : kMinStaticSlots;
        if ((int64_t)fit < need) return PA_E_STATIC;
        if ((size_t)p.n_slots > fit) p.n_slots = (int)fit;
    } else if (workspace_bytes < p.workspace_bytes) {
        return PA_E_WORKSPACE;
    }
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return PA_E_WORKSPACE;

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
    a.slot_stride = p.slot_stride;

    hipStream_t stream = (hipStream_t)stream_;
    reset_work_counter<<<1, 1, 0, stream>>>(a.work_counter);
    p.fn<<<p.n_slots, kWave, p.lds_bytes, stream>>>(a);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int pa_traverse(int64_t *out_I, float *out_D, const int32_t *adj,
                           const int32_t *gid, const int64_t *mapping,
                           const float *storage, const float *query,
                           const int64_t *init_I, const float *init_D,
                           int64_t batch, int64_t n_nodes, int64_t n_storage,
                           int dp, int n_init, int beam, int ef,
                           int n_neighbors, void *workspace,
                           size_t workspace_bytes, uint64_t *counters,
                           void *stream_) {
    return launch_traverse(out_I, out_D, adj, gid, mapping, storage, query,
                           init_I, init_D, batch, n_nodes, n_storage, dp,
                           n_init, beam, ef, n_neighbors, workspace,
                           workspace_bytes, false, counters, stream_);
}

extern "C" int pa_traverse_static(int64_t *out_I, float *out_D,
                                  const int32_t *adj, const int32_t *gid,
                                  const int64_t *mapping, const float *storage,
                                  const float *query, const int64_t *init_I,
                                  const float *init_D, int64_t batch,
                                  int64_t n_nodes, int64_t n_storage, int dp,
                                  int n_init, int beam, int ef, int n_neighbors,
                                  uint64_t *counters, void *stream_) {
    unsigned char *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc != PA_OK) return rc;
    // The work counter is set by a kernel, the visited slices and the result
    // values are cleared by the search itself, per query: nothing of an
    // earlier call is read.
    return launch_traverse(out_I, out_D, adj, gid, mapping, storage, query,
                           init_I, init_D, batch, n_nodes, n_storage, dp,
                           n_init, beam, ef, n_neighbors, ws,
                           PA_STATIC_SCRATCH_BYTES, true, counters, stream_);
}
