// The wide mode of the subgraph traversal for gfx950: a labelled throughput
// mode beside the exact one of traverse.hip.  Never the default.
//
// The exact mode reproduces the reference's host search step for step
// (extension/traverse_cpu.cpp:12-163) and is bound by the dependent chain of
// that emulation: one node per step, each admitted candidate two walks of an
// array heap.  This mode keeps what the search computes and drops how the
// host orders it, in the shape of the reference's own device kernel
// (extension/traverse_cuda.cu:116-226: several nodes expanded per step, one
// shared visited set):
//   * the result list and the open list are one pool of the P best
//     candidates seen, sorted by distance in registers (rank r in lane r % 64
//     of register r / 64), each with a flag "expanded";
//   * a step takes the (up to) `width` best candidates not yet expanded,
//     fetches their rows of neighbour ids together, tests and marks the
//     neighbours in the exact visited set, evaluates all fresh rows in one
//     batch (the distance code of the exact mode: a distance is bit for bit
//     the host's), sorts the candidates that beat the pool's worst with a
//     bitonic network across the wavefront and merges them into the pool,
//     64 at a time, register by register;
//   * the search ends when the pool holds no candidate that is not expanded
//     (what "the popped key is not below the worst kept" means for a sorted
//     pool), or after min(1024, 2 * beam * ef) expansions like the host's.
// What differs from the exact mode: nodes are expanded in groups, so a few
// are expanded that a strict best-first order would not have reached, the
// open list is not the reference's array heap with its large-leaf rule, and
// the entries are part of the pool from the start.  Ids are therefore not
// promised to equal the host search's; distances of returned ids are exact,
// and the recall of the whole search is the measure.
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

#ifndef PA_WIDE_MAX_WIDTH
#define PA_WIDE_MAX_WIDTH 4
#endif
constexpr int kMaxWidth = PA_WIDE_MAX_WIDTH;
constexpr unsigned kDone = 0x80000000u;     // expanded, or nothing to expand
constexpr unsigned kGlobal = 0x40000000u;   // the low bits are a global id, not a storage row
constexpr unsigned kIdMask = 0x3fffffffu;

struct WideArgs {
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
    int batch, n_nodes, n_storage, dp, n_init, k, deg, max_iter, width;
    int words_per_slot;
};

__global__ void reset_wide_counter(int *counter) { *counter = 0; }

// A pool entry: distance key in the high word (order-preserving integer of
// the float), value in the low word; signed 64-bit order = by distance, then
// by value.
typedef long long Entry;
constexpr Entry kEmpty = (Entry)(((unsigned long long)0x7f800000u << 32) | 0xffffffffu);

__device__ __forceinline__ Entry make_entry(int key, unsigned val) {
    return (Entry)(((unsigned long long)(unsigned)key << 32) | val);
}
__device__ __forceinline__ int entry_key(Entry e) { return (int)(e >> 32); }
__device__ __forceinline__ unsigned entry_val(Entry e) { return (unsigned)e; }

// The entry of lane (lane ^ STRIDE).
template <int STRIDE>
__device__ __forceinline__ Entry partner(Entry e, int lane) {
    int lo = (int)(unsigned)e, hi = (int)(e >> 32);
    if (STRIDE == 1) {
        lo = __builtin_amdgcn_update_dpp(lo, lo, 0xB1, 0xF, 0xF, false);
        hi = __builtin_amdgcn_update_dpp(hi, hi, 0xB1, 0xF, 0xF, false);
    } else if (STRIDE == 2) {
        lo = __builtin_amdgcn_update_dpp(lo, lo, 0x4E, 0xF, 0xF, false);
        hi = __builtin_amdgcn_update_dpp(hi, hi, 0x4E, 0xF, 0xF, false);
    } else if (STRIDE <= 16) {
        // swizzle in bit mode: lane ^ STRIDE within 32 lanes
        lo = __builtin_amdgcn_ds_swizzle(lo, (STRIDE << 10) | 0x1f);
        hi = __builtin_amdgcn_ds_swizzle(hi, (STRIDE << 10) | 0x1f);
    } else {
        lo = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, lo);
        hi = __builtin_amdgcn_ds_bpermute((lane ^ 32) << 2, hi);
    }
    return (Entry)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

// One compare-exchange stage of a bitonic network over the 64 lanes: lanes
// STRIDE apart; `up` = this lane's block sorts ascending.
template <int STRIDE>
__device__ __forceinline__ Entry exchange(Entry e, bool up, int lane) {
    const Entry p = partner<STRIDE>(e, lane);
    const bool low_lane = (lane & STRIDE) == 0;
    const bool take_small = low_lane == up;
    const bool p_small = p < e;
    return (p_small == take_small) ? p : e;
}

// A bitonic sequence over the lanes becomes ascending.
__device__ __forceinline__ Entry clean64(Entry e, int lane) {
    e = exchange<32>(e, true, lane);
    e = exchange<16>(e, true, lane);
    e = exchange<8>(e, true, lane);
    e = exchange<4>(e, true, lane);
    e = exchange<2>(e, true, lane);
    e = exchange<1>(e, true, lane);
    return e;
}

// Any 64 entries become ascending over the lanes.
__device__ __forceinline__ Entry sort64(Entry e, int lane) {
    e = exchange<1>(e, (lane & 2) == 0, lane);
    e = exchange<2>(e, (lane & 4) == 0, lane);
    e = exchange<1>(e, (lane & 4) == 0, lane);
    e = exchange<4>(e, (lane & 8) == 0, lane);
    e = exchange<2>(e, (lane & 8) == 0, lane);
    e = exchange<1>(e, (lane & 8) == 0, lane);
    e = exchange<8>(e, (lane & 16) == 0, lane);
    e = exchange<4>(e, (lane & 16) == 0, lane);
    e = exchange<2>(e, (lane & 16) == 0, lane);
    e = exchange<1>(e, (lane & 16) == 0, lane);
    e = exchange<16>(e, (lane & 32) == 0, lane);
    e = exchange<8>(e, (lane & 32) == 0, lane);
    e = exchange<4>(e, (lane & 32) == 0, lane);
    e = exchange<2>(e, (lane & 32) == 0, lane);
    e = exchange<1>(e, (lane & 32) == 0, lane);
    return clean64(e, lane);
}

__device__ __forceinline__ Entry lane_entry(Entry e, int l) {
    const int lo = __builtin_amdgcn_readlane((int)(unsigned)e, l);
    const int hi = __builtin_amdgcn_readlane((int)(e >> 32), l);
    return (Entry)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
}

// The pool: P = 64 * S entries, ascending.
template <int S>
struct Pool {
    Entry e[S];

    __device__ __forceinline__ void reset() {
#pragma unroll
        for (int s = 0; s < S; ++s) e[s] = kEmpty;
    }
    // key of the last entry: a candidate must be below it to enter
    __device__ __forceinline__ int worst() const {
        return __builtin_amdgcn_readlane((int)(e[S - 1] >> 32), kWave - 1);
    }
    // Merges 64 ascending entries (`in`, +inf entries at its end) into the
    // pool; the 64 largest of the union fall out.  Register by register: the
    // smaller half of (register, carry) stays, the larger half is carried on.
    __device__ __forceinline__ void merge(Entry in, int lane) {
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const Entry first_in = lane_entry(in, 0);
            if (entry_key(first_in) == 0x7f800000) return;       // nothing left to place
            if (lane_entry(e[s], kWave - 1) <= first_in) continue;  // all of it below the carry
            // the carry reversed: register and carry together are bitonic
            const int rev = (kWave - 1 - lane) << 2;
            const int lo = __builtin_amdgcn_ds_bpermute(rev, (int)(unsigned)in);
            const int hi = __builtin_amdgcn_ds_bpermute(rev, (int)(in >> 32));
            const Entry r = (Entry)(((unsigned long long)(unsigned)hi << 32) | (unsigned)lo);
            const bool r_small = r < e[s];
            const Entry small = r_small ? r : e[s];
            const Entry large = r_small ? e[s] : r;
            e[s] = clean64(small, lane);
            if (s + 1 < S) in = clean64(large, lane);
        }
    }
};

template <int S, int DP8>
__global__ __launch_bounds__(kWave) void wide_kernel(WideArgs a) {
    constexpr int kCand = kMaxWidth * kWave;
    struct Lds {
        uint32_t seen_cache[kSeenCache];
        int cand_id[kCand];
        float cand_key[kCand];
        int chosen[kMaxWidth];
        float query[DP8 ? query_floats(8 * DP8) : 4];
    };
    __shared__ __align__(16) Lds lds;
    extern __shared__ __align__(16) float query_any_length[];  // DP8 == 0 only
    const int lane = threadIdx.x;
    int *cand_id = lds.cand_id;
    float *cand_key = lds.cand_key;
    float *qv = DP8 ? lds.query : query_any_length;
    const int dp = DP8 ? DP8 * 8 : a.dp;
    uint32_t *seen_cache = lds.seen_cache;
    const bool use_cache = a.n_storage <= (0xffff << kSeenCacheLog2);
    const int deg = a.deg;
    uint32_t *seen = a.seen + (size_t)blockIdx.x * (size_t)a.words_per_slot;

    for (;;) {
        int q = 0;
        if (lane == 0) q = atomicAdd(a.work_counter, 1);
        q = uni(q);
        if (q >= a.batch) break;
        unsigned n_expand = 0, n_adj = 0, n_dist = 0, n_admit = 0;

        for (int w = lane * 4; w < a.words_per_slot; w += kWave * 4)
            *reinterpret_cast<uint4 *>(seen + w) = make_uint4(0, 0, 0, 0);
        for (int i = lane; i < dp; i += kWave)
            qv[query_slot(i, dp >> 3)] = a.query[(size_t)q * dp + i];
        for (int i = lane; i < kSeenCache; i += kWave) seen_cache[i] = 0xffffffffu;
        Pool<S> pool;
        pool.reset();
        // the clearing stores before the first atomic on the slice (only this
        // wavefront touches it)
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        wave_sync();

        // An LDS table of rows whose bit is known to be set in front of the
        // exact bitmask, as in the exact mode.
        auto test_and_set = [&](int v) -> uint32_t {
            uint32_t before = 0xffffffffu;
            if (v >= 0) {
                const int cell = v & (kSeenCache - 1);
                const uint32_t tag = (uint32_t)v >> kSeenCacheLog2;
                const uint32_t ways = use_cache ? seen_cache[cell] : 0xffffffffu;
                if (!use_cache || ((ways & 0xffffu) != tag && (ways >> 16) != tag)) {
                    before = atomicOr(&seen[v >> 5], 1u << (v & 31));
                    if (use_cache) seen_cache[cell] = (ways << 16) | tag;
                }
            }
            return before;
        };

        // One loop: whatever is staged in cand_id / cand_key (values and
        // distances, n of them) goes into the pool; then the next entries of
        // the query are staged, or, when they are all in, the next nodes are
        // expanded and their fresh neighbours staged.
        const int64_t *eI = a.init_I + (size_t)q * a.n_init;
        const float *eD = a.init_D + (size_t)q * a.n_init;
        int entry_base = 0;
        bool searching = false;  // the entries are all in
        int n = 0;
        for (;;) {
            // those below the pool's worst, sorted 64 at a time, merged
            for (int base = 0; base < n; base += kWave) {
                const int i = base + lane;
                const int worst = pool.worst();
                Entry mine = kEmpty;
                if (i < n) {
                    const int key = float_to_key(cand_key[i]);
                    if (key < worst) mine = make_entry(key, (unsigned)cand_id[i]);
                }
                const unsigned long long some = __ballot(mine != kEmpty);
                if (!some) continue;
                if (searching) n_admit += __popcll(some);
                pool.merge(sort64(mine, lane), lane);
            }
            n = 0;
            wave_sync();

            if (entry_base < a.n_init) {
                // the entries: marked, and staged; one without a storage row
                // keeps its global id and counts as expanded
                const int i = entry_base + lane;
                entry_base += kWave;
                unsigned val = 0xffffffffu;
                float d = INFINITY;
                if (i < a.n_init) {
                    const int64_t g = eI[i];
                    if (g >= 0 && g < a.n_nodes) {
                        d = eD[i];
                        const int row = (int)a.mapping[g];
                        if (row >= 0) {
                            atomicOr(&seen[row >> 5], 1u << (row & 31));
                            val = (unsigned)row;
                        } else {
                            val = kDone | kGlobal | (unsigned)g;
                        }
                    }
                }
                cand_id[lane] = (int)val;
                cand_key[lane] = d;
                n = kWave;
                wave_sync();
                continue;
            }
            searching = true;
            if ((int)n_expand >= a.max_iter) break;

            // the best candidates not yet expanded, at most `width`
            const int want = min(a.width, a.max_iter - (int)n_expand);
            int n_chosen = 0;
#pragma unroll
            for (int s = 0; s < S; ++s) {
                if (n_chosen < want) {
                    unsigned long long open = __ballot((entry_val(pool.e[s]) & kDone) == 0);
                    unsigned long long take = 0;
                    for (int t = n_chosen; t < want && open; ++t) {
                        take |= open & (0 - open);
                        open &= open - 1;
                    }
                    if (take) {
                        if ((take >> lane) & 1) {
                            lds.chosen[n_chosen + lane_rank(take)] =
                                (int)(entry_val(pool.e[s]) & kIdMask);
                            pool.e[s] |= (Entry)kDone;
                        }
                        n_chosen += __popcll(take);
                    }
                }
            }
            if (n_chosen == 0) break;
            wave_sync();
            n_expand += n_chosen;
            n_adj += n_chosen * deg;

            // their rows of neighbour ids together, then the visited tests
            int v[kMaxWidth];
#pragma unroll
            for (int w = 0; w < kMaxWidth; ++w) {
                v[w] = -1;
                if (w < n_chosen && lane < deg)
                    v[w] = a.adj[(size_t)lds.chosen[w] * deg + lane];
            }
            uint32_t before[kMaxWidth];
#pragma unroll
            for (int w = 0; w < kMaxWidth; ++w) {
                before[w] = 0xffffffffu;
                if (w < n_chosen) {
                    before[w] = test_and_set(v[w]);
                    // a later row of this step must see the marks of an
                    // earlier one in the table
                    wave_sync();
                }
            }
#pragma unroll
            for (int w = 0; w < kMaxWidth; ++w) {
                const bool fresh = w < n_chosen && v[w] >= 0 &&
                                   !((before[w] >> (v[w] & 31)) & 1u);
                const unsigned long long mask = __ballot(fresh);
                if (fresh) cand_id[n + lane_rank(mask)] = v[w];
                n += __popcll(mask);
            }
            if (n == 0) continue;
            wave_sync();
            eval_rows<DP8>(a.storage, qv, cand_id, cand_key, n, dp, lane);
            n_dist += n;
            wave_sync();
        }

        // the pool is the answer, best first
        int64_t *oI = a.out_I + (size_t)q * a.k;
        float *oD = a.out_D + (size_t)q * a.k;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int r = s * kWave + lane;
            if (r < a.k) {
                const unsigned val = entry_val(pool.e[s]);
                int64_t id = -1;
                if (val != 0xffffffffu)
                    id = (val & kGlobal) ? (int64_t)(val & kIdMask)
                                         : (int64_t)a.gid[val & kIdMask];
                oI[r] = id;
                oD[r] = key_to_float(entry_key(pool.e[s]));
            }
        }
        wave_sync();

        if (a.counters && lane == 0) {
            atomicAdd(&a.counters[0], (unsigned long long)n_expand);
            atomicAdd(&a.counters[1], (unsigned long long)n_adj);
            atomicAdd(&a.counters[2], (unsigned long long)n_dist);
            atomicAdd(&a.counters[3], (unsigned long long)n_admit);
            atomicAdd(&a.counters[4], (unsigned long long)a.k);
        }
    }
}

typedef void (*WideFn)(WideArgs);

template <int S>
WideFn pick_wide_dp(int dp) {
    switch (dp) {
        case 32: return wide_kernel<S, 4>;
        case 64: return wide_kernel<S, 8>;
        case 128: return wide_kernel<S, 16>;
        default: return wide_kernel<S, 0>;
    }
}

// the pool holds the ladder size of the exact mode, rounded up to whole
// registers
WideFn pick_wide(int H, int dp) {
    switch ((H + kWave - 1) / kWave) {
        case 1: return pick_wide_dp<1>(dp);
        case 2: return pick_wide_dp<2>(dp);
        case 3: return pick_wide_dp<3>(dp);
        case 4: return pick_wide_dp<4>(dp);
        case 6: return pick_wide_dp<6>(dp);
        case 8: return pick_wide_dp<8>(dp);
        case 16: return pick_wide_dp<16>(dp);
        case 32: return pick_wide_dp<32>(dp);
        default: return nullptr;
    }
}

struct WidePlan {
    int n_slots, words_per_slot, lds_bytes;
    size_t workspace_bytes;
    WideFn fn;
};

int make_wide_plan(int64_t n_storage, int64_t batch, int dp, int ef_total, WidePlan *p) {
    if (n_storage <= 0 || batch < 0) return PA_E_SHAPE;
    if (n_storage > (int64_t)kIdMask) return PA_E_RANGE;
    if (dp <= 0 || dp % 8) return PA_E_DIM;
    if (ef_total < 1 || ef_total > PA_MAX_EF_TOTAL) return PA_E_EF;
    const int H = pa_heap_size(ef_total);
    p->fn = pick_wide(H, dp);
    if (!p->fn) return PA_E_EF;
    p->lds_bytes = (dp == 32 || dp == 64 || dp == 128) ? 0 : query_floats(dp) * 4;
    int dev = 0, cus = 0, per_cu = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return (int)e;
    {
        static std::mutex mutex;
        static std::map<std::tuple<int, const void *, int>, std::pair<int, int>> known;
        std::lock_guard<std::mutex> guard(mutex);
        const auto key = std::make_tuple(dev, reinterpret_cast<const void *>(p->fn), p->lds_bytes);
        auto it = known.find(key);
        if (it == known.end()) {
            e = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
            if (e == hipSuccess)
                e = hipOccupancyMaxActiveBlocksPerMultiprocessor(
                    &per_cu, reinterpret_cast<const void *>(p->fn), kWave, p->lds_bytes);
            if (e != hipSuccess) return (int)e;
            it = known.emplace(key, std::make_pair(cus, per_cu)).first;
        }
        cus = it->second.first, per_cu = it->second.second;
    }
    if (per_cu < 1) per_cu = 1;
#ifndef PA_WIDE_MAX_WAVES_PER_CU
#define PA_WIDE_MAX_WAVES_PER_CU 20
#endif
    if (per_cu > PA_WIDE_MAX_WAVES_PER_CU) per_cu = PA_WIDE_MAX_WAVES_PER_CU;
    int64_t slots = (int64_t)per_cu * cus;
    if (slots > batch) slots = batch;
    if (slots < 1) slots = 1;
    p->n_slots = (int)slots;
    p->words_per_slot = (int)((((n_storage + 31) / 32 + kSlotAlignWords - 1) / kSlotAlignWords) *
                              kSlotAlignWords);
    p->workspace_bytes = kWorkCounterBytes + (size_t)p->n_slots * p->words_per_slot * 4;
    return PA_OK;
}

}  // namespace

extern "C" int pa_traverse_wide_plan(int64_t n_storage, int64_t batch, int dp,
                                     int ef_total, int *n_slots,
                                     size_t *workspace_bytes) {
    WidePlan p;
    const int rc = make_wide_plan(n_storage, batch, dp, ef_total, &p);
    if (rc != PA_OK) return rc;
    if (n_slots) *n_slots = p.n_slots;
    if (workspace_bytes) *workspace_bytes = p.workspace_bytes;
    return PA_OK;
}

extern "C" int pa_traverse_wide(int64_t *out_I, float *out_D, const int32_t *adj,
                                const int32_t *gid, const int64_t *mapping,
                                const float *storage, const float *query,
                                const int64_t *init_I, const float *init_D,
                                int64_t batch, int64_t n_nodes, int64_t n_storage,
                                int dp, int n_init, int beam, int ef,
                                int n_neighbors, int width, void *workspace,
                                size_t workspace_bytes, uint64_t *counters,
                                void *stream_) {
    if (batch < 0 || n_nodes <= 0 || n_init < 0 || beam < 1 || ef < 1)
        return PA_E_SHAPE;
    if (width < 1 || width > kMaxWidth) return PA_E_SHAPE;
    if (n_nodes > (int64_t)kIdMask || batch >= (1ll << 31)) return PA_E_RANGE;
    if (n_neighbors < 1 || n_neighbors > PA_MAX_NEIGHBORS) return PA_E_NEIGHBORS;
    if ((int64_t)beam * ef > PA_MAX_EF_TOTAL) return PA_E_EF;
    WidePlan p;
    const int rc = make_wide_plan(n_storage, batch, dp, beam * ef, &p);
    if (rc != PA_OK) return rc;
    if (batch == 0) return PA_OK;
    if (!out_I || !out_D || !adj || !gid || !mapping || !storage || !query ||
        !workspace || (n_init > 0 && (!init_I || !init_D)))
        return PA_E_NULL;
    if (workspace_bytes < p.workspace_bytes) return PA_E_WORKSPACE;
    if (reinterpret_cast<uintptr_t>(workspace) % 256) return PA_E_WORKSPACE;

    WideArgs a;
    a.out_I = out_I, a.out_D = out_D;
    a.adj = adj, a.gid = gid, a.mapping = mapping;
    a.storage = storage, a.query = query;
    a.init_I = init_I, a.init_D = init_D;
    a.work_counter = reinterpret_cast<int *>(workspace);
    a.seen = reinterpret_cast<uint32_t *>(
        reinterpret_cast<unsigned char *>(workspace) + kWorkCounterBytes);
    a.counters = reinterpret_cast<unsigned long long *>(counters);
    a.batch = (int)batch, a.n_nodes = (int)n_nodes, a.n_storage = (int)n_storage;
    a.dp = dp, a.n_init = n_init, a.k = beam * ef, a.deg = n_neighbors;
    a.max_iter = 2 * beam * ef < 1024 ? 2 * beam * ef : 1024;
    a.width = width;
    a.words_per_slot = p.words_per_slot;

    hipStream_t stream = (hipStream_t)stream_;
    reset_wide_counter<<<1, 1, 0, stream>>>(a.work_counter);
    p.fn<<<p.n_slots, kWave, p.lds_bytes, stream>>>(a);
    return (int)hipGetLastError();
}
