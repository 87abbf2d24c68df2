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
//     lane a of the quad owns accumulators 2a and 2a+1 and streams its 8
//     bytes of every 32-byte group.
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

using namespace pa;

namespace {

constexpr int kSlotAlignWords = 256;   // bitmask slice: multiple of 1 KiB
constexpr int kWorkCounterBytes = 256; // head of the workspace
#ifndef PA_SEEN_LOG2
#define PA_SEEN_LOG2 10
#endif
constexpr int kSeenCacheLog2 = PA_SEEN_LOG2;
constexpr int kSeenCache = 1 << kSeenCacheLog2;  // LDS words remembering visited rows

// ---- open list: heapq.cuh, top of the heap in registers ----------------------
//
// The reference's open list is an array heap of 2H cells with the sift rules
// of extension/inc/heapq.cuh:13-88.  Here node i of that array is node
// j = i + 1 (children 2j and 2j + 1), level L holds j in [2^L, 2^(L+1)).
//
// Levels 0..7 live in registers, one node per lane: bank A levels 0..5 (node j
// in lane j), bank B level 6 (lane j - 64), banks C and D the left and right
// children of level 7 (lane (j - 128) / 2), so a sibling pair is always two
// v_readlane of known registers.  Deeper nodes sit in LDS at [j - 256] as
// (key, value), a sibling pair per aligned 16 bytes.  Keys are kept as
// order-preserving integers (float_to_key) so that every comparison of a walk
// is a scalar integer compare.  All lanes run the same, uniform, control flow; the walks
// are unrolled by level so that each level is a dozen instructions.  After
// each operation the heap is, cell for cell, the reference's.  Every lane
// stores the same values to the same LDS cells and reads the same cells, so a
// lane only ever reads back its own stores and the walks need no fences.
__device__ __forceinline__ int float_to_key(float x) {
    const int b = __float_as_int(x);
    return b ^ ((b >> 31) & 0x7fffffff);
}
__device__ __forceinline__ float key_to_float(int k) {
    return __int_as_float(k ^ ((k >> 31) & 0x7fffffff));
}

// c + (a != b) on the scalar unit (the compiler routes the boolean of a
// uniform compare through a vector register otherwise).
__device__ __forceinline__ int add_if_ne(int c, int a, int b) {
    int r;
    asm("s_cmp_lg_u32 %1, %2\n\ts_addc_u32 %0, %3, 0"
        : "=s"(r)
        : "s"(a), "s"(b), "s"(c)
        : "scc");
    return r;
}

constexpr int floor_log2(int x) { return x <= 1 ? 0 : 1 + floor_log2(x >> 1); }

// c + bit `idx` of a 64-bit lane mask, on the scalar unit.
__device__ __forceinline__ int add_if_bit(int c, unsigned long long mask, int idx) {
    int r;
    asm("s_bitcmp1_b64 %1, %2\n\ts_addc_u32 %0, %3, 0"
        : "=s"(r)
        : "s"(mask), "s"(idx), "s"(c)
        : "scc");
    return r;
}

template <int H>
struct OpenList {
    static constexpr int kSize = 2 * H;           // cells of the reference heap
    static constexpr int kDepth = floor_log2(kSize);  // deepest level
    static constexpr int kRegNodes = 256;
    static constexpr int kLdsCells = kSize + 2 > kRegNodes ? kSize + 2 - kRegNodes : 0;
    static constexpr int kInf = 0x7f800000;       // float_to_key(+inf)
    int Ak, Av, Bk, Bv, Ck, Cv, Dk, Dv;
    int2 *cells;  // node j >= 256 at [j - 256] as (key, value); 16-byte aligned

    __device__ __forceinline__ static int rl(int x, int l) {
        return __builtin_amdgcn_readlane(x, l);
    }
    // storage class of a level: 0 bank A, 1 bank B, 2 banks C/D, 3 LDS
    __device__ __forceinline__ static constexpr int kind(int level) {
        return level <= 5 ? 0 : level == 6 ? 1 : level == 7 ? 2 : 3;
    }

    __device__ __forceinline__ void reset(int lane) {
        Ak = Bk = Ck = Dk = kInf;
        Av = Bv = Cv = Dv = -1;
        for (int i = lane; i < kLdsCells; i += kWave) cells[i] = make_int2(kInf, -1);
    }

    // keys (and values) of the sibling pair (c, c + 1), c even, of a level.
    // KIND and VALS are constants once the level loops are unrolled.
    __device__ __forceinline__ void pair(const int KIND, const bool VALS, int c,
                                         int &ka, int &kb, int &va,
                                         int &vb) const {
        if (KIND == 0) {
            ka = rl(Ak, c), kb = rl(Ak, c + 1);
            if (VALS) va = rl(Av, c), vb = rl(Av, c + 1);
        } else if (KIND == 1) {
            const int l = c - 64;
            ka = rl(Bk, l), kb = rl(Bk, l + 1);
            if (VALS) va = rl(Bv, l), vb = rl(Bv, l + 1);
        } else if (KIND == 2) {
            const int l = (c - 128) >> 1;
            ka = rl(Ck, l), kb = rl(Dk, l);
            if (VALS) va = rl(Cv, l), vb = rl(Dv, l);
        } else {
            // one 16-byte read: both children with their values
            const int4 p = *reinterpret_cast<const int4 *>(cells + (c - kRegNodes));
            if (VALS) va = uni(p.y), vb = uni(p.w);
            ka = uni(p.x), kb = uni(p.z);
        }
    }
    __device__ __forceinline__ int key_of(const int KIND, int j) const {
        if (KIND == 0) return rl(Ak, j);
        if (KIND == 1) return rl(Bk, j - 64);
        if (KIND == 2) {
            // both banks are read and one result is kept: two instructions
            // more than a branch on the parity of j would need, no branch
            const int l = (j - 128) >> 1;
            const int left = rl(Ck, l), right = rl(Dk, l);
            return (j & 1) ? right : left;
        }
        return uni(cells[j - kRegNodes].x);
    }
    __device__ __forceinline__ int val_of(const int KIND, int j) const {
        if (KIND == 0) return rl(Av, j);
        if (KIND == 1) return rl(Bv, j - 64);
        if (KIND == 2) {
            const int l = (j - 128) >> 1;
            const int left = rl(Cv, l), right = rl(Dv, l);
            return (j & 1) ? right : left;
        }
        return uni(cells[j - kRegNodes].y);
    }
    // lane l of a key bank and of its value bank := two uniform values
    // (v_writelane takes one scalar register besides M0, which holds the lane)
    __device__ __forceinline__ static void set_lane(int &kbank, int &vbank, int k,
                                                    int v, int l) {
        asm("s_mov_b32 m0, %4\n\t"
            "s_nop 0\n\t"
            "v_writelane_b32 %0, %2, m0\n\t"
            "v_writelane_b32 %1, %3, m0"
            : "+v"(kbank), "+v"(vbank)
            : "s"(k), "s"(v), "s"(l)
            : "m0");
    }
    __device__ __forceinline__ void put(const int KIND, int j, int k, int v,
                                        int lane) {
        if (KIND == 0) {
            set_lane(Ak, Av, k, v, j);
        } else if (KIND == 1) {
            set_lane(Bk, Bv, k, v, j - 64);
        } else if (KIND == 2) {
            // lane-masked selects on both banks instead of a branch on the
            // parity of j around two v_writelane
            const int l = (j - 128) >> 1;
            const bool here = lane == l;
            const bool right = j & 1;
            Ck = (here && !right) ? k : Ck;
            Cv = (here && !right) ? v : Cv;
            Dk = (here && right) ? k : Dk;
            Dv = (here && right) ? v : Dv;
        } else {
            // every lane stores the same pair to the same cell: one LDS
            // write, and no divergent branch around it
            cells[j - kRegNodes] = make_int2(k, v);
        }
    }

    // Which child a walk takes, for every sibling pair of the register levels
    // at once: lane-parallel compares against the sibling (one DPP move per
    // bank), read back as lane masks, so that a level of the walk is three
    // scalar instructions and no register read.  LARGER selects the rule of
    // heap_replace (strictly larger right child), else that of the sift of a
    // pop (strictly smaller right child); left wins ties in both.  In banks A
    // and B bit i of the mask tells about the pair whose right child sits in
    // lane i; in banks C/D lane i holds both children.
    struct Choice {
        unsigned long long a, b, cd;
    };
    template <bool LARGER>
    __device__ __forceinline__ Choice choices() const {
        Choice ch;
        const int sa = __builtin_amdgcn_update_dpp(Ak, Ak, 0xB1, 0xF, 0xF, false);
        ch.a = __ballot(LARGER ? Ak > sa : Ak < sa);
        ch.b = 0, ch.cd = 0;
        if (kDepth >= 6) {
            const int sb = __builtin_amdgcn_update_dpp(Bk, Bk, 0xB1, 0xF, 0xF, false);
            ch.b = __ballot(LARGER ? Bk > sb : Bk < sb);
        }
        if (kDepth >= 7) ch.cd = __ballot(LARGER ? Dk > Ck : Dk < Ck);
        return ch;
    }
    // the child of j the walk takes on register level L (1..7), L < kDepth
    // or the pair is known to be complete: 2j + (bit of the pair in the
    // level's mask), three scalar instructions.  s_bitcmp1_b64 looks at the
    // low six bits of its index only, so node numbers serve as lane numbers
    // (bank B holds node j in lane j - 64, banks C/D the children of node j
    // in lane j - 64).
    __device__ __forceinline__ int step_down(const int L, int j,
                                             const Choice &ch) const {
        int r;
        if (kind(L) <= 1) {
            // t = 2j + 1, the right child, whose lane holds the pair's bit
            asm("s_lshl1_add_u32 %0, %1, 1\n\t"
                "s_bitcmp1_b64 %2, %0\n\t"
                "s_addc_u32 %0, %0, -1"
                : "=&s"(r)
                : "s"(j), "s"(kind(L) == 0 ? ch.a : ch.b)
                : "scc");
        } else {
            asm("s_lshl_b32 %0, %1, 1\n\t"
                "s_bitcmp1_b64 %2, %1\n\t"
                "s_addc_u32 %0, %0, 0"
                : "=&s"(r)
                : "s"(j), "s"(ch.cd)
                : "scc");
        }
        return r;
    }

    // heapq.cuh:37-45 with the sift of :13-29: the root leaves, (inf, -1)
    // sinks along the smaller child (left on ties).  The reference stops when
    // that child is (inf, -1) too; going on to the bottom instead only copies
    // (inf, -1) over (inf, -1) — every infinite cell carries -1 — so the
    // final state is the same and the walk is straight-line code.  Levels
    // 1..kDepth-1 are complete; on level kDepth only nodes up to kSize exist
    // and node kSize has no sibling (its absent sibling's cell holds +inf and
    // is never the smaller one).
    __device__ __forceinline__ void pop(int lane, int &out_k, int &out_v) {
        out_k = rl(Ak, 1);
        out_v = rl(Av, 1);
        const Choice ch = choices<false>();
        // Register levels in three passes, so that no read waits for a write
        // of the same bank: the path (masks only), then every entry on it,
        // then the stores.  Reading first is the same thing: a level's store
        // goes to the cell above the one read.
        constexpr int kRegLevels = kDepth < 7 ? kDepth : 7;
        int node[kRegLevels + 1];
        node[0] = 1;
        bool cut = false;  // level kDepth has no node below node[kDepth - 1]
#pragma unroll
        for (int L = 1; L <= kRegLevels; ++L) {
            if (L == kDepth && 2 * node[L - 1] > kSize) {
                cut = true;
                node[L] = node[L - 1];
            } else {
                node[L] = step_down(L, node[L - 1], ch);
            }
        }
        int ck[kRegLevels + 1], cv[kRegLevels + 1];
#pragma unroll
        for (int L = 1; L <= kRegLevels; ++L) {
            ck[L] = key_of(kind(L), node[L]);
            cv[L] = val_of(kind(L), node[L]);
        }
#pragma unroll
        for (int L = 1; L <= kRegLevels; ++L) {
            if (L == kDepth && cut) {
                put(kind(L - 1), node[L - 1], kInf, -1, lane);
                return;
            }
            put(kind(L - 1), node[L - 1], ck[L], cv[L], lane);
        }
        int j = node[kRegLevels];
#pragma unroll
        for (int L = kRegLevels + 1; L <= kDepth; ++L) {
            if (L == kDepth && 2 * j > kSize) {
                put(kind(L - 1), j, kInf, -1, lane);
                return;
            }
            int ka, kb, va, vb;
            pair(3, true, 2 * j, ka, kb, va, vb);
            if (L == kDepth) kb = 2 * j == kSize ? ka : kb;
            const int k = min(ka, kb);
            const int v = k != ka ? vb : va;
            const int c = add_if_ne(2 * j, k, ka);
            put(kind(L - 1), j, k, v, lane);
            j = c;
        }
        put(kind(kDepth), j, kInf, -1, lane);
    }

    // heapq.cuh:47-77: walk to a leaf through the larger child (left on
    // ties), overwrite it when the new key is strictly smaller, let the new
    // entry rise.  In two parts so that the caller can put independent work
    // between them: the walk is straight-line code, the rise branches.
    struct Leaf {
        int j;       // the leaf
        int key;     // its key
        bool bottom; // it is on level kDepth
    };
    __device__ __forceinline__ Leaf walk_to_large_leaf() const {
        const Choice ch = choices<true>();
        int j = 1;
        bool bottom = true;  // the walk reached level kDepth
        int walked_key = 0;  // key of node j when its level is an LDS level
#pragma unroll
        for (int L = 1; L <= kDepth; ++L) {
            if (L == kDepth && 2 * j > kSize) {
                bottom = false;
                break;
            }
            if (kind(L) <= 2) {
                // node kSize has no sibling: the left child it is
                j = (L == kDepth && 2 * j == kSize) ? 2 * j : step_down(L, j, ch);
            } else {
                int ka, kb, va, vb;
                pair(3, false, 2 * j, ka, kb, va, vb);
                if (L == kDepth) kb = 2 * j == kSize ? ka : kb;
                walked_key = max(ka, kb);
                j = add_if_ne(2 * j, walked_key, ka);
            }
        }
        // the leaf's key: the walk has it already when the leaf is in LDS
        Leaf leaf;
        leaf.j = j, leaf.bottom = bottom;
        if (bottom)
            leaf.key = kind(kDepth) == 3 ? walked_key : key_of(kind(kDepth), j);
        else
            leaf.key = kind(kDepth - 1) == 3 ? walked_key : key_of(kind(kDepth - 1), j);
        return leaf;
    }
    // SPARSE: the heap is nearly empty (the entries of a query are pushed),
    // so most ancestors of the leaf are (inf, -1), and so is everything below
    // such an ancestor: moving it down would write (inf, -1) over (inf, -1)
    // and is left out.
    template <bool SPARSE = false>
    __device__ __forceinline__ void replace_leaf(const Leaf &leaf, int k, int v,
                                                 int lane) {
        if (k >= leaf.key) return;
        int j = leaf.j;
        // one store per level: the parent's entry while it is larger than
        // the new key, the new entry where the rise stops
        auto rise = [&](const int L) -> bool {
            const int up = j >> 1;
            const int pk = key_of(kind(L - 1), up);
            if (SPARSE && pk == kInf) {
                j = up;
                return false;
            }
            const int pv = val_of(kind(L - 1), up);
            const bool stop = pk <= k;
            put(kind(L), j, stop ? k : pk, stop ? v : pv, lane);
            j = up;
            return stop;
        };
        if (leaf.bottom && rise(kDepth)) return;
#pragma unroll
        for (int L = kDepth - 1; L >= 1; --L)
            if (rise(L)) return;
        put(0, 1, k, v, lane);
    }
    template <bool SPARSE = false>
    __device__ __forceinline__ void replace(int k, int v, int lane) {
        const Leaf leaf = walk_to_large_leaf();
        replace_leaf<SPARSE>(leaf, k, v, lane);
    }
};

// ---- result list: the H smallest distances ------------------------------------
//
// The reference keeps them in a heap of negated keys whose root is the worst
// kept (traverse_cpu.cpp:21-39): a candidate enters iff its distance is
// strictly below that root, and replaces it.  Which array cell holds what has
// no effect on the search; only the set and its maximum do.  Here the cells
// are a flat LDS array, S per lane (lane l owns cells l*S .. l*S+S-1), of which
// the registers keep only each lane's maximum, the wavefront's maximum and the
// position of one cell that holds it: an insert is one store to that cell,
// one read of every lane's own cells and a wavefront maximum.  Empty cells
// hold +inf (so the maximum is +inf until H candidates came), cells beyond H
// hold -inf and never win.

template <int S>
struct Results {
    static constexpr int kInf = 0x7f800000;      // float_to_key(+inf)
    static constexpr int kNegInf = (int)0x807fffff;  // float_to_key(-inf)
    int *rk;      // LDS: float_to_key of the distance, kWave * S cells
    int *rv;      // device memory: the values, same cells (written once per
                  // insert, read at the end; every lane stores the same value
                  // to a cell and so reads back its own store)
    int lane_max;
    int worst;    // uniform
    int pos;      // uniform: a cell whose key is `worst`

    __device__ __forceinline__ void init(int H, int lane) {
        lane_max = kNegInf;
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int c = lane * S + s;
            const int k = c < H ? kInf : kNegInf;
            rk[c] = k, rv[c] = -1;
            lane_max = max(lane_max, k);
        }
        worst = kInf;
        pos = 0;
    }
    // Caller has checked k < worst.  In two parts so that the caller can put
    // independent work between the LDS traffic and its use.
    __device__ __forceinline__ void begin_insert(int k, int v, int lane, int (&key)[S]) {
        // Every lane stores the same pair to the same cell, so the lane that
        // owns the cell reads back its own store: program order is enough.
        rk[pos] = k, rv[pos] = v;
#pragma unroll
        for (int s = 0; s < S; ++s) key[s] = rk[lane * S + s];
    }
    __device__ __forceinline__ void finish_insert(int lane, const int (&key)[S]) {
        int m = key[0];
#pragma unroll
        for (int s = 1; s < S; ++s) m = max(m, key[s]);
        lane_max = m;
        worst = wave_max_key(lane_max);
        // the first lane that holds the new maximum, its first such cell
        const int holder = __builtin_ctzll(__ballot(lane_max == worst));
        int c = lane * S + S - 1;
#pragma unroll
        for (int s = S - 2; s >= 0; --s) c = key[s] == worst ? lane * S + s : c;
        pos = __builtin_amdgcn_readlane(c, holder);
    }
    __device__ __forceinline__ void insert(int k, int v, int lane) {
        int key[S];
        begin_insert(k, v, lane, key);
        finish_insert(lane, key);
    }
};

// ---- distances ---------------------------------------------------------------

// Squared L2 from the query (LDS) to the storage rows listed in cand_id[0..n),
// written to cand_key: 16 rows per pass, four lanes per row.
template <int DP8>
__device__ __forceinline__ void eval_rows(const float *__restrict__ storage,
                                          const float *qv, const int *cand_id,
                                          float *cand_key, int n, int dp,
                                          int lane) {
    const int quad = lane >> 2, part = lane & 3;
    const float2 *qq = reinterpret_cast<const float2 *>(qv) + part * query_run(dp >> 3);
    for (int base = 0; base < n; base += kRowsPerPass) {
        const int c = base + quad;
        const bool active = c < n;
        const float2 *row = reinterpret_cast<const float2 *>(storage);
        if (active)
            row = reinterpret_cast<const float2 *>(
                      storage + (size_t)cand_id[c] * (size_t)dp) + part;
        const float s = quad_square_dist<DP8>(row, qq, dp >> 3, active);
        if (active && part == 0) cand_key[c] = s;
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
    int words_per_slot, slot_stride, sort_n, lds_cells;
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

template <int H, int DP8>
__global__ __launch_bounds__(kWave) PA_OCCUPANCY(H) void traverse_kernel(TraverseArgs a) {
    // One static block, in this order: the compiler then knows every LDS
    // address, and a heap cell [j - 256] is the scalar j * 8 plus a positive
    // constant that fits the instruction's offset field.
    constexpr int S = (H + kWave - 1) / kWave;
    constexpr int kSortN = H <= kWave ? kWave : 1 << (floor_log2(H - 1) + 1);
    constexpr int kHeapCells =
        OpenList<H>::kLdsCells > kSortN ? OpenList<H>::kLdsCells : kSortN;
    struct Lds {
        uint32_t seen_cache[kSeenCache];
        int cand_id[kWave];
        float cand_key[kWave];
        float query[DP8 ? query_floats(8 * DP8) : 4];
        int2 heap[kHeapCells];  // open list tail; the final sort reuses it
        int res_key[S * kWave];  // result list: keys (the values are in the slot's
                                 // memory behind the visited slice)
    };
    __shared__ __align__(16) Lds lds;
    extern __shared__ __align__(16) float query_any_length[];  // DP8 == 0 only
    const int lane = threadIdx.x;
    float *okey = reinterpret_cast<float *>(lds.heap);
    int *oval = reinterpret_cast<int *>(okey + kHeapCells);
    OpenList<H> open;
    open.cells = lds.heap;
    int *cand_id = lds.cand_id;
    float *cand_key = lds.cand_key;
    float *qv = DP8 ? lds.query : query_any_length;
    const int dp = DP8 ? DP8 * 8 : a.dp;
    uint32_t *seen_cache = lds.seen_cache;
    const bool use_cache = a.n_storage <= (0xffff << kSeenCacheLog2);
    const int deg = a.deg;
    uint32_t *seen = a.seen + (size_t)blockIdx.x * (size_t)a.slot_stride;

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
        for (int w = lane * 4; w < a.words_per_slot; w += kWave * 4)
            *reinterpret_cast<uint4 *>(seen + w) = make_uint4(0, 0, 0, 0);
        for (int i = lane; i < dp; i += kWave)
            qv[query_slot(i, dp >> 3)] = a.query[(size_t)q * dp + i];
        for (int i = lane; i < kSeenCache; i += kWave) seen_cache[i] = 0xffffffffu;
        open.reset(lane);
        Results<S> res;
        res.rk = lds.res_key;
        res.rv = reinterpret_cast<int *>(seen + a.words_per_slot);
        res.init(H, lane);
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
        // the pop (the atomics are in flight while the pop sifts).  Its row of
        // neighbour ids is needed for that, and is requested even earlier,
        // before the inserts, for the node that will most likely be the root
        // after them: the best new candidate if it beats the present root and
        // the admission bound, else the present root.  That load is only a
        // read; when the guess is wrong the row is loaded again.  If the
        // search ends at the next pop instead, the marks set for a node that
        // is never expanded are harmless: the slice is cleared per query.
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
        int v = load_row(OpenList<H>::rl(open.Av, 1));
        uint32_t before = test_and_set(v);
        for (int step = 0; step < a.max_iter; ++step) {
            int uk, u;
            open.pop(lane, uk, u);
            PA_TIMER(0);
            if (u == -1 || uk >= res.worst) break;
            n_expand += 1;
            int guess = -3, guess_row = -1;
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

                    const int d = float_to_key(lane < n ? cand_key[lane] : INFINITY);
                    const int id = lane < n ? cand_id[lane] : -1;
                    // most likely next node; first candidate on ties, as the
                    // rise of an equal key stops below the older one
                    const int d_min = -wave_max_key(-d);
                    guess = OpenList<H>::rl(open.Av, 1);
                    if (d_min < OpenList<H>::rl(open.Ak, 1) && d_min < res.worst)
                        guess = __builtin_amdgcn_readlane(
                            id, __builtin_ctzll(__ballot(d == d_min)));
                    guess_row = load_row(guess);

                    // heap_update, traverse_cpu.cpp:25-39, in adjacency order
                    unsigned long long todo = __ballot(d < res.worst);
                    while (todo) {
                        const int j = __builtin_ctzll(todo);
                        todo &= todo - 1;
                        const int dj = __builtin_amdgcn_readlane(d, j);
                        if (dj >= res.worst) continue;
                        const int vj = __builtin_amdgcn_readlane(id, j);
                        int mine[S];
                        res.begin_insert(dj, vj, lane, mine);
                        const typename OpenList<H>::Leaf leaf = open.walk_to_large_leaf();
                        res.finish_insert(lane, mine);
                        open.replace_leaf(leaf, dj, vj, lane);
                        n_admit += 1;
                    }
                    PA_TIMER(4);
                }
            }
            const int r = OpenList<H>::rl(open.Av, 1);
            v = r == guess ? guess_row : load_row(r);
            before = test_and_set(v);
            PA_TIMER(1);
        }

        // traverse_cpu.cpp:138-148: storage rows -> global ids, then the
        // entries compete for a result slot.
        wave_sync();
#pragma unroll
        for (int s = 0; s < S; ++s) {
            const int row = res.rv[lane * S + s];
            if (row >= 0) res.rv[lane * S + s] = a.gid[row];
        }
        wave_sync();
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
            while (todo) {
                const int j = __builtin_ctzll(todo);
                todo &= todo - 1;
                const int dj = __builtin_amdgcn_readlane(dk, j);
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
            const int e = lane * S + s;
            if (e < H) okey[e] = key_to_float(res.rk[e]), oval[e] = res.rv[e];
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
    int H, sort_n, lds_cells, lds_bytes, n_slots, words_per_slot, slot_stride;
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
    // LDS part of the open list (nodes 256.. of 2H, one spare), reused by the
    // final sort of sort_n cells
    const int tail = 2 * p->H + 2 - 256;
    p->lds_cells = tail > p->sort_n ? tail : p->sort_n;
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
    // a slot: the visited slice, then the values of the result list
    p->slot_stride = p->words_per_slot + round_up(p->H, kWave);
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
    if (workspace_bytes < p.workspace_bytes) return PA_E_WORKSPACE;
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
    a.lds_cells = p.lds_cells;

    hipStream_t stream = (hipStream_t)stream_;
    reset_work_counter<<<1, 1, 0, stream>>>(a.work_counter);
    p.fn<<<p.n_slots, kWave, p.lds_bytes, stream>>>(a);
    return (int)hipGetLastError();
}
