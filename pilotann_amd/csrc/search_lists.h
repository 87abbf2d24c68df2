// Device-side lists of the per-query search, shared by the subgraph traversal
// and the full-dimension refine (gfx950, one 64-lane wavefront per query): the
// open list (the reference's array heap, extension/inc/heapq.cuh:13-88, top
// levels in registers), the result list, the exact visited table of the refine,
// and the batched row distances.
#ifndef PILOTANN_SEARCH_LISTS_H
#define PILOTANN_SEARCH_LISTS_H

#include "device_common.h"

namespace pa {

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
// (key, value), a sibling pair per aligned 16 bytes; with DEEP the levels
// from DEEP on sit in device memory instead (the wavefront's own region, at
// [j - 2^DEEP], same cells): a long list then takes less LDS, more
// wavefronts fit a compute unit, and a walk pays one memory round trip per
// such level.  Keys are kept as
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

// Cells of an open list of 2H cells that sit in device memory when the levels
// from `deep` on do (0: none do).
constexpr int open_list_deep_cells(int H, int deep) {
    return deep >= 8 && deep <= floor_log2(2 * H) ? 2 * H + 2 - (1 << deep) : 0;
}

template <int H, int DEEP = 0>
struct OpenList {
    static constexpr int kSize = 2 * H;           // cells of the reference heap
    static constexpr int kDepth = floor_log2(kSize);  // deepest level
    static constexpr int kRegNodes = 256;
    static constexpr int kDeepCells = open_list_deep_cells(H, DEEP);
    static constexpr int kDeepFrom = kDeepCells ? DEEP : kDepth + 1;
    static constexpr int kDeepBase = 1 << kDeepFrom;  // first node in device memory
    static constexpr int kLdsCells =
        kDeepCells ? kDeepBase - kRegNodes
                   : (kSize + 2 > kRegNodes ? kSize + 2 - kRegNodes : 0);
    static constexpr int kInf = 0x7f800000;       // float_to_key(+inf)
    int Ak, Av, Bk, Bv, Ck, Cv, Dk, Dv;
    int2 *cells;  // node j in [256, kDeepBase) at [j - 256] as (key, value); 16-byte aligned
    int2 *deep;   // node j >= kDeepBase at [j - kDeepBase], device memory, 16-byte aligned
    int4 pending;   // pop(): the requested pair of level kDeepFrom, until pop_finish()
    int pending_j;  // its parent, 0 = nothing pending (uniform)

    __device__ __forceinline__ static int rl(int x, int l) {
        return __builtin_amdgcn_readlane(x, l);
    }
    // storage class of a level: 0 bank A, 1 bank B, 2 banks C/D, 3 LDS,
    // 4 device memory
    __device__ __forceinline__ static constexpr int kind(int level) {
        return level <= 5 ? 0 : level == 6 ? 1 : level == 7 ? 2
                                           : level < kDeepFrom ? 3 : 4;
    }

    __device__ __forceinline__ void reset(int lane) {
        Ak = Bk = Ck = Dk = kInf;
        Av = Bv = Cv = Dv = -1;
        for (int i = lane; i < kLdsCells; i += kWave) cells[i] = make_int2(kInf, -1);
        for (int i = lane; i < kDeepCells; i += kWave) deep[i] = make_int2(kInf, -1);
        pending_j = 0;
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
            const int4 p = KIND == 3
                ? *reinterpret_cast<const int4 *>(cells + (c - kRegNodes))
                : *reinterpret_cast<const int4 *>(deep + (c - kDeepBase));
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
        return uni(KIND == 3 ? cells[j - kRegNodes].x : deep[j - kDeepBase].x);
    }
    __device__ __forceinline__ int val_of(const int KIND, int j) const {
        if (KIND == 0) return rl(Av, j);
        if (KIND == 1) return rl(Bv, j - 64);
        if (KIND == 2) {
            const int l = (j - 128) >> 1;
            const int left = rl(Cv, l), right = rl(Dv, l);
            return (j & 1) ? right : left;
        }
        return uni(KIND == 3 ? cells[j - kRegNodes].y : deep[j - kDeepBase].y);
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
        } else if (KIND == 3) {
            // every lane stores the same pair to the same cell: one LDS
            // write, and no divergent branch around it
            cells[j - kRegNodes] = make_int2(k, v);
        } else {
            deep[j - kDeepBase] = make_int2(k, v);
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
        pending_j = 0;
#pragma unroll
        for (int L = kRegLevels + 1; L <= kDepth; ++L) {
            if (L == kDepth && 2 * j > kSize) {
                put(kind(L - 1), j, kInf, -1, lane);
                return;
            }
            if (kDeepCells && L == kDeepFrom) {
                // the pair is requested; pop_finish() goes on from here
                pending = *reinterpret_cast<const int4 *>(deep + (2 * j - kDeepBase));
                pending_j = j;
                return;
            }
            int ka, kb, va, vb;
            pair(kind(L), true, 2 * j, ka, kb, va, vb);
            if (L == kDepth) kb = 2 * j == kSize ? ka : kb;
            const int k = min(ka, kb);
            const int v = k != ka ? vb : va;
            const int c = add_if_ne(2 * j, k, ka);
            put(kind(L - 1), j, k, v, lane);
            j = c;
        }
        put(kind(kDepth), j, kInf, -1, lane);
    }
    // The levels of a pop that sit in device memory.  pop() only requests the
    // first pair it needs from there; the caller puts the work that does not
    // touch the list (the root is in registers) between the two, and calls
    // this before the next walk or pop.  Nothing to do without such levels.
    __device__ __forceinline__ void pop_finish(int lane) {
        if (!kDeepCells) return;
        int j = pending_j;
        if (j == 0) return;
        pending_j = 0;
#pragma unroll
        for (int L = kDeepFrom; L <= kDepth; ++L) {
            if (L == kDepth && 2 * j > kSize) {
                put(kind(L - 1), j, kInf, -1, lane);
                return;
            }
            int ka, kb, va, vb;
            if (L == kDeepFrom) {
                ka = uni(pending.x), va = uni(pending.y);
                kb = uni(pending.z), vb = uni(pending.w);
            } else {
                pair(kind(L), true, 2 * j, ka, kb, va, vb);
            }
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
        return walk_below(choices<true>(), 0, 1);
    }
    // The walk from node j on level DONE down to a leaf (the levels above
    // were taken elsewhere).
    __device__ __forceinline__ Leaf walk_below(const Choice &ch, const int DONE,
                                               int j) const {
        bool bottom = true;  // the walk reached level kDepth
        int walked_key = 0;  // key of node j when its level is an LDS level
#pragma unroll
        for (int L = DONE + 1; L <= kDepth; ++L) {
            if (L == kDepth && 2 * j > kSize) {
                bottom = false;
                break;
            }
            if (kind(L) <= 2) {
                // node kSize has no sibling: the left child it is
                j = (L == kDepth && 2 * j == kSize) ? 2 * j : step_down(L, j, ch);
            } else {
                int ka, kb, va, vb;
                pair(kind(L), false, 2 * j, ka, kb, va, vb);
                if (L == kDepth) kb = 2 * j == kSize ? ka : kb;
                walked_key = max(ka, kb);
                j = add_if_ne(2 * j, walked_key, ka);
            }
        }
        // the leaf's key: the walk has it already when the leaf is in LDS
        Leaf leaf;
        leaf.j = j, leaf.bottom = bottom;
        if (bottom)
            leaf.key = kind(kDepth) >= 3 ? walked_key : key_of(kind(kDepth), j);
        else
            leaf.key = kind(kDepth - 1) >= 3 ? walked_key : key_of(kind(kDepth - 1), j);
        return leaf;
    }
    // The seven register levels of that walk (lists of 256 cells and more,
    // where they are complete) together with a wavefront maximum of `x`,
    // which comes back in lane 63: the six v_max_i32_dpp of the maximum each
    // need two wait states after the one before, and the three scalar
    // instructions of a level fill them, where apart they would be s_nop.
    // Returns the node on level 7.
    static constexpr bool kFusedTop = kDepth >= 8;
    __device__ __forceinline__ static int top_levels_and_wave_max(const Choice &ch,
                                                                  int &x) {
        int j, t;
        asm("s_bitcmp1_b64 %[a], 3\n\t"
            "s_addc_u32 %[j], 2, 0\n\t"
            "v_max_i32_dpp %[x], %[x], %[x] quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf\n\t"
            "s_lshl1_add_u32 %[j], %[j], 1\n\t"
            "s_bitcmp1_b64 %[a], %[j]\n\t"
            "s_addc_u32 %[j], %[j], -1\n\t"
            "v_max_i32_dpp %[x], %[x], %[x] quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf\n\t"
            "s_lshl1_add_u32 %[j], %[j], 1\n\t"
            "s_bitcmp1_b64 %[a], %[j]\n\t"
            "s_addc_u32 %[j], %[j], -1\n\t"
            "v_max_i32_dpp %[x], %[x], %[x] row_half_mirror row_mask:0xf bank_mask:0xf\n\t"
            "s_lshl1_add_u32 %[j], %[j], 1\n\t"
            "s_bitcmp1_b64 %[a], %[j]\n\t"
            "s_addc_u32 %[j], %[j], -1\n\t"
            "v_max_i32_dpp %[x], %[x], %[x] row_mirror row_mask:0xf bank_mask:0xf\n\t"
            "s_lshl1_add_u32 %[j], %[j], 1\n\t"
            "s_bitcmp1_b64 %[a], %[j]\n\t"
            "s_addc_u32 %[j], %[j], -1\n\t"
            "v_max_i32_dpp %[x], %[x], %[x] row_bcast:15 row_mask:0xa bank_mask:0xf\n\t"
            "s_lshl1_add_u32 %[j], %[j], 1\n\t"
            "s_bitcmp1_b64 %[b], %[j]\n\t"
            "s_addc_u32 %[j], %[j], -1\n\t"
            "v_max_i32_dpp %[x], %[x], %[x] row_bcast:31 row_mask:0xc bank_mask:0xf\n\t"
            "s_lshl_b32 %[t], %[j], 1\n\t"
            "s_bitcmp1_b64 %[cd], %[j]\n\t"
            "s_addc_u32 %[j], %[t], 0"
            : [j] "=&s"(j), [x] "+v"(x), [t] "=&s"(t)
            : [a] "s"(ch.a), [b] "s"(ch.b), [cd] "s"(ch.cd)
            : "scc");
        return j;
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
// hold -inf and never win.  (Long lists keep the keys in registers instead.)

template <int S>
struct Results {
    static constexpr int kInf = 0x7f800000;      // float_to_key(+inf)
    static constexpr int kNegInf = (int)0x807fffff;  // float_to_key(-inf)
    // Long lists (eight cells per lane and more) keep their keys in
    // registers: that is lane-masked selects instead of LDS traffic per
    // insert, and 4 KB of LDS less per wavefront at H = 1024, which is what
    // bounds the residency there (measured 28.1 -> 23.3 ms per 10 000 queries
    // at H = 1024; at H = 256 the LDS form is as fast or faster).
    static constexpr bool kRegKeys = S >= 8;
    static constexpr int kLdsKeys = kRegKeys ? 4 : S * kWave;
    int key_reg[S];  // kRegKeys: the lane's cells
    int *rk;      // !kRegKeys: LDS, float_to_key of the distance, kWave * S cells
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
            if (kRegKeys) key_reg[s] = k;
            else rk[c] = k;
            rv[c] = -1;
            lane_max = max(lane_max, k);
        }
        worst = kInf;
        pos = 0;
    }
    __device__ __forceinline__ int cell_key(int lane, int s) const {
        return kRegKeys ? key_reg[s] : rk[lane * S + s];
    }
    // Caller has checked k < worst.  In two parts so that the caller can put
    // independent work between the LDS traffic and its use.
    __device__ __forceinline__ void begin_insert(int k, int v, int lane, int (&key)[S]) {
        // Every lane stores the same pair to the same cell, so the lane that
        // owns the cell reads back its own store: program order is enough.
        rv[pos] = v;
        if (kRegKeys) {
#pragma unroll
            for (int s = 0; s < S; ++s) {
                key_reg[s] = lane * S + s == pos ? k : key_reg[s];
                key[s] = key_reg[s];
            }
        } else {
            rk[pos] = k;
#pragma unroll
            for (int s = 0; s < S; ++s) key[s] = rk[lane * S + s];
        }
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

// ---- result list of the traversal: sorted keys per lane, entries in a log -------
//
// The same set as Results<S> above, kept so that an insert touches no cell by
// position.  Lane l owns S keys, largest first; the set's maximum is the
// largest first key, `holder` a lane that has it.  A candidate below the
// maximum replaces it: in the holder lane the first key leaves and the new
// key is sorted in, one v_med3_i32 per key (new[s] = the new key clamped
// between old[s + 1] and old[s]); every other lane runs the same
// instructions with the largest integer for a key, which changes nothing.
// Then a wavefront maximum over the first keys.  No key is ever looked up by
// cell, so nothing depends on S but the S clamps: 22 instructions at S = 2,
// 28 at S = 8, against 33 and 71 for the flat cells of Results<S>.
// Which node a key belongs to is not kept here: every admitted candidate is
// also appended to a log in the wavefront's device memory (ResultLog), and
// the final set is read back from the log by its keys.
template <int S>
struct ResultKeys {
    static constexpr int kInf = 0x7f800000;          // float_to_key(+inf)
    static constexpr int kNegInf = (int)0x807fffff;  // float_to_key(-inf)
    int key[S];   // this lane's keys, key[0] >= key[1] >= ...
    int worst;    // uniform: the largest key of the set
    int holder;   // uniform: a lane whose key[0] is `worst`

    // Empty cells hold +inf (the maximum is +inf until H candidates came),
    // cells beyond H hold -inf and never win.
    __device__ __forceinline__ void init(int H, int lane) {
#pragma unroll
        for (int s = 0; s < S; ++s) key[s] = lane * S + s < H ? kInf : kNegInf;
        worst = kInf;
        holder = 0;
    }
    __device__ __forceinline__ static int med3(int a, int b, int c) {
        int r;
        asm("v_med3_i32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
        return r;
    }
    // Caller has checked k < worst.  In two parts for a caller that computes
    // the wavefront maximum of the first keys itself (`reduced`: any register
    // whose lane 63 holds it).
    __device__ __forceinline__ int replace_worst(int k, int lane) {
        const int kk = lane == holder ? k : 0x7fffffff;
#pragma unroll
        for (int s = 0; s + 1 < S; ++s) key[s] = med3(key[s + 1], key[s], kk);
        key[S - 1] = min(key[S - 1], kk);
        return key[0];
    }
    __device__ __forceinline__ void set_worst(int reduced) {
        worst = __builtin_amdgcn_readlane(reduced, kWave - 1);
        holder = __builtin_ctzll(__ballot(key[0] == worst));
    }
    __device__ __forceinline__ void insert(int k, int lane) {
        replace_worst(k, lane);
        worst = wave_max_key(key[0]);
        holder = __builtin_ctzll(__ballot(key[0] == worst));
    }
};

// The log behind ResultKeys: (key, value) of every admitted candidate, in the
// wavefront's device memory.  An entry whose key is below the set's maximum
// is in the set (an entry leaves the set as its maximum, and the maximum only
// falls); entries at the maximum are in it or tie with one that is, at most H
// of them at any time.  So cutting the log down to the entries at or below
// the maximum leaves fewer than 2H, and a log of 2H + 128 entries always has
// room for the 64 candidates of a step after a cut.
struct ResultLog {
    int2 *entry;   // device memory, capacity entries, 8-byte aligned
    int n;         // uniform: entries in use
    int capacity;  // uniform

    __host__ __device__ static constexpr int capacity_for(int H) { return 2 * H + 128; }

    // Lanes whose bit is set in `who` append (k, v), in lane order.
    __device__ __forceinline__ void append(unsigned long long who, int k, int v,
                                           int lane) {
        if ((who >> lane) & 1) entry[n + lane_rank(who)] = make_int2(k, v);
        n += __popcll(who);
    }
    // The wavefront's own stores must be visible to the loads of its other
    // lanes: both go through the compute unit's cache, program order and a
    // wait for the stores are enough.
    __device__ __forceinline__ static void settle() {
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "workgroup");
    }
    // Drops the entries above `worst`, in place, order kept.
    __device__ __forceinline__ void cut(int worst, int lane) {
        settle();
        int m = 0;
        for (int base = 0; base < n; base += kWave) {
            const int i = base + lane;
            int2 e = make_int2(0x7fffffff, -1);
            if (i < n) e = entry[i];
            const bool keep = i < n && e.x <= worst;
            const unsigned long long mask = __ballot(keep);
            // m + rank <= i: the write lands on an entry already read
            if (keep) entry[m + lane_rank(mask)] = e;
            m += __popcll(mask);
        }
        n = m;
        settle();
    }
    __device__ __forceinline__ bool nearly_full() const { return n > capacity - kWave; }
};

// ---- visited set ----------------------------------------------------------------
//
// Exact, like the reference's per-query marks (extension/inc/bitmask.hpp).  An
// LDS table of 2^LOG2 buckets of WAYS 16-bit tags remembers the nodes marked:
// node v lives in bucket v mod 2^LOG2 under the tag v / 2^LOG2 (bucket and tag
// give v back), and nothing is ever evicted.  While a bucket has a free slot,
// every node ever marked for it is in it: a miss means "never marked" and the
// node is added — no memory traffic at all.  A node that finds its bucket full
// is marked in the wavefront's slice of a pooled bitmask in device memory
// instead (atomic OR), which is exact as well; so is every node when the tags
// would not fit 16 bits.  Scattered atomics on a bitmask that does not stay
// in cache cost a random memory access each way and take bandwidth from the
// row reads; with the table they are the exception.  (The subgraph traversal
// keeps its smaller two-way table of recently marked rows in front of the
// bitmask: its bitmask slices are a quarter of the size and stay in cache,
// and the swap loop costs that kernel more than the atomics it saves —
// measured 3.6 against 3.3 ms.)
// The lanes of a wavefront mark their nodes at once: a slot is claimed with
// an LDS compare-and-swap, a lane whose swap fails looks again.
template <int LOG2, int WAYS = 4>
struct Visited {
    static_assert(WAYS % 2 == 0, "two tags per word");
    static constexpr int kBuckets = 1 << LOG2;
    static constexpr int kBucketWords = WAYS / 2;
    static constexpr int kWords = kBucketWords * kBuckets;
    uint32_t *table;  // LDS, kWords
    uint32_t *bits;   // device memory: one bit per node, zero between queries
    bool small;       // tags fit 16 bits (0xffff marks a free slot)
    bool dirty;       // this lane has set a bit in `bits`

    __device__ __forceinline__ void init(uint32_t *lds_words, uint32_t *slice,
                                         int n_nodes) {
        table = lds_words, bits = slice;
        small = n_nodes <= (0xffff << LOG2);
        dirty = false;
    }
    __device__ __forceinline__ void reset(int lane) {
        for (int i = lane; i < kWords; i += kWave) table[i] = 0xffffffffu;
    }
    // Marks node v (>= 0).  Returns 0: it was marked before; 1: it was not;
    // 2: the bitmask was asked, `before` will hold its word as it was (the
    // caller may look at it later, so that the atomic's round trip overlaps
    // other work): fresh() tells.
    __device__ __forceinline__ int probe(int v, uint32_t &before) {
        if (small) {
            const uint32_t tag = (uint32_t)v >> LOG2;
            uint32_t *w = table + kBucketWords * (v & (kBuckets - 1));
            for (;;) {
                uint32_t word[kBucketWords];
#pragma unroll
                for (int i = 0; i < kBucketWords; ++i)
                    word[i] = __hip_atomic_load(w + i, __ATOMIC_RELAXED,
                                                __HIP_MEMORY_SCOPE_WAVEFRONT);
                bool found = false;
                int at = -1;  // first free slot: word at / 2, half at % 2
#pragma unroll
                for (int i = kBucketWords - 1; i >= 0; --i) {
                    found |= (word[i] & 0xffffu) == tag || (word[i] >> 16) == tag;
                    at = (word[i] >> 16) == 0xffffu ? 2 * i + 1 : at;
                    at = (word[i] & 0xffffu) == 0xffffu ? 2 * i : at;
                }
                if (found) return 0;
                if (at < 0) break;  // bucket full
                uint32_t old = word[0];
#pragma unroll
                for (int i = 1; i < kBucketWords; ++i) old = (at >> 1) == i ? word[i] : old;
                const uint32_t neu = (at & 1) ? (old & 0xffffu) | (tag << 16)
                                              : (old & 0xffff0000u) | tag;
                if (atomicCAS(w + (at >> 1), old, neu) == old) return 1;
            }
        }
        dirty = true;
        before = atomicOr(&bits[v >> 5], 1u << (v & 31));
        return 2;
    }
    __device__ __forceinline__ static bool fresh(int state, uint32_t before, int v) {
        return state == 1 || (state == 2 && !((before >> (v & 31)) & 1u));
    }
    // marks node v (>= 0); true if it was not marked before
    __device__ __forceinline__ bool mark(int v) {
        uint32_t before = 0;
        const int state = probe(v, before);
        return fresh(state, before, v);
    }
    // after a query: the slice back to zero if any lane touched it
    __device__ __forceinline__ void clean(int words, int lane) {
        if (__ballot(dirty)) {
            for (int w = lane * 4; w < words; w += kWave * 4)
                *reinterpret_cast<uint4 *>(bits + w) = make_uint4(0, 0, 0, 0);
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            dirty = false;
        }
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
        const float *row = storage;
        if (active) row = storage + (size_t)cand_id[c] * (size_t)dp;
        const float s = quad_square_dist_rows<DP8>(row, qq, dp >> 3, part, active);
        if (active && part == 0) cand_key[c] = s;
    }
}

}  // namespace pa

#endif
