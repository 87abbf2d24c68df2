// Nearest-neighbour candidates for the graph builder, gfx950.
//
// The reference hands graph construction to a library (faiss:
// pilot_ann/utils/graphs.py:15-20,52-56); its first step everywhere is "the
// closest rows of every row".  Here that step is one kernel: half-precision
// products on the matrix cores (v_mfma_f32_32x32x16_f16, float accumulation)
// fused with the selection, so the N x N table of scores never exists in
// memory.  The caller ranks the candidates again with exact float distances.
//
// A workgroup of eight wavefronts owns 256 query rows and walks over the base
// rows 256 at a time.  Per 256 x 256 tile both operands go through LDS in
// chunks of 64 elements, loaded from memory straight into two staging
// buffers; a wavefront multiplies 128 x 64 of the tile as 4 x 2 instruction
// tiles.  score(i, j) = |x_j|^2 - 2 q_i . x_j ranks the base rows of query i
// like the squared distance does.  With tiles of this size every product
// moves 1/64 byte of operands through the memory system, and that traffic,
// not the matrix cores, sets the pace.
//
// Selection: every query row has a list of (score, id) in device memory and,
// in LDS, its length and a limit from the keep-th smallest score at the time
// the list was last cut.  A score below that bound is appended (LDS atomic
// for the position); once a list could overflow with the next tile, the
// wavefront that owns the row cuts it to its `keep` smallest (a radix
// selection over the order-preserving integer image of the scores, in
// registers) and moves the limit.  Late in the walk few scores pass.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "device_common.h"
#include "pilotann.h"

using namespace pa;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int kChunk = 64;        // contraction elements staged at a time; a
                                  // row is a whole number of chunks
constexpr int kSlack = 128;       // appended entries a list may hold beyond
                                  // `keep` before it must be cut
constexpr int kMaxBN = 256;       // the most base rows a tile has in any form
constexpr int kRowPad = 256;      // rows the caller's arrays are padded to

struct KnnArgs {
    const _Float16 *query, *base;
    const float *base_norm;
    float *cand_score;
    int32_t *cand_id, *cand_count;
    int64_t m, n;
    int d, n_seg;
};

__device__ __forceinline__ unsigned ordered(float x) {
    const unsigned b = __float_as_uint(x);
    return (b & 0x80000000u) ? ~b : (b | 0x80000000u);
}
__device__ __forceinline__ float unordered(unsigned u) {
    return __uint_as_float((u & 0x80000000u) ? (u & 0x7fffffffu) : ~u);
}

// The larger of two or three finite numbers (the plain instructions: fmaxf
// first rewrites every operand that could be a signalling NaN).
__device__ __forceinline__ float larger(float x, float y) {
    float r;
    asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(x), "v"(y));
    return r;
}
__device__ __forceinline__ float larger(float x, float y, float z) {
    float r;
    asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(x), "v"(y), "v"(z));
    return r;
}

// Every lane's 16 bytes at `from` go to LDS, side by side from `lds_addr` (the
// same for all lanes) on.  The compiler does not know of the transfer: the
// wavefront waits with bring_wait() before a barrier makes the rows public.
__device__ __forceinline__ void bring_rows(const void *from, unsigned lds_addr) {
    asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off"
                 :: "s"(__builtin_amdgcn_readfirstlane(lds_addr)), "v"(from)
                 : "memory", "m0");
}
template <int LEFT>   // until at most LEFT of the wavefront's transfers are under way
__device__ __forceinline__ void bring_wait() {
    asm volatile("s_waitcnt vmcnt(%0)" :: "n"(LEFT) : "memory");
}

// The wavefront cuts one list of `n` entries (keep < n <= keep + kSlack + BN)
// to its `keep` smallest, which end up in its first `keep` places, and returns
// the largest score kept.
template <int KEEP, int BN>
__device__ __forceinline__ float cut_list(float *score, int32_t *id, int n, int lane) {
    constexpr int kPerLane = (KEEP + kSlack + BN + kWave - 1) / kWave;
    unsigned u[kPerLane];
    int32_t v[kPerLane];
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const int e = lane + kWave * i;
        u[i] = e < n ? ordered(score[e]) : 0xffffffffu;
        v[i] = e < n ? id[e] : -1;
    }
    // the KEEP-th smallest, bit by bit from the top: `bound` stays the largest
    // value with fewer than KEEP entries below it
    unsigned bound = 0;
#pragma unroll 1
    for (int bit = 31; bit >= 0; --bit) {
        const unsigned trial = bound | (1u << bit);
        int below = 0;
#pragma unroll
        for (int i = 0; i < kPerLane; ++i) below += __popcll(__ballot(u[i] < trial));
        if (below < KEEP) bound = trial;
    }
    int n_below = 0;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) n_below += __popcll(__ballot(u[i] < bound));
    // entries below the bound first, then entries equal to it while there is room
    int at_below = 0, at_equal = n_below;
#pragma unroll
    for (int i = 0; i < kPerLane; ++i) {
        const bool below = u[i] < bound;
        const bool equal = u[i] == bound && lane + kWave * i < n;
        const unsigned long long mb = __ballot(below), me = __ballot(equal);
        const int pb = at_below + lane_rank(mb), pe = at_equal + lane_rank(me);
        if (below) {
            score[pb] = unordered(u[i]);
            id[pb] = v[i];
        } else if (equal && pe < KEEP) {
            score[pe] = unordered(u[i]);
            id[pe] = v[i];
        }
        at_below += __popcll(mb);
        at_equal += __popcll(me);
    }
    return unordered(bound);
}

// WR x WC wavefronts, each multiplying WM x WN instruction tiles of 32 x 32:
// the workgroup owns BM = 32 WR WM query rows and takes BN = 32 WC WN base
// rows per tile.
//
// The sums start at -|x_j|^2 / 2 instead of zero, so a finished sum s is
// -score / 2 and "score below the row's bound" is "s above the row's limit",
// limit = -bound / 2: one comparison per product sum, and a row's sums over
// the wavefront's columns are first reduced to their maximum.
//
// Chunks flow through a ring of staging buffers without a break between
// tiles: chunk c is multiplied out of buffer c % 2 while chunk c + 1 travels
// from memory straight into the other buffer (global_load_lds, 16 bytes a
// lane; no registers and no LDS stores in between); one barrier per chunk; the
// chunk after a tile's last is the first of the next tile.
template <int KEEP, int WR, int WC, int WM, int WN>
__global__ __launch_bounds__(64 * WR * WC, (WM * WN > 8 ? 1 : 2)) void knn_kernel(KnnArgs a) {
    constexpr int kThreads = kWave * WR * WC;
    constexpr int BM = 32 * WR * WM, BN = 32 * WC * WN;
    constexpr int kStageRows = kThreads / 8;   // rows one staging step covers
    constexpr int kOwnRows = BM / (WR * WC);   // lists a wavefront looks after
    static_assert(BN <= kMaxBN && kRowPad % BM == 0 && kRowPad % BN == 0, "tile sizes");
    static_assert(kOwnRows == 32 || kOwnRows == 64, "lists per wavefront");
    static_assert(BM % kStageRows == 0 && BN % kStageRows == 0, "staging steps");
    constexpr int kCap = KEEP + kSlack + kMaxBN;  // entries a list can hold
    // a staging buffer: the chunk of the query tile, then that of the base
    // tile, rows of kRow bytes without padding.  LDS has 64 banks of four
    // bytes and serves a 16-byte read to 16 lanes at a time: 16 consecutive
    // rows are 8 pairs that share a 256-byte span, so the 16-byte piece p of
    // row r lies at place p ^ ((r / 2) % 8) of its row, and neither the loads
    // that fill the buffer nor the operand reads meet in a bank
    constexpr int kRow = kChunk * 2;
#define PA_PLACE_MIX(row_) ((unsigned)((row_) / (256 / kRow)) & (unsigned)(kPieces - 1))
    constexpr int kPieces = kRow / 16;             // 16-byte pieces of a row
    constexpr int kInstrRows = kWave / kPieces;    // rows one instruction brings
    constexpr int kStage = (BM + BN) * kRow;
    constexpr int kStages = (128 << 10) / kStage;  // buffers in the ring
    constexpr int kWaves = WR * WC;
    constexpr int kWaveRows = (BM + BN) / kWaves;  // rows a wavefront brings in per chunk
    constexpr int kInstrs = kWaveRows / kInstrRows;
    static_assert(kPieces == 8 || kPieces == 4, "chunk size");
    static_assert(kStages >= 2 && kWaveRows % kInstrRows == 0 && BM % kWaveRows == 0,
                  "rows per wavefront");
    // transfers that may still be under way when the chunk needed next must
    // be there: those of the chunks after it
    constexpr int kAhead = kInstrs * (kStages - 2);
    __shared__ __align__(1024) unsigned char stage[kStages * kStage];
    __shared__ int count[BM];
    __shared__ float limit[BM];
    const int t = threadIdx.x;
    const int lane = t & (kWave - 1), wave = t / kWave;
    const int wr = wave % WR, wc = wave / WR;
    const int col = lane & 31, half = lane >> 5;
    const int64_t q0 = (int64_t)blockIdx.x * BM;
    const int seg = blockIdx.y;
    float *my_score = a.cand_score + ((size_t)seg * a.m + q0) * kCap;
    int32_t *my_id = a.cand_id + ((size_t)seg * a.m + q0) * kCap;

    for (int r = t; r < BM; r += kThreads) {
        count[r] = 0;
        limit[r] = q0 + r < a.m ? -INFINITY : INFINITY;  // rows past the end take nothing
    }

    // staging goes from memory straight into LDS: one instruction of a
    // wavefront brings kInstrRows rows of a chunk, lane l a piece of row
    // l / kPieces, the piece that belongs at place l % kPieces, and the
    // hardware puts the lanes' 16 bytes side by side.
    // The caller's arrays are readable up to the next multiple of kRowPad
    // rows, and a row is a whole number of chunks: no clamping
    const int my_first = wave * kWaveRows;      // among the BM + BN rows of a buffer
    const bool brings_query = my_first < BM;
    const int bring_row = lane / kPieces;
    const unsigned bring_off =
        ((unsigned)((brings_query ? my_first : my_first - BM) + bring_row) * (unsigned)a.d) * 2u;
    const unsigned char *a_base =
        reinterpret_cast<const unsigned char *>(a.query) + (size_t)q0 * a.d * 2;
    const unsigned bring_to =
        (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)stage + my_first * kRow;
    // operand reads: lane l wants elements 16 s + 8 (l / 32) .. + 8 of row
    // l % 32 of an instruction tile, piece 2 s + l / 32 of that row
    const unsigned mix = PA_PLACE_MIX(col);
    const unsigned swizzle = 16u * (half ^ (mix & 1)) + 32u * (mix >> 1);
    const unsigned char *a_tile = stage + (wr * WM * 32 + col) * kRow;
    const unsigned char *b_tile = stage + (BM + wc * WN * 32 + col) * kRow;
    const int64_t n_tiles = (a.n + BN - 1) / BN;

    int64_t f_tile = seg;   // the chunk the next fetch takes: tile and element
    int f_k0 = 0;
    bool pending;           // a chunk is on its way into the other buffer
// the next chunk, if there is one, from memory into staging buffer `buf`
#define PA_FETCH_NEXT(buf)                                                              \
    {                                                                                   \
        pending = f_tile < n_tiles;                                                     \
        if (pending) {                                                                  \
            const unsigned char *from =                                                 \
                (brings_query ? a_base + (size_t)f_k0 * 2                               \
                              : reinterpret_cast<const unsigned char *>(a.base) +       \
                                    ((size_t)f_tile * BN * a.d + f_k0) * 2) + bring_off;\
            _Pragma("unroll") for (int i = 0; i < kInstrs; ++i)                         \
                bring_rows(from + (size_t)(kInstrRows * i) * a.d * 2 +                  \
                               16u * ((lane % kPieces) ^ PA_PLACE_MIX(kInstrRows * i + bring_row)), \
                           bring_to + (buf) * kStage + kInstrRows * i * kRow);          \
            f_k0 += kChunk;                                                             \
            if (f_k0 >= a.d) f_k0 = 0, f_tile += a.n_seg;                               \
        }                                                                               \
    }
// minus half the squared lengths of a tile's base rows, the columns of this
// wavefront (a column past the end: minus infinity, so it never passes)
#define PA_LOAD_NORMS(tile_)                                                            \
    _Pragma("unroll") for (int n = 0; n < WN; ++n) {                                    \
        const int64_t c = (tile_) * BN + (wc * WN + n) * 32 + col;                      \
        start[n] = c < a.n ? -0.5f * a.base_norm[c] : -INFINITY;                        \
    }
    float start[WN];
    if (seg < n_tiles) PA_LOAD_NORMS((int64_t)seg)
#pragma unroll
    for (int b = 0; b < kStages - 1; ++b) PA_FETCH_NEXT(b)
    if (pending) bring_wait<kAhead>(); else bring_wait<0>();
    __syncthreads();
    int buf = 0;

    for (int64_t tile = seg; tile < n_tiles; tile += a.n_seg) {
        floatx16 acc[WM][WN];
#pragma unroll
        for (int m = 0; m < WM; ++m)
#pragma unroll
            for (int n = 0; n < WN; ++n)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[m][n][r] = start[n];

#pragma unroll 1
        for (int k0 = 0; k0 < a.d; k0 += kChunk, buf = (buf + 1) % kStages) {
            // nobody reads the other buffer any more: the next chunk goes there
            PA_FETCH_NEXT((buf + kStages - 1) % kStages)
            // MFMA operands: lane l supplies eight consecutive elements of row
            // l % 32, the first or second eight of a group of 16 by l / 32 —
            // the same for both operands, which is all the sum needs
            const unsigned char *a_now = a_tile + buf * kStage, *b_now = b_tile + buf * kStage;
#pragma unroll
            for (int s = 0; s < kChunk / 16; ++s) {
                half8 av[WM], bv[WN];
                const unsigned at = swizzle ^ (32u * s);
#pragma unroll
                for (int m = 0; m < WM; ++m)
                    av[m] = *reinterpret_cast<const half8 *>(a_now + m * 32 * kRow + at);
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    bv[n] = *reinterpret_cast<const half8 *>(b_now + n * 32 * kRow + at);
#pragma unroll
                for (int m = 0; m < WM; ++m)
#pragma unroll
                    for (int n = 0; n < WN; ++n)
                        acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                            av[m], bv[n], acc[m][n], 0, 0, 0);
            }
            if (pending) bring_wait<kAhead>(); else bring_wait<0>();
            __syncthreads();
        }

        // the next tile's norms travel while this tile's sums are looked at
        if (tile + a.n_seg < n_tiles) PA_LOAD_NORMS(tile + a.n_seg)
        // a lane's 16 results of an instruction tile are
        // D[i = 8 * (r / 4) + 4 * (l / 32) + r % 4][j = l % 32]
        const int32_t c0 = (int32_t)(tile * BN) + wc * WN * 32 + col;
#pragma unroll
        for (int m = 0; m < WM; ++m) {
            // one row of instruction tiles at a time, so that its limits and
            // sums are all that is live
            __builtin_amdgcn_sched_barrier(0);
            const int row0 = (wr * WM + m) * 32 + 4 * half;
            float lim[16];
#pragma unroll
            for (int r = 0; r < 16; ++r) lim[r] = limit[row0 + 8 * (r >> 2) + (r & 3)];
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                float best = acc[m][0][r];
                if constexpr (WN == 4) {
                    best = larger(larger(best, acc[m][1][r], acc[m][2][r]), acc[m][3][r]);
                } else {
#pragma unroll
                    for (int n = 1; n < WN; ++n) best = larger(best, acc[m][n][r]);
                }
                if (best > lim[r]) {  // rare after the first tiles
                    const int row = row0 + 8 * (r >> 2) + (r & 3);
#pragma unroll
                    for (int n = 0; n < WN; ++n) {
                        if (acc[m][n][r] > lim[r]) {
                            const unsigned at = row * kCap + atomicAdd(&count[row], 1);
                            my_score[at] = -2.f * acc[m][n][r];
                            my_id[at] = c0 + 32 * n;
                        }
                    }
                }
            }
        }
        __syncthreads();
        // every wavefront looks after kOwnRows lists: one that the next tile
        // could overflow is cut now
        {
            const int row = wave * kOwnRows + lane % kOwnRows;
            unsigned long long todo =
                __ballot(lane < kOwnRows && count[row] > KEEP + kSlack);
            while (todo) {
                const int r = wave * kOwnRows + __builtin_ctzll(todo);
                todo &= todo - 1;
                const float b = cut_list<KEEP, BN>(my_score + (size_t)r * kCap,
                                                   my_id + (size_t)r * kCap, count[r], lane);
                if (lane == 0) count[r] = KEEP, limit[r] = -0.5f * b;
            }
        }
        // the next tile's first barrier comes before anything reads the
        // counts and limits again
    }
#undef PA_FETCH_NEXT
#undef PA_PLACE_MIX
#undef PA_LOAD_NORMS
    __syncthreads();
    {
        const int row = wave * kOwnRows + lane % kOwnRows;
        unsigned long long todo = __ballot(lane < kOwnRows && count[row] > KEEP);
        while (todo) {
            const int r = wave * kOwnRows + __builtin_ctzll(todo);
            todo &= todo - 1;
            cut_list<KEEP, BN>(my_score + (size_t)r * kCap, my_id + (size_t)r * kCap,
                               count[r], lane);
            if (lane == 0) count[r] = KEEP;
        }
    }
    __syncthreads();
    for (int r = t; r < BM; r += kThreads)
        if (q0 + r < a.m) a.cand_count[(size_t)seg * a.m + q0 + r] = count[r];
}

// Exact squared distances from query row first + q to its candidates, the
// float arithmetic of the search itself (differences, then squares, summed).
// A wavefront per query, its row in LDS; 16 lanes per candidate, four
// candidates at a time, every lane 16 bytes of the candidate's row per step.
// A candidate that is -1, out of range or the query row itself gets infinity.
constexpr int kRankWaves = 4;

__global__ __launch_bounds__(kWave * kRankWaves) void rerank_kernel(
    const float *__restrict__ rows, const int64_t *__restrict__ cand,
    float *__restrict__ out, int64_t m, int64_t first, int64_t n, int d, int k) {
    typedef float floatx4 __attribute__((ext_vector_type(4)));
    extern __shared__ __align__(16) unsigned char rank_lds[];
    const int lane = threadIdx.x & (kWave - 1), wave = threadIdx.x / kWave;
    const int64_t q = (int64_t)blockIdx.x * kRankWaves + wave;
    const int d4 = d / 4;
    floatx4 *mine = reinterpret_cast<floatx4 *>(rank_lds) + wave * d4;
    if (q < m) {
        const floatx4 *src = reinterpret_cast<const floatx4 *>(rows + (size_t)(first + q) * d);
        for (int i = lane; i < d4; i += kWave) mine[i] = src[i];
    }
    __syncthreads();
    if (q >= m) return;
    const int team = lane >> 4, place = lane & 15;
    for (int j0 = 0; j0 < k; j0 += 4) {
        const int j = j0 + team;
        const int64_t id = j < k ? cand[(size_t)q * k + j] : -1;
        const bool ok = id >= 0 && id < n && id != first + q;
        float sum = 0.f;
        if (ok) {
            const floatx4 *row = reinterpret_cast<const floatx4 *>(rows + (size_t)id * d);
            for (int i = place; i < d4; i += 16) {
                const floatx4 x = row[i], y = mine[i];
                const float e0 = x[0] - y[0], e1 = x[1] - y[1], e2 = x[2] - y[2], e3 = x[3] - y[3];
                sum = fmaf(e0, e0, sum);
                sum = fmaf(e1, e1, sum);
                sum = fmaf(e2, e2, sum);
                sum = fmaf(e3, e3, sum);
            }
        }
#pragma unroll
        for (int step = 8; step >= 1; step >>= 1) sum += __shfl_xor(sum, step, 16);
        if (place == 0 && j < k) out[(size_t)q * k + j] = ok ? sum : INFINITY;
    }
}

// Occlusion pruning of a node's candidate list (closest first): candidate j
// is kept unless a candidate kept before it is closer to it than the node
// itself is, until m_keep are kept; with `fill` the closest rejected ones top
// the row up to m_keep.  One wavefront per node; the kept set is a bit mask
// that every lane carries, a step tests one row of the node's table of
// candidate-to-candidate distances against it.
__global__ __launch_bounds__(256) void prune_kernel(
    const float *__restrict__ pair, const float *__restrict__ cand_dist,
    int32_t *__restrict__ selected, int64_t n, int k, int m_keep, int fill) {
    constexpr int kWords = 8;  // k <= 512
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t node = (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (node >= n) return;
    const float *table = pair + (size_t)node * k * k;
    const float *dist = cand_dist + (size_t)node * k;
    int32_t *out = selected + (size_t)node * m_keep;
    unsigned long long kept[kWords];
#pragma unroll
    for (int w = 0; w < kWords; ++w) kept[w] = 0;
    int count = 0;
    for (int j = 0; j < k && count < m_keep; ++j) {
        const float own = dist[j];
        bool hit = false;
        // only candidates before j can have been kept
#pragma unroll
        for (int w = 0; w < kWords; ++w) {
            const int r = 64 * w + lane;
            if (64 * w < j && r < j && ((kept[w] >> lane) & 1ull))
                hit |= table[(size_t)j * k + r] < own;
        }
        if (!__ballot(hit)) {
#pragma unroll
            for (int w = 0; w < kWords; ++w)
                if (j >> 6 == w) kept[w] |= 1ull << (j & 63);
            if (lane == 0) out[count] = j;
            count += 1;
        }
    }
    if (fill) {
        for (int j = 0; j < k && count < m_keep; ++j) {
            bool is_kept = false;
#pragma unroll
            for (int w = 0; w < kWords; ++w)
                if (j >> 6 == w) is_kept = (kept[w] >> (j & 63)) & 1ull;
            if (is_kept) continue;
            if (lane == 0) out[count] = j;
            count += 1;
        }
    }
    for (int i = count + lane; i < m_keep; i += kWave) out[i] = -1;
}

// Occlusion pruning straight from the rows: the same rule as prune_kernel,
// with the candidate-to-candidate distances made on the spot.  A workgroup of
// eight wavefronts takes one node: it gathers the rows of the node's k <= 256
// candidates chunk by chunk into LDS (the transfers of knn_kernel, every lane
// with the address of its own candidate's row), multiplies them with
// themselves on the matrix cores — rows as two half-precision parts, x = hi +
// lo, and hi.hi + hi.lo + lo.hi for the product, which is the float product to
// about 22 bits — and reduces |a|^2 + |b|^2 - 2 a.b < dist(node, a) to one bit
// per pair in LDS; then its first wavefront walks the candidates in order
// against the bits of those kept so far.  The k x k table never leaves the CU.
constexpr int64_t kLaunchNodes = 1ll << 22;

struct PruneRowsArgs {
    const _Float16 *hi, *lo;
    const float *norm;        // squared lengths of the scaled rows
    const int64_t *cand;      // [n, k] row numbers, closest first, -1 after the last
    const float *cand_dist;   // [n, k] squared distances to the node, unscaled
    int32_t *selected;        // [n, m_keep]
    int64_t n, first;         // this launch takes nodes first .. first + gridDim.x
    int64_t n_rows;           // rows behind hi / lo / norm: a candidate at or beyond is no candidate
    int d, k, m_keep, fill;
    float scale2;             // (scaled / unscaled) squared
};

__global__ __launch_bounds__(512, 2) void prune_rows_kernel(PruneRowsArgs a) {
    constexpr int kRows = 256;                 // candidates of a node, padded
    constexpr int kRow = kChunk * 2;           // bytes of a staged row
    constexpr int kPart = kRows * kRow;        // one part (hi or lo) of a chunk
    constexpr int kStage = 2 * kPart;
    constexpr int kWords = kRows / 32;
    __shared__ __align__(1024) unsigned char stage[2 * kStage];
    __shared__ unsigned bits[kRows][kWords];   // bits[a][w]: bit b % 32 of word b / 32 says b blocks a
    __shared__ float len2[kRows], reach[kRows];
    __shared__ int valid_count;
    const int t = threadIdx.x;
    const int lane = t & (kWave - 1), wave = t / kWave;
    const int wr = wave % 2, wc = wave / 2;
    const int col = lane & 31, half = lane >> 5;
    const int64_t node = a.first + blockIdx.x;
    const int64_t *ids = a.cand + (size_t)node * a.k;
    // a candidate: a row number inside the set, else -1 (nothing is read for it)
    auto cand_at = [&](int i) -> int64_t {
        const int64_t id = i < a.k ? ids[i] : -1;
        return id < a.n_rows ? id : -1;
    };

    // the candidates' lengths and distances; what lies behind the list
    // repeats the first candidate and can block nothing
    if (t < kRows) {
        const int64_t id = cand_at(t);
        len2[t] = id >= 0 ? a.norm[id] : 0.f;
        reach[t] = id >= 0 ? a.cand_dist[(size_t)node * a.k + t] * a.scale2 : -INFINITY;
    }
    if (t == 0) valid_count = 0;
    __syncthreads();
    if (cand_at(t) >= 0) atomicAdd(&valid_count, 1);

    // transfers: wavefront w brings rows 32 w .. 32 w + 31 of both parts, 8
    // rows an instruction, lane l the piece that belongs at place l % 8 of row
    // l / 8 (places as in knn_kernel)
    const int bring_row = lane >> 3;
    size_t from[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = 32 * wave + 8 * i + bring_row;
        int64_t id = cand_at(row);
        if (id < 0) id = cand_at(0) >= 0 ? cand_at(0) : 0;
        from[i] = ((size_t)id * a.d) * 2 + 16u * ((lane & 7) ^ (((8 * i + bring_row) >> 1) & 7));
    }
    const unsigned bring_to =
        (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char *)stage +
        32 * wave * kRow;
    const unsigned char *hi = reinterpret_cast<const unsigned char *>(a.hi);
    const unsigned char *lo = reinterpret_cast<const unsigned char *>(a.lo);
#define PA_BRING_CHUNK(k0, buf)                                                          \
    _Pragma("unroll") for (int i = 0; i < 4; ++i) {                                      \
        bring_rows(hi + from[i] + (size_t)(k0) * 2, bring_to + (buf) * kStage + 8 * i * kRow); \
        bring_rows(lo + from[i] + (size_t)(k0) * 2,                                      \
                   bring_to + (buf) * kStage + kPart + 8 * i * kRow);                    \
    }
    const unsigned mix = (col >> 1) & 7;
    const unsigned swizzle = 16u * (half ^ (mix & 1)) + 32u * (mix >> 1);
    const unsigned char *a_tile = stage + (wr * 128 + col) * kRow;
    const unsigned char *b_tile = stage + (wc * 64 + col) * kRow;

    floatx16 acc[4][2];
#pragma unroll
    for (int m = 0; m < 4; ++m)
#pragma unroll
        for (int n = 0; n < 2; ++n)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

    PA_BRING_CHUNK(0, 0)
    bring_wait<0>();
    __syncthreads();
    int buf = 0;
#pragma unroll 1
    for (int k0 = 0; k0 < a.d; k0 += kChunk, buf ^= 1) {
        if (k0 + kChunk < a.d) PA_BRING_CHUNK(k0 + kChunk, buf ^ 1)
        const unsigned char *a_now = a_tile + buf * kStage, *b_now = b_tile + buf * kStage;
#pragma unroll
        for (int s = 0; s < kChunk / 16; ++s) {
            const unsigned at = swizzle ^ (32u * s);
            half8 av[4], bv[2];
            // hi . hi
#pragma unroll
            for (int m = 0; m < 4; ++m)
                av[m] = *reinterpret_cast<const half8 *>(a_now + m * 32 * kRow + at);
#pragma unroll
            for (int n = 0; n < 2; ++n)
                bv[n] = *reinterpret_cast<const half8 *>(b_now + n * 32 * kRow + at);
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[m], bv[n], acc[m][n], 0, 0, 0);
            // hi . lo
#pragma unroll
            for (int n = 0; n < 2; ++n)
                bv[n] = *reinterpret_cast<const half8 *>(b_now + kPart + n * 32 * kRow + at);
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[m], bv[n], acc[m][n], 0, 0, 0);
            // lo . hi
#pragma unroll
            for (int m = 0; m < 4; ++m)
                av[m] = *reinterpret_cast<const half8 *>(a_now + kPart + m * 32 * kRow + at);
#pragma unroll
            for (int n = 0; n < 2; ++n)
                bv[n] = *reinterpret_cast<const half8 *>(b_now + n * 32 * kRow + at);
#pragma unroll
            for (int m = 0; m < 4; ++m)
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(av[m], bv[n], acc[m][n], 0, 0, 0);
        }
        bring_wait<0>();
        __syncthreads();
    }
#undef PA_BRING_CHUNK

    // a lane's 16 results of an instruction tile are
    // D[i = 8 * (r / 4) + 4 * (l / 32) + r % 4][j = l % 32]: one ballot is the
    // word of 32 columns for two rows
#pragma unroll
    for (int n = 0; n < 2; ++n) {
        const int b = (wc * 2 + n) * 32 + col;
        const float len_b = len2[b];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = (wr * 4 + m) * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                const float pair = (len2[row] + len_b) - 2.f * acc[m][n][r];
                const unsigned long long word = __ballot(pair < reach[row]);
                if (col == 0)
                    bits[row][wc * 2 + n] = half ? (unsigned)(word >> 32) : (unsigned)word;
            }
        }
    }
    __syncthreads();
    if (wave != 0) return;

    // the walk: lane w < 8 holds word w of the kept set
    int32_t *out = a.selected + (size_t)node * a.m_keep;
    const int k_valid = valid_count;
    unsigned kept = 0;
    int count = 0;
    for (int j = 0; j < k_valid && count < a.m_keep; ++j) {
        const unsigned hit = lane < kWords ? (bits[j][lane] & kept) : 0u;
        if (!__ballot(hit != 0)) {
            if (lane == (j >> 5)) kept |= 1u << (j & 31);
            if (lane == 0) out[count] = j;
            count += 1;
        }
    }
    if (a.fill) {
        for (int j = 0; j < k_valid && count < a.m_keep; ++j) {
            const unsigned word = __builtin_amdgcn_readlane(kept, j >> 5);
            if ((word >> (j & 31)) & 1u) continue;
            if (lane == 0) out[count] = j;
            count += 1;
        }
    }
    for (int i = count + lane; i < a.m_keep; i += kWave) out[i] = -1;
}

// The form in use: 2 x 4 wavefronts of 4 x 2 instruction tiles, 256 query rows
// against 256 base rows per tile; one workgroup per compute unit (150 KB of
// LDS, 256 registers a lane).
constexpr int kWR = 2, kWC = 4, kWM = 4, kWN = 2;
constexpr int kBM = 32 * kWR * kWM;

template <int KEEP>
int launch_knn(const KnnArgs &a, hipStream_t stream) {
    const dim3 grid((unsigned)((a.m + kBM - 1) / kBM), (unsigned)a.n_seg);
    knn_kernel<KEEP, kWR, kWC, kWM, kWN><<<grid, 64 * kWR * kWC, 0, stream>>>(a);
    return (int)hipGetLastError();
}

}  // namespace

extern "C" int64_t pa_knn_list_capacity(int keep) {
    return keep == 64 || keep == 128 || keep == 256 || keep == 512 ? keep + kSlack + kMaxBN : 0;
}

extern "C" int pa_knn_tile_rows(void) { return kRowPad; }

extern "C" int pa_knn(float *cand_score, int32_t *cand_id, int32_t *cand_count,
                      const void *query_f16, const void *base_f16,
                      const float *base_norm, int64_t m, int64_t n, int d,
                      int keep, int n_seg, void *stream_) {
    if (m < 0 || n < 0 || n_seg < 1 || n_seg > 65535) return PA_E_SHAPE;
    // ids are 32 bits, and a launch holds fewer than 2^32 work-items
    if (n >= (1ll << 31) || (m + kBM - 1) / kBM * n_seg >= (1ll << 32) / (64 * kWR * kWC))
        return PA_E_RANGE;
    if (d <= 0 || d % kChunk) return PA_E_DIM;
    if (keep != 64 && keep != 128 && keep != 256 && keep != 512) return PA_E_SHAPE;
    if (m == 0) return PA_OK;
    if (n == 0) return PA_E_SHAPE;
    if (!cand_score || !cand_id || !cand_count || !query_f16 || !base_f16 || !base_norm)
        return PA_E_NULL;
    KnnArgs a;
    a.query = reinterpret_cast<const _Float16 *>(query_f16);
    a.base = reinterpret_cast<const _Float16 *>(base_f16);
    a.base_norm = base_norm;
    a.cand_score = cand_score, a.cand_id = cand_id, a.cand_count = cand_count;
    a.m = m, a.n = n, a.d = d, a.n_seg = n_seg;
    hipStream_t stream = (hipStream_t)stream_;
    switch (keep) {
        case 64: return launch_knn<64>(a, stream);
        case 128: return launch_knn<128>(a, stream);
        case 256: return launch_knn<256>(a, stream);
        default: return launch_knn<512>(a, stream);
    }
}

extern "C" int pa_knn_rerank(float *dist, const float *rows, const int64_t *cand,
                             int64_t m, int64_t first, int64_t n, int d, int k,
                             void *stream_) {
    if (m < 0 || n < 0 || first < 0 || first + m > n || k < 1) return PA_E_SHAPE;
    if (d <= 0 || d % 4 || d > 4096) return PA_E_DIM;
    if (m >= (1ll << 32) / kWave) return PA_E_RANGE;   // work-items of the launch
    if (m == 0) return PA_OK;
    if (!dist || !rows || !cand) return PA_E_NULL;
    const unsigned lds = (unsigned)(kRankWaves * d * sizeof(float));
    rerank_kernel<<<(unsigned)((m + kRankWaves - 1) / kRankWaves), kWave * kRankWaves, lds,
                    (hipStream_t)stream_>>>(rows, cand, dist, m, first, n, d, k);
    return (int)hipGetLastError();
}

extern "C" int pa_graph_prune_rows(int32_t *selected, const void *rows_hi_f16,
                                   const void *rows_lo_f16, const float *norm,
                                   const int64_t *cand, const float *cand_dist,
                                   int64_t n, int64_t n_rows, int d, int k,
                                   int m_keep, int fill, float scale2,
                                   void *stream_) {
    if (n < 0 || n_rows < 1 || k < 1 || k > 256 || m_keep < 1) return PA_E_SHAPE;
    if (d <= 0 || d % kChunk) return PA_E_DIM;
    if (n == 0) return PA_OK;
    if (!selected || !rows_hi_f16 || !rows_lo_f16 || !norm || !cand || !cand_dist)
        return PA_E_NULL;
    PruneRowsArgs a;
    a.hi = reinterpret_cast<const _Float16 *>(rows_hi_f16);
    a.lo = reinterpret_cast<const _Float16 *>(rows_lo_f16);
    a.norm = norm, a.cand = cand, a.cand_dist = cand_dist, a.selected = selected;
    a.n = n, a.n_rows = n_rows, a.d = d, a.k = k, a.m_keep = m_keep, a.fill = fill;
    a.scale2 = scale2;
    // a launch holds fewer than 2^32 work-items: at most 2^22 nodes of 512
    for (a.first = 0; a.first < n; a.first += kLaunchNodes) {
        const int64_t count = n - a.first < kLaunchNodes ? n - a.first : kLaunchNodes;
        prune_rows_kernel<<<(unsigned)count, 512, 0, (hipStream_t)stream_>>>(a);
        const hipError_t err = hipGetLastError();
        if (err != hipSuccess) return (int)err;
    }
    return PA_OK;
}

extern "C" int pa_graph_prune(int32_t *selected, const float *pair,
                              const float *cand_dist, int64_t n, int k,
                              int m_keep, int fill, void *stream_) {
    if (n < 0 || k < 1 || k > 512 || m_keep < 1) return PA_E_SHAPE;
    if (n >= (1ll << 32) / kWave) return PA_E_RANGE;   // work-items of the launch
    if (n == 0) return PA_OK;
    if (!selected || !pair || !cand_dist) return PA_E_NULL;
    prune_kernel<<<(unsigned)((n + 3) / 4), 256, 0, (hipStream_t)stream_>>>(
        pair, cand_dist, selected, n, k, m_keep, fill);
    return (int)hipGetLastError();
}
