// Nearest-neighbour candidates for the graph builder, gfx950.
//
// The reference hands graph construction to a library (faiss:
// pilot_ann/utils/graphs.py:15-20,52-56); its first step everywhere is "the
// closest rows of every row".  Here that step is one kernel: half-precision
// products on the matrix cores (v_mfma_f32_32x32x16_f16, float accumulation)
// fused with the selection, so the N x N table of scores never exists in
// memory.  The caller ranks the candidates again with exact float distances.
//
// A workgroup of four wavefronts owns 128 query rows and walks over the base
// rows 128 at a time.  Per 128 x 128 tile both operands go through LDS in
// chunks of 64 elements (16-byte loads, the next chunk waiting in registers
// while the present one is multiplied); a wavefront multiplies 64 x 64 of the
// tile as 2 x 2 instructions tiles.  score(i, j) = |x_j|^2 - 2 q_i . x_j ranks
// the base rows of query i like the squared distance does.
//
// Selection: every query row has a list of (score, id) in device memory and,
// in LDS, its length and a bound: the keep-th smallest score at the time the
// list was last cut.  A score below the bound is appended (LDS atomic for the
// position); once a list could overflow with the next tile, the wavefront
// that owns the row cuts it to its `keep` smallest (a radix selection over
// the order-preserving integer image of the scores, in registers) and lowers
// the bound.  After the first few tiles almost nothing passes the bound, so
// the matrix instructions are what the kernel spends its time on.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdint.h>

#include "device_common.h"
#include "pilotann.h"

using namespace pa;

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned int uintx4 __attribute__((ext_vector_type(4)));

constexpr int kBM = 128;          // query rows per workgroup
constexpr int kBN = 128;          // base rows per tile
constexpr int kChunk = 64;        // contraction elements staged at a time
// LDS row pitch in bytes: 128 of data + 16, so that consecutive rows start
// four banks apart and the 16-byte reads of eight lanes cover every bank once
constexpr int kPitch = kChunk * 2 + 16;
constexpr int kSlack = 128;       // appended entries a list may hold beyond
                                  // `keep` before it must be cut

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

// The wavefront cuts one list of `n` entries (keep < n <= keep + kSlack + kBN)
// to its `keep` smallest, which end up in its first `keep` places, and returns
// the largest score kept.
template <int KEEP>
__device__ __forceinline__ float cut_list(float *score, int32_t *id, int n, int lane) {
    constexpr int kPerLane = (KEEP + kSlack + kBN + kWave - 1) / kWave;
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

template <int KEEP>
__global__ __launch_bounds__(256) void knn_kernel(KnnArgs a) {
    constexpr int kCap = KEEP + kSlack + kBN;  // entries a list can hold
    __shared__ __align__(16) unsigned char a_s[kBM * kPitch];
    __shared__ __align__(16) unsigned char b_s[kBN * kPitch];
    __shared__ int count[kBM];
    __shared__ float bound[kBM];
    const int t = threadIdx.x;
    const int lane = t & (kWave - 1), wave = t / kWave;
    const int col = lane & 31, half = lane >> 5;
    const int64_t q0 = (int64_t)blockIdx.x * kBM;
    const int seg = blockIdx.y;
    float *my_score = a.cand_score + ((size_t)seg * a.m + q0) * kCap;
    int32_t *my_id = a.cand_id + ((size_t)seg * a.m + q0) * kCap;

    if (t < kBM) {
        count[t] = 0;
        bound[t] = q0 + t < a.m ? INFINITY : -INFINITY;  // rows past the end take nothing
    }

    // staging: lane t copies 16-byte piece t % 8 of rows t / 8 + 32 i.  The
    // caller's arrays are readable up to the next multiple of 128 rows, and a
    // row is a whole number of chunks: no clamping, and addresses are a
    // uniform base plus one 32-bit offset per lane
    const int srow = t >> 3, spiece = t & 7;
    const unsigned lane_off = ((unsigned)srow * (unsigned)a.d + 8u * spiece) * 2u;
    const unsigned char *a_base =
        reinterpret_cast<const unsigned char *>(a.query) + (size_t)q0 * a.d * 2;
    const unsigned char *a_tile = a_s + ((wave & 1) * 64 + col) * kPitch + 16 * half;
    const unsigned char *b_tile = b_s + ((wave >> 1) * 64 + col) * kPitch + 16 * half;
    const int64_t n_tiles = (a.n + kBN - 1) / kBN;
    __syncthreads();

    for (int64_t tile = seg; tile < n_tiles; tile += a.n_seg) {
        const int64_t n0 = tile * kBN;
        const unsigned char *b_base =
            reinterpret_cast<const unsigned char *>(a.base) + (size_t)n0 * a.d * 2;
        floatx16 acc[2][2];
#pragma unroll
        for (int m = 0; m < 2; ++m)
#pragma unroll
            for (int n = 0; n < 2; ++n)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

        uintx4 a_reg[kBM / 32], b_reg[kBN / 32];
// the chunk that starts at element k0, from memory into registers
#define PA_FETCH_CHUNK(k0)                                                              \
    {                                                                                   \
        _Pragma("unroll") for (int i = 0; i < kBM / 32; ++i) a_reg[i] =                 \
            *reinterpret_cast<const uintx4 *>(                                          \
                a_base + ((size_t)(32 * i) * a.d + (k0)) * 2 + lane_off);               \
        _Pragma("unroll") for (int i = 0; i < kBN / 32; ++i) b_reg[i] =                 \
            *reinterpret_cast<const uintx4 *>(                                          \
                b_base + ((size_t)(32 * i) * a.d + (k0)) * 2 + lane_off);               \
    }
        PA_FETCH_CHUNK(0)
#pragma unroll 1
        for (int k0 = 0; k0 < a.d; k0 += kChunk) {
#pragma unroll
            for (int i = 0; i < kBM / 32; ++i)
                *reinterpret_cast<uintx4 *>(a_s + (srow + 32 * i) * kPitch + 16 * spiece) = a_reg[i];
#pragma unroll
            for (int i = 0; i < kBN / 32; ++i)
                *reinterpret_cast<uintx4 *>(b_s + (srow + 32 * i) * kPitch + 16 * spiece) = b_reg[i];
            __syncthreads();
            if (k0 + kChunk < a.d) PA_FETCH_CHUNK(k0 + kChunk)
            // MFMA operands: lane l supplies eight consecutive elements of row
            // l % 32, the first or second eight of a group of 16 by l / 32 —
            // the same for both operands, which is all the sum needs
#pragma unroll 2
            for (int s = 0; s < kChunk / 16; ++s) {
                half8 av[2], bv[2];
#pragma unroll
                for (int m = 0; m < 2; ++m)
                    av[m] = *reinterpret_cast<const half8 *>(a_tile + m * 32 * kPitch + 32 * s);
#pragma unroll
                for (int n = 0; n < 2; ++n)
                    bv[n] = *reinterpret_cast<const half8 *>(b_tile + n * 32 * kPitch + 32 * s);
#pragma unroll
                for (int m = 0; m < 2; ++m)
#pragma unroll
                    for (int n = 0; n < 2; ++n)
                        acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x16_f16(
                            av[m], bv[n], acc[m][n], 0, 0, 0);
            }
            __syncthreads();
        }
#undef PA_FETCH_CHUNK

        // a lane's 16 results of an instruction tile are
        // D[i = 8 * (r / 4) + 4 * (l / 32) + r % 4][j = l % 32]
#pragma unroll
        for (int n = 0; n < 2; ++n) {
            const int64_t cg = n0 + (wave >> 1) * 64 + n * 32 + col;
            const bool col_ok = cg < a.n;
            const float xn = col_ok ? a.base_norm[cg] : 0.f;
#pragma unroll
            for (int m = 0; m < 2; ++m) {
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = (wave & 1) * 64 + m * 32 + 8 * (r >> 2) + 4 * half + (r & 3);
                    const float sc = fmaf(-2.f, acc[m][n][r], xn);
                    const bool pass = col_ok && sc < bound[row];
                    if (__ballot(pass)) {  // rare after the first tiles
                        if (pass) {
                            const int pos = atomicAdd(&count[row], 1);
                            my_score[(size_t)row * kCap + pos] = sc;
                            my_id[(size_t)row * kCap + pos] = (int32_t)cg;
                        }
                    }
                }
            }
        }
        __syncthreads();
        // wavefront w looks after rows 32 w .. 32 w + 31: a list that the
        // next tile could overflow is cut now
        {
            const int row = wave * 32 + col;
            unsigned long long todo = __ballot(half == 0 && count[row] > KEEP + kSlack);
            while (todo) {
                const int r = wave * 32 + __builtin_ctzll(todo);
                todo &= todo - 1;
                const float b = cut_list<KEEP>(my_score + (size_t)r * kCap,
                                               my_id + (size_t)r * kCap, count[r], lane);
                if (lane == 0) count[r] = KEEP, bound[r] = b;
            }
        }
        // the next tile's first barrier comes before anything reads the
        // counts and bounds again
    }
    __syncthreads();
    {
        const int row = wave * 32 + col;
        unsigned long long todo = __ballot(half == 0 && count[row] > KEEP);
        while (todo) {
            const int r = wave * 32 + __builtin_ctzll(todo);
            todo &= todo - 1;
            cut_list<KEEP>(my_score + (size_t)r * kCap, my_id + (size_t)r * kCap, count[r], lane);
            if (lane == 0) count[r] = KEEP;
        }
    }
    __syncthreads();
    if (t < kBM && q0 + t < a.m) a.cand_count[(size_t)seg * a.m + q0 + t] = count[t];
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

}  // namespace

extern "C" int64_t pa_knn_list_capacity(int keep) {
    return keep == 64 || keep == 128 || keep == 256 || keep == 512 ? keep + kSlack + kBN : 0;
}

extern "C" int pa_knn(float *cand_score, int32_t *cand_id, int32_t *cand_count,
                      const void *query_f16, const void *base_f16,
                      const float *base_norm, int64_t m, int64_t n, int d,
                      int keep, int n_seg, void *stream_) {
    if (m < 0 || n < 0 || n_seg < 1 || n_seg > 65535) return PA_E_SHAPE;
    if (n >= (1ll << 31) || (m + kBM - 1) / kBM >= (1ll << 31)) return PA_E_RANGE;
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
    const dim3 grid((unsigned)((m + kBM - 1) / kBM), (unsigned)n_seg);
    hipStream_t stream = (hipStream_t)stream_;
    switch (keep) {
        case 64: knn_kernel<64><<<grid, 256, 0, stream>>>(a); break;
        case 128: knn_kernel<128><<<grid, 256, 0, stream>>>(a); break;
        case 256: knn_kernel<256><<<grid, 256, 0, stream>>>(a); break;
        default: knn_kernel<512><<<grid, 256, 0, stream>>>(a);
    }
    return (int)hipGetLastError();
}

extern "C" int pa_graph_prune(int32_t *selected, const float *pair,
                              const float *cand_dist, int64_t n, int k,
                              int m_keep, int fill, void *stream_) {
    if (n < 0 || k < 1 || k > 512 || m_keep < 1) return PA_E_SHAPE;
    if ((n + 3) / 4 >= (1ll << 31)) return PA_E_RANGE;
    if (n == 0) return PA_OK;
    if (!selected || !pair || !cand_dist) return PA_E_NULL;
    prune_kernel<<<(unsigned)((n + 3) / 4), 256, 0, (hipStream_t)stream_>>>(
        pair, cand_dist, selected, n, k, m_keep, fill);
    return (int)hipGetLastError();
}
