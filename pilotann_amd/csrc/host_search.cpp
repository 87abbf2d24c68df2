// Host (CPU) search stages: the single-stage search and the two-stage refine
// that follows the device traversal.  These are the product's own version of
// the reference's host code, which the pipeline leaves on the CPU
// (extension/traverse_cpu.cpp:12-369, extension/inc/heapq.cuh,
// extension/inc/distance.h, extension/inc/bitmask.hpp).  AVX2 + FMA, OpenMP
// over queries.
//
// Floating point follows distance.h:31-55 literally: eight FMA lanes, lanes
// added left to right.  This file is built without -ffast-math, so the sums
// are the ones written here; the device kernels use the same order, which
// makes a candidate's distance the same number on both sides.
#include <immintrin.h>
#include <omp.h>

#include <cmath>
#include <cstdint>
#include <cstring>
#include <limits>
#include <vector>

#include "pilotann.h"

namespace {

constexpr float kInf = std::numeric_limits<float>::infinity();
constexpr int kTile = 4;       // rows per batched distance, traverse_cpu.cpp:8
constexpr int kRefineSteps = 2;  // traverse_cpu.cpp:9

// ---- distance ---------------------------------------------------------------

inline float lanes_sum(__m256 acc) {
    alignas(32) float lane[8];
    _mm256_store_ps(lane, acc);
    float r = 0.0f;
    for (int j = 0; j < 8; ++j) r += lane[j];
    return r;
}

// distance.h:31-55; [from, d) of one row.
inline float square_dist(const float *q, const float *row, int d, int from = 0) {
    __m256 acc = _mm256_setzero_ps();
    for (int o = from; o < d; o += 8) {
        const __m256 t = _mm256_sub_ps(_mm256_loadu_ps(q + o), _mm256_loadu_ps(row + o));
        acc = _mm256_fmadd_ps(t, t, acc);
    }
    return lanes_sum(acc);
}

// distance.h:73-111; four rows share each load of the query.
inline void square_dist4(float *out, const float *q, const float *storage,
                         const int64_t *rows, int d) {
    __m256 acc[kTile];
    const float *p[kTile];
    for (int i = 0; i < kTile; ++i) {
        acc[i] = _mm256_setzero_ps();
        p[i] = storage + rows[i] * (int64_t)d;
    }
    for (int o = 0; o < d; o += 8) {
        const __m256 qq = _mm256_loadu_ps(q + o);
        for (int i = 0; i < kTile; ++i) {
            const __m256 t = _mm256_sub_ps(qq, _mm256_loadu_ps(p[i] + o));
            acc[i] = _mm256_fmadd_ps(t, t, acc[i]);
        }
    }
    for (int i = 0; i < kTile; ++i) out[i] = lanes_sum(acc[i]);
}

inline void prefetch(const void *p) {
    _mm_prefetch(reinterpret_cast<const char *>(p), _MM_HINT_T1);
}

// ---- heaps: heapq.cuh ---------------------------------------------------------

struct HeapView {
    float *key;
    int64_t *val;
    int size;

    void fill(float k) {
        for (int i = 0; i < size; ++i) key[i] = k, val[i] = -1;
    }
    // heapq.cuh:13-29
    void sink_root() {
        int at = 0;
        const float k = key[0];
        const int64_t v = val[0];
        for (;;) {
            int c = 2 * at + 1;
            if (c >= size) break;
            if (c + 1 < size && key[c + 1] < key[c]) ++c;
            if (k <= key[c]) break;
            key[at] = key[c], val[at] = val[c];
            at = c;
        }
        key[at] = k, val[at] = v;
    }
    // heapq.cuh:37-45
    void pop(float *k, int64_t *v) {
        *k = key[0], *v = val[0];
        key[0] = kInf, val[0] = -1;
        sink_root();
    }
    // heapq.cuh:79-88
    void pushpop(float k, int64_t v) {
        if (k <= key[0]) return;
        key[0] = k, val[0] = v;
        sink_root();
    }
    // heapq.cuh:47-77
    void replace(float k, int64_t v) {
        int at = 0;
        for (;;) {
            int c = 2 * at + 1;
            if (c >= size) break;
            if (c + 1 < size && key[c + 1] > key[c]) ++c;
            at = c;
        }
        if (k >= key[at]) return;
        while (at > 0) {
            const int up = (at - 1) / 2;
            if (key[up] <= k) break;
            key[at] = key[up], val[at] = val[up];
            at = up;
        }
        key[at] = k, val[at] = v;
    }
};

// ---- per-thread state -----------------------------------------------------------

// bitmask.hpp:11-46: an int32 per node, a node is visited when its word holds
// the current marker; a new marker per query makes clearing unnecessary.
struct ThreadState {
    std::vector<int32_t> seen;
    int32_t marker = 0;
    std::vector<float> keys;
    std::vector<int64_t> vals;

    int32_t *visited(int64_t n) {
        if ((int64_t)seen.size() != n || marker == std::numeric_limits<int32_t>::max()) {
            seen.assign((size_t)n, 0);
            marker = 0;
        }
        marker += 1;
        return seen.data();
    }
    void heaps(int H, HeapView *result, HeapView *open) {
        keys.resize((size_t)3 * H);
        vals.resize((size_t)3 * H);
        *result = HeapView{keys.data(), vals.data(), H};
        *open = HeapView{keys.data() + H, vals.data() + H, 2 * H};
    }
};

thread_local ThreadState tls;

// ---- one query: traverse_cpu.cpp:12-163 --------------------------------------------

void search_one(int64_t *out_I, float *out_D, int32_t *seen, int32_t marker,
                const int64_t *init_I, float *init_D, const int64_t *indptr,
                const int64_t *indices, const float *storage, const float *q,
                int d_model, int d_principle, int n_init, int ef_search, int k,
                int max_iter, HeapView result, HeapView open) {
    // :42-62 the entries' distances cover [0, d_principle); add the rest
    if (d_principle < d_model) {
        for (int i = 0; i < n_init; ++i)
            if (init_I[i] >= 0) prefetch(storage + init_I[i] * (int64_t)d_model + d_principle);
        for (int i = 0; i < n_init; ++i)
            if (init_I[i] >= 0)
                init_D[i] += square_dist(q, storage + init_I[i] * (int64_t)d_model,
                                         d_model, d_principle);
    }
    // :65-79
    result.fill(-kInf);
    open.fill(kInf);
    for (int i = 0; i < n_init; ++i) {
        const int64_t u = init_I[i];
        if (u < 0) continue;
        seen[u] = marker;
        open.replace(init_D[i], u);
    }
    auto admit = [&](const float *d, const int64_t *v, int n) {  // :25-39
        for (int i = 0; i < n; ++i) {
            if (d[i] >= -result.key[0]) continue;
            result.pushpop(-d[i], v[i]);
            open.replace(d[i], v[i]);
        }
    };
    // :82-136
    if (2 * ef_search < max_iter) max_iter = 2 * ef_search;
    for (int step = 0; step < max_iter; ++step) {
        float uk;
        int64_t u;
        open.pop(&uk, &u);
        if (u < 0 || uk >= -result.key[0]) break;
        const int64_t lo = indptr[u], hi = indptr[u + 1];
        for (int64_t e = lo; e < hi; ++e)
            if (indices[e] >= 0) prefetch(&seen[indices[e]]);
        int n = 0;
        float d[kTile];
        int64_t v[kTile];
        for (int64_t e = lo; e < hi; ++e) {
            const int64_t w = indices[e];
            if (w < 0) break;
            if (seen[w] == -1 || seen[w] == marker) continue;
            seen[w] = marker;
            v[n++] = w;
            prefetch(storage + w * (int64_t)d_model);
            if (n == kTile) {
                square_dist4(d, q, storage, v, d_model);
                admit(d, v, n);
                n = 0;
            }
        }
        for (int i = 0; i < n; ++i) d[i] = square_dist(q, storage + v[i] * (int64_t)d_model, d_model);
        admit(d, v, n);
    }
    // :138-148
    for (int i = 0; i < n_init; ++i)
        if (init_I[i] >= 0) result.pushpop(-init_D[i], init_I[i]);
    // :150-162
    float key;
    int64_t val;
    for (int i = k; i < result.size; ++i) result.pop(&key, &val);
    for (int i = 0; i < k; ++i) {
        result.pop(&key, &val);
        out_I[k - 1 - i] = val;
        out_D[k - 1 - i] = -key;
    }
}

}  // namespace

// Replaces `traverse_cpu` (extension/traverse_cpu.cpp:167-257,
// pilot_ann/kernels/__init__.py:47-59).  All pointers are host memory; rows of
// `storage` are addressed by node id; k is the row length of the outputs.
extern "C" int pa_traverse_cpu(int64_t *out_I, float *out_D, int64_t *init_I,
                               float *init_D, const int64_t *indptr,
                               const int64_t *indices, const float *storage,
                               const float *query, int64_t batch,
                               int64_t n_storage, int d_model, int n_init, int k,
                               int ef_search) {
    if (batch < 0 || n_storage <= 0 || n_init < 0 || k < 1) return PA_E_SHAPE;
    if (d_model <= 0 || d_model % 8) return PA_E_DIM;
    const int H = pa_heap_size(ef_search);
    if (H < 0 || ef_search < 1) return PA_E_EF;
    if (batch == 0) return PA_OK;
    if (!out_I || !out_D || !indptr || !indices || !storage || !query ||
        (n_init > 0 && (!init_I || !init_D)))
        return PA_E_NULL;
#pragma omp parallel for schedule(guided)
    for (int64_t b = 0; b < batch; ++b) {
        HeapView result, open;
        tls.heaps(H, &result, &open);
        int32_t *seen = tls.visited(n_storage);
        search_one(out_I + b * k, out_D + b * k, seen, tls.marker,
                   init_I + b * n_init, init_D + b * n_init, indptr, indices,
                   storage, query + b * (int64_t)d_model, d_model, d_model,
                   n_init, ef_search, k, 1024, result, open);
    }
    return PA_OK;
}

// Replaces `traverse_refine` (extension/traverse_cpu.cpp:261-369,
// pilot_ann/kernels/__init__.py:78-94): at most two expansions on the subgraph
// in full dimension from the device stage's candidates (whose distances cover
// the first d_principle coordinates; the rest is added in place), then a
// search of the full graph seeded with that stage's n_buffers results.  Both
// stages share the visited marks.  buf_* may alias init_*
// (pipeline_cpu.cpp:110-114).
extern "C" int pa_traverse_refine(
    int64_t *out_I, float *out_D, int64_t *buf_I, float *buf_D, int64_t *init_I,
    float *init_D, const int64_t *sub_indptr, const int64_t *sub_indices,
    const int64_t *full_indptr, const int64_t *full_indices,
    const float *storage, const float *query, int64_t batch, int64_t n_storage,
    int d_model, int d_principle, int n_init, int n_buffers, int k,
    int ef_search) {
    if (batch < 0 || n_storage <= 0 || n_init < 0 || n_buffers < 1 || k < 1)
        return PA_E_SHAPE;
    if (d_model <= 0 || d_model % 8 || d_principle <= 0 || d_principle % 8 ||
        d_principle > d_model)
        return PA_E_DIM;
    const int H = pa_heap_size(ef_search);
    if (H < 0 || ef_search < 1) return PA_E_EF;
    if (batch == 0) return PA_OK;
    if (!out_I || !out_D || !buf_I || !buf_D || !init_I || !init_D ||
        !sub_indptr || !sub_indices || !full_indptr || !full_indices ||
        !storage || !query)
        return PA_E_NULL;
#pragma omp parallel for schedule(guided)
    for (int64_t b = 0; b < batch; ++b) {
        HeapView result, open;
        tls.heaps(H, &result, &open);
        int32_t *seen = tls.visited(n_storage);
        const float *q = query + b * (int64_t)d_model;
        search_one(buf_I + b * n_buffers, buf_D + b * n_buffers, seen,
                   tls.marker, init_I + b * n_init, init_D + b * n_init,
                   sub_indptr, sub_indices, storage, q, d_model, d_principle,
                   n_init, ef_search, n_buffers, kRefineSteps, result, open);
        search_one(out_I + b * k, out_D + b * k, seen, tls.marker,
                   buf_I + b * n_buffers, buf_D + b * n_buffers, full_indptr,
                   full_indices, storage, q, d_model, d_model, n_buffers,
                   ef_search, k, 1024, result, open);
    }
    return PA_OK;
}

// ---- the reference's operator hooks (extension/ops_cpu.cpp:8-95) -------------
//
// pilot_ann/kernels/__init__.py:5-35 exposes the heap primitives, the visited
// marks and the row distance of the host search one call at a time; the
// reference's operator tests (test/kernel/test_operators.py) are written
// against them.  These run the same code the searches above run.

namespace {
bool heap_args_ok(const float *keys, const int64_t *values, int64_t n) {
    return keys && values && n >= 1 && n < (1ll << 31);
}
}  // namespace

// heapq_pop_cpu, ops_cpu.cpp:8-13: the root leaves, (inf, -1) takes its place.
extern "C" int pa_heapq_pop(float *keys, int64_t *values, int64_t n) {
    if (n == 0) return PA_OK;
    if (!heap_args_ok(keys, values, n)) return n < 0 || n >= (1ll << 31) ? PA_E_SHAPE : PA_E_NULL;
    float k;
    int64_t v;
    HeapView{keys, values, (int)n}.pop(&k, &v);
    return PA_OK;
}

// heapq_pushpop_cpu, ops_cpu.cpp:15-24.
extern "C" int pa_heapq_pushpop(float *keys, int64_t *values, int64_t n,
                                float key, int64_t value) {
    if (n == 0) return PA_OK;
    if (!heap_args_ok(keys, values, n)) return n < 0 || n >= (1ll << 31) ? PA_E_SHAPE : PA_E_NULL;
    HeapView{keys, values, (int)n}.pushpop(key, value);
    return PA_OK;
}

// heapq_replace_cpu, ops_cpu.cpp:26-35.
extern "C" int pa_heapq_replace(float *keys, int64_t *values, int64_t n,
                                float key, int64_t value) {
    if (n == 0) return PA_OK;
    if (!heap_args_ok(keys, values, n)) return n < 0 || n >= (1ll << 31) ? PA_E_SHAPE : PA_E_NULL;
    HeapView{keys, values, (int)n}.replace(key, value);
    return PA_OK;
}

// bitmask_put_cpu, ops_cpu.cpp:37-51: a fresh set of n visited marks (all
// zero), advanced once, with the marker written at every key.  A key outside
// [0, n) is an error here (the reference writes out of bounds).
extern "C" int pa_bitmask_put(int32_t *marks, int64_t n, const int64_t *keys,
                              int64_t n_keys) {
    if (n < 0 || n_keys < 0) return PA_E_SHAPE;
    if ((n && !marks) || (n_keys && !keys)) return PA_E_NULL;
    for (int64_t i = 0; i < n_keys; ++i)
        if (keys[i] < 0 || keys[i] >= n) return PA_E_RANGE;
    std::memset(marks, 0, (size_t)n * sizeof(int32_t));
    const int32_t marker = 1;  // bitmask.hpp:16-31: the first marker
    for (int64_t i = 0; i < n_keys; ++i) marks[keys[i]] = marker;
    return PA_OK;
}

// square_dist_cpu, ops_cpu.cpp:53-85: squared L2 distance of the query to the
// rows nodelist[i] of storage, four rows at a time while more than four are
// left, then one by one (both forms add in the same order).
extern "C" int pa_square_dist(float *out, const float *query,
                              const float *storage, const int64_t *nodelist,
                              int64_t n_nodes, int64_t n_storage, int d_model) {
    if (n_nodes < 0 || n_storage < 0) return PA_E_SHAPE;
    if (d_model <= 0 || d_model % 8) return PA_E_DIM;
    if (n_nodes == 0) return PA_OK;
    if (!out || !query || !storage || !nodelist) return PA_E_NULL;
    for (int64_t i = 0; i < n_nodes; ++i)
        if (nodelist[i] < 0 || nodelist[i] >= n_storage) return PA_E_RANGE;
    int64_t at = 0;
    for (; at + kTile < n_nodes; at += kTile)
        square_dist4(out + at, query, storage, nodelist + at, d_model);
    for (; at < n_nodes; ++at)
        out[at] = square_dist(query, storage + nodelist[at] * (int64_t)d_model, d_model);
    return PA_OK;
}
