/*
 * CPU oracle: a plain-C restatement of PilotANN's host traversal.
 *
 * THIS IS TEST INFRASTRUCTURE.  Nothing that ships (the package, the HIP
 * library, the C-ABI) may call, link or import it; only the test-suite, the
 * smoke check and the benchmark's cpu_baseline leg use it, and only as the
 * checker / the timed CPU baseline.
 *
 * What it restates (all paths are under the reference repository):
 *   heap primitives ............ extension/inc/heapq.cuh:13-88
 *   squared-L2 distance ........ extension/inc/distance.h:31-111
 *   visited epoch array ........ extension/inc/bitmask.hpp:11-46
 *   single-query search ........ extension/traverse_cpu.cpp:12-163
 *   batch driver (one stage) ... extension/traverse_cpu.cpp:167-257
 *   batch driver (refine) ...... extension/traverse_cpu.cpp:261-369
 *   leaf distances of the router extension/routing_cuda.cu:10-66
 * and, with no counterpart in the reference, the library's own wide mode
 * (orc_traverse_wide, at the end): restated here so that the device kernel of
 * that mode has a checker too; what pins it is stated there.
 *
 * Floating point: the reference accumulates (q-x)^2 with one FMA per element
 * into eight independent lanes (element j goes to lane j mod 8) and then adds
 * the eight lanes left to right (distance.h:39-55).  This file fixes exactly
 * that order in IEEE arithmetic (no reassociation), so that a device kernel
 * that follows the same order can be compared bit for bit.  The reference is
 * built with -ffast-math, which lets its compiler reassociate the final
 * eight-term sum; that can move a result by an ulp, never more.
 *
 * Parity pins (see tests/test_oracle_*.py): heaps against Python's heapq and
 * hand-derived states; distance against float64; the search against brute
 * force on small connected graphs, and against hand-built graphs that
 * isolate each rule (iteration cap, stop at the first negative neighbour,
 * entries merged after the loop, front padding when k exceeds the heap, an
 * open list of exactly 2 * HEAP_SIZE cells, the gate in front of both lists,
 * the stop on a popped key equal to the worst kept, the two expansions of
 * the refine's first stage, the visited marks its stages share, and what
 * happens to equal keys in every heap primitive).  Each of these rules was
 * also changed on purpose in a copy of this file; every such copy fails one
 * of those tests.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define ORC_LANES 8

typedef struct {
    float *key;
    int64_t *val;
    int size;
} orc_heap;

/* ---- heaps: heapq.cuh ---------------------------------------------------- */

/* heapq.cuh:13-29 — restore the min-heap below the root after the root
 * changed.  The smaller child wins, the left one on equal keys. */
static void orc_sift_root(orc_heap *h) {
    int at = 0;
    for (;;) {
        int c = 2 * at + 1;
        if (c >= h->size) return;
        if (c + 1 < h->size && h->key[c + 1] < h->key[c]) c += 1;
        if (h->key[at] <= h->key[c]) return;
        float k = h->key[at];
        int64_t v = h->val[at];
        h->key[at] = h->key[c];
        h->val[at] = h->val[c];
        h->key[c] = k;
        h->val[c] = v;
        at = c;
    }
}

/* heapq.cuh:37-45 — take the root, refill it with (inf, -1). */
void orc_heap_pop(float *keys, int64_t *vals, int size, float *out_key,
                  int64_t *out_val) {
    orc_heap h = {keys, vals, size};
    if (out_key) *out_key = keys[0];
    if (out_val) *out_val = vals[0];
    keys[0] = INFINITY;
    vals[0] = -1;
    orc_sift_root(&h);
}

/* heapq.cuh:79-88 — replace the root when the new key is strictly larger. */
void orc_heap_pushpop(float *keys, int64_t *vals, int size, float k,
                      int64_t v) {
    orc_heap h = {keys, vals, size};
    if (k <= keys[0]) return;
    keys[0] = k;
    vals[0] = v;
    orc_sift_root(&h);
}

/* heapq.cuh:47-77 — walk from the root to a leaf through the larger child
 * (the left one on equal keys); overwrite that leaf when the new key is
 * strictly smaller, then let it rise.  The leaf reached is a large one, not
 * necessarily the largest: an insert can displace a live entry while empty
 * slots remain elsewhere. */
void orc_heap_replace(float *keys, int64_t *vals, int size, float k,
                      int64_t v) {
    int at = 0;
    for (;;) {
        int c = 2 * at + 1;
        if (c >= size) break;
        if (c + 1 < size && keys[c + 1] > keys[c]) c += 1;
        at = c;
    }
    if (k >= keys[at]) return;
    keys[at] = k;
    vals[at] = v;
    while (at > 0) {
        int up = (at - 1) / 2;
        if (keys[up] <= keys[at]) break;
        float tk = keys[up];
        int64_t tv = vals[up];
        keys[up] = keys[at];
        vals[up] = vals[at];
        keys[at] = tk;
        vals[at] = tv;
        at = up;
    }
}

/* ---- distance: distance.h ------------------------------------------------ */

/* distance.h:31-55 — squared L2 over [offset, d) of row `row`, eight FMA
 * lanes, lanes added left to right starting from zero. */
float orc_square_dist(const float *q, const float *row, int d, int offset) {
    float lane[ORC_LANES];
    for (int j = 0; j < ORC_LANES; j++) lane[j] = 0.0f;
    for (int o = offset; o < d; o += ORC_LANES) {
        for (int j = 0; j < ORC_LANES; j++) {
            float t = q[o + j] - row[o + j];
            lane[j] = fmaf(t, t, lane[j]);
        }
    }
    float r = 0.0f;
    for (int j = 0; j < ORC_LANES; j++) r += lane[j];
    return r;
}

/* ops_cpu.cpp:53-85 — distances from one query to a list of rows. */
int orc_square_dist_list(float *out, const float *q, const float *storage,
                         const int64_t *nodes, int64_t n, int d) {
    if (d % ORC_LANES) return -1;
    for (int64_t i = 0; i < n; i++)
        out[i] = orc_square_dist(q, storage + nodes[i] * (int64_t)d, d, 0);
    return 0;
}

/* ---- the heap-size ladder: traverse_cpu.cpp:228-254 ----------------------- */

int orc_heap_size(int ef_search) {
    static const int ladder[] = {16,  32,  48,  64,  96,   128,
                                 192, 256, 384, 512, 1024, 2048};
    for (unsigned i = 0; i < sizeof(ladder) / sizeof(ladder[0]); i++)
        if (ef_search <= ladder[i]) return ladder[i];
    return -1;
}

/* ---- one query: traverse_cpu.cpp:12-163 ---------------------------------- */

/* Work counters a caller may ask for (all summed over the queries of a call):
 *   [0] nodes expanded (loop iterations that did not stop the search)
 *   [1] adjacency entries read before the scan of a row ended
 *   [2] distances evaluated in the loop (unvisited neighbours)
 *   [3] candidates admitted to the queues
 *   [4] admitted candidates that displaced a live (finite) entry of the
 *       open heap, or were dropped against one, while it had free slots —
 *       how often the large-leaf rule of heap_replace mattered            */
#define ORC_N_COUNTERS 5

typedef struct {
    float *res_key, *open_key;
    int64_t *res_val, *open_val;
} orc_scratch;

static void orc_search_one(int64_t *out_I, float *out_D, int32_t *seen,
                           const int64_t *init_I, float *init_D,
                           const int64_t *indptr, const int64_t *indices,
                           const float *storage, const float *query,
                           int d_model, int d_principle, int n_init,
                           int ef_search, int k, int32_t marker, int max_iter,
                           int heap_size, orc_scratch *ws, int64_t *counters) {
    const int H = heap_size, O = 2 * heap_size;
    float *res_key = ws->res_key, *open_key = ws->open_key;
    int64_t *res_val = ws->res_val, *open_val = ws->open_val;

    /* :42-62 — entries arrive with the distance over the first d_principle
     * coordinates; add the rest, in place. */
    if (d_principle < d_model) {
        for (int i = 0; i < n_init; i++) {
            int64_t u = init_I[i];
            if (u < 0) continue;
            init_D[i] += orc_square_dist(query, storage + u * (int64_t)d_model,
                                         d_model, d_principle);
        }
    }

    /* :65-79 — result heap holds negated distances (root = worst kept),
     * the open heap plain distances; entries go to the open heap only. */
    for (int i = 0; i < H; i++) res_key[i] = -INFINITY, res_val[i] = -1;
    for (int i = 0; i < O; i++) open_key[i] = INFINITY, open_val[i] = -1;
    for (int i = 0; i < n_init; i++) {
        int64_t u = init_I[i];
        if (u < 0) continue;
        seen[u] = marker;
        orc_heap_replace(open_key, open_val, O, init_D[i], u);
    }

    /* :82-136 */
    if (2 * ef_search < max_iter) max_iter = 2 * ef_search;
    for (int step = 0; step < max_iter; step++) {
        float uk;
        int64_t u;
        orc_heap_pop(open_key, open_val, O, &uk, &u);
        if (u < 0 || uk >= -res_key[0]) break;
        if (counters) counters[0] += 1;
        for (int64_t e = indptr[u]; e < indptr[u + 1]; e++) {
            int64_t v = indices[e];
            if (counters) counters[1] += 1;
            if (v < 0) break; /* :107-109 — ends the row, not just the entry */
            if (seen[v] == -1 || seen[v] == marker) continue;
            seen[v] = marker;
            /* :118-135 batch four rows per distance call; each row's value
             * and the order in which they reach the heaps are those of
             * a one-at-a-time loop, which is what is written here.  The
             * threshold is re-read per candidate as in heap_update :25-39. */
            float d = orc_square_dist(query, storage + v * (int64_t)d_model,
                                      d_model, 0);
            if (counters) counters[2] += 1;
            if (d >= -res_key[0]) continue;
            orc_heap_pushpop(res_key, res_val, H, -d, v);
            if (counters) {
                counters[3] += 1;
                int free_slots = 0;
                for (int i = 0; i < O; i++) free_slots += isinf(open_key[i]);
                int at = 0;
                for (;;) {
                    int c = 2 * at + 1;
                    if (c >= O) break;
                    if (c + 1 < O && open_key[c + 1] > open_key[c]) c += 1;
                    at = c;
                }
                if (free_slots && !isinf(open_key[at])) counters[4] += 1;
            }
            orc_heap_replace(open_key, open_val, O, d, v);
        }
    }

    /* :138-148 — only now do the entries compete for a result slot. */
    for (int i = 0; i < n_init; i++) {
        int64_t u = init_I[i];
        if (u < 0) continue;
        orc_heap_pushpop(res_key, res_val, H, -init_D[i], u);
    }

    /* :150-162 — drop the worst H-k, emit best first.  With k > H the pops
     * past the heap's content return (inf, -1) and land, negated, in front. */
    for (int i = k; i < H; i++) orc_heap_pop(res_key, res_val, H, NULL, NULL);
    for (int i = 0; i < k; i++) {
        float key;
        int64_t val;
        orc_heap_pop(res_key, res_val, H, &key, &val);
        out_I[k - 1 - i] = val;
        out_D[k - 1 - i] = -key;
    }
}

static int orc_scratch_init(orc_scratch *ws, int heap_size) {
    ws->res_key = (float *)malloc(sizeof(float) * heap_size);
    ws->open_key = (float *)malloc(sizeof(float) * 2 * heap_size);
    ws->res_val = (int64_t *)malloc(sizeof(int64_t) * heap_size);
    ws->open_val = (int64_t *)malloc(sizeof(int64_t) * 2 * heap_size);
    return ws->res_key && ws->open_key && ws->res_val && ws->open_val;
}

static void orc_scratch_free(orc_scratch *ws) {
    free(ws->res_key);
    free(ws->open_key);
    free(ws->res_val);
    free(ws->open_val);
}

/* ---- batch drivers ------------------------------------------------------- */

/* traverse_cpu.cpp:167-257.  One search per query over (indptr, indices)
 * with rows of `storage` addressed by node id; k = row length of the output.
 * The reference keeps a pool of int32[n_storage] epoch arrays and hands one
 * to each query (bitmask.hpp:11-76); a fresh marker per query on a per-thread
 * array is the same thing.  Returns 0, or a negative argument error. */
int orc_traverse_cpu(int64_t *out_I, float *out_D, int64_t *init_I,
                     float *init_D, const int64_t *indptr,
                     const int64_t *indices, const float *storage,
                     const float *query, int64_t batch, int64_t n_storage,
                     int d_model, int n_init, int k, int ef_search,
                     int64_t *counters) {
    const int H = orc_heap_size(ef_search);
    if (H < 0) return -1;
    if (d_model % ORC_LANES) return -2;
    int failed = 0;
#pragma omp parallel
    {
        orc_scratch ws;
        int32_t *seen = (int32_t *)calloc((size_t)n_storage, sizeof(int32_t));
        int ok = orc_scratch_init(&ws, H) && seen;
        int32_t marker = 0;
        int64_t local[ORC_N_COUNTERS] = {0};
        if (!ok) {
#pragma omp atomic write
            failed = 1;
        }
#pragma omp for schedule(guided)
        for (int64_t b = 0; b < batch; b++) {
            if (!ok) continue;
            marker += 1;
            orc_search_one(out_I + b * k, out_D + b * k, seen,
                           init_I + b * n_init, init_D + b * n_init, indptr,
                           indices, storage, query + b * (int64_t)d_model,
                           d_model, d_model, n_init, ef_search, k, marker, 1024,
                           H, &ws, counters ? local : NULL);
        }
        if (counters)
            for (int i = 0; i < ORC_N_COUNTERS; i++) {
#pragma omp atomic
                counters[i] += local[i];
            }
        orc_scratch_free(&ws);
        free(seen);
    }
    return failed ? -3 : 0;
}

/* traverse_cpu.cpp:261-369.  Stage 2: at most two expansions on the subgraph
 * starting from the device stage's candidates, whose distances cover the
 * first d_principle coordinates only; the output row has n_buffers slots.
 * Stage 3: ordinary search on the full graph seeded from stage 2's row.
 * Both stages share one marker, so stage 3 never re-evaluates a node stage 2
 * has seen.  buffer_* may alias initial_* (pipeline_cpu.cpp:110-114): stage
 * 2 reads every entry before it writes its output. */
int orc_traverse_refine(int64_t *out_I, float *out_D, int64_t *buf_I,
                        float *buf_D, int64_t *init_I, float *init_D,
                        const int64_t *sub_indptr, const int64_t *sub_indices,
                        const int64_t *full_indptr, const int64_t *full_indices,
                        const float *storage, const float *query, int64_t batch,
                        int64_t n_storage, int d_model, int d_principle,
                        int n_init, int n_buffers, int k, int ef_search) {
    const int H = orc_heap_size(ef_search);
    if (H < 0) return -1;
    if (d_model % ORC_LANES || d_principle % ORC_LANES) return -2;
    int failed = 0;
#pragma omp parallel
    {
        orc_scratch ws;
        int32_t *seen = (int32_t *)calloc((size_t)n_storage, sizeof(int32_t));
        int ok = orc_scratch_init(&ws, H) && seen;
        int32_t marker = 0;
        if (!ok) {
#pragma omp atomic write
            failed = 1;
        }
#pragma omp for schedule(guided)
        for (int64_t b = 0; b < batch; b++) {
            if (!ok) continue;
            marker += 1;
            const float *q = query + b * (int64_t)d_model;
            orc_search_one(buf_I + b * n_buffers, buf_D + b * n_buffers, seen,
                           init_I + b * n_init, init_D + b * n_init, sub_indptr,
                           sub_indices, storage, q, d_model, d_principle,
                           n_init, ef_search, n_buffers, marker, 2, H, &ws,
                           NULL);
            orc_search_one(out_I + b * k, out_D + b * k, seen,
                           buf_I + b * n_buffers, buf_D + b * n_buffers,
                           full_indptr, full_indices, storage, q, d_model,
                           d_model, n_buffers, ef_search, k, marker, 1024, H,
                           &ws, NULL);
        }
        orc_scratch_free(&ws);
        free(seen);
    }
    return failed ? -3 : 0;
}

/* ---- router: routing_cuda.cu:70-113 --------------------------------------- */

/* The route of a query is the nearest route vector; the reference takes it
 * from a library cdist+argmin (routing_cuda.cu:93-95).  Here the distances
 * are formed in double precision so that the oracle's choice is the exact
 * argmin (first index on an exact tie); a float implementation may differ
 * from it only where two routes tie within float rounding.  The leaf
 * distances are direct sums of squared differences (routing_cuda.cu:53-61);
 * they use the same eight-lane order as every other distance here, which the
 * reference's own test accepts (atol 1e-3, test_routing.py:82-85). */
int orc_route(int64_t *router, float *dist, const float *query,
              const float *route_vectors, const float *entry_vectors,
              int64_t batch, int n_routers, int n_leaves, int d) {
    if (d % ORC_LANES) return -2;
#pragma omp parallel for schedule(static)
    for (int64_t b = 0; b < batch; b++) {
        const float *q = query + b * (int64_t)d;
        int best = 0;
        double best_d = INFINITY;
        for (int r = 0; r < n_routers; r++) {
            const float *p = route_vectors + r * (int64_t)d;
            double s = 0.0;
            for (int j = 0; j < d; j++) {
                double t = (double)q[j] - (double)p[j];
                s += t * t;
            }
            if (s < best_d) best_d = s, best = r;
        }
        router[b] = best;
        const float *leaves = entry_vectors + (int64_t)best * n_leaves * d;
        for (int l = 0; l < n_leaves; l++)
            dist[b * n_leaves + l] =
                orc_square_dist(q, leaves + l * (int64_t)d, d, 0);
    }
    return 0;
}

/* ---- the wide mode of the device traversal ---------------------------------
 *
 * Not a restatement of anything in the reference: the library's labelled
 * throughput mode (pa_traverse_wide), written down once more in plain C so
 * that the device kernel can be compared id for id.  A best-first search
 * whose result list and open list are one pool of the P best candidates seen
 * (P = the heap size of the ladder for k, rounded up to a multiple of 64),
 * ordered by (distance, storage row):
 *   - the entries are marked and offered to the pool, 64 at a time (one
 *     without a storage row keeps its global id and is never expanded);
 *   - a step takes the `width` first candidates of the pool that are not yet
 *     expanded, walks their rows of neighbours in that order (a row ends at
 *     its first negative id; nodes without a storage row are skipped), marks
 *     what is new and offers it, with its distance, to the pool, 64 at a
 *     time in that order: of a group of 64 those strictly below the pool's
 *     last key enter, the pool keeps its P smallest;
 *   - the search ends when no candidate of the pool is left to expand, or
 *     after min(1024, 2k) expansions.
 * Pins: the distances are orc_square_dist's; with width 1 and a pool that
 * holds every node the result is the exact nearest neighbours on a connected
 * graph (brute force, tests/test_oracle_wide.py); the stop rule, the cap and
 * the order of a step are stepped by hand there on small graphs.
 */
#define ORC_WIDE_DONE 0x80000000u
#define ORC_WIDE_GLOBAL 0x40000000u
#define ORC_WIDE_ID 0x3fffffffu

typedef struct {
    int32_t key;   /* order-preserving integer image of the float distance */
    uint32_t val;  /* storage row, or DONE | GLOBAL | global id */
} orc_wide_entry;

static int32_t orc_float_key(float x) {
    int32_t b;
    memcpy(&b, &x, 4);
    return b ^ ((b >> 31) & 0x7fffffff);
}

static float orc_key_float(int32_t k) {
    int32_t b = k ^ ((k >> 31) & 0x7fffffff);
    float x;
    memcpy(&x, &b, 4);
    return x;
}

static int orc_wide_less(const orc_wide_entry *a, const orc_wide_entry *b) {
    if (a->key != b->key) return a->key < b->key;
    return a->val < b->val;
}

static int orc_wide_cmp(const void *a, const void *b) {
    const orc_wide_entry *x = a, *y = b;
    return orc_wide_less(x, y) ? -1 : orc_wide_less(y, x) ? 1 : 0;
}

/* offers `n` staged entries to the pool, 64 at a time */
static void orc_wide_offer(orc_wide_entry *pool, int P, orc_wide_entry *staged,
                           int n, orc_wide_entry *tmp, int64_t *admitted) {
    for (int base = 0; base < n; base += 64) {
        const int32_t worst = pool[P - 1].key;
        int m = 0;
        memcpy(tmp, pool, (size_t)P * sizeof(*pool));
        for (int i = base; i < n && i < base + 64; ++i)
            if (staged[i].key < worst) tmp[P + m++] = staged[i];
        if (!m) continue;
        if (admitted) *admitted += m;
        qsort(tmp, (size_t)(P + m), sizeof(*tmp), orc_wide_cmp);
        memcpy(pool, tmp, (size_t)P * sizeof(*pool));
    }
}

int orc_traverse_wide(int64_t *out_I, float *out_D, const int64_t *init_I,
                      const float *init_D, const int64_t *indptr,
                      const int64_t *indices, const int64_t *mapping,
                      const float *storage, const float *query, int64_t batch,
                      int64_t n_nodes, int d, int n_init, int k, int width,
                      int64_t *counters) {
    const int H = orc_heap_size(k);
    if (H < 0 || d % ORC_LANES || width < 1 || width > 4) return -1;
    const int P = (H + 63) / 64 * 64;
    const int max_iter = 2 * k < 1024 ? 2 * k : 1024;
    int64_t n_rows = 0;
    for (int64_t g = 0; g < n_nodes; ++g)
        if (mapping[g] >= n_rows) n_rows = mapping[g] + 1;
    int64_t *gid = malloc((size_t)(n_rows ? n_rows : 1) * sizeof(*gid));
    for (int64_t g = 0; g < n_nodes; ++g)
        if (mapping[g] >= 0) gid[mapping[g]] = g;
    int64_t total[ORC_N_COUNTERS] = {0, 0, 0, 0, 0};
#pragma omp parallel
    {
        unsigned char *seen = malloc((size_t)(n_rows ? n_rows : 1));
        orc_wide_entry *pool = malloc((size_t)(P + 64) * sizeof(*pool));
        orc_wide_entry *tmp = malloc((size_t)(P + 64) * sizeof(*tmp));
        orc_wide_entry *staged = malloc(4 * 64 * sizeof(*staged));
        int64_t mine[ORC_N_COUNTERS] = {0, 0, 0, 0, 0};
#pragma omp for schedule(guided)
        for (int64_t b = 0; b < batch; ++b) {
            const float *q = query + b * d;
            memset(seen, 0, (size_t)n_rows);
            for (int i = 0; i < P; ++i) {
                pool[i].key = 0x7f800000;
                pool[i].val = 0xffffffffu;
            }
            /* the entries */
            for (int base = 0; base < n_init; base += 64) {
                int n = 0;
                for (int i = base; i < n_init && i < base + 64; ++i) {
                    const int64_t g = init_I[b * n_init + i];
                    if (g < 0 || g >= n_nodes) continue;
                    staged[n].key = orc_float_key(init_D[b * n_init + i]);
                    if (mapping[g] >= 0) {
                        seen[mapping[g]] = 1;
                        staged[n].val = (uint32_t)mapping[g];
                    } else {
                        staged[n].val = ORC_WIDE_DONE | ORC_WIDE_GLOBAL | (uint32_t)g;
                    }
                    ++n;
                }
                orc_wide_offer(pool, P, staged, n, tmp, NULL);
            }
            int n_expand = 0;
            while (n_expand < max_iter) {
                int want = width < max_iter - n_expand ? width : max_iter - n_expand;
                int64_t chosen[4];
                int n_chosen = 0;
                for (int i = 0; i < P && n_chosen < want; ++i)
                    if (!(pool[i].val & ORC_WIDE_DONE)) {
                        chosen[n_chosen++] = pool[i].val & ORC_WIDE_ID;
                        pool[i].val |= ORC_WIDE_DONE;
                    }
                if (!n_chosen) break;
                n_expand += n_chosen;
                int n = 0;
                for (int w = 0; w < n_chosen; ++w) {
                    const int64_t u = gid[chosen[w]];
                    for (int64_t e = indptr[u]; e < indptr[u + 1]; ++e) {
                        const int64_t v = indices[e];
                        if (v < 0) break;
                        mine[1] += 1;
                        const int64_t row = v < n_nodes ? mapping[v] : -1;
                        if (row < 0 || seen[row]) continue;
                        seen[row] = 1;
                        staged[n].key = orc_float_key(
                            orc_square_dist(q, storage + v * d, d, 0));
                        staged[n].val = (uint32_t)row;
                        ++n;
                    }
                }
                mine[2] += n;
                orc_wide_offer(pool, P, staged, n, tmp, &mine[3]);
            }
            mine[0] += n_expand;
            mine[4] += k;
            for (int i = 0; i < k; ++i) {
                const uint32_t val = pool[i].val;
                int64_t id = -1;
                if (val != 0xffffffffu)
                    id = (val & ORC_WIDE_GLOBAL) ? (int64_t)(val & ORC_WIDE_ID)
                                                 : gid[val & ORC_WIDE_ID];
                out_I[b * k + i] = id;
                out_D[b * k + i] = orc_key_float(pool[i].key);
            }
        }
#pragma omp critical
        for (int c = 0; c < ORC_N_COUNTERS; ++c) total[c] += mine[c];
        free(seen);
        free(pool);
        free(tmp);
        free(staged);
    }
    if (counters)
        for (int c = 0; c < ORC_N_COUNTERS; ++c) counters[c] += total[c];
    free(gid);
    return 0;
}

int orc_num_threads(void) {
#ifdef _OPENMP
    return omp_get_max_threads();
#else
    return 1;
#endif
}
