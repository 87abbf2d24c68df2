/*
 * pilotann.h — C ABI of the MI355X search stage of PilotANN.
 *
 * Plain pointers and sizes only; every device pointer is memory of the GPU
 * that is current when the call is made, every call enqueues on the HIP
 * stream it is given (hipStream_t passed as void*, NULL = the null stream)
 * and returns without synchronising unless it says otherwise.
 *
 * Return value: 0 on success; < 0 an argument error (PA_E_*), detected on the
 * host before anything is launched; > 0 a hipError_t from the runtime.
 * pa_error_string() turns either into text.
 *
 * Each entry point names the reference interface it replaces (paths under
 * the reference repository).
 */
#ifndef PILOTANN_H
#define PILOTANN_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PA_BEAM_WIDTH 4     /* traverse_cuda.cu:13  — output is [B, 4, ef]      */
#define PA_MAX_NEIGHBORS 64 /* traverse_cuda.cu:280 — 4 * n_neighbors <= 256    */
#define PA_MAX_EF_TOTAL 2048 /* traverse_cpu.cpp:250 — largest heap of the ladder */

enum {
    PA_OK = 0,
    PA_E_NULL = -1,        /* a required pointer is NULL                         */
    PA_E_SHAPE = -2,       /* a size is negative or inconsistent                 */
    PA_E_DIM = -3,         /* vector length not a multiple of 8 (distance.h:35-36) */
    PA_E_NEIGHBORS = -4,   /* n_neighbors outside 1..64                          */
    PA_E_EF = -5,          /* beam * ef outside 1..2048                          */
    PA_E_WORKSPACE = -6,   /* workspace too small or not 256-byte aligned          */
    PA_E_GRAPH = -7,       /* pa_graph_prepare found a malformed graph           */
    PA_E_LEAVES = -8,      /* n_leaves not a multiple of 32 (routing_cuda.cu:90) */
    PA_E_CHUNK = -9,       /* batch not a multiple of chunk (pipeline_cpu.cpp:58) */
    PA_E_RANGE = -10,      /* an id does not fit 31 bits                         */
    PA_E_STATIC = -11      /* index too large for pa_traverse_static's scratch   */
};

const char *pa_error_string(int code);

/* Heap size the host search uses for a given ef_search
 * (traverse_cpu.cpp:228-254): 16,32,48,64,96,128,192,256,384,512,1024,2048;
 * -1 above 2048. */
int pa_heap_size(int ef_search);

/* ---- device graph -------------------------------------------------------- */

/*
 * Builds the device-resident form of a subgraph once per index
 * (the reference re-reads indptr / indices / mapping as int64 on every
 * expansion: traverse_cuda.cu:130-140,199).
 *
 *   indptr  [n_nodes + 1], indices [nnz], mapping [n_nodes]:
 *           the int64 device arrays `traverse_cuda` receives
 *           (traverse_cuda.cu:249-258); indices are global ids, mapping is
 *           global id -> row of `storage` or -1.
 *   adj     [n_storage * n_neighbors] int32, out: row r lists, in order, the
 *           storage rows of the neighbours of the node stored in row r, cut
 *           at the first negative id (traverse_cpu.cpp:107-109), without
 *           self loops, repeats of an earlier entry of the same row, or
 *           neighbours that have no storage row; -1 pads.  Dropping those
 *           entries does not change what a search does: each of them is
 *           already marked visited when the row is scanned.
 *   gid     [n_storage] int32, out: storage row -> global id.
 *   status  [1] int32 device word, out: 0, or a bit set: 1 = mapping is not
 *           a bijection onto 0..n_storage-1, 2 = a row is longer than
 *           n_neighbors, 4 = an id is >= n_nodes, 8 = a row of a stored node
 *           does not lie inside indices[0..nnz) (it is read as empty).
 *
 * Synchronises the stream and returns PA_E_GRAPH when status != 0.
 */
int pa_graph_prepare(const int64_t *indptr, const int64_t *indices,
                     const int64_t *mapping, int64_t n_nodes,
                     int64_t n_storage, int64_t nnz, int n_neighbors,
                     int32_t *adj, int32_t *gid, int32_t *status, void *stream);

/*
 * Builds the device layout of vector rows, once per index: copies plain rows
 * src [n_rows * d] into dst (another buffer of the same size) such that
 * within every 16 floats (two groups of eight) the four 8-byte pairs of the
 * first group and those of the second are interleaved, pair a of both next to
 * each other.  The distance kernels give lane a of a quad accumulators 2a and
 * 2a + 1 of the reference's eight (extension/inc/distance.h:31-55); in this
 * layout the lane reads its share of two groups with one 16-byte load and a
 * quad covers 64 contiguous bytes per instruction.  A last group without a
 * partner (d / 8 odd) stays as it is.  d must be a multiple of 8.
 * Asynchronous on `stream`.
 */
int pa_rows_prepare(float *dst, const float *src, int64_t n_rows, int d,
                    void *stream);

/* ---- traversal ----------------------------------------------------------- */

/*
 * Sizes the scratch memory pa_traverse needs: one visited bitmask of
 * n_storage bits per resident wavefront plus a work counter.  n_slots
 * (out, may be NULL) is the number of wavefronts that will be launched.
 */
int pa_traverse_plan(int64_t n_storage, int64_t batch, int dp, int ef_total,
                     int *n_slots, size_t *workspace_bytes);

/*
 * Replaces `traverse_cuda` (extension/traverse_cuda.cu:249-316,
 * pilot_ann/kernels/__init__.py:62-75).
 *
 * Per query: the best-first search of the host kernel
 * (extension/traverse_cpu.cpp:12-163) with ef_search = k = beam * ef on the
 * prepared subgraph, distances over the dp stored coordinates.  One
 * wavefront runs one query.
 *
 *   out_I [batch * beam * ef] int64, out_D [same] float: the k results of
 *         query b start at b * k, best first; unused slots hold -1 / +inf
 *         at the end.  Ids are global.
 *   adj, gid: from pa_graph_prepare.   mapping [n_nodes] int64 as there.
 *   storage [n_storage * dp] float in the layout of pa_rows_prepare,
 *         query [batch * dp] float (plain).
 *   init_I / init_D [batch * n_init]: entry ids (global, negative = unused)
 *         and their squared distances over the same dp coordinates.
 *   counters: NULL, or 5 uint64 device words that are incremented by
 *         {nodes expanded, adjacency entries read, distances evaluated,
 *          candidates admitted, result slots written}.
 *   workspace: at least pa_traverse_plan()'s bytes, 256-byte aligned, not
 *         shared with a call that may run at the same time.
 */
int pa_traverse(int64_t *out_I, float *out_D, const int32_t *adj,
                const int32_t *gid, const int64_t *mapping,
                const float *storage, const float *query,
                const int64_t *init_I, const float *init_D, int64_t batch,
                int64_t n_nodes, int64_t n_storage, int dp, int n_init,
                int beam, int ef, int n_neighbors, void *workspace,
                size_t workspace_bytes, uint64_t *counters, void *stream);

/*
 * pa_traverse for callers that cannot allocate device memory (code under HIP
 * graph capture, serving loops and harnesses that forbid it).  No counterpart
 * in the reference.  Same arguments and same results as pa_traverse, without
 * the workspace: the scratch is a static device array of
 * PA_STATIC_SCRATCH_BYTES inside the library (each GPU the library runs on
 * holds one until the process ends), and the call allocates nothing.
 *
 * A resident wavefront needs its visited slice (ceil(n_storage / 32) words
 * rounded up to 1 KiB), 8 bytes per entry of its log of admitted candidates
 * (2 H + 128 entries, H = pa_heap_size(beam * ef)) and, with the longest
 * lists only (H = 2048), 16.6 KB for the last two levels of its open list; as
 * many wavefronts are launched as the array holds (fewer than pa_traverse
 * would use when the index is large, which costs time, not correctness).
 * PA_E_STATIC when fewer than min(batch, 256) fit: with the longest lists
 * that is n_storage above about 3.7 million rows (4.1 million at H = 512).
 *
 * All calls on one GPU share the array: calls that may overlap on one GPU
 * (different streams, different threads) race; serialise them.  Nothing is
 * kept between calls.
 */
#define PA_STATIC_SCRATCH_BYTES (128u << 20)
int pa_traverse_static(int64_t *out_I, float *out_D, const int32_t *adj,
                       const int32_t *gid, const int64_t *mapping,
                       const float *storage, const float *query,
                       const int64_t *init_I, const float *init_D,
                       int64_t batch, int64_t n_nodes, int64_t n_storage,
                       int dp, int n_init, int beam, int ef, int n_neighbors,
                       uint64_t *counters, void *stream);

/*
 * The wide mode of the traversal: a labelled throughput mode beside
 * pa_traverse, never the default.  No counterpart in the reference's host
 * search, which pa_traverse reproduces; its shape is that of the reference's
 * device kernel (extension/traverse_cuda.cu:116-226: several nodes expanded
 * per step, one shared visited set).  The result list and the open list are
 * one pool of the best candidates seen (as many as pa_traverse's result list,
 * rounded up to a multiple of 64), sorted by distance; a step expands the
 * `width` (1..4) best candidates not yet expanded together and merges their
 * fresh neighbours into the pool with a bitonic network; the search ends when
 * every candidate in the pool is expanded, or after min(1024, 2 * beam * ef)
 * expansions.  Same arguments, output layout, distance arithmetic and visited
 * set as pa_traverse: the distance returned for an id is bit for bit the host
 * search's.  The ids are those of a best-first search that expands in groups
 * and keeps its open list as long as its result list; they are not promised
 * to equal traverse_cpu's (the recall of the whole search is the measure).
 * Ids must fit 30 bits.  workspace: pa_traverse_wide_plan()'s bytes.
 */
int pa_traverse_wide_plan(int64_t n_storage, int64_t batch, int dp,
                          int ef_total, int *n_slots, size_t *workspace_bytes);
int pa_traverse_wide(int64_t *out_I, float *out_D, const int32_t *adj,
                     const int32_t *gid, const int64_t *mapping,
                     const float *storage, const float *query,
                     const int64_t *init_I, const float *init_D, int64_t batch,
                     int64_t n_nodes, int64_t n_storage, int dp, int n_init,
                     int beam, int ef, int n_neighbors, int width,
                     void *workspace, size_t workspace_bytes,
                     uint64_t *counters, void *stream);

/* ---- entry router -------------------------------------------------------- */

/*
 * Replaces `routing_cuda` (extension/routing_cuda.cu:70-113,
 * pilot_ann/kernels/__init__.py:97-103).
 *
 *   router [batch] int64, out: index of the nearest route vector.
 *   dist   [batch * n_leaves] float, out: squared L2 from the query to each
 *          leaf vector of its route, entry_vectors[router[b], l, :].
 *   query [batch * dp], route_vectors [n_routers * dp],
 *   entry_vectors [n_routers * n_leaves * dp], all float.
 *   entry_nodes [n_routers * n_leaves] int64 and entry_ids [batch * n_leaves]
 *          int64, out: both NULL, or the ids of the chosen route's leaves are
 *          written as well, entry_ids[b][l] = entry_nodes[router[b]][l] — the
 *          `index_select` that follows the call in pilot_ann/layers/entry.py:86.
 * With n_routers == 0 every query uses group 0 of entry_vectors and `router`
 * may be NULL: the distances of a fixed entry list
 * (pilot_ann/layers/entry.py:70-77).
 */
int pa_route(int64_t *router, float *dist, const float *query,
             const float *route_vectors, const float *entry_vectors,
             int64_t batch, int n_routers, int n_leaves, int dp,
             const int64_t *entry_nodes, int64_t *entry_ids, void *stream);

/*
 * Replaces the query rotation of `IndexStaged.search`
 * (pilot_ann/layers/staged.py:198-201: `query @ VT.T`, then the first
 * d_principle coordinates for the device stage), on the matrix cores.
 *
 *   out   [batch * n_out] float, out: out[b][j] = sum_k query[b][k] * VT[j][k]
 *         for j < n_out (n_out = d for the whole rotation, d_principle for
 *         the device stage's part).
 *   query [batch * d], VT [d * d] (row j = basis vector j), float, device.
 * d must be a multiple of 8, 1 <= n_out <= d.  Float32 accumulation in another
 * order than a host matmul: results agree to rounding, not bit for bit.
 */
int pa_rotate(float *out, const float *query, const float *VT, int64_t batch,
              int d, int n_out, void *stream);

/* ---- host stages and the chunk pipeline ------------------------------------- */

/*
 * Replaces `traverse_cpu` (extension/traverse_cpu.cpp:167-257,
 * pilot_ann/kernels/__init__.py:47-59): one best-first search per query on the
 * CPU (OpenMP over queries).  Host pointers.  out_* are [batch * k], init_*
 * [batch * n_init], rows of storage [n_storage * d_model] are addressed by
 * node id.  Heap size = pa_heap_size(ef_search); at most min(1024,
 * 2 * ef_search) expansions.
 */
int pa_traverse_cpu(int64_t *out_I, float *out_D, int64_t *init_I,
                    float *init_D, const int64_t *indptr,
                    const int64_t *indices, const float *storage,
                    const float *query, int64_t batch, int64_t n_storage,
                    int d_model, int n_init, int k, int ef_search);

/*
 * Replaces `traverse_refine` (extension/traverse_cpu.cpp:261-369,
 * pilot_ann/kernels/__init__.py:78-94).  Host pointers.  init_* [batch *
 * n_init] hold the device stage's candidates with distances over the first
 * d_principle coordinates; the remaining coordinates are added to init_D in
 * place.  Stage 2 (at most two expansions on the subgraph) writes buf_*
 * [batch * n_buffers], stage 3 (full graph) writes out_* [batch * k].  buf_*
 * may be the same memory as init_*.
 */
int pa_traverse_refine(int64_t *out_I, float *out_D, int64_t *buf_I,
                       float *buf_D, int64_t *init_I, float *init_D,
                       const int64_t *sub_indptr, const int64_t *sub_indices,
                       const int64_t *full_indptr, const int64_t *full_indices,
                       const float *storage, const float *query, int64_t batch,
                       int64_t n_storage, int d_model, int d_principle,
                       int n_init, int n_buffers, int k, int ef_search);

/*
 * Nearest-neighbour candidates for graph construction, the step the reference
 * leaves to faiss (pilot_ann/utils/graphs.py:15-20,52-56; no entry point of
 * the reference's extension corresponds to it).  For each of m query rows the
 * `keep` (64, 128, 256 or 512) base rows with the smallest
 * |x_j|^2 - 2 q_i . x_j, products in half precision with float accumulation,
 * unordered.  query_f16 and base_f16 hold m and n IEEE half rows of d
 * elements, d % 64 == 0 (pad rows with zeros), and must be readable up to the
 * next multiple of pa_knn_tile_rows() (256) rows: the kernel loads whole tiles,
 * and what the padding rows hold does not matter; base_norm [n] are the
 * squared lengths of the base rows; n >= 1, and pa_knn_list_capacity() is 0
 * for any other `keep`.  Values must fit the half range: scale both sets by
 * one factor first.  The base rows are dealt to n_seg workgroups per tile of
 * query rows (n_seg > 1 when m is too small to fill the device; a segment
 * starts its lists from nothing, so many segments cost more than they
 * spread); segment s of query i leaves its list at
 * cand_score / cand_id [(s * m + i) * pa_knn_list_capacity(keep)], of which
 * the first cand_count [s * m + i] (at most keep) entries are valid.  Device
 * pointers; enqueued on `stream`.
 */
int64_t pa_knn_list_capacity(int keep);
int pa_knn_tile_rows(void);
int pa_knn(float *cand_score, int32_t *cand_id, int32_t *cand_count,
           const void *query_f16, const void *base_f16, const float *base_norm,
           int64_t m, int64_t n, int d, int keep, int n_seg, void *stream);

/*
 * The exact ranking that follows pa_knn (faiss' part in the reference,
 * pilot_ann/utils/graphs.py:15-20; no entry point of the reference's extension
 * corresponds to it): dist [m * k] receives the squared float32 distances
 * from rows first .. first + m of `rows` [n * d] to their candidates
 * cand [m * k] (int64 row numbers); infinity for a candidate that is -1, out
 * of range or the row itself.  d % 4 == 0, d <= 4096.  Device pointers;
 * enqueued on `stream`.
 */
int pa_knn_rerank(float *dist, const float *rows, const int64_t *cand,
                  int64_t m, int64_t first, int64_t n, int d, int k, void *stream);

/*
 * Occlusion pruning of candidate lists, the edge selection of the graph
 * builder (faiss' part in the reference, pilot_ann/utils/graphs.py:15-20,52-56;
 * no entry point of the reference's extension corresponds to it).  For each of
 * n nodes: cand_dist [n * k] are the distances of its k <= 512 candidates,
 * closest first, pair [n * k * k] the distances between its candidates.
 * Candidate j is kept unless an earlier kept candidate r has
 * pair[j][r] < cand_dist[j]; selected [n * m_keep] receives the positions of
 * the kept candidates in order, then (with fill != 0) the closest rejected
 * ones, then -1.  Device pointers; enqueued on `stream`.
 */
int pa_graph_prune(int32_t *selected, const float *pair, const float *cand_dist,
                   int64_t n, int k, int m_keep, int fill, void *stream);

/*
 * The same pruning straight from the rows (no counterpart in the reference's
 * extension either): the distances between a node's k <= 256 candidates are
 * made inside the kernel and never stored.  rows_hi_f16 / rows_lo_f16 hold
 * every row as two half-precision parts (row * s = hi + lo, rows of d
 * elements, d % 64 == 0, padded with zeros), norm [rows] the squared lengths
 * of the scaled rows, n_rows the number of rows behind them, cand [n * k] the
 * candidates' row numbers (closest first, -1 after the last; a number at or
 * beyond n_rows counts as -1 and nothing is read for it), cand_dist [n * k] their squared distances to the node in
 * the rows' own units and scale2 = s * s.  A pair's distance is
 * |a|^2 + |b|^2 - 2 (hi.hi + hi.lo + lo.hi): the float32 value to about 22
 * bits.  selected as for pa_graph_prune.  Device pointers; enqueued on
 * `stream`.
 */
int pa_graph_prune_rows(int32_t *selected, const void *rows_hi_f16,
                        const void *rows_lo_f16, const float *norm,
                        const int64_t *cand, const float *cand_dist, int64_t n,
                        int64_t n_rows, int d, int k, int m_keep, int fill,
                        float scale2, void *stream);

/*
 * The reference's operator hooks (extension/ops_cpu.cpp:8-95,
 * pilot_ann/kernels/__init__.py:5-35): one call of a heap primitive of
 * extension/inc/heapq.cuh on a host array heap of n (key, value) cells, a set
 * of visited marks, and the row distance of extension/inc/distance.h.  Host
 * pointers; the code is the one pa_traverse_cpu runs.
 *
 * pa_heapq_pop: heapq_pop_cpu (:8-13) - the root is dropped, (inf, -1) sinks
 * from its place.  pa_heapq_pushpop: heapq_pushpop_cpu (:15-24) - a key larger
 * than the root replaces it and sinks.  pa_heapq_replace: heapq_replace_cpu
 * (:26-35) - a key smaller than the leaf reached through the larger children
 * overwrites that leaf and rises.
 */
int pa_heapq_pop(float *keys, int64_t *values, int64_t n);
int pa_heapq_pushpop(float *keys, int64_t *values, int64_t n, float key,
                     int64_t value);
int pa_heapq_replace(float *keys, int64_t *values, int64_t n, float key,
                     int64_t value);

/*
 * bitmask_put_cpu (ops_cpu.cpp:37-51, extension/inc/bitmask.hpp:11-46): marks
 * [n] := 0, then the first marker (1) at every key.  Keys outside [0, n) are
 * refused with PA_E_RANGE before anything is written.
 */
int pa_bitmask_put(int32_t *marks, int64_t n, const int64_t *keys,
                   int64_t n_keys);

/*
 * square_dist_cpu (ops_cpu.cpp:53-85): out[i] = squared L2 distance between
 * query [d_model] and row nodelist[i] of storage [n_storage * d_model], in the
 * summation order of distance.h:31-55.  d_model % 8 == 0.
 */
int pa_square_dist(float *out, const float *query, const float *storage,
                   const int64_t *nodelist, int64_t n_nodes, int64_t n_storage,
                   int d_model);

/*
 * Replaces `pipeline` (extension/pipeline_cpu.cpp:32-145,
 * pilot_ann/kernels/__init__.py:106-124): splits the batch into chunks, runs
 * pa_traverse for chunk i+1 and i+2 on two internal streams while
 * pa_traverse_refine finishes chunk i on the host.
 *
 *   topk_I / topk_D [batch * k]: host, out.
 *   full_* / sub_* : host CSR of the full graph and of the subgraph (global
 *   ids), storage [n_nodes * d_model] and query [batch * d_model]: host.
 *   adj, gid, mapping, storage_dev [n_storage * d_principle] (in the layout
 *   of pa_rows_prepare),
 *   query_dev [batch * d_principle], init_I / init_D [batch * n_init]: device.
 *   caller_stream: the stream that produced query_dev / init_*; it is
 *   synchronised before the first chunk starts (pipeline_cpu.cpp:74-75).
 *
 * Blocking.  Device and pinned buffers are kept between calls.  Calls are
 * serialised by a lock.
 */
int pa_pipeline(int64_t *topk_I, float *topk_D, const int64_t *full_indptr,
                const int64_t *full_indices, const int64_t *sub_indptr,
                const int64_t *sub_indices, const float *storage,
                const float *query, const int32_t *adj, const int32_t *gid,
                const int64_t *mapping, const float *storage_dev,
                const float *query_dev, const int64_t *init_I,
                const float *init_D, int64_t batch, int64_t n_nodes,
                int64_t n_storage, int d_model, int d_principle, int n_init,
                int n_neighbors, int ef_search, int k, int chunk_size,
                void *caller_stream);

/* ---- refine on the device ---------------------------------------------------- */

/*
 * `traverse_refine` (extension/traverse_cpu.cpp:261-369) run on the device
 * instead of the host: same arguments, same two searches per query, same
 * results (distances bit for bit, ids up to exact distance ties), with every
 * pointer in device memory.  The reference has no device version of this
 * stage; it is for indexes whose full-dimension rows fit device memory.
 *
 *   sub_adj, sub_gid, sub_mapping: the subgraph as pa_graph_prepare made it
 *         for pa_traverse (rows of sampled-node ranks, rank -> node, node ->
 *         rank), sub_neighbors its row length.
 *   full_adj: the full graph from pa_graph_prepare with the identity mapping
 *         (n_storage == n_nodes), full_neighbors its row length.
 *   storage [n_nodes * d_model]: all rows in full dimension, in the layout
 *         of pa_rows_prepare.   query [batch * d_model] (plain).
 *   init_I / init_D [batch * n_init]: the candidates; init_D is completed in
 *         place.  buf_* [batch * n_buffers] receives the first search's
 *         result and may be the same memory as init_*.  out_* [batch * k].
 *         Where a row is longer than pa_heap_size(ef_search) the surplus
 *         slots come first and hold -1 / -inf (traverse_cpu.cpp:150-162).
 *   counters: NULL, or 6 uint64 device words incremented by {expansions on
 *         the subgraph, expansions on the full graph, full-dimension
 *         distances, candidates admitted, distances completed, adjacency
 *         entries read}.
 *   workspace: at least pa_refine_plan()'s bytes, 256-byte aligned, not
 *         shared with a call that may run at the same time.
 * Asynchronous on `stream`.
 */
int pa_refine_plan(int64_t n_nodes, int64_t batch, int d_model, int ef_search,
                   int *n_slots, size_t *workspace_bytes);
int pa_refine(int64_t *out_I, float *out_D, int64_t *buf_I, float *buf_D,
              const int64_t *init_I, float *init_D, const int32_t *sub_adj,
              const int32_t *sub_gid, const int64_t *sub_mapping,
              const int32_t *full_adj, const float *storage,
              const float *query, int64_t batch, int64_t n_nodes, int d_model,
              int d_principle, int n_init, int n_buffers, int k, int ef_search,
              int sub_neighbors, int full_neighbors, void *workspace,
              size_t workspace_bytes, uint64_t *counters, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* PILOTANN_H */
