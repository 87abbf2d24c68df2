// Chunk pipeline: device traversal of chunk i+1 and i+2 overlaps the host
// refine of chunk i.  Replaces `pipeline` (extension/pipeline_cpu.cpp:32-145).
//
// Two HIP streams (default priority) each own a device result buffer, a
// pinned host buffer and a traversal workspace.  All of them live for the
// life of the process and only grow: the reference allocates its four
// buffers, pinned ones included, on every call (pipeline_cpu.cpp:78-96).
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <mutex>

#include "pilotann.h"

extern "C" int pa_traverse_refine(
    int64_t *out_I, float *out_D, int64_t *buf_I, float *buf_D, int64_t *init_I,
    float *init_D, const int64_t *sub_indptr, const int64_t *sub_indices,
    const int64_t *full_indptr, const int64_t *full_indices,
    const float *storage, const float *query, int64_t batch, int64_t n_storage,
    int d_model, int d_principle, int n_init, int n_buffers, int k,
    int ef_search);

namespace {

constexpr int kSlots = 2;  // N_PREFETCH, pipeline_cpu.cpp:6

struct Slot {
    hipStream_t stream = nullptr;
    int64_t *dev_I = nullptr, *host_I = nullptr;
    float *dev_D = nullptr, *host_D = nullptr;
    void *workspace = nullptr;
    size_t cells = 0, workspace_bytes = 0;
};

struct DeviceState {
    Slot slot[kSlots];
};

constexpr int kMaxDevices = 16;
DeviceState g_state[kMaxDevices];
std::mutex g_mutex;

#define PA_TRY(expr)                           \
    do {                                       \
        hipError_t e_ = (expr);                \
        if (e_ != hipSuccess) return (int)e_;  \
    } while (0)

int ensure_slot(Slot *s, size_t cells, size_t workspace_bytes) {
    if (!s->stream)
        PA_TRY(hipStreamCreateWithFlags(&s->stream, hipStreamNonBlocking));
    if (s->cells < cells) {
        PA_TRY(hipStreamSynchronize(s->stream));
        if (s->dev_I) (void)hipFree(s->dev_I);
        if (s->dev_D) (void)hipFree(s->dev_D);
        if (s->host_I) (void)hipHostFree(s->host_I);
        if (s->host_D) (void)hipHostFree(s->host_D);
        s->dev_I = nullptr, s->dev_D = nullptr, s->host_I = nullptr, s->host_D = nullptr;
        s->cells = 0;
        PA_TRY(hipMalloc(reinterpret_cast<void **>(&s->dev_I), cells * sizeof(int64_t)));
        PA_TRY(hipMalloc(reinterpret_cast<void **>(&s->dev_D), cells * sizeof(float)));
        PA_TRY(hipHostMalloc(reinterpret_cast<void **>(&s->host_I), cells * sizeof(int64_t), hipHostMallocDefault));
        PA_TRY(hipHostMalloc(reinterpret_cast<void **>(&s->host_D), cells * sizeof(float), hipHostMallocDefault));
        s->cells = cells;
    }
    if (s->workspace_bytes < workspace_bytes) {
        PA_TRY(hipStreamSynchronize(s->stream));
        if (s->workspace) (void)hipFree(s->workspace);
        s->workspace = nullptr, s->workspace_bytes = 0;
        PA_TRY(hipMalloc(&s->workspace, workspace_bytes));
        s->workspace_bytes = workspace_bytes;
    }
    return PA_OK;
}

}  // namespace

extern "C" int pa_pipeline(
    int64_t *topk_I, float *topk_D, const int64_t *full_indptr,
    const int64_t *full_indices, const int64_t *sub_indptr,
    const int64_t *sub_indices, const float *storage, const float *query,
    const int32_t *adj, const int32_t *gid, const int64_t *mapping,
    const float *storage_dev, const float *query_dev, const int64_t *init_I,
    const float *init_D, int64_t batch, int64_t n_nodes, int64_t n_storage,
    int d_model, int d_principle, int n_init, int n_neighbors, int ef_search,
    int k, int chunk_size, void *caller_stream) {
    if (batch < 0 || chunk_size < 1 || k < 1) return PA_E_SHAPE;
    if (batch % chunk_size) return PA_E_CHUNK;  // pipeline_cpu.cpp:58
    if (d_model <= 0 || d_model % 8 || d_principle <= 0 || d_principle % 8 ||
        d_principle > d_model)
        return PA_E_DIM;
    if (ef_search < 1 || (int64_t)PA_BEAM_WIDTH * ef_search > PA_MAX_EF_TOTAL)
        return PA_E_EF;
    if (batch == 0) return PA_OK;
    if (!topk_I || !topk_D || !full_indptr || !full_indices || !sub_indptr ||
        !sub_indices || !storage || !query)
        return PA_E_NULL;

    int dev = 0;
    PA_TRY(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return PA_E_SHAPE;
    std::lock_guard<std::mutex> guard(g_mutex);
    DeviceState &st = g_state[dev];

    const size_t cells = (size_t)chunk_size * PA_BEAM_WIDTH * ef_search;
    size_t workspace_bytes = 0;
    int rc = pa_traverse_plan(n_storage, chunk_size, d_principle,
                              PA_BEAM_WIDTH * ef_search, nullptr, &workspace_bytes);
    if (rc != PA_OK) return rc;
    for (int s = 0; s < kSlots; ++s) {
        rc = ensure_slot(&st.slot[s], cells, workspace_bytes);
        if (rc != PA_OK) return rc;
    }
    // entries and queries were produced on the caller's stream
    // (pipeline_cpu.cpp:74-75)
    PA_TRY(hipStreamSynchronize((hipStream_t)caller_stream));

    const int n_buffers = PA_BEAM_WIDTH * ef_search;
    const int64_t n_chunks = batch / chunk_size;
    int failure = PA_OK;
    for (int64_t i = 0; i < n_chunks + kSlots; ++i) {
        Slot &s = st.slot[i % kSlots];
        if (i >= kSlots) {
            hipError_t e = hipStreamSynchronize(s.stream);
            if (e != hipSuccess && failure == PA_OK) failure = (int)e;
            if (failure == PA_OK) {
                const int64_t lo = (i - kSlots) * chunk_size;
                // the device stage's rows are both entries and scratch of
                // stage 2 (pipeline_cpu.cpp:110-117)
                rc = pa_traverse_refine(
                    topk_I + lo * k, topk_D + lo * k, s.host_I, s.host_D,
                    s.host_I, s.host_D, sub_indptr, sub_indices, full_indptr,
                    full_indices, storage, query + lo * (int64_t)d_model,
                    chunk_size, n_nodes, d_model, d_principle, n_buffers,
                    n_buffers, k, ef_search);
                if (rc != PA_OK) failure = rc;
            }
        }
        if (i < n_chunks && failure == PA_OK) {
            const int64_t lo = i * chunk_size;
            rc = pa_traverse(s.dev_I, s.dev_D, adj, gid, mapping, storage_dev,
                             query_dev + lo * (int64_t)d_principle,
                             init_I + lo * n_init, init_D + lo * n_init,
                             chunk_size, n_nodes, n_storage, d_principle, n_init,
                             PA_BEAM_WIDTH, ef_search, n_neighbors, s.workspace,
                             s.workspace_bytes, nullptr, s.stream);
            hipError_t e = hipSuccess;
            if (rc == PA_OK)
                e = hipMemcpyAsync(s.host_I, s.dev_I, cells * sizeof(int64_t),
                                   hipMemcpyDeviceToHost, s.stream);
            if (rc == PA_OK && e == hipSuccess)
                e = hipMemcpyAsync(s.host_D, s.dev_D, cells * sizeof(float),
                                   hipMemcpyDeviceToHost, s.stream);
            if (rc != PA_OK) failure = rc;
            else if (e != hipSuccess) failure = (int)e;
        }
    }
    if (failure != PA_OK)
        for (int s = 0; s < kSlots; ++s) (void)hipStreamSynchronize(st.slot[s].stream);
    return failure;
}
