// Query rotation for gfx950: out = query . VT^T, first n_out columns.
//
// The reference rotates a batch of queries onto the index's SVD basis with a
// host matmul and then slices off the first d_principle coordinates for the
// device stage (pilot_ann/layers/staged.py:198-201).  That is a plain dense
// contraction, queries x basis vectors, so it runs on the matrix cores in
// float32 (v_mfma_f32_32x32x2_f32).  Both operands are row major with the
// contraction along the row (out[b][j] = sum_k query[b][k] * VT[j][k]).
//
// A workgroup of four wavefronts owns a tile of the output (up to 128 queries
// x 128 basis vectors) and walks the row length in chunks of 32 elements:
// all 256 lanes copy the chunk of both operands into LDS with 16-byte loads
// (every row piece is fetched from memory once per workgroup), then each
// wavefront reads its operands back with 16-byte LDS loads and feeds up to
// 2 x 2 tiles of 32 x 32, so that one operand register serves two
// instructions.  The next chunk's global loads are issued before the matrix
// instructions of the present one and wait in registers.
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "device_common.h"
#include "pilotann.h"

using namespace pa;

namespace {

typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kTile = 32;        // rows and columns of one matrix instruction
constexpr int kChunk = 32;       // contraction elements staged in LDS at a time
// row pitch in LDS: 36 floats = 144 bytes keeps 16-byte alignment and moves
// consecutive rows by four banks, so the 16-byte reads of eight lanes (eight
// consecutive rows, same column) cover all banks once
constexpr int kPitch = kChunk + 4;

// MFMA operands: lane l supplies A[i = l % 32][k] and B[k][j = l % 32] with
// k = l / 32 of the instruction's two.  The contraction index is a free
// relabelling: within every group of eight elements lanes 0..31 take elements
// 0..3 and lanes 32..63 elements 4..7, so one 16-byte read per operand feeds
// four instructions.  The 16 results of a lane are
// D[i = 8 * (r / 4) + 4 * (l / 32) + r % 4][j = l % 32].
//
// WM, WN: 32 x 32 tiles per wavefront along the queries / the basis vectors;
// the workgroup's 2 x 2 wavefronts cover (64 WM) x (64 WN) outputs.
template <int WM, int WN>
__global__ __launch_bounds__(256) void rotate_kernel(
    const float *__restrict__ query, const float *__restrict__ basis,
    float *__restrict__ out, int batch, int d, int n_out) {
    constexpr int BM = 2 * kTile * WM, BN = 2 * kTile * WN;
    __shared__ __align__(16) float a_s[BM * kPitch];
    __shared__ __align__(16) float b_s[BN * kPitch];
    const int t = threadIdx.x;
    const int lane = t & (kWave - 1), wave = t / kWave;
    const int col = lane & 31, half = lane >> 5;
    const int q0 = blockIdx.x * BM, j0 = blockIdx.y * BN;

    // staging: lane t copies float4 number t % 8 of rows t / 8 + 32 i.  Rows
    // past the end are clamped (their outputs are never stored); elements
    // past the row length are zeros.
    const int srow = t >> 3, scol = 4 * (t & 7);
    const float *a_src[BM / 32], *b_src[BN / 32];
#pragma unroll
    for (int i = 0; i < BM / 32; ++i) {
        const int r = min(q0 + srow + 32 * i, batch - 1);
        a_src[i] = query + (size_t)r * d + scol;
    }
#pragma unroll
    for (int i = 0; i < BN / 32; ++i) {
        const int r = min(j0 + srow + 32 * i, n_out - 1);
        b_src[i] = basis + (size_t)r * d + scol;
    }
    floatx4 a_reg[BM / 32], b_reg[BN / 32];
    const floatx4 zero = {0.f, 0.f, 0.f, 0.f};
// the chunk that starts at element k0, from memory into registers
#define PA_FETCH_CHUNK(k0)                                                            \
    {                                                                                 \
        const bool in = (k0) + scol < d;                                              \
        _Pragma("unroll") for (int i = 0; i < BM / 32; ++i) a_reg[i] =                \
            in ? *reinterpret_cast<const floatx4 *>(a_src[i] + (k0)) : zero;           \
        _Pragma("unroll") for (int i = 0; i < BN / 32; ++i) b_reg[i] =                \
            in ? *reinterpret_cast<const floatx4 *>(b_src[i] + (k0)) : zero;           \
    }

    floatx16 acc[WM][WN];
#pragma unroll
    for (int m = 0; m < WM; ++m)
#pragma unroll
        for (int n = 0; n < WN; ++n)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[m][n][r] = 0.f;

    const float *a_tile = a_s + ((wave & 1) * kTile * WM + col) * kPitch + 4 * half;
    const float *b_tile = b_s + ((wave >> 1) * kTile * WN + col) * kPitch + 4 * half;

    PA_FETCH_CHUNK(0)
    for (int k0 = 0; k0 < d; k0 += kChunk) {
#pragma unroll
        for (int i = 0; i < BM / 32; ++i)
            *reinterpret_cast<floatx4 *>(a_s + (srow + 32 * i) * kPitch + scol) = a_reg[i];
#pragma unroll
        for (int i = 0; i < BN / 32; ++i)
            *reinterpret_cast<floatx4 *>(b_s + (srow + 32 * i) * kPitch + scol) = b_reg[i];
        __syncthreads();
        if (k0 + kChunk < d) PA_FETCH_CHUNK(k0 + kChunk)
#pragma unroll
        for (int g = 0; g < kChunk / 8; ++g) {
            floatx4 a[WM], b[WN];
#pragma unroll
            for (int m = 0; m < WM; ++m)
                a[m] = *reinterpret_cast<const floatx4 *>(a_tile + m * kTile * kPitch + 8 * g);
#pragma unroll
            for (int n = 0; n < WN; ++n)
                b[n] = *reinterpret_cast<const floatx4 *>(b_tile + n * kTile * kPitch + 8 * g);
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[m].x, b[n].x, acc[m][n], 0, 0, 0);
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[m].y, b[n].y, acc[m][n], 0, 0, 0);
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[m].z, b[n].z, acc[m][n], 0, 0, 0);
#pragma unroll
            for (int m = 0; m < WM; ++m)
#pragma unroll
                for (int n = 0; n < WN; ++n)
                    acc[m][n] = __builtin_amdgcn_mfma_f32_32x32x2f32(a[m].w, b[n].w, acc[m][n], 0, 0, 0);
        }
        __syncthreads();
    }
#undef PA_FETCH_CHUNK

#pragma unroll
    for (int m = 0; m < WM; ++m) {
        const int qb = q0 + ((wave & 1) * WM + m) * kTile;
#pragma unroll
        for (int n = 0; n < WN; ++n) {
            const int j = j0 + ((wave >> 1) * WN + n) * kTile + col;
            if (j >= n_out) continue;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int i = qb + 8 * (r >> 2) + 4 * half + (r & 3);
                if (i < batch) out[(size_t)i * n_out + j] = acc[m][n][r];
            }
        }
    }
}

template <int WM, int WN>
void launch_rotate(const float *query, const float *basis, float *out, int batch, int d,
                   int n_out, hipStream_t stream) {
    constexpr int BM = 2 * kTile * WM, BN = 2 * kTile * WN;
    const dim3 grid((unsigned)((batch + BM - 1) / BM), (unsigned)((n_out + BN - 1) / BN));
    rotate_kernel<WM, WN><<<grid, 256, 0, stream>>>(query, basis, out, batch, d, n_out);
}

// A larger tile reads its operands from LDS less often, but only pays when
// the launch still has workgroups for every compute unit: measured on
// 10 000 x 768 rows, 768 outputs run 14 % faster with 128 x 128 tiles than
// with 64 x 64 (474 against 1884 workgroups), 128 outputs 44 % slower (79
// against 314).
constexpr int64_t kMinWorkgroups = 400;

int64_t tiles(int64_t batch, int n_out, int bm, int bn) {
    return ((batch + bm - 1) / bm) * ((n_out + bn - 1) / bn);
}

}  // namespace

extern "C" int pa_rotate(float *out, const float *query, const float *basis,
                         int64_t batch, int d, int n_out, void *stream_) {
    if (batch < 0 || n_out < 1 || n_out > d) return PA_E_SHAPE;
    if (batch >= (1ll << 31)) return PA_E_RANGE;
    if (d <= 0 || d % 8) return PA_E_DIM;
    if (batch == 0) return PA_OK;
    if (!out || !query || !basis) return PA_E_NULL;
    hipStream_t stream = (hipStream_t)stream_;
    if (tiles(batch, n_out, 128, 128) >= kMinWorkgroups)
        launch_rotate<2, 2>(query, basis, out, (int)batch, d, n_out, stream);
    else if (tiles(batch, n_out, 64, 128) >= kMinWorkgroups)
        launch_rotate<1, 2>(query, basis, out, (int)batch, d, n_out, stream);
    else
        launch_rotate<1, 1>(query, basis, out, (int)batch, d, n_out, stream);
    return (int)hipGetLastError();
}
