// Builds the 8-bit sketch of a vector table (layout and use: sketch_device.h).  No counterpart in the
// reference, which evaluates every candidate distance in full (kernels.py:204-257).
#include "sketch_device.h"

namespace {

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
    for (int h = kWave / 2; h >= 1; h >>= 1) x = fmaxf(x, __shfl_xor(x, h));
    return x;
}
__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
    for (int h = kWave / 2; h >= 1; h >>= 1) x += __shfl_xor(x, h);
    return x;
}

// One wavefront per row; a lane packs four elements into one 32-bit store.
__global__ __launch_bounds__(256) void sketch_build_kernel(const float *__restrict__ vectors, int64_t n, int dim,
                                                           int64_t row0, uint8_t *__restrict__ table) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = row0 + (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (row >= n) return;
    const float *v = vectors + row * dim;
    const int chunks = (int)sketch_data_chunks(dim);
    uint8_t *out = table + row * sketch_data_bytes(dim);

    float mx = 0.f;
    bool finite = true;
    for (int j = lane; j < dim; j += kWave) {
        const float x = v[j];
        finite = finite && (x - x == 0.0f);  // false for NaN and for either infinity
        mx = fmaxf(mx, __builtin_fabsf(x));
    }
    mx = wave_max(mx);
    finite = __ballot(!finite) == 0;
    const float scale = mx / 127.0f;
    const float inv = mx > 0.f ? 127.0f / mx : 0.f;

    float r2 = 0.f, n2 = 0.f;
    for (int g = lane; g < chunks * 4; g += kWave) {
        uint32_t word = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int j = 4 * g + k;
            float qv = 0.f;
            if (j < dim) {
                const float x = v[j];
                qv = fminf(fmaxf(rintf(x * inv), -127.0f), 127.0f);
                const float e = x - scale * qv;
                r2 = __builtin_fmaf(e, e, r2);
                n2 = __builtin_fmaf(x, x, n2);
            }
            word |= (uint32_t)((int)qv & 0xff) << (8 * k);
        }
        reinterpret_cast<uint32_t *>(out)[g] = word;
    }
    r2 = wave_sum(r2);
    n2 = wave_sum(n2);
    if (lane == 0) {
        // 1.001: the float32 sums above are off by at most dim * 2^-24 of their value, the products
        // scale * q by 2^-24 of |v_j|; the floor covers squares that underflow (elements below 1e-19);
        // a row that holds a NaN or an infinity promises nothing
        const float floor_ = 1.1e-19f * __builtin_sqrtf((float)dim);
        const float resid = finite ? __builtin_sqrtf(r2) * 1.001f + floor_ : __builtin_inff();
        const float norm = finite ? __builtin_sqrtf(n2) * 1.001f + floor_ : __builtin_inff();
        uint2 tail;
        tail.x = __builtin_bit_cast(uint32_t, finite ? scale : 0.f);
        tail.y = half_bits_not_below(resid) | (half_bits_not_below(norm) << 16);
        *reinterpret_cast<uint2 *>(table + sketch_tails_offset(n, dim) + row * kSketchTailBytes) = tail;
    }
}

// Rounds the query rows of a call to 15 bits per element for the sketch (sketch_device.h): one wavefront per
// row, a lane rounds four elements at a time.
__global__ __launch_bounds__(256) void sketch_query_kernel(const float *__restrict__ queries, int64_t n, int dim,
                                                           int64_t row0, uint8_t *__restrict__ out_rows) {
    const int lane = threadIdx.x & (kWave - 1);
    const int64_t row = row0 + (int64_t)blockIdx.x * (blockDim.x / kWave) + threadIdx.x / kWave;
    if (row >= n) return;
    const float *q = queries + row * dim;
    const int chunks = (int)sketch_data_chunks(dim);
    uint8_t *out = out_rows + row * sketch_query_bytes(dim);
    float mx = 0.f, n2 = 0.f;
    for (int j = lane; j < dim; j += kWave) {
        const float x = q[j];
        mx = fmaxf(mx, __builtin_fabsf(x));   // a NaN is not seen here but makes n2 a NaN
        n2 = __builtin_fmaf(x, x, n2);
    }
    mx = wave_max(mx);
    n2 = wave_sum(n2);
    // a row of zeros, of denormals, or one with a NaN: rounded to zero, and the bound is the row's whole length
    const bool tiny = !(mx > 1e-30f) || !(n2 == n2);
    const float inv = tiny ? 0.f : 16256.0f / mx;
    for (int g = lane; g < chunks * 4; g += kWave) {   // word g of the row: elements 4g .. 4g + 3
        uint32_t hi = 0, lo = 0;
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            const int j = 4 * g + k;
            int v = 0;
            if (j < dim) v = (int)fminf(fmaxf(rintf(q[j] * inv), -16256.0f), 16256.0f);
            const int l = ((v + 64) & 127) - 64;   // [-64, 63]
            const int h = (v - l) >> 7;            // [-127, 127], v = 128 h + l
            hi |= (uint32_t)(h & 0xff) << (8 * k);
            lo |= (uint32_t)(l & 0xff) << (8 * k);
        }
        const int c = g >> 2, w = g & 3;
        reinterpret_cast<uint32_t *>(out)[c * 8 + w] = hi;
        reinterpret_cast<uint32_t *>(out)[c * 8 + 4 + w] = lo;
    }
    if (lane == 0) {
        float4 tail;
        tail.x = mx / 16256.0f;
        tail.y = __builtin_sqrtf(n2) * 1.001f;
        // an element moves by at most half a step (0.51: q * inv and the step itself are rounded floats); a NaN or
        // an infinity in the query makes the bound a NaN or an infinity, which the callers read as "evaluate"
        tail.z = tiny ? tail.y : 0.51f * tail.x * __builtin_sqrtf((float)(16 * chunks));
        tail.w = (float)(dim + 16) * 5.9604645e-8f * tail.y;  // terms |q_j v_j| sum to at most ||q||_2 ||v||_2
        *reinterpret_cast<float4 *>(out + (int64_t)chunks * 32) = tail;
    }
}

// Bounds of gathered distances: one workgroup per query row, a wavefront per 64 ids; the very code
// (sketch_query_load, wave_sketch) the beam-search step runs.
template <int SCPL, int SLPR>
__global__ __launch_bounds__(256) void sketch_bounds_kernel(const uint8_t *__restrict__ rounded, int64_t rounded_bytes,
                                                            int chunks, const uint8_t *__restrict__ table,
                                                            const uint8_t *__restrict__ tails, int64_t n_vectors,
                                                            const int32_t *__restrict__ ids, int m, int64_t row0,
                                                            float *__restrict__ lo, float *__restrict__ hi) {
    const int64_t row = row0 + blockIdx.x;
    const int lane = threadIdx.x & (kWave - 1);
    const int wave = threadIdx.x / kWave;
    __shared__ float out_lo[256 / kWave][kWave], out_hi[256 / kWave][kWave];
    __shared__ uint8_t order[256 / kWave][kWave];
    SketchQuery<SCPL> sq;
    sketch_query_load<SCPL, SLPR>(sq, rounded + row * rounded_bytes, chunks);
    for (int c0 = wave * kWave; c0 < m; c0 += 256) {
        const int slot = c0 + lane;
        const int32_t id = slot < m ? ids[row * m + slot] : VL_MAXINT;
        const bool ok = slot < m && id != VL_MAXINT && id >= 0 && (int64_t)id < n_vectors;
        out_lo[wave][lane] = VL_MAXFLOAT;
        out_hi[wave][lane] = VL_MAXFLOAT;
        wave_sketch<SCPL, SLPR, 2>(sq, table, tails, chunks, id, ok, out_lo[wave], out_hi[wave], order[wave]);
        // (the wavefront's own LDS writes and reads are in program order)
        if (slot < m) {
            lo[row * m + slot] = out_lo[wave][lane];
            hi[row * m + slot] = out_hi[wave][lane];
        }
    }
}

template <int SCPL, int SLPR>
int launch_sketch_bounds(const uint8_t *rounded, int64_t dim, const uint8_t *table, int64_t n_vectors, const int32_t *ids,
                         int64_t n_rows, int64_t m, float *lo, float *hi, hipStream_t st) {
    for (int64_t row0 = 0; row0 < n_rows; row0 += kMaxBlocks) {
        int64_t rows = n_rows - row0 < kMaxBlocks ? n_rows - row0 : kMaxBlocks;
        hipLaunchKernelGGL((sketch_bounds_kernel<SCPL, SLPR>), dim3((unsigned)rows), dim3(256), 0, st, rounded,
                           sketch_query_bytes(dim), (int)sketch_data_chunks(dim), table, table + sketch_tails_offset(n_vectors, dim), n_vectors,
                           ids, (int)m, row0, lo, hi);
        VL_LAUNCH_CHECK("sketch_bounds_kernel");
    }
    return VL_OK;
}

}  // namespace

// Rounded query rows for a beam-search call that uses the sketch; out_rows: n_rows x sketch_query_bytes(dim),
// 16-byte aligned (part of the call's workspace).
int vl_launch_sketch_queries(const float *queries, int64_t n_rows, int64_t dim, uint8_t *out_rows, hipStream_t st) {
    const int rows_per_block = 256 / kWave;
    for (int64_t row0 = 0; row0 < n_rows; row0 += kMaxBlocks * rows_per_block) {
        int64_t rows = n_rows - row0 < kMaxBlocks * rows_per_block ? n_rows - row0 : kMaxBlocks * rows_per_block;
        hipLaunchKernelGGL(sketch_query_kernel, dim3((unsigned)((rows + rows_per_block - 1) / rows_per_block)), dim3(256),
                           0, st, queries, n_rows, (int)dim, row0, out_rows);
        VL_LAUNCH_CHECK("sketch_query_kernel");
    }
    return VL_OK;
}

VL_EXPORT int64_t vl_sketch_row_bytes(int64_t dim) {
    if (dim <= 0) {
        vl_set_error("dim must be positive");
        return VL_ERR_ARG;
    }
    return sketch_row_bytes(dim);
}

VL_EXPORT int vl_sketch_build(const float *vectors, int64_t n_vectors, int64_t dim, uint8_t *table, void *stream) {
    VL_REQUIRE(vectors && table, "null pointer");
    VL_REQUIRE(n_vectors >= 0 && dim > 0 && dim < (1 << 24), "bad sizes");
    VL_REQUIRE(((uintptr_t)table & 15) == 0, "the sketch table must be 16-byte aligned");
    const int rows_per_block = 256 / kWave;
    for (int64_t row0 = 0; row0 < n_vectors; row0 += kMaxBlocks * rows_per_block) {
        int64_t rows = n_vectors - row0 < kMaxBlocks * rows_per_block ? n_vectors - row0 : kMaxBlocks * rows_per_block;
        hipLaunchKernelGGL(sketch_build_kernel, dim3((unsigned)((rows + rows_per_block - 1) / rows_per_block)), dim3(256),
                           0, (hipStream_t)stream, vectors, n_vectors, (int)dim, row0, table);
        VL_LAUNCH_CHECK("sketch_build_kernel");
    }
    return VL_OK;
}

VL_EXPORT int64_t vl_sketch_bounds_workspace_bytes(int64_t n_rows, int64_t dim) {
    if (n_rows < 0 || dim <= 0) {
        vl_set_error("bad sizes");
        return VL_ERR_ARG;
    }
    return n_rows * sketch_query_bytes(dim) + 256;
}

VL_EXPORT int vl_sketch_bounds(const float *queries, int64_t n_rows, int64_t dim, const uint8_t *table,
                               int64_t n_vectors, const int32_t *ids, int64_t m, float *lo, float *hi,
                               void *workspace, int64_t workspace_bytes, void *stream) {
    VL_REQUIRE(n_rows >= 0 && m >= 0 && n_vectors >= 0 && dim > 0, "bad sizes");
    if (n_rows == 0 || m == 0) return VL_OK;
    VL_REQUIRE(queries && table && ids && lo && hi && workspace, "null pointer");
    VL_REQUIRE(dim % 4 == 0 && dim <= 2048 && ((uintptr_t)queries & 15) == 0 && ((uintptr_t)table & 15) == 0,
               "the sketch serves 16-byte aligned rows of up to 2048 columns, a multiple of 4");
    VL_REQUIRE(((uintptr_t)workspace & 15) == 0 && workspace_bytes >= n_rows * sketch_query_bytes(dim),
               "workspace too small or not 16-byte aligned");
    hipStream_t st = (hipStream_t)stream;
    uint8_t *rounded = (uint8_t *)workspace;
    int rc = vl_launch_sketch_queries(queries, n_rows, dim, rounded, st);
    if (rc < 0) return rc;
    const int chunks = (int)sketch_data_chunks(dim);
    if (chunks <= 8) return launch_sketch_bounds<1, 8>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    if (chunks <= 16) return launch_sketch_bounds<2, 8>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    if (chunks <= 24) return launch_sketch_bounds<3, 8>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    if (chunks <= 32) return launch_sketch_bounds<2, 16>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    if (chunks <= 48) return launch_sketch_bounds<3, 16>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    if (chunks <= 64) return launch_sketch_bounds<4, 16>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    if (chunks <= 96) return launch_sketch_bounds<3, 32>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
    return launch_sketch_bounds<4, 32>(rounded, dim, table, n_vectors, ids, n_rows, m, lo, hi, st);
}
