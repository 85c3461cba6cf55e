// Elementwise / row-copy kernels of the expert path for gfx950: SwiGLU with an
// optional per-row probability (forward and backward) and the chunk re-ordering
// used after the all-to-all.  All are HBM-bound: 16-byte vectors per lane, fp32
// math, one rounding.
#include "common.h"

namespace ms {
namespace {

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + __expf(-x)); }

template <typename DT, int VEC>
__global__ __launch_bounds__(256) void swiglu_kernel(const typename DT::storage *__restrict__ x,
                                                     const void *__restrict__ probs, int probs_dtype,
                                                     typename DT::storage *__restrict__ y, int64_t rows, int ffn) {
    using S = typename DT::storage;
    const int vecs = ffn / VEC;
    const int64_t total = rows * vecs;
    for (int64_t v = blockIdx.x * static_cast<int64_t>(blockDim.x) + threadIdx.x; v < total;
         v += static_cast<int64_t>(gridDim.x) * blockDim.x) {
        const int64_t r = v / vecs;
        const int c = static_cast<int>(v - r * vecs) * VEC;
        const S *xg = x + r * 2 * ffn + c;
        const S *xu = xg + ffn;
        S g[VEC], u[VEC], o[VEC];
        if constexpr (VEC * sizeof(S) == 16) {
            *reinterpret_cast<v16 *>(g) = MS_NT_LOAD(reinterpret_cast<const v16 *>(xg));
            *reinterpret_cast<v16 *>(u) = MS_NT_LOAD(reinterpret_cast<const v16 *>(xu));
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { g[e] = xg[e]; u[e] = xu[e]; }
        }
        const float p = probs != nullptr ? load_scalar_as_float(probs, r, probs_dtype) : 1.f;
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float gf = DT::to_float(g[e]);
            o[e] = DT::from_float(gf * sigmoidf_(gf) * DT::to_float(u[e]) * p);
        }
        S *dst = y + r * ffn + c;
        if constexpr (VEC * sizeof(S) == 16) {
            MS_NT_STORE(*reinterpret_cast<v16 *>(o), reinterpret_cast<v16 *>(dst));
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) dst[e] = o[e];
        }
    }
}

// One block per row (so grad_probs can be reduced in the same pass).
template <typename DT, int VEC>
__global__ __launch_bounds__(256) void swiglu_grad_kernel(const typename DT::storage *__restrict__ gy,
                                                          const typename DT::storage *__restrict__ x,
                                                          const void *__restrict__ probs, int probs_dtype,
                                                          typename DT::storage *__restrict__ gx,
                                                          void *__restrict__ gprobs, int ffn) {
    using S = typename DT::storage;
    __shared__ float partial[4];
    const int64_t r = blockIdx.x;
    const int vecs = ffn / VEC;
    const float p = probs != nullptr ? load_scalar_as_float(probs, r, probs_dtype) : 1.f;
    float dot = 0.f;
    for (int v = threadIdx.x; v < vecs; v += blockDim.x) {
        const int c = v * VEC;
        const S *xg = x + r * 2 * ffn + c;
        const S *xu = xg + ffn;
        const S *gp = gy + r * ffn + c;
        S g[VEC], u[VEC], d[VEC], og[VEC], ou[VEC];
        if constexpr (VEC * sizeof(S) == 16) {
            *reinterpret_cast<v16 *>(g) = MS_NT_LOAD(reinterpret_cast<const v16 *>(xg));
            *reinterpret_cast<v16 *>(u) = MS_NT_LOAD(reinterpret_cast<const v16 *>(xu));
            *reinterpret_cast<v16 *>(d) = MS_NT_LOAD(reinterpret_cast<const v16 *>(gp));
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { g[e] = xg[e]; u[e] = xu[e]; d[e] = gp[e]; }
        }
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
            const float gf = DT::to_float(g[e]), uf = DT::to_float(u[e]), df = DT::to_float(d[e]);
            const float sig = sigmoidf_(gf);
            const float act = gf * sig;
            dot = fmaf(df, act * uf, dot);
            const float dp = df * p;
            og[e] = DT::from_float(dp * uf * (sig * (1.f + gf * (1.f - sig))));
            ou[e] = DT::from_float(dp * act);
        }
        S *dg = gx + r * 2 * ffn + c;
        S *du = dg + ffn;
        if constexpr (VEC * sizeof(S) == 16) {
            MS_NT_STORE(*reinterpret_cast<v16 *>(og), reinterpret_cast<v16 *>(dg));
            MS_NT_STORE(*reinterpret_cast<v16 *>(ou), reinterpret_cast<v16 *>(du));
        } else {
#pragma unroll
            for (int e = 0; e < VEC; ++e) { dg[e] = og[e]; du[e] = ou[e]; }
        }
    }
    if (gprobs != nullptr) {
#pragma unroll
        for (int dlt = 32; dlt > 0; dlt >>= 1) dot += __shfl_down(dot, dlt, 64);
        if ((threadIdx.x & 63) == 0) partial[threadIdx.x >> 6] = dot;
        __syncthreads();
        if (threadIdx.x == 0) {
            float s = 0.f;
            for (int w = 0; w < (blockDim.x + 63) / 64; ++w) s += partial[w];
            store_float_as(gprobs, r, probs_dtype, s);
        }
    }
}

// row_map[r] = source row of output row r for out = cat(chunks[sorted_idxs[i]]).
// One block; num_chunks is small (experts x ranks).
__global__ __launch_bounds__(256) void chunk_row_map_kernel(const int64_t *__restrict__ split_sizes,
                                                            const int64_t *__restrict__ sorted_idxs,
                                                            int num_chunks, int rows, int32_t *row_map) {
    extern __shared__ int64_t sh[];  // src_start[num_chunks], dst_start[num_chunks]
    int64_t *src_start = sh;
    int64_t *dst_start = sh + num_chunks;
    if (threadIdx.x == 0) {
        int64_t acc = 0;
        for (int i = 0; i < num_chunks; ++i) { src_start[i] = acc; acc += split_sizes[i]; }
        acc = 0;
        for (int i = 0; i < num_chunks; ++i) {
            const int64_t src = sorted_idxs[i];
            dst_start[i] = acc;
            if (src >= 0 && src < num_chunks) acc += split_sizes[src];
        }
    }
    __syncthreads();
    for (int i = 0; i < num_chunks; ++i) {
        const int64_t src = sorted_idxs[i];
        if (src < 0 || src >= num_chunks) continue;  // malformed index: skip rather than read out of bounds
        const int64_t len = split_sizes[src];
        for (int64_t r = threadIdx.x; r < len; r += blockDim.x) {
            const int64_t o = dst_start[i] + r;
            if (o < rows) row_map[o] = static_cast<int32_t>(src_start[src] + r);
        }
    }
}

template <typename VecT>
__global__ __launch_bounds__(256) void gather_rows_kernel(const VecT *__restrict__ in, VecT *__restrict__ out,
                                                          const int32_t *__restrict__ row_map, int rows,
                                                          int vecs_per_row, int lanes, int inverse) {
    const int local_row = threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    const int r = blockIdx.x * (256 / lanes) + local_row;
    if (r >= rows) return;
    const int m = row_map[r];
    if (static_cast<unsigned>(m) >= static_cast<unsigned>(rows)) return;   // corrupt map entry: touch nothing
    const int64_t s = inverse ? r : m;
    const int64_t d = inverse ? m : r;
    for (int c = lane; c < vecs_per_row; c += lanes)
        MS_NT_STORE(MS_NT_LOAD(in + s * vecs_per_row + c), out + d * vecs_per_row + c);
}

template <typename VecT>
int launch_gather_rows(hipStream_t stream, const void *in, void *out, const int32_t *map, int64_t rows,
                       int64_t row_bytes, int inverse) {
    const int64_t vecs = row_bytes / sizeof(VecT);
    int lanes = 1;
    while (lanes < 256 && lanes < vecs) lanes <<= 1;
    const int64_t blocks = ceil_div(rows, 256 / lanes);
    hipLaunchKernelGGL(gather_rows_kernel<VecT>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                       static_cast<const VecT *>(in), static_cast<VecT *>(out), map, static_cast<int>(rows),
                       static_cast<int>(vecs), lanes, inverse);
    MS_CHECK_LAUNCH("gather_rows_kernel");
    return MS_OK;
}

int gather_rows_any(hipStream_t stream, const void *in, void *out, const int32_t *map, int64_t rows, int64_t hidden,
                    int dtype, int inverse) {
    const int64_t row_bytes = hidden * dtype_size(dtype);
    if (row_bytes % 16 == 0 && aligned16(in) && aligned16(out))
        return launch_gather_rows<v16>(stream, in, out, map, rows, row_bytes, inverse);
    if (dtype == MS_FP32) return launch_gather_rows<uint32_t>(stream, in, out, map, rows, row_bytes, inverse);
    return launch_gather_rows<uint16_t>(stream, in, out, map, rows, row_bytes, inverse);
}

template <typename DT>
int launch_swiglu(hipStream_t stream, const void *x, const void *probs, int probs_dtype, int64_t rows, int64_t ffn,
                  void *y) {
    using S = typename DT::storage;
    constexpr int VEC = 16 / sizeof(S);
    const bool vec_ok = ffn % VEC == 0 && aligned16(x) && aligned16(y);
    const int64_t total = rows * (vec_ok ? ffn / VEC : ffn);
    int64_t blocks = ceil_div(total, 256);
    if (blocks > 256 * 64) blocks = 256 * 64;
    if (vec_ok)
        hipLaunchKernelGGL((swiglu_kernel<DT, VEC>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const S *>(x), probs, probs_dtype, static_cast<S *>(y), rows,
                           static_cast<int>(ffn));
    else
        hipLaunchKernelGGL((swiglu_kernel<DT, 1>), dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const S *>(x), probs, probs_dtype, static_cast<S *>(y), rows,
                           static_cast<int>(ffn));
    MS_CHECK_LAUNCH("swiglu_kernel");
    return MS_OK;
}

template <typename DT>
int launch_swiglu_grad(hipStream_t stream, const void *gy, const void *x, const void *probs, int probs_dtype,
                       int64_t rows, int64_t ffn, void *gx, void *gprobs) {
    using S = typename DT::storage;
    constexpr int VEC = 16 / sizeof(S);
    const bool vec_ok = ffn % VEC == 0 && aligned16(x) && aligned16(gy) && aligned16(gx);
    if (vec_ok)
        hipLaunchKernelGGL((swiglu_grad_kernel<DT, VEC>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, stream,
                           static_cast<const S *>(gy), static_cast<const S *>(x), probs, probs_dtype,
                           static_cast<S *>(gx), gprobs, static_cast<int>(ffn));
    else
        hipLaunchKernelGGL((swiglu_grad_kernel<DT, 1>), dim3(static_cast<unsigned>(rows)), dim3(256), 0, stream,
                           static_cast<const S *>(gy), static_cast<const S *>(x), probs, probs_dtype,
                           static_cast<S *>(gx), gprobs, static_cast<int>(ffn));
    MS_CHECK_LAUNCH("swiglu_grad_kernel");
    return MS_OK;
}

int check_swiglu(const char *fn, int64_t rows, int64_t ffn, int dtype, const void *probs, int probs_dtype) {
    MS_REQUIRE(rows >= 0 && ffn >= 1 && ffn < (1ll << 30) && rows < (1ll << 31), MS_ERR_INVALID_ARGUMENT,
               "%s: bad sizes rows=%lld ffn=%lld", fn, (long long)rows, (long long)ffn);
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED, "%s: bad dtype %d", fn,
               dtype);
    MS_REQUIRE(probs == nullptr || probs_dtype == MS_BF16 || probs_dtype == MS_FP16 || probs_dtype == MS_FP32,
               MS_ERR_UNSUPPORTED, "%s: bad probs dtype %d", fn, probs_dtype);
    return MS_OK;
}

}  // namespace
}  // namespace ms

using namespace ms;

extern "C" int ms_swiglu(ms_stream_t stream_, const void *x, const void *probs, int probs_dtype, int64_t rows,
                         int64_t ffn, int dtype, void *y) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_swiglu("ms_swiglu", rows, ffn, dtype, probs, probs_dtype)) return rc;
    if (rows == 0) return MS_OK;
    MS_REQUIRE(x && y, MS_ERR_INVALID_ARGUMENT, "ms_swiglu: NULL tensor pointer");
    switch (dtype) {
        case MS_BF16: return launch_swiglu<BF16>(stream, x, probs, probs_dtype, rows, ffn, y);
        case MS_FP16: return launch_swiglu<FP16>(stream, x, probs, probs_dtype, rows, ffn, y);
        default: return launch_swiglu<FP32>(stream, x, probs, probs_dtype, rows, ffn, y);
    }
}

extern "C" int ms_swiglu_grad(ms_stream_t stream_, const void *grad_y, const void *x, const void *probs,
                              int probs_dtype, int64_t rows, int64_t ffn, int dtype, void *grad_x, void *grad_probs) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_swiglu("ms_swiglu_grad", rows, ffn, dtype, probs, probs_dtype)) return rc;
    MS_REQUIRE(grad_probs == nullptr || probs != nullptr, MS_ERR_INVALID_ARGUMENT,
               "ms_swiglu_grad: grad_probs needs probs");
    if (rows == 0) return MS_OK;
    MS_REQUIRE(grad_y && x && grad_x, MS_ERR_INVALID_ARGUMENT, "ms_swiglu_grad: NULL tensor pointer");
    switch (dtype) {
        case MS_BF16: return launch_swiglu_grad<BF16>(stream, grad_y, x, probs, probs_dtype, rows, ffn, grad_x, grad_probs);
        case MS_FP16: return launch_swiglu_grad<FP16>(stream, grad_y, x, probs, probs_dtype, rows, ffn, grad_x, grad_probs);
        default: return launch_swiglu_grad<FP32>(stream, grad_y, x, probs, probs_dtype, rows, ffn, grad_x, grad_probs);
    }
}

extern "C" int ms_gather_rows(ms_stream_t stream_, const void *input, const int32_t *row_map, int64_t rows,
                              int64_t hidden, int dtype, int inverse, void *out) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MS_REQUIRE(rows >= 0 && rows < (1ll << 31) && hidden >= 1 && hidden < (1ll << 31), MS_ERR_INVALID_ARGUMENT,
               "ms_gather_rows: bad sizes");
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED, "ms_gather_rows: bad dtype");
    if (rows == 0) return MS_OK;
    MS_REQUIRE(input && row_map && out, MS_ERR_INVALID_ARGUMENT, "ms_gather_rows: NULL tensor pointer");
    return gather_rows_any(stream, input, out, row_map, rows, hidden, dtype, inverse);
}

extern "C" int ms_sort_chunks(ms_stream_t stream_, const void *input, const int64_t *split_sizes,
                              const int64_t *sorted_idxs, int64_t num_chunks, int64_t rows, int64_t hidden, int dtype,
                              const void *probs, int probs_dtype, void *out, void *out_probs, int32_t *row_map) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MS_REQUIRE(rows >= 0 && rows < (1ll << 31) && hidden >= 1 && hidden < (1ll << 31), MS_ERR_INVALID_ARGUMENT,
               "ms_sort_chunks: bad sizes");
    MS_REQUIRE(num_chunks >= 1 && num_chunks <= 4096, MS_ERR_UNSUPPORTED, "ms_sort_chunks: num_chunks %lld outside [1, 4096]",
               (long long)num_chunks);
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED, "ms_sort_chunks: bad dtype");
    MS_REQUIRE((probs == nullptr) == (out_probs == nullptr), MS_ERR_INVALID_ARGUMENT,
               "ms_sort_chunks: probs and out_probs must be given together");
    if (rows == 0) return MS_OK;
    MS_REQUIRE(input && split_sizes && sorted_idxs && out && row_map, MS_ERR_INVALID_ARGUMENT,
               "ms_sort_chunks: NULL tensor pointer");
    hipLaunchKernelGGL(chunk_row_map_kernel, dim3(1), dim3(256), 2 * num_chunks * sizeof(int64_t), stream, split_sizes,
                       sorted_idxs, static_cast<int>(num_chunks), static_cast<int>(rows), row_map);
    MS_CHECK_LAUNCH("chunk_row_map_kernel");
    if (int rc = gather_rows_any(stream, input, out, row_map, rows, hidden, dtype, 0)) return rc;
    if (probs != nullptr) return gather_rows_any(stream, probs, out_probs, row_map, rows, 1, probs_dtype, 0);
    return MS_OK;
}
