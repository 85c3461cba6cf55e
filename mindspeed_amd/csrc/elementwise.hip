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

// Exclusive scan of one int per thread over a block of up to 1024 threads (scratch: 16 ints).
__device__ __forceinline__ int block_exclusive_scan(int v, int *scratch) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    int incl = v;
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        const int up = __shfl_up(incl, d, 64);
        if (lane >= d) incl += up;
    }
    if (lane == 63) scratch[wave] = incl;
    __syncthreads();
    if (wave == 0) {
        const int nw = (blockDim.x + 63) >> 6;
        int w = lane < nw ? scratch[lane] : 0;
        int wi = w;
#pragma unroll
        for (int d = 1; d < 16; d <<= 1) {
            const int up = __shfl_up(wi, d, 64);
            if (lane >= d) wi += up;
        }
        if (lane < nw) scratch[lane] = wi - w;
    }
    __syncthreads();
    return incl - v + scratch[wave];
}

// out = cat(chunks[sorted_idxs[i]] for i) in one launch: row_map[r] = source row of output row r, the rows
// themselves, and optionally one probability per row.  Every workgroup scans the chunk sizes itself (in input
// order -> first source row of every chunk; in output order -> first output row of every position; num_chunks is
// experts x ranks, a few thousand at most), finds the position of each of its output rows by bisection, and
// copies the rows with `lanes` threads per row, eight 16-byte loads in flight per thread.  Output rows past the
// sum of the sizes get row_map = -1 and are left alone; malformed chunk indices count as empty chunks.
template <typename VecT>
__global__ __launch_bounds__(1024) void sort_chunks_kernel(
    const VecT *__restrict__ in, VecT *__restrict__ out, const int64_t *__restrict__ split_sizes,
    const int64_t *__restrict__ sorted_idxs, int num_chunks, int rows, int vecs_per_row, int lanes,
    const void *__restrict__ probs, void *__restrict__ out_probs, int probs_bytes, int32_t *__restrict__ row_map) {
    extern __shared__ int lds[];   // src_start[num_chunks], dst_start[num_chunks + 1], src_of[num_chunks], scratch[32]
    int *src_start = lds;
    int *dst_start = lds + num_chunks;
    int *src_of = dst_start + num_chunks + 1;
    int *scratch = src_of + num_chunks;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    int carry_s = 0, carry_d = 0;
    for (int c0 = 0; c0 < num_chunks; c0 += nthreads) {
        const int i = c0 + tid;
        int size = 0, moved = 0, src = -1;
        if (i < num_chunks) {
            const int64_t sz = split_sizes[i];
            size = static_cast<int>(sz < 0 ? 0 : (sz > rows ? rows : sz));
            const int64_t sidx = sorted_idxs[i];
            if (sidx >= 0 && sidx < num_chunks) {
                src = static_cast<int>(sidx);
                const int64_t ms = split_sizes[src];
                moved = static_cast<int>(ms < 0 ? 0 : (ms > rows ? rows : ms));
            }
        }
        const int s_ex = carry_s + block_exclusive_scan(size, scratch);
        const int d_ex = carry_d + block_exclusive_scan(moved, scratch);
        if (i < num_chunks) {
            src_start[i] = s_ex;
            dst_start[i] = d_ex;
            src_of[i] = src;
        }
        if (tid == nthreads - 1) {
            scratch[16] = s_ex + size;
            scratch[17] = d_ex + moved;
        }
        __syncthreads();
        carry_s = scratch[16];
        carry_d = scratch[17];
        __syncthreads();
    }
    if (tid == 0) dst_start[num_chunks] = carry_d;
    __syncthreads();

    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int r = blockIdx.x * (nthreads / lanes) + local_row;
    if (r >= rows) return;
    int lo = 0, hi = num_chunks + 1;            // last position with dst_start <= r
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (dst_start[mid] <= r) lo = mid; else hi = mid;
    }
    int m = -1;
    if (lo < num_chunks && r < dst_start[num_chunks] && src_of[lo] >= 0) {
        m = src_start[src_of[lo]] + (r - dst_start[lo]);
        if (static_cast<unsigned>(m) >= static_cast<unsigned>(rows)) m = -1;   // sizes that run past the input
    }
    if (lane == 0) {
        row_map[r] = m;
        if (probs != nullptr && m >= 0) {
            if (probs_bytes == 4) static_cast<uint32_t *>(out_probs)[r] = static_cast<const uint32_t *>(probs)[m];
            else static_cast<uint16_t *>(out_probs)[r] = static_cast<const uint16_t *>(probs)[m];
        }
    }
    if (m < 0) return;
    const VecT *src_row = in + static_cast<int64_t>(m) * vecs_per_row;
    VecT *dst_row = out + static_cast<int64_t>(r) * vecs_per_row;
    for (int c0 = lane; c0 < vecs_per_row; c0 += 8 * lanes) {
        VecT v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (c0 + u * lanes < vecs_per_row) v[u] = MS_NT_LOAD(src_row + c0 + u * lanes);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (c0 + u * lanes < vecs_per_row) MS_NT_STORE(v[u], dst_row + c0 + u * lanes);
    }
}

// The chunk sort's row map by itself, in the direction the reference's make_chunk_sort_map returns it
// (mindspeed/lite/ops/triton/sort_chunks_by_idx.py:67-115): map[source row] = output row.  Every workgroup scans the
// chunk sizes in input order (first source row of every chunk) and in output order (first output row of every position),
// inverts sorted_idxs in LDS, and locates each of its source rows by bisection.  Rows past the sum of the sizes, and
// rows of chunks that sorted_idxs never names, get -1.
__global__ __launch_bounds__(256) void chunk_sort_map_kernel(const int64_t *__restrict__ split_sizes,
                                                             const int64_t *__restrict__ sorted_idxs, int num_chunks,
                                                             int rows, int32_t *__restrict__ map) {
    extern __shared__ int lds[];   // src_start[num_chunks + 1], dst_start[num_chunks], pos_of[num_chunks], scratch[32]
    int *src_start = lds;
    int *dst_start = lds + num_chunks + 1;
    int *pos_of = dst_start + num_chunks;
    int *scratch = pos_of + num_chunks;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    for (int i = tid; i < num_chunks; i += nthreads) pos_of[i] = -1;
    __syncthreads();
    int carry_s = 0, carry_d = 0;
    for (int c0 = 0; c0 < num_chunks; c0 += nthreads) {
        const int i = c0 + tid;
        int size = 0, moved = 0;
        if (i < num_chunks) {
            const int64_t sz = split_sizes[i];
            size = static_cast<int>(sz < 0 ? 0 : (sz > rows ? rows : sz));
            const int64_t sidx = sorted_idxs[i];
            if (sidx >= 0 && sidx < num_chunks) {
                const int64_t ms = split_sizes[sidx];
                moved = static_cast<int>(ms < 0 ? 0 : (ms > rows ? rows : ms));
                pos_of[sidx] = i;
            }
        }
        const int s_ex = carry_s + block_exclusive_scan(size, scratch);
        const int d_ex = carry_d + block_exclusive_scan(moved, scratch);
        if (i < num_chunks) {
            src_start[i] = s_ex;
            dst_start[i] = d_ex;
        }
        if (tid == nthreads - 1) {
            scratch[16] = s_ex + size;
            scratch[17] = d_ex + moved;
        }
        __syncthreads();
        carry_s = scratch[16];
        carry_d = scratch[17];
        __syncthreads();
    }
    if (tid == 0) src_start[num_chunks] = carry_s;
    __syncthreads();
    const int r = blockIdx.x * nthreads + tid;
    if (r >= rows) return;
    int lo = 0, hi = num_chunks + 1;            // last chunk with src_start <= r
    while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (src_start[mid] <= r) lo = mid; else hi = mid;
    }
    int m = -1;
    if (lo < num_chunks && r < src_start[num_chunks] && pos_of[lo] >= 0) {
        m = dst_start[pos_of[lo]] + (r - src_start[lo]);
        if (static_cast<unsigned>(m) >= static_cast<unsigned>(rows)) m = -1;
    }
    map[r] = m;
}

// out[r] = in[row_map[r]] (inverse: out[row_map[r]] = in[r]); `lanes` threads per row, eight 16-byte loads in
// flight per thread.  Map entries outside [0, rows) move nothing.
template <typename VecT>
__global__ __launch_bounds__(256) void gather_rows_kernel(const VecT *__restrict__ in, VecT *__restrict__ out,
                                                          const int32_t *__restrict__ row_map, int rows,
                                                          int vecs_per_row, int lanes, int inverse) {
    const int local_row = threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    const int r = blockIdx.x * (256 / lanes) + local_row;
    if (r >= rows) return;
    const int m = row_map[r];
    if (static_cast<unsigned>(m) >= static_cast<unsigned>(rows)) return;
    const VecT *src_row = in + static_cast<int64_t>(inverse ? r : m) * vecs_per_row;
    VecT *dst_row = out + static_cast<int64_t>(inverse ? m : r) * vecs_per_row;
    for (int c0 = lane; c0 < vecs_per_row; c0 += 8 * lanes) {
        VecT v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (c0 + u * lanes < vecs_per_row) v[u] = MS_NT_LOAD(src_row + c0 + u * lanes);
#pragma unroll
        for (int u = 0; u < 8; ++u)
            if (c0 + u * lanes < vecs_per_row) MS_NT_STORE(v[u], dst_row + c0 + u * lanes);
    }
}

inline int row_lanes(int64_t vecs) {
    int lanes = 1;
    while (lanes < 64 && lanes < vecs) lanes <<= 1;   // one wavefront per row at most
    return lanes;
}

template <typename VecT>
int launch_gather_rows(hipStream_t stream, const void *in, void *out, const int32_t *map, int64_t rows,
                       int64_t row_bytes, int inverse) {
    const int64_t vecs = row_bytes / sizeof(VecT);
    const int lanes = row_lanes(vecs);
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

template <typename VecT>
int launch_sort_chunks(hipStream_t stream, const void *in, void *out, const int64_t *split_sizes,
                       const int64_t *sorted_idxs, int64_t num_chunks, int64_t rows, int64_t row_bytes, const void *probs,
                       void *out_probs, int probs_bytes, int32_t *row_map) {
    const int64_t vecs = row_bytes / sizeof(VecT);
    const int lanes = row_lanes(vecs);
    // fat workgroups repeat the scan of the chunk sizes less often; keep one per compute unit
    int threads = 1024;
    while (threads > 256 && ceil_div(rows, threads / lanes) < 256) threads >>= 1;
    const size_t lds = (3 * static_cast<size_t>(num_chunks) + 1 + 32) * sizeof(int);
    hipLaunchKernelGGL(sort_chunks_kernel<VecT>, dim3(static_cast<unsigned>(ceil_div(rows, threads / lanes))), dim3(threads),
                       lds, stream, static_cast<const VecT *>(in), static_cast<VecT *>(out), split_sizes, sorted_idxs,
                       static_cast<int>(num_chunks), static_cast<int>(rows), static_cast<int>(vecs), lanes, probs,
                       out_probs, probs_bytes, row_map);
    MS_CHECK_LAUNCH("sort_chunks_kernel");
    return MS_OK;
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

extern "C" int ms_chunk_sort_map(ms_stream_t stream_, const int64_t *split_sizes, const int64_t *sorted_idxs,
                                 int64_t num_chunks, int64_t rows, int32_t *row_id_map) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MS_REQUIRE(rows >= 0 && rows < (1ll << 31), MS_ERR_INVALID_ARGUMENT, "ms_chunk_sort_map: bad sizes");
    MS_REQUIRE(num_chunks >= 1 && num_chunks <= 4096, MS_ERR_UNSUPPORTED,
               "ms_chunk_sort_map: num_chunks %lld outside [1, 4096]", (long long)num_chunks);
    if (rows == 0) return MS_OK;
    MS_REQUIRE(split_sizes && sorted_idxs && row_id_map, MS_ERR_INVALID_ARGUMENT, "ms_chunk_sort_map: NULL tensor pointer");
    const size_t lds = (3 * static_cast<size_t>(num_chunks) + 1 + 32) * sizeof(int);
    hipLaunchKernelGGL(chunk_sort_map_kernel, dim3(static_cast<unsigned>(ceil_div(rows, 256))), dim3(256), lds, stream,
                       split_sizes, sorted_idxs, static_cast<int>(num_chunks), static_cast<int>(rows), row_id_map);
    MS_CHECK_LAUNCH("chunk_sort_map_kernel");
    return MS_OK;
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
    MS_REQUIRE(probs == nullptr || probs_dtype == MS_BF16 || probs_dtype == MS_FP16 || probs_dtype == MS_FP32,
               MS_ERR_UNSUPPORTED, "ms_sort_chunks: bad probs dtype");
    if (rows == 0) return MS_OK;
    MS_REQUIRE(input && split_sizes && sorted_idxs && out && row_map, MS_ERR_INVALID_ARGUMENT,
               "ms_sort_chunks: NULL tensor pointer");
    const int64_t row_bytes = hidden * dtype_size(dtype);
    const int probs_bytes = probs != nullptr ? static_cast<int>(dtype_size(probs_dtype)) : 0;
    if (row_bytes % 16 == 0 && aligned16(input) && aligned16(out))
        return launch_sort_chunks<v16>(stream, input, out, split_sizes, sorted_idxs, num_chunks, rows, row_bytes, probs,
                                       out_probs, probs_bytes, row_map);
    if (dtype == MS_FP32)
        return launch_sort_chunks<uint32_t>(stream, input, out, split_sizes, sorted_idxs, num_chunks, rows, row_bytes, probs,
                                            out_probs, probs_bytes, row_map);
    return launch_sort_chunks<uint16_t>(stream, input, out, split_sizes, sorted_idxs, num_chunks, rows, row_bytes, probs,
                                        out_probs, probs_bytes, row_map);
}
