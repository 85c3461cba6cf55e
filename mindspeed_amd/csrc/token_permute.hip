// MoE token permute / unpermute for gfx950 (MI355X).
//
// permute  = stable counting sort of the flattened expert ids (wavefront-ballot
//            match, per-wave histogram rows, LDS prefix scan, no atomics, so
//            the order is deterministic) followed by a coalesced 16-byte row
//            scatter that reads every token row once and writes its topk
//            copies.
// unpermute = per-token top-k gather with fp32 accumulation in registers and
//            one rounding; its backward scatters prob-scaled rows and reduces
//            the per-(token, slot) dot products for grad_probs.
//
// All kernels are HBM-bound; rows move as 16-byte vectors per lane.
#include "common.h"

namespace ms {
namespace {

constexpr int kSortBlockWaves = 16;          // single-block sort: 1024 threads
constexpr int kSmallSortMax = 16384;         // flat positions handled by one block (16 waves x 1024 keys)
constexpr int kHistWavesPerBlock = 4;        // multi-block sort: 256 threads
constexpr int kMaxSegments = 4096;

// ---- wavefront helpers ---------------------------------------------------------
template <typename IdxT>
__device__ __forceinline__ int load_key(const IdxT *idx, int64_t i, int nbins) {
    long long v = static_cast<long long>(idx[i]);
    v = v < 0 ? 0 : v;
    v = v >= nbins ? nbins - 1 : v;
    return static_cast<int>(v);
}

// Mask of the valid lanes of this wavefront that hold the same key as the caller.
__device__ __forceinline__ unsigned long long match_key(int key, bool valid, int nbits) {
    unsigned long long m = __ballot(valid);
    for (int b = 0; b < nbits; ++b) {
        const bool bit = (key >> b) & 1;
        const unsigned long long bal = __ballot(valid && bit);
        m &= bit ? bal : ~bal;
    }
    return m;
}

constexpr int kKeysPerLane = 16;               // one register-resident chunk: 64 lanes x 16 keys
constexpr int kChunk = 64 * kKeysPerLane;

// Load up to kChunk keys of idx[begin, end) into registers (-1 past the end).  All loads are issued
// before any is used, so a chunk costs one memory latency instead of one per 64 keys.
template <typename IdxT>
__device__ __forceinline__ void load_keys(const IdxT *idx, int begin, int end, int nbins, int (&keys)[kKeysPerLane]) {
    const int lane = threadIdx.x & 63;
    if (begin >= end) {
#pragma unroll
        for (int u = 0; u < kKeysPerLane; ++u) keys[u] = -1;
        return;
    }
    // Unconditional loads from clamped positions (no per-load branch, so nothing waits in between),
    // then mask what lies past the end.
    IdxT raw[kKeysPerLane];
#pragma unroll
    for (int u = 0; u < kKeysPerLane; ++u) raw[u] = idx[min(begin + u * 64 + lane, end - 1)];
#pragma unroll
    for (int u = 0; u < kKeysPerLane; ++u) {
        long long v = static_cast<long long>(raw[u]);
        v = v < 0 ? 0 : v;
        v = v >= nbins ? nbins - 1 : v;
        keys[u] = begin + u * 64 + lane < end ? static_cast<int>(v) : -1;
    }
}

// Histogram of a register-resident chunk into one table row owned by this wavefront.  One lane per
// distinct key (the lowest lane holding it) adds the key's multiplicity with a fire-and-forget LDS add.
__device__ __forceinline__ void hist_keys(int *row, const int (&keys)[kKeysPerLane], int count, int nbits) {
    const int lane = threadIdx.x & 63;
#pragma unroll
    for (int u = 0; u < kKeysPerLane; ++u) {
        if (u * 64 >= count) break;
        const bool valid = keys[u] >= 0;
        const int key = valid ? keys[u] : 0;
        const unsigned long long m = match_key(key, valid, nbits);
        if (valid && lane == __ffsll(static_cast<long long>(m)) - 1) atomicAdd(&row[key], __popcll(m));
    }
}

// Stable scatter of a register-resident chunk that starts at flat position `begin`: row[key] holds
// the next output row of `key` for this wavefront's segment.  The lowest lane of every key fetches
// and advances that counter with one returning LDS add and hands the old value to the key's lanes.
__device__ __forceinline__ void scatter_keys(int *row, const int (&keys)[kKeysPerLane], int begin, int count,
                                             int nbits, int num_out, int32_t *row_id_map, int32_t *sorted_indices) {
    const int lane = threadIdx.x & 63;
    const unsigned long long lt = (1ull << lane) - 1ull;
#pragma unroll
    for (int u = 0; u < kKeysPerLane; ++u) {
        if (u * 64 >= count) break;
        const bool valid = keys[u] >= 0;
        const int key = valid ? keys[u] : 0;
        const unsigned long long m = match_key(key, valid, nbits);
        const int leader = valid ? __ffsll(static_cast<long long>(m)) - 1 : lane;
        int first = 0;
        if (valid && lane == leader) first = atomicAdd(&row[key], __popcll(m));
        first = __shfl(first, leader, 64);
        if (valid) {
            const int rank = first + __popcll(m & lt);
            const int i = begin + u * 64 + lane;
            row_id_map[i] = rank;
            if (sorted_indices != nullptr && rank < num_out) sorted_indices[rank] = i;
        }
    }
}

// ---- few bins (<= NB): one ballot per bin, counters in scalar registers ---------------------------
// With at most 16 bins a ballot per bin is cheaper than matching lanes pairwise: the per-bin counts and
// running offsets are wave-uniform (scalar registers), and a lane's rank inside the chunk is the number
// of lower lanes in its bin's ballot.
__device__ __forceinline__ int lanes_below(unsigned long long mask) {
    return __builtin_amdgcn_mbcnt_hi(static_cast<unsigned>(mask >> 32),
                                     __builtin_amdgcn_mbcnt_lo(static_cast<unsigned>(mask), 0u));
}

template <int NB>
__device__ __forceinline__ void hist_keys_few(int *row, const int (&keys)[kKeysPerLane], int count, int nbins) {
    const int lane = threadIdx.x & 63;
    int cnt[NB];
#pragma unroll
    for (int e = 0; e < NB; ++e) cnt[e] = 0;
#pragma unroll
    for (int u = 0; u < kKeysPerLane; ++u) {
        if (u * 64 >= count) break;
#pragma unroll
        for (int e = 0; e < NB; ++e) cnt[e] += __popcll(__ballot(keys[u] == e));
    }
    int mine = 0;
#pragma unroll
    for (int e = 0; e < NB; ++e) mine = lane == e ? cnt[e] : mine;
    if (lane < nbins) row[lane] += mine;   // the row has nbins (<= NB) entries
}

template <int NB>
__device__ __forceinline__ void scatter_keys_few(int *row, const int (&keys)[kKeysPerLane], int begin, int count,
                                                 int nbins, int num_out, int32_t *row_id_map, int32_t *sorted_indices) {
    const int lane = threadIdx.x & 63;
    int base[NB];
    const int mine = lane < nbins ? row[lane] : 0;
#pragma unroll
    for (int e = 0; e < NB; ++e) base[e] = __builtin_amdgcn_readlane(mine, e);
#pragma unroll
    for (int u = 0; u < kKeysPerLane; ++u) {
        if (u * 64 >= count) break;
        int rank = 0;
#pragma unroll
        for (int e = 0; e < NB; ++e) {
            const unsigned long long bal = __ballot(keys[u] == e);
            rank = keys[u] == e ? base[e] + lanes_below(bal) : rank;
            base[e] += __popcll(bal);
        }
        if (keys[u] >= 0) {
            const int i = begin + u * 64 + lane;
            row_id_map[i] = rank;
            if (sorted_indices != nullptr && rank < num_out) sorted_indices[rank] = i;
        }
    }
    int upd = 0;
#pragma unroll
    for (int e = 0; e < NB; ++e) upd = lane == e ? base[e] : upd;
    if (lane < nbins) row[lane] = upd;
}

// Dispatch on the bin count.
__device__ __forceinline__ void hist_chunk(int *row, const int (&keys)[kKeysPerLane], int count, int nbins, int nbits) {
    if (nbins <= 8) hist_keys_few<8>(row, keys, count, nbins);
    else if (nbins <= 16) hist_keys_few<16>(row, keys, count, nbins);
    else hist_keys(row, keys, count, nbits);
}
__device__ __forceinline__ void scatter_chunk(int *row, const int (&keys)[kKeysPerLane], int begin, int count, int nbins,
                                              int nbits, int num_out, int32_t *row_id_map, int32_t *sorted_indices) {
    if (nbins <= 8) scatter_keys_few<8>(row, keys, begin, count, nbins, num_out, row_id_map, sorted_indices);
    else if (nbins <= 16) scatter_keys_few<16>(row, keys, begin, count, nbins, num_out, row_id_map, sorted_indices);
    else scatter_keys(row, keys, begin, count, nbits, num_out, row_id_map, sorted_indices);
}

// Histogram of idx[begin, end) into one table row owned by this wavefront.
template <typename IdxT>
__device__ __forceinline__ void wave_histogram(int *row, const IdxT *idx, int begin, int end,
                                               int nbins, int nbits) {
    int keys[kKeysPerLane];
    for (int c = begin; c < end; c += kChunk) {
        const int ce = min(c + kChunk, end);
        load_keys(idx, c, ce, nbins, keys);
        hist_chunk(row, keys, ce - c, nbins, nbits);
    }
}

// Stable scatter of idx[begin, end).
template <typename IdxT>
__device__ __forceinline__ void wave_scatter(int *row, const IdxT *idx, int begin, int end,
                                             int nbins, int nbits, int num_out, int32_t *row_id_map,
                                             int32_t *sorted_indices) {
    int keys[kKeysPerLane];
    for (int c = begin; c < end; c += kChunk) {
        const int ce = min(c + kChunk, end);
        load_keys(idx, c, ce, nbins, keys);
        scatter_chunk(row, keys, c, ce - c, nbins, nbits, num_out, row_id_map, sorted_indices);
    }
}

// Exclusive scan of one int per thread over a block of up to 1024 threads.
__device__ __forceinline__ int block_exclusive_scan(int v, int *scratch /* >= 16 ints */) {
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

// ---- single-block sort (small inputs): one launch ---------------------------------
template <typename IdxT>
__global__ __launch_bounds__(kSortBlockWaves * 64) void sort_small_kernel(
    const IdxT *__restrict__ idx, int n, int nbins, int nbits, int num_out, int32_t *row_id_map,
    int32_t *sorted_indices, int64_t *tokens_per_expert, int tpe_n) {
    extern __shared__ int lds[];  // [kSortBlockWaves][nbins] table, then 16 ints of scan scratch
    int *scratch = lds + kSortBlockWaves * nbins;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    for (int i = tid; i < kSortBlockWaves * nbins; i += blockDim.x) lds[i] = 0;
    __syncthreads();
    int seg = (n + kSortBlockWaves - 1) / kSortBlockWaves;
    seg = (seg + 63) & ~63;
    const int begin = min(wave * seg, n);
    const int end = min(begin + seg, n);
    int keys[kKeysPerLane];                    // seg <= kChunk: the whole segment stays in registers
    load_keys(idx, begin, end, nbins, keys);
    hist_chunk(lds + wave * nbins, keys, end - begin, nbins, nbits);
    __syncthreads();
    int total = 0;
    int cnt[kSortBlockWaves];
    if (tid < nbins) {
#pragma unroll
        for (int w = 0; w < kSortBlockWaves; ++w) cnt[w] = lds[w * nbins + tid];
#pragma unroll
        for (int w = 0; w < kSortBlockWaves; ++w) total += cnt[w];
    }
    int run = block_exclusive_scan(total, scratch);
    if (tid < nbins) {
#pragma unroll
        for (int w = 0; w < kSortBlockWaves; ++w) {
            lds[w * nbins + tid] = run;
            run += cnt[w];
        }
        if (tokens_per_expert != nullptr && tid < tpe_n) tokens_per_expert[tid] = total;
    }
    __syncthreads();
    scatter_chunk(lds + wave * nbins, keys, begin, end - begin, nbins, nbits, num_out, row_id_map, sorted_indices);
}

// ---- multi-block sort (large inputs): histogram, scan, scatter ----------------------
template <typename IdxT>
__global__ __launch_bounds__(kHistWavesPerBlock * 64) void sort_hist_kernel(
    const IdxT *__restrict__ idx, int n, int seg, int nseg, int nbins, int nbits, int *table) {
    extern __shared__ int lds[];  // [kHistWavesPerBlock][nbins]
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int s = blockIdx.x * kHistWavesPerBlock + wave;
    int *row = lds + wave * nbins;
    for (int e = lane; e < nbins; e += 64) row[e] = 0;
    __builtin_amdgcn_wave_barrier();
    if (s < nseg) {
        const int begin = min(s * seg, n);
        const int end = min(begin + seg, n);
        wave_histogram(row, idx, begin, end, nbins, nbits);
        __builtin_amdgcn_wave_barrier();
        for (int e = lane; e < nbins; e += 64) table[static_cast<int64_t>(s) * nbins + e] = row[e];
    }
}

__global__ __launch_bounds__(1024) void sort_scan_kernel(int *table, int nseg, int nbins,
                                                         int64_t *tokens_per_expert, int tpe_n) {
    __shared__ int scratch[16];
    const int tid = threadIdx.x;
    int total = 0;
    if (tid < nbins) {
#pragma unroll 8
        for (int s = 0; s < nseg; ++s) total += table[static_cast<int64_t>(s) * nbins + tid];
    }
    int run = block_exclusive_scan(total, scratch);
    if (tid < nbins) {
#pragma unroll 8
        for (int s = 0; s < nseg; ++s) {
            const int64_t at = static_cast<int64_t>(s) * nbins + tid;
            const int c = table[at];
            table[at] = run;
            run += c;
        }
        if (tokens_per_expert != nullptr && tid < tpe_n) tokens_per_expert[tid] = total;
    }
}

template <typename IdxT>
__global__ __launch_bounds__(kHistWavesPerBlock * 64) void sort_scatter_kernel(
    const IdxT *__restrict__ idx, int n, int seg, int nseg, int nbins, int nbits, const int *table,
    int num_out, int32_t *row_id_map, int32_t *sorted_indices) {
    extern __shared__ int lds[];
    const int wave = threadIdx.x >> 6;
    const int lane = threadIdx.x & 63;
    const int s = blockIdx.x * kHistWavesPerBlock + wave;
    if (s >= nseg) return;
    int *row = lds + wave * nbins;
    for (int e = lane; e < nbins; e += 64) row[e] = table[static_cast<int64_t>(s) * nbins + e];
    __builtin_amdgcn_wave_barrier();
    const int begin = min(s * seg, n);
    const int end = min(begin + seg, n);
    wave_scatter(row, idx, begin, end, nbins, nbits, num_out, row_id_map, sorted_indices);
}

// ---- row movers ---------------------------------------------------------------------
// Thread layout shared by the row kernels: a block of 256 threads covers
// rows_per_block rows, `lanes` threads per row, each thread striding over the
// row's vectors.
struct RowLayout {
    int lanes;           // threads per row (power of two, 1..64)
    int rows_per_block;  // 256 / lanes
};
inline RowLayout row_layout(int64_t vecs_per_row) {
    int lanes = 1;
    while (lanes < 64 && lanes < vecs_per_row) lanes <<= 1;   // one wavefront per row at most
    return RowLayout{lanes, 256 / lanes};
}

constexpr int kSlotBatch = 8;   // top-k slots whose row ids / weights are kept in registers at a time

// permuted[row_id_map[t*k+j]] = tokens[t] for every kept (t, j).  Row ids are read once per thread,
// and four independent 16-byte loads are in flight per thread before the first store.
template <typename VecT>
__global__ __launch_bounds__(256) void permute_rows_kernel(const VecT *__restrict__ tokens,
                                                           VecT *__restrict__ permuted,
                                                           const int32_t *__restrict__ row_id_map,
                                                           int num_tokens, int topk, int vecs_per_row,
                                                           int num_out, int lanes) {
    const int local_row = threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    const int t = blockIdx.x * (256 / lanes) + local_row;
    if (t >= num_tokens) return;
    const VecT *src = tokens + static_cast<int64_t>(t) * vecs_per_row;
    for (int j0 = 0; j0 < topk; j0 += kSlotBatch) {
        int d[kSlotBatch];
#pragma unroll
        for (int j = 0; j < kSlotBatch; ++j)
            d[j] = j0 + j < topk ? row_id_map[static_cast<int64_t>(t) * topk + j0 + j] : num_out;
        for (int c0 = lane; c0 < vecs_per_row; c0 += 4 * lanes) {
            VecT v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (c0 + u * lanes < vecs_per_row) v[u] = src[c0 + u * lanes];
#pragma unroll
            for (int j = 0; j < kSlotBatch; ++j) {
                if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_out)) continue;   // dropped (or corrupt) id
                VecT *dst = permuted + static_cast<int64_t>(d[j]) * vecs_per_row;
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (c0 + u * lanes < vecs_per_row) dst[c0 + u * lanes] = v[u];
            }
        }
    }
}

// out[t] = sum_j w[t,j] * rows[row_id_map[t*k+j]] ; w == nullptr -> unweighted.
// VEC: elements per thread access (16 bytes worth, or 1 for the unaligned path).
// Row ids and weights are read once per thread; per pair of output vectors all topk row loads are
// independent and issued together; accumulation is fp32 in registers, one rounding.
template <typename DT, int VEC>
__global__ __launch_bounds__(256) void gather_combine_kernel(
    const typename DT::storage *__restrict__ rows, const int32_t *__restrict__ row_id_map,
    const typename DT::storage *__restrict__ probs, typename DT::storage *__restrict__ out,
    int num_tokens, int topk, int hidden, int num_rows, int lanes) {
    using S = typename DT::storage;
    const int local_row = threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    const int t = blockIdx.x * (256 / lanes) + local_row;
    if (t >= num_tokens) return;
    const int vecs = hidden / VEC;
    constexpr int U = 2;
    for (int c0 = lane; c0 < vecs; c0 += U * lanes) {
        float acc[U][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[u][e] = 0.f;
        for (int j0 = 0; j0 < topk; j0 += kSlotBatch) {
            int d[kSlotBatch];
            float w[kSlotBatch];
#pragma unroll
            for (int j = 0; j < kSlotBatch; ++j) {
                const int64_t flat = static_cast<int64_t>(t) * topk + j0 + j;
                d[j] = j0 + j < topk ? row_id_map[flat] : num_rows;
                w[j] = (probs != nullptr && j0 + j < topk) ? DT::to_float(probs[flat]) : 1.f;
            }
            S tmp[kSlotBatch][U][VEC];
#pragma unroll
            for (int j = 0; j < kSlotBatch; ++j) {
                if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_rows)) continue;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int c = c0 + u * lanes;
                    if (c >= vecs) continue;
                    const S *src = rows + static_cast<int64_t>(d[j]) * hidden + static_cast<int64_t>(c) * VEC;
                    if constexpr (VEC * sizeof(S) == 16) {
                        *reinterpret_cast<v16 *>(tmp[j][u]) = *reinterpret_cast<const v16 *>(src);
                    } else {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) tmp[j][u][e] = src[e];
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < kSlotBatch; ++j) {
                if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_rows)) continue;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    if (c0 + u * lanes >= vecs) continue;
#pragma unroll
                    for (int e = 0; e < VEC; ++e) acc[u][e] = fmaf(w[j], DT::to_float(tmp[j][u][e]), acc[u][e]);
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int c = c0 + u * lanes;
            if (c >= vecs) continue;
            S res[VEC];
#pragma unroll
            for (int e = 0; e < VEC; ++e) res[e] = DT::from_float(acc[u][e]);
            S *dst = out + static_cast<int64_t>(t) * hidden + static_cast<int64_t>(c) * VEC;
            if constexpr (VEC * sizeof(S) == 16) {
                *reinterpret_cast<v16 *>(dst) = *reinterpret_cast<v16 *>(res);
            } else {
#pragma unroll
                for (int e = 0; e < VEC; ++e) dst[e] = res[e];
            }
        }
    }
}

// One block per token: grad_permuted[row] = w * dY[t]; grad_probs[t,j] = <dY[t], permuted[row]>.
template <typename DT, int VEC>
__global__ __launch_bounds__(256) void unpermute_grad_kernel(
    const typename DT::storage *__restrict__ permuted, const typename DT::storage *__restrict__ grad_out,
    const int32_t *__restrict__ row_id_map, const typename DT::storage *__restrict__ probs,
    typename DT::storage *__restrict__ grad_permuted, typename DT::storage *__restrict__ grad_probs,
    int topk, int hidden, int num_rows) {
    using S = typename DT::storage;
    __shared__ float partial[4];
    const int t = blockIdx.x;
    const int vecs = hidden / VEC;
    const S *gy = grad_out + static_cast<int64_t>(t) * hidden;
    for (int j = 0; j < topk; ++j) {
        const int64_t flat = static_cast<int64_t>(t) * topk + j;
        const int d = row_id_map[flat];
        const bool kept = static_cast<unsigned>(d) < static_cast<unsigned>(num_rows);   // negative ids count as dropped
        const float w = probs != nullptr ? DT::to_float(probs[flat]) : 1.f;
        float dot = 0.f;
        if (kept) {
            for (int c = threadIdx.x; c < vecs; c += blockDim.x) {
                S g[VEC], x[VEC], o[VEC];
                const S *gp = gy + static_cast<int64_t>(c) * VEC;
                const int64_t off = static_cast<int64_t>(d) * hidden + static_cast<int64_t>(c) * VEC;
                if constexpr (VEC * sizeof(S) == 16) {
                    *reinterpret_cast<v16 *>(g) = *reinterpret_cast<const v16 *>(gp);
                    if (grad_probs != nullptr)
                        *reinterpret_cast<v16 *>(x) =
                            MS_NT_LOAD(reinterpret_cast<const v16 *>(permuted + off));
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) g[e] = gp[e];
                    if (grad_probs != nullptr) {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) x[e] = permuted[off + e];
                    }
                }
#pragma unroll
                for (int e = 0; e < VEC; ++e) {
                    const float gf = DT::to_float(g[e]);
                    o[e] = DT::from_float(w * gf);
                    if (grad_probs != nullptr) dot = fmaf(gf, DT::to_float(x[e]), dot);
                }
                if constexpr (VEC * sizeof(S) == 16) {
                    MS_NT_STORE(*reinterpret_cast<v16 *>(o),
                                                reinterpret_cast<v16 *>(grad_permuted + off));
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) grad_permuted[off + e] = o[e];
                }
            }
        }
        if (grad_probs != nullptr) {
#pragma unroll
            for (int dlt = 32; dlt > 0; dlt >>= 1) dot += __shfl_down(dot, dlt, 64);
            const int wave = threadIdx.x >> 6;
            if ((threadIdx.x & 63) == 0) partial[wave] = dot;
            __syncthreads();
            if (threadIdx.x == 0) {
                float s = 0.f;
                for (int w2 = 0; w2 < (blockDim.x + 63) / 64; ++w2) s += partial[w2];
                grad_probs[flat] = DT::from_float(s);
            }
            __syncthreads();
        }
    }
}

__global__ __launch_bounds__(256) void copy_bytes_kernel(const v16 *__restrict__ src, v16 *__restrict__ dst,
                                                         size_t nvec) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < nvec;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        dst[i] = src[i];
}
__global__ void copy_tail_kernel(const unsigned char *src, unsigned char *dst, size_t begin, size_t end) {
    const size_t i = begin + blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (i < end) dst[i] = src[i];
}

// ---- sort + row scatter in one launch (small inputs, few bins) ------------------------------------
// The single-workgroup sort is latency, not work: ~12 us for 8192 keys, after which the row scatter still has to
// be launched.  Here every scatter workgroup works out the rows of its own tokens itself: its four wavefronts
// count, per bin, the keys in front of the workgroup's first flat position and the keys from there on (two
// histograms over all keys, read from L2 after the first workgroup has touched them), a scan over the bins
// turns that into each bin's next free row as seen from this workgroup, and wavefront 0 ranks the
// workgroup's own positions with the same stable scatter the sort kernels use.  Counting is redundant across
// workgroups (every one reads all keys) but cheap, and it overlaps with the row traffic of the workgroups
// that are already copying.  The integer outputs are the same as the sort kernels' by construction.
constexpr int kFusedMaxBins = 16;   // the per-bin ballot counting; measured slower than two launches with 1024 bins

template <typename IdxT, typename VecT>
__global__ __launch_bounds__(256) void permute_fused_kernel(
    const VecT *__restrict__ tokens, VecT *__restrict__ permuted, const IdxT *__restrict__ idx, int n, int nbins,
    int nbits, int num_out, int32_t *__restrict__ row_id_map, int32_t *__restrict__ sorted_indices,
    int64_t *__restrict__ tokens_per_expert, int tpe_n, int num_tokens, int topk, int vecs_per_row, int lanes) {
    extern __shared__ int lds[];               // before[4][nbins], after[4][nbins], base[nbins], 16 ints scratch
    int *before = lds;
    int *after = lds + 4 * nbins;
    int *base = lds + 8 * nbins;
    int *scratch = base + nbins;
    const int tid = threadIdx.x;
    const int wave = tid >> 6;
    const int rows_per_block = 256 / lanes;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int p0 = t0 * topk, p1 = t1 * topk;  // this workgroup's flat positions
    for (int i = tid; i < 8 * nbins; i += 256) lds[i] = 0;
    __syncthreads();
    int seg = (n + 3) / 4;
    seg = (seg + 63) & ~63;
    const int b = min(wave * seg, n);
    const int e = min(b + seg, n);
    const int mid = min(max(p0, b), e);
    wave_histogram(before + wave * nbins, idx, b, mid, nbins, nbits);
    wave_histogram(after + wave * nbins, idx, mid, e, nbins, nbits);
    __syncthreads();
    // bins in passes of 256 (one per thread), the running row count carried from pass to pass
    int carry = 0;
    for (int e0 = 0; e0 < nbins; e0 += 256) {
        const int bin = e0 + tid;
        int bef = 0, tot = 0;
        if (bin < nbins) {
#pragma unroll
            for (int w = 0; w < 4; ++w) {
                bef += before[w * nbins + bin];
                tot += after[w * nbins + bin];
            }
            tot += bef;
        }
        const int first = carry + block_exclusive_scan(tot, scratch);   // first row of this bin
        if (bin < nbins) {
            base[bin] = first + bef;
            if (blockIdx.x == 0 && tokens_per_expert != nullptr && bin < tpe_n) tokens_per_expert[bin] = tot;
        }
        if (tid == 255) scratch[15] = first + tot;
        __syncthreads();
        carry = scratch[15];
        __syncthreads();
    }
    if (wave == 0) wave_scatter(base, idx, p0, p1, nbins, nbits, num_out, row_id_map, sorted_indices);
    // Workgroup-scope release / acquire (part of __syncthreads) is all the other wavefronts need to see the
    // row ids: they run on the same compute unit.  A device-scope fence here would write the L2 back, rows
    // of other workgroups included, once per workgroup.
    __syncthreads();

    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    if (t >= num_tokens) return;
    const VecT *src = tokens + static_cast<int64_t>(t) * vecs_per_row;
    for (int j0 = 0; j0 < topk; j0 += kSlotBatch) {
        int d[kSlotBatch];
#pragma unroll
        for (int j = 0; j < kSlotBatch; ++j)
            d[j] = j0 + j < topk ? row_id_map[static_cast<int64_t>(t) * topk + j0 + j] : num_out;
        for (int c0 = lane; c0 < vecs_per_row; c0 += 4 * lanes) {
            VecT v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (c0 + u * lanes < vecs_per_row) v[u] = src[c0 + u * lanes];
#pragma unroll
            for (int j = 0; j < kSlotBatch; ++j) {
                if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_out)) continue;   // dropped (or corrupt) id
                VecT *dst = permuted + static_cast<int64_t>(d[j]) * vecs_per_row;
#pragma unroll
                for (int u = 0; u < 4; ++u)
                    if (c0 + u * lanes < vecs_per_row) dst[c0 + u * lanes] = v[u];
            }
        }
    }
}

// ---- routing-map (mask) mode ----------------------------------------------------------
// The [T, E] boolean routing map is sorted with the same counting sort as the index form: flat position
// i = t*E + e gets the key e when the entry is set and the extra last key E when it is not, so the set
// entries come out expert-major, token-ascending (rows 0 .. nnz-1) and the unset ones after them.  In
// drop-and-pad mode the key is 2*e + (entry unset): every expert's block then holds all T tokens, routed
// ones first, and the first `capacity` of each block are kept, which is what
// argsort(descending, stable)[:, :capacity] on the transposed int8 map selects.
__global__ __launch_bounds__(256) void routing_map_keys_kernel(const unsigned char *__restrict__ map, int n, int E,
                                                               int pad, int32_t *__restrict__ keys,
                                                               int32_t *__restrict__ sorted_flat, int num_rows) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        const int e = i % E;
        const bool set = map[i] != 0;
        keys[i] = pad ? 2 * e + (set ? 0 : 1) : (set ? e : E);
    }
    if (i < num_rows) sorted_flat[i] = -1;   // rows nobody maps to stay marked
}

// rank[i] (position of flat entry i in the sorted order) -> output row, in place; the inverse list
// sorted_flat[row] = i; rows per expert.  counts: per-key totals of the sort (E+1 keys, or 2E in pad mode).
__global__ __launch_bounds__(256) void routing_map_rows_kernel(const int32_t *__restrict__ keys, int n, int T, int E,
                                                               int capacity, int num_rows,
                                                               int32_t *__restrict__ row_id_map,
                                                               int32_t *__restrict__ sorted_flat,
                                                               const int64_t *__restrict__ counts,
                                                               int64_t *__restrict__ tokens_per_expert) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (tokens_per_expert != nullptr && i < E) tokens_per_expert[i] = capacity > 0 ? capacity : counts[i];
    if (i >= n) return;
    const int rank = row_id_map[i];
    int row = -1;
    if (capacity > 0) {
        const int e = rank / T, j = rank - e * T;
        if (j < capacity) row = e * capacity + j;
    } else if (keys[i] < E) {
        row = rank;
    }
    if (static_cast<unsigned>(row) >= static_cast<unsigned>(num_rows)) row = -1;
    row_id_map[i] = row < 0 ? 0x7fffffff : row;   // dropped: an id no row count reaches
    if (row >= 0) sorted_flat[row] = i;
}

// permuted_probs[r] = probs.flat[sorted_flat[r]], sorted_token_ids[r] = sorted_flat[r] / E (0 for unmapped rows)
template <typename S>
__global__ __launch_bounds__(256) void routing_map_probs_kernel(const int32_t *__restrict__ sorted_flat, int num_rows,
                                                                int E, const S *__restrict__ probs,
                                                                S *__restrict__ permuted_probs,
                                                                int64_t *__restrict__ sorted_token_ids) {
    const int r = blockIdx.x * blockDim.x + threadIdx.x;
    if (r >= num_rows) return;
    const int i = sorted_flat[r];
    if (permuted_probs != nullptr) permuted_probs[r] = i >= 0 ? probs[i] : S(0);
    if (sorted_token_ids != nullptr) sorted_token_ids[r] = i >= 0 ? i / E : 0;
}

// grad_probs.flat[i] = grad_permuted_probs[row_id_map[i]] for mapped entries, 0 otherwise
template <typename S>
__global__ __launch_bounds__(256) void routing_map_probs_grad_kernel(const int32_t *__restrict__ row_id_map, int n,
                                                                     const S *__restrict__ grad_permuted_probs,
                                                                     int num_rows, S *__restrict__ grad_probs) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= n) return;
    const int r = row_id_map[i];
    grad_probs[i] = static_cast<unsigned>(r) < static_cast<unsigned>(num_rows) ? grad_permuted_probs[r] : S(0);
}

// Mask mode, rows laid out and moved in one launch (no drop-and-pad, experts a power of two up to 16, so that
// a 16-byte vector of the map holds whole tokens and byte position b of a vector always belongs to expert
// b % E).  Every scatter workgroup counts, per expert column, the set entries of the tokens in front of its
// own and of all tokens (byte-wise over the map, read from L2), turns that into the next free row of every
// expert as seen from its first token, walks its own few tokens in order, and copies their rows.  Same
// outputs as the sort-based path.
__global__ __launch_bounds__(256) void routing_map_fused_kernel(
    const v16 *__restrict__ tokens, v16 *__restrict__ permuted, const unsigned char *__restrict__ map, int num_tokens,
    int E, int num_rows, int32_t *__restrict__ row_id_map, int32_t *__restrict__ sorted_flat,
    int64_t *__restrict__ tokens_per_expert, int vecs_per_row, int lanes) {
    extern __shared__ int lds[];     // before[16], total[16], base[16], rows[rows_per_block][E]
    int *before = lds, *total = lds + 16, *base = lds + 32, *rows = lds + 48;
    const int tid = threadIdx.x;
    const int rows_per_block = 256 / lanes;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int64_t n = static_cast<int64_t>(num_tokens) * E;
    const int64_t split = static_cast<int64_t>(t0) * E;          // flat entries in front of this workgroup
    if (tid < 32) lds[tid] = 0;
    __syncthreads();
    // counters per byte position of a vector (position b <-> expert b % E); folded per expert afterwards
    int cb[16], ct[16];
#pragma unroll
    for (int b = 0; b < 16; ++b) cb[b] = ct[b] = 0;
    const int64_t nvec = n / 16;
    const v16 *mv = reinterpret_cast<const v16 *>(map);
    for (int64_t v = tid; v < nvec; v += 256) {
        const v16 w = mv[v];
        const int64_t first = v * 16;
        const bool all_before = first + 16 <= split;
        const bool none_before = first >= split;
#pragma unroll
        for (int b = 0; b < 16; ++b) {
            const int bit = ((w[b >> 2] >> (8 * (b & 3))) & 0xffu) != 0u ? 1 : 0;
            ct[b] += bit;
            cb[b] += (all_before || (!none_before && first + b < split)) ? bit : 0;
        }
    }
    // entries past the last whole vector (n is not a multiple of 16 only for small maps)
    for (int64_t i = nvec * 16 + tid; i < n; i += 256) {
        const int bit = map[i] != 0 ? 1 : 0;
        const int e = static_cast<int>(i % E);
        atomicAdd(&total[e], bit);
        if (i < split) atomicAdd(&before[e], bit);
    }
    // fold byte positions into experts, then lanes, then wavefronts
#pragma unroll
    for (int e = 0; e < 16; ++e) {
        if (e >= E) break;
        int sb = 0, st = 0;
#pragma unroll
        for (int b = 0; b < 16; ++b)
            if ((b & (E - 1)) == e) { sb += cb[b]; st += ct[b]; }   // E is a power of two
#pragma unroll
        for (int d = 32; d > 0; d >>= 1) {
            sb += __shfl_down(sb, d, 64);
            st += __shfl_down(st, d, 64);
        }
        if ((tid & 63) == 0) {
            atomicAdd(&before[e], sb);
            atomicAdd(&total[e], st);
        }
    }
    __syncthreads();
    if (tid < E) {
        int first = 0;
        for (int e = 0; e < tid; ++e) first += total[e];
        base[tid] = first + before[tid];
        if (blockIdx.x == 0 && tokens_per_expert != nullptr) tokens_per_expert[tid] = total[tid];
    }
    if (blockIdx.x == 0) {   // rows that nothing maps to (only if the caller's row count exceeds the set entries)
        int nnz = 0;
        for (int e = 0; e < E; ++e) nnz += total[e];
        for (int r = nnz + tid; r < num_rows; r += 256) sorted_flat[r] = -1;
    }
    __syncthreads();
    // own tokens, in order, one thread per expert column
    if (tid < E) {
        int next = base[tid];
        for (int t = t0; t < t1; ++t) {
            const int64_t i = static_cast<int64_t>(t) * E + tid;
            int row = 0x7fffffff;
            if (map[i] != 0) {
                if (next < num_rows) {
                    row = next;
                    sorted_flat[row] = static_cast<int32_t>(i);
                }
                ++next;
            }
            row_id_map[i] = row;
            rows[(t - t0) * E + tid] = row;
        }
    }
    __syncthreads();
    if (tokens == nullptr) return;
    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    if (t >= num_tokens) return;
    const v16 *src = tokens + static_cast<int64_t>(t) * vecs_per_row;
    int d[16];
#pragma unroll
    for (int j = 0; j < 16; ++j) d[j] = j < E ? rows[local_row * E + j] : 0x7fffffff;
    for (int c0 = lane; c0 < vecs_per_row; c0 += 4 * lanes) {
        v16 v[4];
#pragma unroll
        for (int u = 0; u < 4; ++u)
            if (c0 + u * lanes < vecs_per_row) v[u] = src[c0 + u * lanes];
#pragma unroll
        for (int j = 0; j < 16; ++j) {
            if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_rows)) continue;
            v16 *dst = permuted + static_cast<int64_t>(d[j]) * vecs_per_row;
#pragma unroll
            for (int u = 0; u < 4; ++u)
                if (c0 + u * lanes < vecs_per_row) dst[c0 + u * lanes] = v[u];
        }
    }
}

// ---- host helpers -------------------------------------------------------------------
struct SortPlan {
    int n, nbins, nbits, seg, nseg;
    bool small;
};

inline SortPlan make_sort_plan(int64_t n, int64_t experts_hint) {
    SortPlan p{};
    p.n = static_cast<int>(n);
    int64_t want = experts_hint > 0 ? experts_hint : MS_MAX_EXPERTS;
    p.nbins = 2;
    p.nbits = 1;
    while (p.nbins < want) {
        p.nbins <<= 1;
        p.nbits++;
    }
    p.small = n <= kSmallSortMax;
    int64_t seg = 1024;
    if (ceil_div(n, seg) > kMaxSegments) seg = (ceil_div(n, kMaxSegments) + 63) / 64 * 64;
    p.seg = static_cast<int>(seg);
    p.nseg = static_cast<int>(ceil_div(n, seg));
    return p;
}

template <typename IdxT>
int launch_sort(hipStream_t stream, const SortPlan &p, const IdxT *idx, int num_out, int32_t *row_id_map,
                int32_t *sorted_indices, int64_t *tpe, int tpe_n, void *workspace) {
    if (p.n == 0) return MS_OK;
    if (p.small) {
        const size_t lds = (static_cast<size_t>(kSortBlockWaves) * p.nbins + 16) * sizeof(int);
        static thread_local bool configured[2] = {false, false};
        constexpr int which = sizeof(IdxT) == 8 ? 1 : 0;
        if (!configured[which]) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&sort_small_kernel<IdxT>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize,
                                               (kSortBlockWaves * MS_MAX_EXPERTS + 16) * sizeof(int));
            MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "hipFuncSetAttribute(sort_small): %s", hipGetErrorString(e));
            configured[which] = true;
        }
        hipLaunchKernelGGL(sort_small_kernel<IdxT>, dim3(1), dim3(kSortBlockWaves * 64), lds, stream, idx, p.n,
                           p.nbins, p.nbits, num_out, row_id_map, sorted_indices, tpe, tpe_n);
        MS_CHECK_LAUNCH("sort_small_kernel");
        return MS_OK;
    }
    int *table = static_cast<int *>(workspace);
    const int blocks = static_cast<int>(ceil_div(p.nseg, kHistWavesPerBlock));
    const size_t lds = static_cast<size_t>(kHistWavesPerBlock) * p.nbins * sizeof(int);
    hipLaunchKernelGGL(sort_hist_kernel<IdxT>, dim3(blocks), dim3(kHistWavesPerBlock * 64), lds, stream, idx, p.n,
                       p.seg, p.nseg, p.nbins, p.nbits, table);
    MS_CHECK_LAUNCH("sort_hist_kernel");
    hipLaunchKernelGGL(sort_scan_kernel, dim3(1), dim3(1024), 0, stream, table, p.nseg, p.nbins, tpe, tpe_n);
    MS_CHECK_LAUNCH("sort_scan_kernel");
    hipLaunchKernelGGL(sort_scatter_kernel<IdxT>, dim3(blocks), dim3(kHistWavesPerBlock * 64), lds, stream, idx,
                       p.n, p.seg, p.nseg, p.nbins, p.nbits, table, num_out, row_id_map, sorted_indices);
    MS_CHECK_LAUNCH("sort_scatter_kernel");
    return MS_OK;
}

template <typename VecT>
int launch_permute_rows(hipStream_t stream, const void *tokens, void *permuted, const int32_t *map, int64_t T,
                        int64_t k, int64_t row_bytes, int64_t num_out) {
    const int64_t vecs = row_bytes / sizeof(VecT);
    const RowLayout rl = row_layout(vecs);
    const int64_t blocks = ceil_div(T, rl.rows_per_block);
    hipLaunchKernelGGL(permute_rows_kernel<VecT>, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                       static_cast<const VecT *>(tokens), static_cast<VecT *>(permuted), map, static_cast<int>(T),
                       static_cast<int>(k), static_cast<int>(vecs), static_cast<int>(num_out), rl.lanes);
    MS_CHECK_LAUNCH("permute_rows_kernel");
    return MS_OK;
}

template <typename IdxT, typename VecT>
int launch_permute_fused(hipStream_t stream, const SortPlan &p, const void *tokens, void *permuted, const IdxT *idx,
                         int num_out, int32_t *row_id_map, int32_t *sorted_indices, int64_t *tpe, int tpe_n,
                         int64_t T, int64_t k, int64_t row_bytes) {
    const int64_t vecs = row_bytes / sizeof(VecT);
    const RowLayout rl = row_layout(vecs);
    const int64_t blocks = ceil_div(T, rl.rows_per_block);
    const size_t lds = (static_cast<size_t>(9) * p.nbins + 16) * sizeof(int);
    hipLaunchKernelGGL((permute_fused_kernel<IdxT, VecT>), dim3(static_cast<unsigned>(blocks)), dim3(256), lds, stream,
                       static_cast<const VecT *>(tokens), static_cast<VecT *>(permuted), idx, p.n, p.nbins, p.nbits,
                       num_out, row_id_map, sorted_indices, tpe, tpe_n, static_cast<int>(T), static_cast<int>(k),
                       static_cast<int>(vecs), rl.lanes);
    MS_CHECK_LAUNCH("permute_fused_kernel");
    return MS_OK;
}

template <typename IdxT>
int permute_fused_dispatch(hipStream_t stream, const SortPlan &p, const void *tokens, void *permuted, const IdxT *idx,
                           int num_out, int32_t *row_id_map, int32_t *sorted_indices, int64_t *tpe, int tpe_n,
                           int64_t T, int64_t k, int64_t row_bytes, int dtype) {
    if (row_bytes % 16 == 0 && aligned16(tokens) && aligned16(permuted))
        return launch_permute_fused<IdxT, v16>(stream, p, tokens, permuted, idx, num_out, row_id_map, sorted_indices, tpe,
                                               tpe_n, T, k, row_bytes);
    if (dtype == MS_FP32)
        return launch_permute_fused<IdxT, uint32_t>(stream, p, tokens, permuted, idx, num_out, row_id_map, sorted_indices,
                                                    tpe, tpe_n, T, k, row_bytes);
    return launch_permute_fused<IdxT, uint16_t>(stream, p, tokens, permuted, idx, num_out, row_id_map, sorted_indices, tpe,
                                                tpe_n, T, k, row_bytes);
}

template <typename DT>
int launch_gather_combine(hipStream_t stream, const void *rows, const int32_t *map, const void *probs, void *out,
                          int64_t T, int64_t k, int64_t H, int64_t num_rows) {
    using S = typename DT::storage;
    constexpr int VEC = 16 / sizeof(S);
    const bool vec_ok = (H % VEC == 0) && aligned16(rows) && aligned16(out);
    const int64_t vecs = vec_ok ? H / VEC : H;
    const RowLayout rl = row_layout(vecs);
    const unsigned blocks = static_cast<unsigned>(ceil_div(T, rl.rows_per_block));
    if (vec_ok) {
        hipLaunchKernelGGL((gather_combine_kernel<DT, VEC>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const S *>(rows), map, static_cast<const S *>(probs), static_cast<S *>(out),
                           static_cast<int>(T), static_cast<int>(k), static_cast<int>(H),
                           static_cast<int>(num_rows), rl.lanes);
    } else {
        hipLaunchKernelGGL((gather_combine_kernel<DT, 1>), dim3(blocks), dim3(256), 0, stream,
                           static_cast<const S *>(rows), map, static_cast<const S *>(probs), static_cast<S *>(out),
                           static_cast<int>(T), static_cast<int>(k), static_cast<int>(H),
                           static_cast<int>(num_rows), rl.lanes);
    }
    MS_CHECK_LAUNCH("gather_combine_kernel");
    return MS_OK;
}

template <typename DT>
int launch_unpermute_grad(hipStream_t stream, const void *permuted, const void *gy, const int32_t *map,
                          const void *probs, void *gperm, void *gprobs, int64_t T, int64_t k, int64_t H,
                          int64_t num_rows) {
    using S = typename DT::storage;
    constexpr int VEC = 16 / sizeof(S);
    const bool vec_ok = (H % VEC == 0) && aligned16(gy) && aligned16(gperm) && (permuted == nullptr || aligned16(permuted));
    const int64_t vecs = vec_ok ? H / VEC : H;
    int threads = 64;
    while (threads < 256 && threads < vecs) threads <<= 1;
    if (vec_ok) {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, VEC>), dim3(static_cast<unsigned>(T)), dim3(threads), 0, stream,
                           static_cast<const S *>(permuted), static_cast<const S *>(gy), map,
                           static_cast<const S *>(probs), static_cast<S *>(gperm), static_cast<S *>(gprobs),
                           static_cast<int>(k), static_cast<int>(H), static_cast<int>(num_rows));
    } else {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, 1>), dim3(static_cast<unsigned>(T)), dim3(threads), 0, stream,
                           static_cast<const S *>(permuted), static_cast<const S *>(gy), map,
                           static_cast<const S *>(probs), static_cast<S *>(gperm), static_cast<S *>(gprobs),
                           static_cast<int>(k), static_cast<int>(H), static_cast<int>(num_rows));
    }
    MS_CHECK_LAUNCH("unpermute_grad_kernel");
    return MS_OK;
}

int check_common(const char *fn, int64_t T, int64_t k, int64_t H, int dtype) {
    MS_REQUIRE(T >= 0 && k >= 1 && H >= 1, MS_ERR_INVALID_ARGUMENT,
               "%s: need num_tokens >= 0, topk >= 1, hidden >= 1 (got %lld, %lld, %lld)", fn, (long long)T,
               (long long)k, (long long)H);
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "%s: dtype %d is not one of bf16/fp16/fp32", fn, dtype);
    MS_REQUIRE(T * k < (1ll << 31) - 64 && H < (1ll << 31), MS_ERR_UNSUPPORTED,
               "%s: num_tokens*topk and hidden must fit int32", fn);
    return MS_OK;
}

}  // namespace
}  // namespace ms

using namespace ms;

extern "C" int ms_moe_token_permute_workspace_size(int64_t num_tokens, int64_t topk, int64_t num_experts_hint,
                                                   size_t *bytes) {
    MS_REQUIRE(bytes != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_moe_token_permute_workspace_size: bytes is NULL");
    MS_REQUIRE(num_tokens >= 0 && topk >= 1, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_permute_workspace_size: bad sizes");
    MS_REQUIRE(num_experts_hint >= 0 && num_experts_hint <= MS_MAX_EXPERTS, MS_ERR_UNSUPPORTED,
               "ms_moe_token_permute_workspace_size: num_experts_hint %lld exceeds %d", (long long)num_experts_hint,
               MS_MAX_EXPERTS);
    const SortPlan p = make_sort_plan(num_tokens * topk, num_experts_hint);
    *bytes = p.small ? 0 : static_cast<size_t>(p.nseg) * p.nbins * sizeof(int);
    return MS_OK;
}

extern "C" int ms_moe_token_permute(ms_stream_t stream_, const void *tokens, const void *indices, int index_dtype,
                                    int64_t T, int64_t k, int64_t H, int dtype, int64_t num_out,
                                    int64_t experts_hint, void *permuted, int32_t *row_id_map,
                                    int32_t *sorted_indices, int64_t *tokens_per_expert, void *workspace,
                                    size_t workspace_bytes) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_common("ms_moe_token_permute", T, k, H, dtype)) return rc;
    MS_REQUIRE(index_dtype == MS_INT32 || index_dtype == MS_INT64, MS_ERR_UNSUPPORTED,
               "ms_moe_token_permute: indices must be int32 or int64");
    MS_REQUIRE(experts_hint >= 0 && experts_hint <= MS_MAX_EXPERTS, MS_ERR_UNSUPPORTED,
               "ms_moe_token_permute: num_experts_hint %lld exceeds %d", (long long)experts_hint, MS_MAX_EXPERTS);
    MS_REQUIRE(num_out >= 0 && num_out <= T * k, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_permute: num_out_tokens %lld outside [0, %lld]", (long long)num_out, (long long)(T * k));
    MS_REQUIRE(tokens_per_expert == nullptr || experts_hint > 0, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_permute: tokens_per_expert needs num_experts_hint > 0");
    if (T == 0) return MS_OK;
    MS_REQUIRE(tokens && indices && row_id_map && (permuted || num_out == 0), MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_permute: NULL tensor pointer");
    const SortPlan p = make_sort_plan(T * k, experts_hint);
    const size_t need = p.small ? 0 : static_cast<size_t>(p.nseg) * p.nbins * sizeof(int);
    MS_REQUIRE(workspace_bytes >= need && (need == 0 || workspace != nullptr), MS_ERR_WORKSPACE_TOO_SMALL,
               "ms_moe_token_permute: workspace %zu < %zu bytes", workspace_bytes, need);
    const int64_t row_bytes = H * dtype_size(dtype);
    // small inputs with a known, modest number of experts: sort and row scatter in one launch
    if (p.small && p.nbins <= kFusedMaxBins && num_out > 0) {
        if (index_dtype == MS_INT32)
            return permute_fused_dispatch(stream, p, tokens, permuted, static_cast<const int32_t *>(indices), (int)num_out,
                                          row_id_map, sorted_indices, tokens_per_expert, (int)experts_hint, T, k, row_bytes,
                                          dtype);
        return permute_fused_dispatch(stream, p, tokens, permuted, static_cast<const int64_t *>(indices), (int)num_out,
                                      row_id_map, sorted_indices, tokens_per_expert, (int)experts_hint, T, k, row_bytes, dtype);
    }
    int rc;
    if (index_dtype == MS_INT32)
        rc = launch_sort(stream, p, static_cast<const int32_t *>(indices), (int)num_out, row_id_map, sorted_indices,
                         tokens_per_expert, (int)experts_hint, workspace);
    else
        rc = launch_sort(stream, p, static_cast<const int64_t *>(indices), (int)num_out, row_id_map, sorted_indices,
                         tokens_per_expert, (int)experts_hint, workspace);
    if (rc) return rc;
    if (num_out == 0) return MS_OK;
    if (row_bytes % 16 == 0 && aligned16(tokens) && aligned16(permuted))
        return launch_permute_rows<v16>(stream, tokens, permuted, row_id_map, T, k, row_bytes, num_out);
    if (dtype == MS_FP32) return launch_permute_rows<uint32_t>(stream, tokens, permuted, row_id_map, T, k, row_bytes, num_out);
    return launch_permute_rows<uint16_t>(stream, tokens, permuted, row_id_map, T, k, row_bytes, num_out);
}

extern "C" int ms_moe_token_unpermute(ms_stream_t stream_, const void *permuted, const int32_t *row_id_map,
                                      const void *probs, int64_t T, int64_t k, int64_t H, int dtype,
                                      int64_t num_rows, void *out) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_common("ms_moe_token_unpermute", T, k, H, dtype)) return rc;
    MS_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31), MS_ERR_INVALID_ARGUMENT, "ms_moe_token_unpermute: bad num_permuted_rows");
    if (T == 0) return MS_OK;
    MS_REQUIRE((permuted || num_rows == 0) && row_id_map && out, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_unpermute: NULL tensor pointer");
    switch (dtype) {
        case MS_BF16: return launch_gather_combine<BF16>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows);
        case MS_FP16: return launch_gather_combine<FP16>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows);
        default: return launch_gather_combine<FP32>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows);
    }
}

extern "C" int ms_moe_token_permute_grad(ms_stream_t stream, const void *grad_permuted, const int32_t *row_id_map,
                                         int64_t T, int64_t k, int64_t H, int dtype, int64_t num_rows,
                                         void *grad_tokens) {
    // The backward of a row gather is the unweighted top-k gather-sum.
    return ms_moe_token_unpermute(stream, grad_permuted, row_id_map, nullptr, T, k, H, dtype, num_rows, grad_tokens);
}

extern "C" int ms_moe_token_unpermute_grad(ms_stream_t stream_, const void *permuted, const void *grad_out,
                                           const int32_t *row_id_map, const void *probs, int64_t T, int64_t k,
                                           int64_t H, int dtype, int64_t num_rows, void *grad_permuted,
                                           void *grad_probs) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_common("ms_moe_token_unpermute_grad", T, k, H, dtype)) return rc;
    MS_REQUIRE(num_rows >= 0 && num_rows <= T * k, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_unpermute_grad: num_permuted_rows %lld outside [0, %lld]", (long long)num_rows,
               (long long)(T * k));
    MS_REQUIRE((grad_probs == nullptr) == (probs == nullptr), MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_unpermute_grad: probs and grad_probs must be given together");
    MS_REQUIRE(grad_probs == nullptr || permuted != nullptr || num_rows == 0, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_unpermute_grad: grad_probs needs permuted_tokens");
    if (T == 0) return MS_OK;
    MS_REQUIRE(grad_out && row_id_map && (grad_permuted || num_rows == 0), MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_unpermute_grad: NULL tensor pointer");
    switch (dtype) {
        case MS_BF16: return launch_unpermute_grad<BF16>(stream, permuted, grad_out, row_id_map, probs, grad_permuted, grad_probs, T, k, H, num_rows);
        case MS_FP16: return launch_unpermute_grad<FP16>(stream, permuted, grad_out, row_id_map, probs, grad_permuted, grad_probs, T, k, H, num_rows);
        default: return launch_unpermute_grad<FP32>(stream, permuted, grad_out, row_id_map, probs, grad_permuted, grad_probs, T, k, H, num_rows);
    }
}

// ---- routing-map mode entry points ------------------------------------------------------
namespace {
struct RoutingPlan {
    int64_t n;          // T * E flat entries
    int nkeys;          // E + 1, or 2 * E in drop-and-pad mode
    ms::SortPlan sort;
    size_t keys_off, counts_off, sort_off, total;
};
RoutingPlan make_routing_plan(int64_t T, int64_t E, int pad) {
    RoutingPlan r{};
    r.n = T * E;
    r.nkeys = static_cast<int>(pad ? 2 * E : E + 1);
    r.sort = ms::make_sort_plan(r.n, r.nkeys);
    auto up = [](size_t v) { return (v + 255) & ~static_cast<size_t>(255); };
    r.keys_off = 0;
    r.counts_off = up(static_cast<size_t>(r.n) * sizeof(int32_t));
    r.sort_off = r.counts_off + up(static_cast<size_t>(r.nkeys) * sizeof(int64_t));
    r.total = r.sort_off + up(r.sort.small ? 0 : static_cast<size_t>(r.sort.nseg) * r.sort.nbins * sizeof(int));
    return r;
}
int check_routing(const char *fn, int64_t T, int64_t E, int pad) {
    MS_REQUIRE(T >= 0 && E >= 1, MS_ERR_INVALID_ARGUMENT, "%s: need num_tokens >= 0, num_experts >= 1", fn);
    MS_REQUIRE((pad ? 2 * E : E + 1) <= MS_MAX_EXPERTS, MS_ERR_UNSUPPORTED, "%s: num_experts %lld too large (limit %d%s)",
               fn, (long long)E, pad ? MS_MAX_EXPERTS / 2 : MS_MAX_EXPERTS - 1, pad ? " in drop-and-pad mode" : "");
    MS_REQUIRE(T * E < (1ll << 31) - 64, MS_ERR_UNSUPPORTED, "%s: num_tokens*num_experts must fit int32", fn);
    return MS_OK;
}
}  // namespace

extern "C" int ms_moe_routing_map_workspace_size(int64_t T, int64_t E, int drop_and_pad, size_t *bytes) {
    MS_REQUIRE(bytes != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_moe_routing_map_workspace_size: bytes is NULL");
    if (int rc = check_routing("ms_moe_routing_map_workspace_size", T, E, drop_and_pad)) return rc;
    *bytes = make_routing_plan(T, E, drop_and_pad).total;
    return MS_OK;
}

extern "C" int ms_moe_routing_map_permute(ms_stream_t stream_, const void *tokens, const void *routing_map, int64_t T,
                                          int64_t E, int64_t H, int dtype, int64_t num_rows, int drop_and_pad,
                                          void *permuted, int32_t *row_id_map, int32_t *sorted_flat,
                                          int64_t *tokens_per_expert, void *workspace, size_t workspace_bytes) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char *fn = "ms_moe_routing_map_permute";
    if (int rc = check_routing(fn, T, E, drop_and_pad)) return rc;
    MS_REQUIRE(num_rows >= 0 && num_rows <= T * E, MS_ERR_INVALID_ARGUMENT, "%s: num_out_tokens %lld outside [0, %lld]", fn,
               (long long)num_rows, (long long)(T * E));
    MS_REQUIRE(!drop_and_pad || (num_rows % E == 0 && num_rows / E <= T), MS_ERR_INVALID_ARGUMENT,
               "%s: drop-and-pad needs num_out_tokens = num_experts * capacity with capacity <= num_tokens (got %lld)", fn,
               (long long)num_rows);
    if (tokens != nullptr)
        if (int rc = check_common(fn, T, E, H, dtype)) return rc;
    if (T == 0) return MS_OK;
    MS_REQUIRE(routing_map && row_id_map && sorted_flat, MS_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", fn);
    MS_REQUIRE(tokens == nullptr || permuted != nullptr || num_rows == 0, MS_ERR_INVALID_ARGUMENT, "%s: permuted is NULL", fn);
    // one launch when whole tokens fit a 16-byte vector of the map and rows move as 16-byte vectors
    const int64_t row_bytes_f = H * dtype_size(dtype);
    const bool pow2 = (E & (E - 1)) == 0 && E <= 16;
    if (!drop_and_pad && pow2 && aligned16(routing_map) &&
        (tokens == nullptr || (row_bytes_f % 16 == 0 && aligned16(tokens) && aligned16(permuted)))) {
        const int64_t vecs = tokens != nullptr ? row_bytes_f / 16 : 1;
        const RowLayout rl = tokens != nullptr ? row_layout(vecs) : RowLayout{1, 256};
        const int64_t blocks = ceil_div(T, rl.rows_per_block);
        const size_t lds = (48 + static_cast<size_t>(rl.rows_per_block) * E) * sizeof(int);
        hipLaunchKernelGGL(routing_map_fused_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), lds, stream,
                           static_cast<const v16 *>(tokens), static_cast<v16 *>(permuted),
                           static_cast<const unsigned char *>(routing_map), static_cast<int>(T), static_cast<int>(E),
                           static_cast<int>(num_rows), row_id_map, sorted_flat, tokens_per_expert, static_cast<int>(vecs),
                           rl.lanes);
        MS_CHECK_LAUNCH("routing_map_fused_kernel");
        return MS_OK;
    }
    const RoutingPlan r = make_routing_plan(T, E, drop_and_pad);
    MS_REQUIRE(workspace != nullptr && workspace_bytes >= r.total, MS_ERR_WORKSPACE_TOO_SMALL, "%s: workspace %zu < %zu bytes",
               fn, workspace_bytes, r.total);
    MS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7u) == 0, MS_ERR_INVALID_ARGUMENT, "%s: workspace must be 8-byte aligned", fn);
    char *ws = static_cast<char *>(workspace);
    int32_t *keys = reinterpret_cast<int32_t *>(ws + r.keys_off);
    int64_t *counts = reinterpret_cast<int64_t *>(ws + r.counts_off);
    const int n = static_cast<int>(r.n);
    const int capacity = drop_and_pad ? static_cast<int>(num_rows / E) : 0;
    const int64_t cover = r.n > num_rows ? r.n : num_rows;
    hipLaunchKernelGGL(routing_map_keys_kernel, dim3(static_cast<unsigned>(ceil_div(cover, 256))), dim3(256), 0, stream,
                       static_cast<const unsigned char *>(routing_map), n, static_cast<int>(E), drop_and_pad ? 1 : 0, keys,
                       sorted_flat, static_cast<int>(num_rows));
    MS_CHECK_LAUNCH("routing_map_keys_kernel");
    if (int rc = launch_sort(stream, r.sort, keys, 0, row_id_map, nullptr, counts, r.nkeys, ws + r.sort_off)) return rc;
    hipLaunchKernelGGL(routing_map_rows_kernel, dim3(static_cast<unsigned>(ceil_div(r.n, 256))), dim3(256), 0, stream, keys, n,
                       static_cast<int>(T), static_cast<int>(E), capacity, static_cast<int>(num_rows), row_id_map, sorted_flat,
                       counts, tokens_per_expert);
    MS_CHECK_LAUNCH("routing_map_rows_kernel");
    if (tokens == nullptr || num_rows == 0) return MS_OK;
    const int64_t row_bytes = H * dtype_size(dtype);
    if (row_bytes % 16 == 0 && aligned16(tokens) && aligned16(permuted))
        return launch_permute_rows<v16>(stream, tokens, permuted, row_id_map, T, E, row_bytes, num_rows);
    if (dtype == MS_FP32) return launch_permute_rows<uint32_t>(stream, tokens, permuted, row_id_map, T, E, row_bytes, num_rows);
    return launch_permute_rows<uint16_t>(stream, tokens, permuted, row_id_map, T, E, row_bytes, num_rows);
}

extern "C" int ms_moe_routing_map_probs(ms_stream_t stream_, const int32_t *sorted_flat, int64_t num_rows, int64_t E,
                                        const void *probs, int dtype, void *permuted_probs, int64_t *sorted_token_ids) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char *fn = "ms_moe_routing_map_probs";
    MS_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && E >= 1, MS_ERR_INVALID_ARGUMENT, "%s: bad sizes", fn);
    MS_REQUIRE((probs == nullptr) == (permuted_probs == nullptr), MS_ERR_INVALID_ARGUMENT,
               "%s: probs and permuted_probs must be given together", fn);
    MS_REQUIRE(probs == nullptr || dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "%s: dtype %d is not one of bf16/fp16/fp32", fn, dtype);
    if (num_rows == 0) return MS_OK;
    MS_REQUIRE(sorted_flat != nullptr, MS_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", fn);
    const dim3 grid(static_cast<unsigned>(ceil_div(num_rows, 256)));
    // a probability is only moved, never computed with: 2-byte types share one instantiation
    if (probs != nullptr && dtype == MS_FP32)
        hipLaunchKernelGGL(routing_map_probs_kernel<uint32_t>, grid, dim3(256), 0, stream, sorted_flat, static_cast<int>(num_rows),
                           static_cast<int>(E), static_cast<const uint32_t *>(probs), static_cast<uint32_t *>(permuted_probs),
                           sorted_token_ids);
    else
        hipLaunchKernelGGL(routing_map_probs_kernel<uint16_t>, grid, dim3(256), 0, stream, sorted_flat, static_cast<int>(num_rows),
                           static_cast<int>(E), static_cast<const uint16_t *>(probs), static_cast<uint16_t *>(permuted_probs),
                           sorted_token_ids);
    MS_CHECK_LAUNCH("routing_map_probs_kernel");
    return MS_OK;
}

extern "C" int ms_moe_routing_map_probs_grad(ms_stream_t stream_, const int32_t *row_id_map, int64_t num_entries,
                                             const void *grad_permuted_probs, int dtype, int64_t num_rows,
                                             void *grad_probs) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char *fn = "ms_moe_routing_map_probs_grad";
    MS_REQUIRE(num_entries >= 0 && num_entries < (1ll << 31) && num_rows >= 0 && num_rows < (1ll << 31),
               MS_ERR_INVALID_ARGUMENT, "%s: bad sizes", fn);
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "%s: dtype %d is not one of bf16/fp16/fp32", fn, dtype);
    if (num_entries == 0) return MS_OK;
    MS_REQUIRE(row_id_map && grad_probs && (grad_permuted_probs || num_rows == 0), MS_ERR_INVALID_ARGUMENT,
               "%s: NULL tensor pointer", fn);
    const dim3 grid(static_cast<unsigned>(ceil_div(num_entries, 256)));
    if (dtype == MS_FP32)
        hipLaunchKernelGGL(routing_map_probs_grad_kernel<uint32_t>, grid, dim3(256), 0, stream, row_id_map,
                           static_cast<int>(num_entries), static_cast<const uint32_t *>(grad_permuted_probs),
                           static_cast<int>(num_rows), static_cast<uint32_t *>(grad_probs));
    else
        hipLaunchKernelGGL(routing_map_probs_grad_kernel<uint16_t>, grid, dim3(256), 0, stream, row_id_map,
                           static_cast<int>(num_entries), static_cast<const uint16_t *>(grad_permuted_probs),
                           static_cast<int>(num_rows), static_cast<uint16_t *>(grad_probs));
    MS_CHECK_LAUNCH("routing_map_probs_grad_kernel");
    return MS_OK;
}

extern "C" int ms_copy_bytes(ms_stream_t stream_, const void *src, void *dst, size_t bytes) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (bytes == 0) return MS_OK;
    MS_REQUIRE(src && dst, MS_ERR_INVALID_ARGUMENT, "ms_copy_bytes: NULL pointer");
    size_t nvec = (aligned16(src) && aligned16(dst)) ? bytes / 16 : 0;
    if (nvec) {
        size_t blocks = (nvec + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;
        hipLaunchKernelGGL(copy_bytes_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const v16 *>(src), static_cast<v16 *>(dst), nvec);
        MS_CHECK_LAUNCH("copy_bytes_kernel");
    }
    const size_t done = nvec * 16;
    if (done < bytes) {
        const size_t rest = bytes - done;
        hipLaunchKernelGGL(copy_tail_kernel, dim3(static_cast<unsigned>((rest + 255) / 256)), dim3(256), 0, stream,
                           static_cast<const unsigned char *>(src), static_cast<unsigned char *>(dst), done, bytes);
        MS_CHECK_LAUNCH("copy_tail_kernel");
    }
    return MS_OK;
}
