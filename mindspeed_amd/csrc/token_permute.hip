// MoE token permute / unpermute for gfx950 (MI355X).
//
// permute  = stable counting sort of the flattened expert ids (wavefront-ballot
//            match, histogram rows in LDS, LDS prefix scan; no atomic decides an
//            order, so the result is deterministic) and a coalesced 16-byte row
//            scatter that reads every token row once and writes its topk
//            copies.  Up to 16384 positions both happen in one launch
//            (permute_fused_kernel for at most 16 bins, permute_fused_bins_kernel
//            for more); beyond that a histogram launch is followed by
//            permute_scatter_rows_kernel.  The routing-map form counts per expert
//            column instead of sorting (routing_map_fused_kernel,
//            routing_map_hist_kernel + routing_map_ranked_kernel); the separate
//            sort_* / permute_rows kernels serve what is left (no rows to move,
//            drop-and-pad, shapes the fused forms do not take).
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
                                             int nbits, int num_out, int32_t *row_id_map, int32_t *sorted_indices,
                                             int *echo = nullptr, int echo_begin = 0) {
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
            if (echo != nullptr) echo[i - echo_begin] = rank;
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
                                                 int nbins, int num_out, int32_t *row_id_map, int32_t *sorted_indices,
                                                 int *echo = nullptr, int echo_begin = 0) {
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
            if (echo != nullptr) echo[i - echo_begin] = rank;
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
// `echo` (optional, LDS): the row of flat position i is also written to echo[i - echo_begin].
__device__ __forceinline__ void scatter_chunk(int *row, const int (&keys)[kKeysPerLane], int begin, int count, int nbins,
                                              int nbits, int num_out, int32_t *row_id_map, int32_t *sorted_indices,
                                              int *echo = nullptr, int echo_begin = 0) {
    if (nbins <= 8)
        scatter_keys_few<8>(row, keys, begin, count, nbins, num_out, row_id_map, sorted_indices, echo, echo_begin);
    else if (nbins <= 16)
        scatter_keys_few<16>(row, keys, begin, count, nbins, num_out, row_id_map, sorted_indices, echo, echo_begin);
    else
        scatter_keys(row, keys, begin, count, nbits, num_out, row_id_map, sorted_indices, echo, echo_begin);
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
                                             int32_t *sorted_indices, int *echo = nullptr) {
    int keys[kKeysPerLane];
    for (int c = begin; c < end; c += kChunk) {
        const int ce = min(c + kChunk, end);
        load_keys(idx, c, ce, nbins, keys);
        scatter_chunk(row, keys, c, ce - c, nbins, nbits, num_out, row_id_map, sorted_indices, echo, begin);
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
// table[s][bin] = keys of `bin` in segment s.  One workgroup of 256 threads per segment: every thread requests all its
// keys at once (unconditional loads from clamped positions) and counts them into the segment's LDS row with
// fire-and-forget adds (a count does not depend on the order of its additions).  At 65536 positions in 64 segments
// this takes a third of the time of one wavefront per segment matching its lanes' keys against each other, which left
// the launch with 64 busy wavefronts on the whole chip.
constexpr int kHistThreads = 256;
constexpr int kHistKeysPerThread = 16;       // one pass over a segment of up to 4096 positions
template <typename IdxT>
__global__ __launch_bounds__(kHistThreads) void sort_hist_kernel(
    const IdxT *__restrict__ idx, int n, int seg, int nseg, int nbins, int nbits, int *table) {
    extern __shared__ int lds[];  // [nbins]
    (void)nbits;
    const int s = blockIdx.x;
    const int tid = threadIdx.x;
    for (int e = tid; e < nbins; e += kHistThreads) lds[e] = 0;
    const int begin = min(s * seg, n);
    const int end = min(begin + seg, n);
    __syncthreads();
    // (one pass for segments of up to 4096 positions, which is all but inputs beyond 16 M positions)
    for (int c = begin; c < end; c += kHistThreads * kHistKeysPerThread) {
        IdxT raw[kHistKeysPerThread];
#pragma unroll
        for (int u = 0; u < kHistKeysPerThread; ++u) raw[u] = idx[min(c + u * kHistThreads + tid, end - 1)];
#pragma unroll
        for (int u = 0; u < kHistKeysPerThread; ++u) {
            if (c + u * kHistThreads + tid < end) {
                long long v = static_cast<long long>(raw[u]);
                v = v < 0 ? 0 : v;
                v = v >= nbins ? nbins - 1 : v;
                __hip_atomic_fetch_add(&lds[static_cast<int>(v)], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            }
        }
    }
    __syncthreads();
    for (int e = tid; e < nbins; e += kHistThreads) table[static_cast<int64_t>(s) * nbins + e] = lds[e];
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

// The slots of token t whose row id lies in [0, num_rows), in slot order, into an LDS list (row id, weight and,
// if asked for, slot number); returns their count.  For the routing-map form, where a token has one slot per
// expert and only a few are set: the row loops then run over the list instead of over all slots.  The `lanes`
// threads of a token (a power of two, part of one wavefront) look at `lanes` slots at a time and place the
// valid ones with a ballot.  Probability gradients of the other slots are zeroed here when `zero` is given.
constexpr int kCompactMaxLocal = 2048;   // (token, slot) pairs of one workgroup that the lists hold
template <typename PT>
__device__ __forceinline__ int compact_slots(const int32_t *__restrict__ row_id_map,
                                             const typename PT::storage *__restrict__ probs, int t, int topk,
                                             int num_rows, int lane, int lanes, int *ld, float *lw, int *lj,
                                             typename PT::storage *__restrict__ zero) {
    const int wl = threadIdx.x & 63;
    const int group0 = wl - lane;
    const unsigned long long group = (lanes == 64 ? ~0ull : ((1ull << lanes) - 1ull)) << group0;
    const unsigned long long below = (1ull << wl) - 1ull;
    int count = 0;
    for (int j0 = 0; j0 < topk; j0 += lanes) {
        const int j = j0 + lane;
        const int64_t flat = static_cast<int64_t>(t) * topk + j;
        const int d = j < topk ? row_id_map[flat] : num_rows;
        const bool valid = j < topk && static_cast<unsigned>(d) < static_cast<unsigned>(num_rows);
        const unsigned long long bal = __ballot(valid) & group;
        if (valid) {
            const int pos = count + __popcll(bal & below);
            ld[pos] = d;
            lw[pos] = probs != nullptr ? PT::to_float(probs[flat]) : 1.f;
            if (lj != nullptr) lj[pos] = j;
        } else if (zero != nullptr && j < topk) {
            zero[flat] = PT::from_float(0.f);
        }
        count += __popcll(bal);
    }
    __builtin_amdgcn_wave_barrier();   // the list is read by the same lanes' wavefront only
    return count;
}

// out[t] = sum_j w[t,j] * rows[row_id_map[t*k+j]] ; w == nullptr -> unweighted.
// VEC: elements per thread access (16 bytes worth, or 1 for the unaligned path).
// Row ids and weights are read once per thread; per group of U output vectors the row loads of up to JB
// slots are independent and issued together; accumulation is fp32 in registers, slot by slot, one rounding.
template <typename DT, typename PT, int VEC, int JB, int U, bool COMPACT>
__global__ __launch_bounds__(256) void gather_combine_kernel(
    const typename DT::storage *__restrict__ rows, const int32_t *__restrict__ row_id_map,
    const typename PT::storage *__restrict__ probs, typename DT::storage *__restrict__ out,
    int num_tokens, int topk, int hidden, int num_rows, int lanes) {
    using S = typename DT::storage;
    extern __shared__ int lds[];   // COMPACT: row ids [rows_per_block][topk], then weights
    const int local_row = threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    const int t = blockIdx.x * (256 / lanes) + local_row;
    if (t >= num_tokens) return;
    const int vecs = hidden / VEC;
    int *ld = lds + local_row * topk;
    float *lw = reinterpret_cast<float *>(lds + (256 / lanes) * topk) + local_row * topk;
    int nslots = topk;
    if constexpr (COMPACT)
        nslots = compact_slots<PT>(row_id_map, probs, t, topk, num_rows, lane, lanes, ld, lw, nullptr, nullptr);
    for (int c0 = lane; c0 < vecs; c0 += U * lanes) {
        float acc[U][VEC];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int e = 0; e < VEC; ++e) acc[u][e] = 0.f;
        for (int j0 = 0; j0 < nslots; j0 += JB) {
            int d[JB];
            float w[JB];
#pragma unroll
            for (int j = 0; j < JB; ++j) {
                if constexpr (COMPACT) {
                    d[j] = j0 + j < nslots ? ld[j0 + j] : num_rows;
                    w[j] = j0 + j < nslots ? lw[j0 + j] : 1.f;
                } else {
                    const int64_t flat = static_cast<int64_t>(t) * topk + j0 + j;
                    d[j] = j0 + j < topk ? row_id_map[flat] : num_rows;
                    w[j] = (probs != nullptr && j0 + j < topk) ? PT::to_float(probs[flat]) : 1.f;
                }
            }
            S tmp[JB][U][VEC];
#pragma unroll
            for (int j = 0; j < JB; ++j) {
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
            for (int j = 0; j < JB; ++j) {
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

// grad_permuted[row] = w * dY[t]; grad_probs[t,j] = <dY[t], permuted[row]> for row = row_id_map[t*k+j].
// `lanes` threads (a power of two, one wavefront at most) share a token, so the dot products are folded with
// lane shuffles and the kernel has no barrier.  Per chunk of U vectors a thread reads dY once and has the
// loads of up to JB slots' rows in flight together.
template <typename DT, typename PT, int VEC, int JB, int U, bool COMPACT>
__global__ __launch_bounds__(256) void unpermute_grad_kernel(
    const typename DT::storage *__restrict__ permuted, const typename DT::storage *__restrict__ grad_out,
    const int32_t *__restrict__ row_id_map, const typename PT::storage *__restrict__ probs,
    typename DT::storage *__restrict__ grad_permuted, typename PT::storage *__restrict__ grad_probs,
    int num_tokens, int topk, int hidden, int num_rows, int lanes) {
    using S = typename DT::storage;
    const int local_row = threadIdx.x / lanes;
    const int lane = threadIdx.x % lanes;
    const int t = blockIdx.x * (256 / lanes) + local_row;
    if (t >= num_tokens) return;
    const int vecs = hidden / VEC;
    const S *gy = grad_out + static_cast<int64_t>(t) * hidden;
    const bool want_dot = grad_probs != nullptr;
    extern __shared__ int lds[];   // COMPACT: row ids [rows_per_block][topk], weights, slot numbers
    int *ld = lds + local_row * topk;
    float *lw = reinterpret_cast<float *>(lds + (256 / lanes) * topk) + local_row * topk;
    int *lj = lds + 2 * (256 / lanes) * topk + local_row * topk;
    int nslots = topk;
    if constexpr (COMPACT)
        nslots = compact_slots<PT>(row_id_map, probs, t, topk, num_rows, lane, lanes, ld, lw, lj, grad_probs);
    for (int j0 = 0; j0 < nslots; j0 += JB) {
        int d[JB];
        float w[JB], dot[JB];
#pragma unroll
        for (int j = 0; j < JB; ++j) {
            if constexpr (COMPACT) {
                d[j] = j0 + j < nslots ? ld[j0 + j] : num_rows;
                w[j] = j0 + j < nslots ? lw[j0 + j] : 1.f;
            } else {
                const int64_t flat = static_cast<int64_t>(t) * topk + j0 + j;
                d[j] = j0 + j < topk ? row_id_map[flat] : num_rows;          // ids outside [0, num_rows): dropped
                w[j] = (probs != nullptr && j0 + j < topk) ? PT::to_float(probs[flat]) : 1.f;
            }
            dot[j] = 0.f;
        }
        for (int c0 = lane; c0 < vecs; c0 += U * lanes) {
            S g[U][VEC], x[JB][U][VEC];
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int c = c0 + u * lanes;
                if (c >= vecs) continue;
                const S *gp = gy + static_cast<int64_t>(c) * VEC;
                if constexpr (VEC * sizeof(S) == 16) {
                    *reinterpret_cast<v16 *>(g[u]) = *reinterpret_cast<const v16 *>(gp);
                } else {
#pragma unroll
                    for (int e = 0; e < VEC; ++e) g[u][e] = gp[e];
                }
            }
            if (want_dot) {
#pragma unroll
                for (int j = 0; j < JB; ++j) {
                    if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_rows)) continue;
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int c = c0 + u * lanes;
                        if (c >= vecs) continue;
                        const S *xp = permuted + static_cast<int64_t>(d[j]) * hidden + static_cast<int64_t>(c) * VEC;
                        if constexpr (VEC * sizeof(S) == 16) {
                            // plain loads measured faster with two slots per token, non-temporal ones with more
                            if constexpr (JB == 2) *reinterpret_cast<v16 *>(x[j][u]) = *reinterpret_cast<const v16 *>(xp);
                            else *reinterpret_cast<v16 *>(x[j][u]) = MS_NT_LOAD(reinterpret_cast<const v16 *>(xp));
                        } else {
#pragma unroll
                            for (int e = 0; e < VEC; ++e) x[j][u][e] = xp[e];
                        }
                    }
                }
            }
#pragma unroll
            for (int j = 0; j < JB; ++j) {
                if (static_cast<unsigned>(d[j]) >= static_cast<unsigned>(num_rows)) continue;
#pragma unroll
                for (int u = 0; u < U; ++u) {
                    const int c = c0 + u * lanes;
                    if (c >= vecs) continue;
                    S o[VEC];
#pragma unroll
                    for (int e = 0; e < VEC; ++e) {
                        const float gf = DT::to_float(g[u][e]);
                        o[e] = DT::from_float(w[j] * gf);
                        if (want_dot) dot[j] = fmaf(gf, DT::to_float(x[j][u][e]), dot[j]);
                    }
                    S *op = grad_permuted + static_cast<int64_t>(d[j]) * hidden + static_cast<int64_t>(c) * VEC;
                    if constexpr (VEC * sizeof(S) == 16) {
                        MS_NT_STORE(*reinterpret_cast<v16 *>(o), reinterpret_cast<v16 *>(op));
                    } else {
#pragma unroll
                        for (int e = 0; e < VEC; ++e) op[e] = o[e];
                    }
                }
            }
        }
        if (want_dot) {
#pragma unroll
            for (int j = 0; j < JB; ++j) {
                float s = dot[j];
                for (int dlt = lanes >> 1; dlt > 0; dlt >>= 1) s += __shfl_xor(s, dlt, 64);
                if (lane == 0 && j0 + j < nslots) {
                    const int slot = COMPACT ? lj[j0 + j] : j0 + j;
                    grad_probs[static_cast<int64_t>(t) * topk + slot] = PT::from_float(s);
                }
            }
        }
    }
}

// ---- pieces shared by the one-launch permute kernels ---------------------------------------
// The first eight vectors of a thread's source row, as unconditional loads from clamped positions: straight-line
// code, so that the compiler's waits for loads issued before these can leave them in flight.
template <typename VecT>
__device__ __forceinline__ void prefetch_row(VecT (&v)[8], const VecT *__restrict__ src, int lane, int lanes,
                                             int vecs_per_row) {
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = src[min(lane + u * lanes, vecs_per_row - 1)];
}

// Write one source row to the rows listed in dest[0 .. count) (entries outside [0, limit) are skipped), `lanes`
// threads per row, eight vectors per thread at a time; v holds the row's first eight vectors already.
template <typename VecT>
__device__ __forceinline__ void scatter_row(VecT (&v)[8], const VecT *__restrict__ src, VecT *__restrict__ permuted,
                                            const int *dest, int count, int limit, int lane, int lanes,
                                            int vecs_per_row) {
    for (int c0 = lane; c0 < vecs_per_row; c0 += 8 * lanes) {
        if (c0 != lane) {
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + u * lanes < vecs_per_row) v[u] = src[c0 + u * lanes];
        }
        for (int j = 0; j < count; ++j) {
            const int row = dest[j];
            if (static_cast<unsigned>(row) >= static_cast<unsigned>(limit)) continue;   // dropped
            VecT *dst = permuted + static_cast<int64_t>(row) * vecs_per_row;
#pragma unroll
            for (int u = 0; u < 8; ++u)
                if (c0 + u * lanes < vecs_per_row) MS_NT_STORE(v[u], dst + c0 + u * lanes);
        }
    }
}

// ---- sort and row scatter in one launch ------------------------------------------------
constexpr int kFusedMaxBins = 16;     // one private LDS counter column per thread and bin; more bins: two launches
constexpr int kFusedMaxLocal = 4096;  // flat positions of one workgroup whose rows are handed over through LDS

// Key of a raw index, clamped to [0, last] like load_keys does.  The quick form looks at the low half of a
// 64-bit index only and reports (`bad`) whether any high half was set; the caller then counts again exactly.
template <bool EXACT>
__device__ __forceinline__ int fused_key(int32_t raw, int last, unsigned &) {
    return min(max(raw, 0), last);
}
template <bool EXACT>
__device__ __forceinline__ int fused_key(int64_t raw, int last, unsigned &bad) {
    if constexpr (EXACT) {
        const long long v = raw < 0 ? 0 : raw;
        return static_cast<int>(v > last ? last : v);
    } else {
        bad |= static_cast<unsigned>(static_cast<unsigned long long>(raw) >> 32);
        return static_cast<int>(min(static_cast<unsigned>(raw), static_cast<unsigned>(last)));
    }
}

constexpr int kScanInKernelMax = 16384;  // histogram entries (segments x bins) a scatter workgroup adds up itself
constexpr int kFusedKeys = 8;         // keys per thread in flight at a time

// One batch of raw indices: flat positions c + u * blockDim.x + tid.
template <typename IdxT>
__device__ __forceinline__ void fused_load(IdxT (&raw)[kFusedKeys], const IdxT *__restrict__ idx, int c, int n) {
#pragma unroll
    for (int u = 0; u < kFusedKeys; ++u)
        raw[u] = idx[min(c + u * static_cast<int>(blockDim.x) + static_cast<int>(threadIdx.x), n - 1)];
}

// Add the batch to the counter table: table[bin][tid % 256] for positions in front of `split`,
// table[NB + bin][tid % 256] for the others, with fire-and-forget LDS adds.
template <typename IdxT, int NB, bool EXACT>
__device__ __forceinline__ void fused_add(int *table, const IdxT (&raw)[kFusedKeys], int c, int n, int split, int last,
                                          unsigned &bad) {
    const int tid = threadIdx.x;
#pragma unroll
    for (int u = 0; u < kFusedKeys; ++u) {
        const int pos = c + u * static_cast<int>(blockDim.x) + tid;
        const int key = fused_key<EXACT>(raw[u], last, bad);
        // positions past the end read the last index again and add nothing: straight-line code, so the
        // waits stay per load
        __hip_atomic_fetch_add(table + ((pos < split ? 0 : NB) + key) * 256 + (tid & 255), pos < n ? 1 : 0,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}

// sums[r] = sum of the 256 columns of table row r, for the 2 NB rows; the first 256 threads do it,
// 256 / (2 NB) threads per row with 2 NB columns each.
template <int NB>
__device__ __forceinline__ void fused_fold(const int *table, int *sums) {
    const int tid = threadIdx.x;
    if (tid >= 256) return;
    constexpr int TPR = 256 / (2 * NB);
    constexpr int CPT = 2 * NB;
    const int r = tid / TPR, part = tid % TPR;
    int acc = 0;
#pragma unroll
    for (int j = 0; j < CPT; ++j) acc += table[r * 256 + ((j + part) % CPT) * TPR + part];
#pragma unroll
    for (int d = TPR >> 1; d > 0; d >>= 1) acc += __shfl_xor(acc, d, 64);
    if (part == 0) sums[r] = acc;
}

// Sort and row scatter in one launch, for at most kFusedMaxBins keys and inputs one workgroup can count
// (n <= kSmallSortMax).  Every workgroup (256, 512 or 1024 threads) moves the rows of rows_per_block tokens.  To
// place them it needs, per key, the number of flat positions in front of its own (-> rank of its first
// entry) and the total (-> first row of the key): it counts all n keys itself into 256 LDS counter columns,
// folds the columns, and ranks its own positions with the same stable scatter the sort kernels use, which
// also writes this workgroup's part of row_id_map / sorted_indices.  The counting is redundant across
// workgroups but short (the keys come from L2) and needs no communication between workgroups; the first
// vectors of the workgroup's source rows are requested before it starts, so the row reads are under way while
// it runs.  The destination rows reach the copying threads through LDS.  The integer outputs are the same
// as the sort kernels' by construction.
template <typename IdxT, typename VecT, int NB>
__global__ __launch_bounds__(1024) void permute_fused_kernel(
    const VecT *__restrict__ tokens, VecT *__restrict__ permuted, const IdxT *__restrict__ idx, int n, int nbins,
    int nbits, int num_out, int32_t *__restrict__ row_id_map, int32_t *__restrict__ sorted_indices,
    int64_t *__restrict__ tokens_per_expert, int tpe_n, int num_tokens, int topk, int vecs_per_row, int lanes) {
    extern __shared__ int lds[];               // table[2 * NB][256], sums[2 * NB], base[NB], dest[rows_per_block * topk]
    int *table = lds;
    int *sums = lds + 2 * NB * 256;
    int *base = sums + 2 * NB;
    int *dest = base + NB;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int rows_per_block = nthreads / lanes;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int p0 = t0 * topk, p1 = t1 * topk;  // this workgroup's flat positions
    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    const bool mover = t < num_tokens;
    const VecT *src = tokens + static_cast<int64_t>(mover ? t : 0) * vecs_per_row;

    if (tid < 256) {
#pragma unroll
        for (int r = 0; r < 2 * NB; ++r) table[r * 256 + tid] = 0;
    }
    IdxT raw[kFusedKeys];
    fused_load(raw, idx, 0, n);
    // the workgroup's own indices, for the ranking below (first wavefront, up to 64 of them)
    const bool few_own = p1 - p0 <= 64;
    IdxT own = 0;
    if (tid < 64) own = idx[min(p0 + tid, n - 1)];
    VecT v[8];   // the first vectors of this thread's row; unconditional loads from clamped positions, so that
                 // the waits for the indices above can leave these in flight
    prefetch_row(v, src, lane, lanes, vecs_per_row);
    __syncthreads();
    unsigned bad = 0;
    fused_add<IdxT, NB, false>(table, raw, 0, n, p0, nbins - 1, bad);
    for (int c = kFusedKeys * nthreads; c < n; c += kFusedKeys * nthreads) {
        fused_load(raw, idx, c, n);
        fused_add<IdxT, NB, false>(table, raw, c, n, p0, nbins - 1, bad);
    }
    if (__syncthreads_or(bad != 0u)) {          // some index does not fit 32 bits: count again with the full clamp
        if (tid < 256) {
#pragma unroll
            for (int r = 0; r < 2 * NB; ++r) table[r * 256 + tid] = 0;
        }
        __syncthreads();
        for (int c = 0; c < n; c += kFusedKeys * nthreads) {
            fused_load(raw, idx, c, n);
            fused_add<IdxT, NB, true>(table, raw, c, n, p0, nbins - 1, bad);
        }
        __syncthreads();
    }
    fused_fold<NB>(table, sums);
    __syncthreads();
    if (tid < nbins) {
        int first = 0;
        for (int e = 0; e < tid; ++e) first += sums[e] + sums[NB + e];
        base[tid] = first + sums[tid];
        if (blockIdx.x == 0 && tokens_per_expert != nullptr && tid < tpe_n)
            tokens_per_expert[tid] = sums[tid] + sums[NB + tid];
    }
    __syncthreads();
    if (tid < 64) {
        if (few_own) {
            int keys[kKeysPerLane];
#pragma unroll
            for (int u = 1; u < kKeysPerLane; ++u) keys[u] = -1;
            unsigned unused = 0;
            keys[0] = p0 + tid < p1 ? fused_key<true>(own, nbins - 1, unused) : -1;
            scatter_keys_few<NB>(base, keys, p0, p1 - p0, nbins, num_out, row_id_map, sorted_indices, dest, p0);
        } else {
            wave_scatter(base, idx, p0, p1, nbins, nbits, num_out, row_id_map, sorted_indices, dest);
        }
    }
    __syncthreads();

    if (!mover) return;
    scatter_row(v, src, permuted, dest + local_row * topk, topk, num_out, lane, lanes, vecs_per_row);
}

// The one-launch permute for more than kFusedMaxBins bins (up to MS_MAX_EXPERTS, which is what a call without
// an expert count sorts into) and n <= kSmallSortMax.  Same scheme as permute_fused_kernel, but the counters are
// one LDS word per bin and per side (in front of the workgroup's first position / all), added to directly: with
// many bins the lanes of an instruction rarely meet on a word, and a table of private columns would not fit.
template <typename IdxT, typename VecT>
__global__ __launch_bounds__(1024) void permute_fused_bins_kernel(
    const VecT *__restrict__ tokens, VecT *__restrict__ permuted, const IdxT *__restrict__ idx, int n, int nbins,
    int nbits, int num_out, int32_t *__restrict__ row_id_map, int32_t *__restrict__ sorted_indices,
    int64_t *__restrict__ tokens_per_expert, int tpe_n, int num_tokens, int topk, int vecs_per_row, int lanes) {
    extern __shared__ int lds[];               // bef[nbins], tot[nbins], scratch[32], dest[rows_per_block * topk]
    int *bef = lds;
    int *tot = lds + nbins;
    int *scratch = tot + nbins;
    int *dest = scratch + 32;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int rows_per_block = nthreads / lanes;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int p0 = t0 * topk, p1 = t1 * topk;  // this workgroup's flat positions
    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    const bool mover = t < num_tokens;
    const VecT *src = tokens + static_cast<int64_t>(mover ? t : 0) * vecs_per_row;

    for (int e = tid; e < 2 * nbins; e += nthreads) lds[e] = 0;
    IdxT raw[kFusedKeys];
    fused_load(raw, idx, 0, n);
    const bool few_own = p1 - p0 <= 64;
    IdxT own = 0;
    if (tid < 64) own = idx[min(p0 + tid, n - 1)];
    VecT v[8];   // first vectors of this thread's row: unconditional loads from clamped positions, in flight
                 // while the keys are counted
    prefetch_row(v, src, lane, lanes, vecs_per_row);
    __syncthreads();
    unsigned unused = 0;
    for (int c = 0; c < n; c += kFusedKeys * nthreads) {
        if (c != 0) fused_load(raw, idx, c, n);
#pragma unroll
        for (int u = 0; u < kFusedKeys; ++u) {
            const int pos = c + u * nthreads + tid;
            const int key = fused_key<true>(raw[u], nbins - 1, unused);
            __hip_atomic_fetch_add(tot + key, pos < n ? 1 : 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
            __hip_atomic_fetch_add(bef + key, pos < p0 ? 1 : 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
        }
    }
    __syncthreads();
    // bins in passes of one per thread, the running row count carried from pass to pass; bef[bin] becomes the
    // bin's next free row as seen from this workgroup
    int carry = 0;
    for (int e0 = 0; e0 < nbins; e0 += nthreads) {
        const int bin = e0 + tid;
        const int total = bin < nbins ? tot[bin] : 0;
        const int first = carry + block_exclusive_scan(total, scratch);
        if (bin < nbins) {
            bef[bin] += first;
            if (blockIdx.x == 0 && tokens_per_expert != nullptr && bin < tpe_n) tokens_per_expert[bin] = total;
        }
        if (tid == nthreads - 1) scratch[16] = first + total;
        __syncthreads();
        carry = scratch[16];
        __syncthreads();
    }
    if (tid < 64) {
        if (few_own) {
            int keys[kKeysPerLane];
#pragma unroll
            for (int u = 1; u < kKeysPerLane; ++u) keys[u] = -1;
            keys[0] = p0 + tid < p1 ? fused_key<true>(own, nbins - 1, unused) : -1;
            scatter_chunk(bef, keys, p0, p1 - p0, nbins, nbits, num_out, row_id_map, sorted_indices, dest, p0);
        } else {
            wave_scatter(bef, idx, p0, p1, nbins, nbits, num_out, row_id_map, sorted_indices, dest);
        }
    }
    __syncthreads();
    if (!mover) return;
    scatter_row(v, src, permuted, dest + local_row * topk, topk, num_out, lane, lanes, vecs_per_row);
}

// Stable scatter and row movement in one launch, behind the histogram launch of the multi-block sort (any bin
// count, any number of positions).  A workgroup ranks its own flat positions.  For the segment its first
// position lies in it needs, per bin, the first row of that (segment, bin):
//   SCANNED = true:  table[s][bin] holds it (sort_scan_kernel has run);
//   SCANNED = false: table[s][bin] is still the segment's histogram, and the workgroup adds up, per bin, all
//                    segments (-> first row of the bin, after a scan over the bins) and the segments in front of
//                    its own; the host picks this form while the table is small enough to read per workgroup.
// To that it adds the keys of its segment in front of its first position, counted by all threads with LDS adds,
// and its first wavefront runs the same stable scatter as sort_scatter_kernel over the workgroup's positions,
// piece by piece where they cross a segment boundary.  The rows reach the copying threads through LDS.
template <typename IdxT, typename VecT, bool SCANNED>
__global__ __launch_bounds__(1024) void permute_scatter_rows_kernel(
    const VecT *__restrict__ tokens, VecT *__restrict__ permuted, const IdxT *__restrict__ idx, int n, int seg, int nseg,
    int nbins, int nbits, const int *__restrict__ table, int num_out, int32_t *__restrict__ row_id_map,
    int32_t *__restrict__ sorted_indices, int64_t *__restrict__ tokens_per_expert, int tpe_n, int num_tokens, int topk,
    int vecs_per_row, int lanes) {
    extern __shared__ int lds[];               // cnt[nbins], first[nbins], pre[nbins], scratch[32], dest[rows_per_block * topk]
    int *cnt = lds;
    int *first = lds + nbins;
    int *pre = first + nbins;
    int *scratch = pre + nbins;
    int *dest = scratch + 32;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int rows_per_block = nthreads / lanes;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int p0 = t0 * topk, p1 = t1 * topk;  // this workgroup's flat positions
    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    const bool mover = t < num_tokens;
    const VecT *src = tokens + static_cast<int64_t>(mover ? t : 0) * vecs_per_row;
    const int s0 = p0 / seg;
    const int seg_begin = s0 * seg;

    for (int e = tid; e < 3 * nbins; e += nthreads) lds[e] = 0;
    constexpr int KU = 4;
    IdxT raw[KU];
#pragma unroll
    for (int u = 0; u < KU; ++u) raw[u] = idx[min(seg_begin + u * nthreads + tid, n - 1)];
    __syncthreads();
    for (int c = seg_begin; c < p0; c += KU * nthreads) {
        if (c != seg_begin) {
#pragma unroll
            for (int u = 0; u < KU; ++u) raw[u] = idx[min(c + u * nthreads + tid, n - 1)];
        }
#pragma unroll
        for (int u = 0; u < KU; ++u) {
            long long key = static_cast<long long>(raw[u]);
            key = key < 0 ? 0 : key;
            key = key >= nbins ? nbins - 1 : key;
            if (c + u * nthreads + tid < p0) atomicAdd(&cnt[static_cast<int>(key)], 1);
        }
    }
    if constexpr (!SCANNED) {
        for (int i = tid; i < nseg * nbins; i += nthreads) {
            const int sg = i / nbins;
            const int e = i - sg * nbins;
            const int c = table[i];
            atomicAdd(&first[e], c);                 // per-bin total for now
            if (sg < s0) atomicAdd(&pre[e], c);
        }
    }
    // The first vectors of this thread's row (clamped, unconditional loads), requested after the last load the
    // counting needs - loads retire in order, so an earlier request would stall the counting until the rows are
    // in - and in flight during the scan and the ranking below.
    VecT v[8];
    prefetch_row(v, src, lane, lanes, vecs_per_row);
    if constexpr (!SCANNED) {
        __syncthreads();
        int carry = 0;
        for (int e0 = 0; e0 < nbins; e0 += nthreads) {
            const int bin = e0 + tid;
            const int total = bin < nbins ? first[bin] : 0;
            const int start = carry + block_exclusive_scan(total, scratch);
            if (bin < nbins) {
                first[bin] = start;
                if (blockIdx.x == 0 && tokens_per_expert != nullptr && bin < tpe_n) tokens_per_expert[bin] = total;
            }
            if (tid == nthreads - 1) scratch[16] = start + total;
            __syncthreads();
            carry = scratch[16];
            __syncthreads();
        }
    } else {
        __syncthreads();
    }
    if (tid < 64) {
        int begin = p0;
        for (int sgm = s0; begin < p1; ++sgm) {
            const int end = min(p1, (sgm + 1) * seg);
            for (int e = tid; e < nbins; e += 64) {
                if constexpr (SCANNED) {
                    cnt[e] = table[static_cast<int64_t>(sgm) * nbins + e] + (sgm == s0 ? cnt[e] : 0);
                } else {
                    if (sgm != s0) pre[e] += table[static_cast<int64_t>(sgm - 1) * nbins + e];
                    cnt[e] = first[e] + pre[e] + (sgm == s0 ? cnt[e] : 0);
                }
            }
            __builtin_amdgcn_wave_barrier();
            wave_scatter(cnt, idx, begin, end, nbins, nbits, num_out, row_id_map, sorted_indices, dest + (begin - p0));
            __builtin_amdgcn_wave_barrier();
            begin = end;
        }
    }
    __syncthreads();
    if (!mover) return;
    scatter_row(v, src, permuted, dest + local_row * topk, topk, num_out, lane, lanes, vecs_per_row);
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

// Permuted rows [first, num_rows) that no map entry leads to (the caller's row count exceeds the number of set
// entries) are written as zeros, shared out over the workgroups of the launch.
template <typename VecT>
__device__ __forceinline__ void zero_unmapped_rows(VecT *__restrict__ permuted, int first, int num_rows, int vecs_per_row) {
    for (int r = first + blockIdx.x; r < num_rows; r += gridDim.x) {
        VecT *dst = permuted + static_cast<int64_t>(r) * vecs_per_row;
        for (int c = threadIdx.x; c < vecs_per_row; c += blockDim.x) dst[c] = VecT{};
    }
}

// The same for the sort-based path, which marks those rows in sorted_flat: one workgroup per 4 rows.
template <typename VecT>
__global__ __launch_bounds__(256) void zero_marked_rows_kernel(const int32_t *__restrict__ sorted_flat, int num_rows,
                                                               int vecs_per_row, VecT *__restrict__ permuted) {
    const int r = blockIdx.x * 4 + (threadIdx.x >> 6);
    if (r >= num_rows || sorted_flat[r] >= 0) return;
    VecT *dst = permuted + static_cast<int64_t>(r) * vecs_per_row;
    for (int c = threadIdx.x & 63; c < vecs_per_row; c += 64) dst[c] = VecT{};
}

// Mask mode, rows laid out and moved in one launch (no drop-and-pad, experts a power of two up to 16, so that
// a 16-byte vector of the map holds whole tokens and byte position b of a vector always belongs to expert
// b % E; maps up to kFusedMapMax entries).  Same scheme as permute_fused_kernel: every workgroup counts, per
// expert column, the set entries of the tokens in front of its own and of the others into 256 LDS counter
// columns (the map comes from L2), folds them into the next free row of every expert as seen from its first
// token, ranks its own entries in order with wavefront ballots, and copies its tokens' rows, whose first
// vectors were requested before the counting.  Same outputs as the sort-based path.
constexpr int kFusedMapMax = 1 << 17;

__device__ __forceinline__ void mask_vector_add(int *table, const v16 &w, int first, int live, int split, int E) {
    const int col = threadIdx.x & 255;
#pragma unroll
    for (int b = 0; b < 16; ++b) {
        const unsigned byte = (w[b >> 2] >> (8 * (b & 3))) & 0xffu;
        const int row = (first + b < split ? 0 : 16) + (b & (E - 1));
        __hip_atomic_fetch_add(table + row * 256 + col, static_cast<int>(min(byte, 1u)) & live, __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_WORKGROUP);
    }
}

__global__ __launch_bounds__(1024) void routing_map_fused_kernel(
    const v16 *__restrict__ tokens, v16 *__restrict__ permuted, const unsigned char *__restrict__ map, int num_tokens,
    int E, int num_rows, int32_t *__restrict__ row_id_map, int32_t *__restrict__ sorted_flat,
    int64_t *__restrict__ tokens_per_expert, int vecs_per_row, int lanes) {
    extern __shared__ int lds[];     // table[32][256], sums[32], base[16], rows[rows_per_block * E]
    int *table = lds;
    int *sums = lds + 32 * 256;
    int *base = sums + 32;
    int *rows = base + 16;
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int rows_per_block = nthreads / lanes;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int n = num_tokens * E;
    const int split = t0 * E;                   // flat entries in front of this workgroup
    const int own = (t1 - t0) * E;              // this workgroup's entries
    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    const bool mover = tokens != nullptr && t < num_tokens;
    const v16 *src = tokens + static_cast<int64_t>(mover ? t : 0) * vecs_per_row;

    if (tid < 256) {
#pragma unroll
        for (int r = 0; r < 32; ++r) table[r * 256 + tid] = 0;
    }
    const int nvec = n / 16;
    const v16 *mv = reinterpret_cast<const v16 *>(map);
    v16 w = {0u, 0u, 0u, 0u};
    if (nvec > 0) w = mv[min(tid, nvec - 1)];
    unsigned char own0 = 0;
    if (tid < 64) own0 = map[min(split + tid, n - 1)];
    v16 v[8];                                   // the first vectors of this thread's row (clamped, unconditional)
    if (tokens != nullptr) {
        prefetch_row(v, src, lane, lanes, vecs_per_row);
    }
    __syncthreads();
    mask_vector_add(table, w, tid * 16, tid < nvec ? 1 : 0, split, E);
    for (int vi = tid + nthreads; vi < nvec; vi += nthreads) mask_vector_add(table, mv[vi], vi * 16, 1, split, E);
    for (int i = nvec * 16 + tid; i < n; i += nthreads)     // entries past the last whole vector (small maps only)
        __hip_atomic_fetch_add(table + ((i < split ? 0 : 16) + (i & (E - 1))) * 256 + (tid & 255), map[i] != 0 ? 1 : 0,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_WORKGROUP);
    __syncthreads();
    fused_fold<16>(table, sums);
    __syncthreads();
    if (tid < E) {
        int first = 0;
        for (int e = 0; e < tid; ++e) first += sums[e] + sums[16 + e];
        base[tid] = first + sums[tid];
        if (blockIdx.x == 0 && tokens_per_expert != nullptr) tokens_per_expert[tid] = sums[tid] + sums[16 + tid];
    }
    {   // rows that nothing maps to (only if the caller's row count exceeds the set entries)
        int nnz = 0;
        for (int e = 0; e < E; ++e) nnz += sums[e] + sums[16 + e];
        if (blockIdx.x == 0)
            for (int r = nnz + tid; r < num_rows; r += nthreads) sorted_flat[r] = -1;
        if (tokens != nullptr) zero_unmapped_rows(permuted, nnz, num_rows, vecs_per_row);
    }
    __syncthreads();
    // Own entries in flat order, 64 at a time: lane l always sees expert l % E (E divides 64).  An entry's row
    // is its expert's next free row plus the set entries of the same expert on lower lanes.
    if (tid < 64) {
        const int e = tid & (E - 1);
        unsigned long long same = 1ull << e;
        for (int sft = E; sft < 64; sft <<= 1) same |= same << sft;
        int next = base[e];
        for (int q0 = 0; q0 < own; q0 += 64) {
            const int q = q0 + tid;
            const bool valid = q < own;
            const unsigned char byte = q0 == 0 ? own0 : (valid ? map[split + q] : 0);
            const bool set = valid && byte != 0;
            const unsigned long long mine = __ballot(set) & same;
            const int rank = next + lanes_below(mine);
            int row = 0x7fffffff;                // unset or dropped: an id no row count reaches
            if (set && rank < num_rows) {
                row = rank;
                sorted_flat[row] = split + q;
            }
            if (valid) {
                row_id_map[split + q] = row;
                rows[q] = row;
            }
            next += __popcll(mine);
        }
    }
    __syncthreads();
    if (!mover) return;
    scatter_row(v, src, permuted, rows + local_row * E, E, num_rows, lane, lanes, vecs_per_row);
}

// Mask mode for any expert count (no drop-and-pad), two launches.  The map is cut into chunks of `chunk` tokens
// (a power of two): routing_map_hist_kernel counts the set entries per (chunk, expert); every workgroup of
// routing_map_ranked_kernel then owns a few tokens of one chunk, adds up the table (per expert: all chunks ->
// first row of the expert after a scan over the experts; the chunks in front of its own), counts its chunk's
// set entries in front of its first token, walks its own tokens in order, one thread per expert column, and
// copies its tokens' rows, whose first vectors were requested before the counting.  Same outputs as the
// sort-based path.
__global__ __launch_bounds__(256) void routing_map_hist_kernel(const unsigned char *__restrict__ map, int num_tokens, int E,
                                                               int chunk, int *__restrict__ hist) {
    extern __shared__ int lds[];   // cnt[E]
    const int tid = threadIdx.x;
    for (int e = tid; e < E; e += 256) lds[e] = 0;
    __syncthreads();
    const int begin = blockIdx.x * chunk * E;
    const int end = min(num_tokens, (static_cast<int>(blockIdx.x) + 1) * chunk) * E;
    for (int i = begin + tid; i < end; i += 256)
        if (map[i] != 0) atomicAdd(&lds[i % E], 1);
    __syncthreads();
    for (int e = tid; e < E; e += 256) hist[blockIdx.x * E + e] = lds[e];
}

template <typename VecT>
__global__ __launch_bounds__(1024) void routing_map_ranked_kernel(
    const VecT *__restrict__ tokens, VecT *__restrict__ permuted, const unsigned char *__restrict__ map, int num_tokens,
    int E, int chunk, int nchunk, const int *__restrict__ hist, int num_rows, int32_t *__restrict__ row_id_map,
    int32_t *__restrict__ sorted_flat, int64_t *__restrict__ tokens_per_expert, int vecs_per_row, int lanes,
    int rows_per_block) {
    // first[E], pre[E], cnt[E], scratch[32], ntok[rows_per_block], list[rows_per_block * E] (movers only),
    // own[rows_per_block * E] bytes
    extern __shared__ int lds[];
    int *first = lds;
    int *pre = first + E;
    int *cnt = pre + E;
    int *scratch = cnt + E;
    int *ntok = scratch + 32;
    int *list = ntok + rows_per_block;
    unsigned char *own = reinterpret_cast<unsigned char *>(list + (tokens != nullptr ? rows_per_block * E : 0));
    const int tid = threadIdx.x;
    const int nthreads = blockDim.x;
    const int t0 = blockIdx.x * rows_per_block;
    const int t1 = min(t0 + rows_per_block, num_tokens);
    const int c0 = t0 / chunk;                  // rows_per_block divides chunk: all own tokens lie in chunk c0
    const int split = t0 * E;                   // first own flat entry
    const int own_n = (t1 - t0) * E;
    const int local_row = tid / lanes;
    const int lane = tid % lanes;
    const int t = t0 + local_row;
    const bool mover = tokens != nullptr && local_row < rows_per_block && t < num_tokens;
    const VecT *src = tokens + static_cast<int64_t>(mover ? t : 0) * vecs_per_row;

    for (int e = tid; e < 3 * E + 32 + rows_per_block; e += nthreads) lds[e] = 0;
    for (int q = tid; q < own_n; q += nthreads) own[q] = map[split + q];
    __syncthreads();
    for (int i = c0 * chunk * E + tid; i < split; i += nthreads)       // this chunk's entries in front of the own ones
        if (map[i] != 0) atomicAdd(&cnt[i % E], 1);
    for (int i = tid; i < nchunk * E; i += nthreads) {
        const int c = i / E;
        const int count = hist[i];
        atomicAdd(&first[i - c * E], count);    // per-expert total for now
        if (c < c0) atomicAdd(&pre[i - c * E], count);
    }
    // The first vectors of this thread's row (clamped, unconditional loads), requested after the last load the
    // ranking needs - loads retire in order, so an earlier request would stall the counting above until the rows
    // are in - and in flight during the scan and the ranking below, which work out of LDS.
    VecT v[8];
    if (tokens != nullptr) {
        prefetch_row(v, src, lane, lanes, vecs_per_row);
    }
    __syncthreads();
    int carry = 0;
    for (int e0 = 0; e0 < E; e0 += nthreads) {
        const int e = e0 + tid;
        const int total = e < E ? first[e] : 0;
        const int start = carry + block_exclusive_scan(total, scratch);
        if (e < E) {
            first[e] = start;
            if (blockIdx.x == 0 && tokens_per_expert != nullptr) tokens_per_expert[e] = total;
        }
        if (tid == nthreads - 1) scratch[16] = start + total;
        __syncthreads();
        carry = scratch[16];
        __syncthreads();
    }
    if (blockIdx.x == 0)   // rows that nothing maps to (only if the caller's row count exceeds the set entries)
        for (int r = carry + tid; r < num_rows; r += nthreads) sorted_flat[r] = -1;
    if (tokens != nullptr) zero_unmapped_rows(permuted, carry, num_rows, vecs_per_row);
    for (int e = tid; e < E; e += nthreads) {
        int next = first[e] + pre[e] + cnt[e];
        for (int lt = 0; lt < t1 - t0; ++lt) {
            const int q = lt * E + e;
            int row = 0x7fffffff;               // unset or dropped: an id no row count reaches
            if (own[q] != 0) {
                if (next < num_rows) {
                    row = next;
                    sorted_flat[row] = split + q;
                    if (tokens != nullptr) list[lt * E + atomicAdd(&ntok[lt], 1)] = row;
                }
                ++next;
            }
            row_id_map[split + q] = row;
        }
    }
    __syncthreads();
    if (!mover) return;
    scatter_row(v, src, permuted, list + local_row * E, ntok[local_row], num_rows, lane, lanes, vecs_per_row);
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
    // 1024 positions per segment; beyond 128 segments the segments grow (up to 4096 positions) before their number
    // does: the scan over the segments is a serial loop per bin, while a scatter workgroup counts at most one
    // segment's keys in front of its own positions
    int64_t seg = 1024;
    if (ceil_div(n, seg) > 128) seg = (ceil_div(n, 128) + 63) / 64 * 64;
    if (seg > 4096) seg = 4096;
    if (ceil_div(n, seg) > kMaxSegments) seg = (ceil_div(n, kMaxSegments) + 63) / 64 * 64;
    p.seg = static_cast<int>(seg);
    p.nseg = static_cast<int>(ceil_div(n, seg));
    return p;
}

// Histogram launch of the multi-block sort (table[s][bin] = keys of `bin` in segment s) and, with `scan`, the scan
// launch behind it (table[s][bin] = first row of `bin` for segment s).
template <typename IdxT>
int launch_sort_offsets(hipStream_t stream, const SortPlan &p, const IdxT *idx, int64_t *tpe, int tpe_n, int *table,
                        bool scan = true) {
    hipLaunchKernelGGL(sort_hist_kernel<IdxT>, dim3(p.nseg), dim3(kHistThreads), static_cast<size_t>(p.nbins) * sizeof(int),
                       stream, idx, p.n, p.seg, p.nseg, p.nbins, p.nbits, table);
    MS_CHECK_LAUNCH("sort_hist_kernel");
    if (!scan) return MS_OK;
    hipLaunchKernelGGL(sort_scan_kernel, dim3(1), dim3(1024), 0, stream, table, p.nseg, p.nbins, tpe, tpe_n);
    MS_CHECK_LAUNCH("sort_scan_kernel");
    return MS_OK;
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
    if (int rc = launch_sort_offsets(stream, p, idx, tpe, tpe_n, table)) return rc;
    const int blocks = static_cast<int>(ceil_div(p.nseg, kHistWavesPerBlock));
    const size_t lds = static_cast<size_t>(kHistWavesPerBlock) * p.nbins * sizeof(int);
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
    // Fat workgroups repeat the counting less often; keep at least one workgroup per compute unit, and the
    // workgroup's flat positions within what its LDS hand-over holds.
    int threads = 1024;
    while (threads > 256 && (ceil_div(T, threads / rl.lanes) < 256 || (threads / rl.lanes) * k > kFusedMaxLocal))
        threads >>= 1;
    const int rows_per_block = threads / rl.lanes;
    const size_t local = static_cast<size_t>(rows_per_block) * k;
    if (local > static_cast<size_t>(kFusedMaxLocal)) return -1;   // very short rows with a large top-k: two launches
    const dim3 grid(static_cast<unsigned>(ceil_div(T, rows_per_block)));
#define MS_FUSED_ARGS                                                                                                  \
    static_cast<const VecT *>(tokens), static_cast<VecT *>(permuted), idx, p.n, p.nbins, p.nbits, num_out, row_id_map, \
        sorted_indices, tpe, tpe_n, static_cast<int>(T), static_cast<int>(k), static_cast<int>(vecs), rl.lanes
    if (p.nbins > kFusedMaxBins) {
        const size_t lds = (static_cast<size_t>(2) * p.nbins + 32 + local) * sizeof(int);
        hipLaunchKernelGGL((permute_fused_bins_kernel<IdxT, VecT>), grid, dim3(threads), lds, stream, MS_FUSED_ARGS);
    } else if (p.nbins <= 8) {
        const size_t lds = (static_cast<size_t>(16) * 256 + 16 + 8 + local) * sizeof(int);
        hipLaunchKernelGGL((permute_fused_kernel<IdxT, VecT, 8>), grid, dim3(threads), lds, stream, MS_FUSED_ARGS);
    } else {
        const size_t lds = (static_cast<size_t>(32) * 256 + 32 + 16 + local) * sizeof(int);
        hipLaunchKernelGGL((permute_fused_kernel<IdxT, VecT, 16>), grid, dim3(threads), lds, stream, MS_FUSED_ARGS);
    }
#undef MS_FUSED_ARGS
    MS_CHECK_LAUNCH("permute_fused_kernel");
    return MS_OK;
}

// Histogram, scan, then scatter + row movement in one launch.  Returns -1 when a workgroup's positions do not
// fit the LDS hand-over (very short rows with a large top-k).
template <typename IdxT, typename VecT>
int launch_permute_scatter_rows(hipStream_t stream, const SortPlan &p, const void *tokens, void *permuted, const IdxT *idx,
                                int num_out, int32_t *row_id_map, int32_t *sorted_indices, int64_t *tpe, int tpe_n,
                                int64_t T, int64_t k, int64_t row_bytes, int *table) {
    const int64_t vecs = row_bytes / sizeof(VecT);
    const RowLayout rl = row_layout(vecs);
    int threads = 1024;
    while (threads > 256 && (ceil_div(T, threads / rl.lanes) < 256 || (threads / rl.lanes) * k > kFusedMaxLocal))
        threads >>= 1;
    const int rows_per_block = threads / rl.lanes;
    const size_t local = static_cast<size_t>(rows_per_block) * k;
    if (local > static_cast<size_t>(kFusedMaxLocal)) return -1;
    // a small table is summed by every scatter workgroup itself; a large one gets its own scan launch
    const bool scan_launch = static_cast<int64_t>(p.nseg) * p.nbins > kScanInKernelMax;
    if (int rc = launch_sort_offsets(stream, p, idx, tpe, tpe_n, table, scan_launch)) return rc;
    const size_t lds = (static_cast<size_t>(3) * p.nbins + 32 + local) * sizeof(int);
    const dim3 grid(static_cast<unsigned>(ceil_div(T, rows_per_block)));
#define MS_SR_ARGS                                                                                                    \
    static_cast<const VecT *>(tokens), static_cast<VecT *>(permuted), idx, p.n, p.seg, p.nseg, p.nbins, p.nbits, table, \
        num_out, row_id_map, sorted_indices, tpe, tpe_n, static_cast<int>(T), static_cast<int>(k),                     \
        static_cast<int>(vecs), rl.lanes
    if (scan_launch)
        hipLaunchKernelGGL((permute_scatter_rows_kernel<IdxT, VecT, true>), grid, dim3(threads), lds, stream, MS_SR_ARGS);
    else
        hipLaunchKernelGGL((permute_scatter_rows_kernel<IdxT, VecT, false>), grid, dim3(threads), lds, stream, MS_SR_ARGS);
#undef MS_SR_ARGS
    MS_CHECK_LAUNCH("permute_scatter_rows_kernel");
    return MS_OK;
}

template <typename IdxT>
int permute_scatter_rows_dispatch(hipStream_t stream, const SortPlan &p, const void *tokens, void *permuted,
                                  const IdxT *idx, int num_out, int32_t *row_id_map, int32_t *sorted_indices, int64_t *tpe,
                                  int tpe_n, int64_t T, int64_t k, int64_t row_bytes, int dtype, int *table) {
    if (row_bytes % 16 == 0 && aligned16(tokens) && aligned16(permuted))
        return launch_permute_scatter_rows<IdxT, v16>(stream, p, tokens, permuted, idx, num_out, row_id_map,
                                                      sorted_indices, tpe, tpe_n, T, k, row_bytes, table);
    if (dtype == MS_FP32)
        return launch_permute_scatter_rows<IdxT, uint32_t>(stream, p, tokens, permuted, idx, num_out, row_id_map,
                                                           sorted_indices, tpe, tpe_n, T, k, row_bytes, table);
    return launch_permute_scatter_rows<IdxT, uint16_t>(stream, p, tokens, permuted, idx, num_out, row_id_map,
                                                       sorted_indices, tpe, tpe_n, T, k, row_bytes, table);
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

// PT: the probabilities' own type (the tokens' type, or fp32 beside 16-bit tokens)
template <typename DT, typename PT>
int launch_gather_combine(hipStream_t stream, const void *rows, const int32_t *map, const void *probs, void *out,
                          int64_t T, int64_t k, int64_t H, int64_t num_rows) {
    using S = typename DT::storage;
    using PS = typename PT::storage;
    constexpr int VEC = 16 / sizeof(S);
    const bool vec_ok = (H % VEC == 0) && aligned16(rows) && aligned16(out);
    const int64_t vecs = vec_ok ? H / VEC : H;
    const RowLayout rl = row_layout(vecs);
    const unsigned blocks = static_cast<unsigned>(ceil_div(T, rl.rows_per_block));
#define MS_GC_ARGS                                                                                                  \
    static_cast<const S *>(rows), map, static_cast<const PS *>(probs), static_cast<S *>(out), static_cast<int>(T),  \
        static_cast<int>(k), static_cast<int>(H), static_cast<int>(num_rows), rl.lanes
    // many slots per token, or a map most of whose slots lead nowhere (the routing-map form has one slot per expert
    // and only top-k of them set): list the valid ones first.  With at most two valid slots per token on average the
    // listed rows are read like a top-2 map's, four vectors per slot in flight (measured on the 8-expert top-2 mask
    // with buffers that do not fit the last-level cache: 26.0 -> 21 us; with all slots tested in place only the valid
    // quarter of the eight-slot batch has loads in flight).
    const bool sparse = k > 2 && 2 * num_rows <= T * k;
    const bool compact = (k > 8 || sparse) && rl.rows_per_block * k <= kCompactMaxLocal;
    const bool pairs = compact && num_rows <= 2 * T;
    const size_t lds = compact ? static_cast<size_t>(2) * rl.rows_per_block * k * sizeof(int) : 0;
    if (!vec_ok && compact) {
        hipLaunchKernelGGL((gather_combine_kernel<DT, PT, 1, 8, 2, true>), dim3(blocks), dim3(256), lds, stream, MS_GC_ARGS);
    } else if (!vec_ok) {
        hipLaunchKernelGGL((gather_combine_kernel<DT, PT, 1, 8, 2, false>), dim3(blocks), dim3(256), 0, stream, MS_GC_ARGS);
    } else if (pairs) {
        hipLaunchKernelGGL((gather_combine_kernel<DT, PT, VEC, 2, 4, true>), dim3(blocks), dim3(256), lds, stream, MS_GC_ARGS);
    } else if (compact) {
        hipLaunchKernelGGL((gather_combine_kernel<DT, PT, VEC, 8, 2, true>), dim3(blocks), dim3(256), lds, stream, MS_GC_ARGS);
    } else if (k <= 2) {
        hipLaunchKernelGGL((gather_combine_kernel<DT, PT, VEC, 2, 4, false>), dim3(blocks), dim3(256), 0, stream, MS_GC_ARGS);
    } else {
        hipLaunchKernelGGL((gather_combine_kernel<DT, PT, VEC, 8, 2, false>), dim3(blocks), dim3(256), 0, stream, MS_GC_ARGS);
    }
#undef MS_GC_ARGS
    MS_CHECK_LAUNCH("gather_combine_kernel");
    return MS_OK;
}

template <typename DT, typename PT>
int launch_unpermute_grad(hipStream_t stream, const void *permuted, const void *gy, const int32_t *map,
                          const void *probs, void *gperm, void *gprobs, int64_t T, int64_t k, int64_t H,
                          int64_t num_rows) {
    using S = typename DT::storage;
    using PS = typename PT::storage;
    constexpr int VEC = 16 / sizeof(S);
    const bool vec_ok = (H % VEC == 0) && aligned16(gy) && aligned16(gperm) && (permuted == nullptr || aligned16(permuted));
    const int64_t vecs = vec_ok ? H / VEC : H;
    const RowLayout rl = row_layout(vecs);
    const dim3 grid(static_cast<unsigned>(ceil_div(T, rl.rows_per_block)));
#define MS_UG_ARGS                                                                                                   \
    static_cast<const S *>(permuted), static_cast<const S *>(gy), map, static_cast<const PS *>(probs),               \
        static_cast<S *>(gperm), static_cast<PS *>(gprobs), static_cast<int>(T), static_cast<int>(k),                \
        static_cast<int>(H), static_cast<int>(num_rows), rl.lanes
    // (the same choice as the gather's: list the valid slots of a many-slot or mostly empty map first)
    const bool sparse = k > 2 && 2 * num_rows <= T * k;
    const bool compact = (k > 8 || sparse) && rl.rows_per_block * k <= kCompactMaxLocal;
    const bool pairs = compact && num_rows <= 2 * T;
    const size_t lds = compact ? static_cast<size_t>(3) * rl.rows_per_block * k * sizeof(int) : 0;
    if (!vec_ok && compact) {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, PT, 1, 4, 4, true>), grid, dim3(256), lds, stream, MS_UG_ARGS);
    } else if (!vec_ok) {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, PT, 1, 4, 4, false>), grid, dim3(256), 0, stream, MS_UG_ARGS);
    } else if (pairs) {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, PT, VEC, 2, 4, true>), grid, dim3(256), lds, stream, MS_UG_ARGS);
    } else if (compact) {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, PT, VEC, 4, 2, true>), grid, dim3(256), lds, stream, MS_UG_ARGS);
    } else if (k <= 2) {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, PT, VEC, 2, 4, false>), grid, dim3(256), 0, stream, MS_UG_ARGS);
    } else {
        hipLaunchKernelGGL((unpermute_grad_kernel<DT, PT, VEC, 4, 2, false>), grid, dim3(256), 0, stream, MS_UG_ARGS);
    }
#undef MS_UG_ARGS
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
    // inputs one workgroup can count: sort and row scatter in one launch
    if (p.small && num_out > 0) {
        const int fused =
            index_dtype == MS_INT32
                ? permute_fused_dispatch(stream, p, tokens, permuted, static_cast<const int32_t *>(indices), (int)num_out,
                                         row_id_map, sorted_indices, tokens_per_expert, (int)experts_hint, T, k, row_bytes,
                                         dtype)
                : permute_fused_dispatch(stream, p, tokens, permuted, static_cast<const int64_t *>(indices), (int)num_out,
                                         row_id_map, sorted_indices, tokens_per_expert, (int)experts_hint, T, k, row_bytes,
                                         dtype);
        if (fused != -1) return fused;
    }
    // otherwise: histogram and scan launches, then scatter and row movement in one launch
    if (num_out > 0 && !p.small) {
        int *table = static_cast<int *>(workspace);
        const int three =
            index_dtype == MS_INT32
                ? permute_scatter_rows_dispatch(stream, p, tokens, permuted, static_cast<const int32_t *>(indices),
                                                (int)num_out, row_id_map, sorted_indices, tokens_per_expert,
                                                (int)experts_hint, T, k, row_bytes, dtype, table)
                : permute_scatter_rows_dispatch(stream, p, tokens, permuted, static_cast<const int64_t *>(indices),
                                                (int)num_out, row_id_map, sorted_indices, tokens_per_expert,
                                                (int)experts_hint, T, k, row_bytes, dtype, table);
        if (three != -1) return three;
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
                                      const void *probs, int probs_dtype, int64_t T, int64_t k, int64_t H, int dtype,
                                      int64_t num_rows, void *out) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_common("ms_moe_token_unpermute", T, k, H, dtype)) return rc;
    MS_REQUIRE(probs == nullptr || probs_dtype == dtype || probs_dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "ms_moe_token_unpermute: probs dtype %d must be the tokens' dtype (%d) or fp32", probs_dtype, dtype);
    const bool p32 = probs != nullptr && probs_dtype == MS_FP32;
    MS_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31), MS_ERR_INVALID_ARGUMENT, "ms_moe_token_unpermute: bad num_permuted_rows");
    if (T == 0) return MS_OK;
    MS_REQUIRE((permuted || num_rows == 0) && row_id_map && out, MS_ERR_INVALID_ARGUMENT,
               "ms_moe_token_unpermute: NULL tensor pointer");
    switch (dtype) {
        case MS_BF16:
            return p32 ? launch_gather_combine<BF16, FP32>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows)
                       : launch_gather_combine<BF16, BF16>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows);
        case MS_FP16:
            return p32 ? launch_gather_combine<FP16, FP32>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows)
                       : launch_gather_combine<FP16, FP16>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows);
        default: return launch_gather_combine<FP32, FP32>(stream, permuted, row_id_map, probs, out, T, k, H, num_rows);
    }
}

extern "C" int ms_moe_token_permute_grad(ms_stream_t stream, const void *grad_permuted, const int32_t *row_id_map,
                                         int64_t T, int64_t k, int64_t H, int dtype, int64_t num_rows,
                                         void *grad_tokens) {
    // The backward of a row gather is the unweighted top-k gather-sum.
    return ms_moe_token_unpermute(stream, grad_permuted, row_id_map, nullptr, dtype, T, k, H, dtype, num_rows, grad_tokens);
}

extern "C" int ms_moe_token_unpermute_grad(ms_stream_t stream_, const void *permuted, const void *grad_out,
                                           const int32_t *row_id_map, const void *probs, int probs_dtype, int64_t T,
                                           int64_t k, int64_t H, int dtype, int64_t num_rows, void *grad_permuted,
                                           void *grad_probs) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (int rc = check_common("ms_moe_token_unpermute_grad", T, k, H, dtype)) return rc;
    MS_REQUIRE(probs == nullptr || probs_dtype == dtype || probs_dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "ms_moe_token_unpermute_grad: probs dtype %d must be the tokens' dtype (%d) or fp32", probs_dtype, dtype);
    const bool p32 = probs != nullptr && probs_dtype == MS_FP32;
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
#define MS_UG_CALL(DT_, PT_) \
    launch_unpermute_grad<DT_, PT_>(stream, permuted, grad_out, row_id_map, probs, grad_permuted, grad_probs, T, k, H, num_rows)
        case MS_BF16: return p32 ? MS_UG_CALL(BF16, FP32) : MS_UG_CALL(BF16, BF16);
        case MS_FP16: return p32 ? MS_UG_CALL(FP16, FP32) : MS_UG_CALL(FP16, FP16);
        default: return MS_UG_CALL(FP32, FP32);
#undef MS_UG_CALL
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
template <typename VecT>
void launch_routing_map_ranked(hipStream_t stream, const void *tokens, void *permuted, const unsigned char *map, int64_t T,
                               int64_t E, int chunk, int nchunk, const int *hist, int64_t num_rows, int32_t *row_id_map,
                               int32_t *sorted_flat, int64_t *tpe, int64_t vecs, int lanes, int threads,
                               int rows_per_block) {
    const size_t ints = 3 * static_cast<size_t>(E) + 32 + rows_per_block +
                        (tokens != nullptr ? static_cast<size_t>(rows_per_block) * E : 0);
    const size_t lds = ints * sizeof(int) + ((static_cast<size_t>(rows_per_block) * E + 3) & ~static_cast<size_t>(3));
    hipLaunchKernelGGL((ms::routing_map_ranked_kernel<VecT>), dim3(static_cast<unsigned>(ms::ceil_div(T, rows_per_block))),
                       dim3(threads), lds, stream, static_cast<const VecT *>(tokens), static_cast<VecT *>(permuted), map,
                       static_cast<int>(T), static_cast<int>(E), chunk, nchunk, hist, static_cast<int>(num_rows),
                       row_id_map, sorted_flat, tpe, static_cast<int>(vecs), lanes, rows_per_block);
}

// Mask mode in two launches (chunk histogram, then ranking + row movement).  Returns -1 when the shape does not
// fit (a workgroup's entries beyond what LDS holds, or chunks too large to count per workgroup): the caller
// then takes the sort-based path.
int routing_map_two_launches(hipStream_t stream, const void *tokens, const unsigned char *map, int64_t T, int64_t E,
                             int64_t row_bytes, int dtype, int64_t num_rows, void *permuted, int32_t *row_id_map,
                             int32_t *sorted_flat, int64_t *tpe, int *hist) {
    using namespace ms;
    int lanes = 1, threads = 1024, rows_per_block;
    int64_t vecs = 1;
    int vec_bytes = 16;
    if (tokens != nullptr) {
        if (!(row_bytes % 16 == 0 && aligned16(tokens) && aligned16(permuted))) vec_bytes = dtype == MS_FP32 ? 4 : 2;
        vecs = row_bytes / vec_bytes;
        lanes = row_layout(vecs).lanes;
        while (threads > 256 && (ceil_div(T, threads / lanes) < 256 || (threads / lanes) * E > kFusedMaxLocal)) threads >>= 1;
        rows_per_block = threads / lanes;
        if (static_cast<int64_t>(rows_per_block) * E > kFusedMaxLocal) return -1;
    } else {
        rows_per_block = 1024;
        while (rows_per_block > 1 && rows_per_block * E > 4 * kFusedMaxLocal) rows_per_block >>= 1;
        threads = rows_per_block < 256 ? 256 : rows_per_block;
    }
    int chunk = rows_per_block;
    while (ceil_div(T, chunk) * E > kScanInKernelMax) chunk <<= 1;
    if (static_cast<int64_t>(chunk) * E > (1 << 16)) return -1;
    const int nchunk = static_cast<int>(ceil_div(T, chunk));
    hipLaunchKernelGGL(routing_map_hist_kernel, dim3(nchunk), dim3(256), static_cast<size_t>(E) * sizeof(int), stream, map,
                       static_cast<int>(T), static_cast<int>(E), chunk, hist);
    MS_CHECK_LAUNCH("routing_map_hist_kernel");
    if (vec_bytes == 16)
        launch_routing_map_ranked<v16>(stream, tokens, permuted, map, T, E, chunk, nchunk, hist, num_rows, row_id_map,
                                       sorted_flat, tpe, vecs, lanes, threads, rows_per_block);
    else if (vec_bytes == 4)
        launch_routing_map_ranked<uint32_t>(stream, tokens, permuted, map, T, E, chunk, nchunk, hist, num_rows, row_id_map,
                                            sorted_flat, tpe, vecs, lanes, threads, rows_per_block);
    else
        launch_routing_map_ranked<uint16_t>(stream, tokens, permuted, map, T, E, chunk, nchunk, hist, num_rows, row_id_map,
                                            sorted_flat, tpe, vecs, lanes, threads, rows_per_block);
    MS_CHECK_LAUNCH("routing_map_ranked_kernel");
    return MS_OK;
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
    MS_REQUIRE(routing_map && row_id_map && (sorted_flat || num_rows == 0), MS_ERR_INVALID_ARGUMENT,
               "%s: NULL tensor pointer", fn);
    MS_REQUIRE(tokens == nullptr || permuted != nullptr || num_rows == 0, MS_ERR_INVALID_ARGUMENT, "%s: permuted is NULL", fn);
    // one launch when whole tokens fit a 16-byte vector of the map and rows move as 16-byte vectors
    const int64_t row_bytes_f = H * dtype_size(dtype);
    const bool pow2 = (E & (E - 1)) == 0 && E <= 16;
    if (!drop_and_pad && pow2 && T * E <= kFusedMapMax && aligned16(routing_map) &&
        (tokens == nullptr || (row_bytes_f % 16 == 0 && aligned16(tokens) && aligned16(permuted)))) {
        const int64_t vecs = tokens != nullptr ? row_bytes_f / 16 : 1;
        const int lanes = tokens != nullptr ? row_layout(vecs).lanes : 1;
        // fat workgroups repeat the counting less often; keep one per compute unit, and the own entries within
        // what the LDS hand-over holds
        int threads = 1024;
        while (threads > 256 && (ceil_div(T, threads / lanes) < 256 || (threads / lanes) * E > kFusedMaxLocal)) threads >>= 1;
        const int rows_per_block = threads / lanes;
        if (static_cast<int64_t>(rows_per_block) * E <= kFusedMaxLocal) {
            const size_t lds = (static_cast<size_t>(32) * 256 + 48 + static_cast<size_t>(rows_per_block) * E) * sizeof(int);
            hipLaunchKernelGGL(routing_map_fused_kernel, dim3(static_cast<unsigned>(ceil_div(T, rows_per_block))),
                               dim3(threads), lds, stream, static_cast<const v16 *>(tokens), static_cast<v16 *>(permuted),
                               static_cast<const unsigned char *>(routing_map), static_cast<int>(T), static_cast<int>(E),
                               static_cast<int>(num_rows), row_id_map, sorted_flat, tokens_per_expert,
                               static_cast<int>(vecs), lanes);
            MS_CHECK_LAUNCH("routing_map_fused_kernel");
            return MS_OK;
        }
    }
    const RoutingPlan r = make_routing_plan(T, E, drop_and_pad);
    MS_REQUIRE(workspace != nullptr && workspace_bytes >= r.total, MS_ERR_WORKSPACE_TOO_SMALL, "%s: workspace %zu < %zu bytes",
               fn, workspace_bytes, r.total);
    MS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7u) == 0, MS_ERR_INVALID_ARGUMENT, "%s: workspace must be 8-byte aligned", fn);
    char *ws = static_cast<char *>(workspace);
    if (!drop_and_pad) {
        const int rc = routing_map_two_launches(stream, tokens, static_cast<const unsigned char *>(routing_map), T, E,
                                                row_bytes_f, dtype, num_rows, permuted, row_id_map, sorted_flat,
                                                tokens_per_expert, reinterpret_cast<int *>(ws + r.keys_off));
        if (rc != -1) return rc;
    }
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
    // rows that no entry maps to (never in drop-and-pad mode, which fills every expert's block) are zeroed
    const dim3 zgrid(static_cast<unsigned>(ceil_div(num_rows, 4)));
    if (row_bytes % 16 == 0 && aligned16(tokens) && aligned16(permuted)) {
        if (int rc = launch_permute_rows<v16>(stream, tokens, permuted, row_id_map, T, E, row_bytes, num_rows)) return rc;
        if (!drop_and_pad)
            hipLaunchKernelGGL(zero_marked_rows_kernel<v16>, zgrid, dim3(256), 0, stream, sorted_flat, static_cast<int>(num_rows),
                               static_cast<int>(row_bytes / 16), static_cast<v16 *>(permuted));
    } else if (dtype == MS_FP32) {
        if (int rc = launch_permute_rows<uint32_t>(stream, tokens, permuted, row_id_map, T, E, row_bytes, num_rows)) return rc;
        if (!drop_and_pad)
            hipLaunchKernelGGL(zero_marked_rows_kernel<uint32_t>, zgrid, dim3(256), 0, stream, sorted_flat,
                               static_cast<int>(num_rows), static_cast<int>(row_bytes / 4), static_cast<uint32_t *>(permuted));
    } else {
        if (int rc = launch_permute_rows<uint16_t>(stream, tokens, permuted, row_id_map, T, E, row_bytes, num_rows)) return rc;
        if (!drop_and_pad)
            hipLaunchKernelGGL(zero_marked_rows_kernel<uint16_t>, zgrid, dim3(256), 0, stream, sorted_flat,
                               static_cast<int>(num_rows), static_cast<int>(row_bytes / 2), static_cast<uint16_t *>(permuted));
    }
    if (!drop_and_pad) MS_CHECK_LAUNCH("zero_marked_rows_kernel");
    return MS_OK;
}

extern "C" int ms_moe_routing_map_probs(ms_stream_t stream_, const int32_t *sorted_flat, int64_t num_rows, int64_t E,
                                        const void *probs, int dtype, void *permuted_probs, int64_t *sorted_token_ids) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char *fn = "ms_moe_routing_map_probs";
    MS_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && E >= 1, MS_ERR_INVALID_ARGUMENT, "%s: bad sizes", fn);
    MS_REQUIRE(probs == nullptr || dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "%s: dtype %d is not one of bf16/fp16/fp32", fn, dtype);
    if (num_rows == 0) return MS_OK;   // empty outputs may come as NULL
    MS_REQUIRE((probs == nullptr) == (permuted_probs == nullptr), MS_ERR_INVALID_ARGUMENT,
               "%s: probs and permuted_probs must be given together", fn);
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

// Rows of a permuted-layout matrix that no map entry leads to (marked by a negative entry of sorted_flat) are written
// as zeros; all other rows are left alone.
extern "C" int ms_moe_zero_unmapped_rows(ms_stream_t stream_, const int32_t *sorted_flat, int64_t num_rows, int64_t hidden,
                                         int dtype, void *rows) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    const char *fn = "ms_moe_zero_unmapped_rows";
    MS_REQUIRE(num_rows >= 0 && num_rows < (1ll << 31) && hidden >= 1 && hidden < (1ll << 31), MS_ERR_INVALID_ARGUMENT,
               "%s: bad sizes", fn);
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "%s: dtype %d is not one of bf16/fp16/fp32", fn, dtype);
    if (num_rows == 0) return MS_OK;
    MS_REQUIRE(sorted_flat && rows, MS_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", fn);
    const int64_t row_bytes = hidden * dtype_size(dtype);
    const dim3 zgrid(static_cast<unsigned>(ceil_div(num_rows, 4)));
    if (row_bytes % 16 == 0 && aligned16(rows))
        hipLaunchKernelGGL(zero_marked_rows_kernel<v16>, zgrid, dim3(256), 0, stream, sorted_flat, static_cast<int>(num_rows),
                           static_cast<int>(row_bytes / 16), static_cast<v16 *>(rows));
    else if (dtype == MS_FP32)
        hipLaunchKernelGGL(zero_marked_rows_kernel<uint32_t>, zgrid, dim3(256), 0, stream, sorted_flat,
                           static_cast<int>(num_rows), static_cast<int>(row_bytes / 4), static_cast<uint32_t *>(rows));
    else
        hipLaunchKernelGGL(zero_marked_rows_kernel<uint16_t>, zgrid, dim3(256), 0, stream, sorted_flat,
                           static_cast<int>(num_rows), static_cast<int>(row_bytes / 2), static_cast<uint16_t *>(rows));
    MS_CHECK_LAUNCH("zero_marked_rows_kernel");
    return MS_OK;
}
