// Grouped matmul for gfx950 (MI355X): y[rows of group g] = x[rows of g] @ w[g]
// (split on rows) and y[g] = x[:, red range of g] @ w[red range of g] (split on
// the reduction dim), for forward, dX and dW from one weight storage.
//
// Structure
//   * gmm_schedule_kernel turns the device-resident group_list into a table of
//     per-group tile ranges (no host read of group_list, empty groups emit no
//     row tiles, a trailing pseudo-group zero-fills rows past the last offset;
//     ragged groups may end in a 64- or 128-row tile; per-group weight offsets
//     may come from a list of separately allocated matrices).  In launches with
//     few rounds of tiles those small tiles run last, and with room in the
//     workspace their reduction is cut into parts (fp32 partial sums, added up
//     by gmm_split_reduce_kernel) so that they fill one round instead of
//     running long on a few compute units.
//   * every XCD takes a contiguous eighth of every group's tiles (workgroup b
//     runs on XCD b % 8), in blocks of 4 row tiles x 8 column panels, so the
//     workgroups running together on an XCD share operand panels in its L2;
//     with many small groups whole groups are dealt out to single XCDs instead
//     (one list of entries per XCD).
//   * the fast 16-bit kernels live in gmm_fast.hip.  Here: gmm16_kernel, the
//     16-bit kernel for operands that do not allow 16-byte vector access
//     (element-wise guarded loads, operands that are not contiguous along the
//     reduction dim transposed in registers on their way to LDS), same
//     256x256x64 tile and 4x4 v_mfma_f32_32x32x16 per wavefront; and
//     gmm32_kernel for fp32 inputs (v_mfma_f32_32x32x2f32, 128x128x16 or 64x64x32 tiles).
#include <mutex>
#include <type_traits>

#include "gmm_common.h"

namespace ms {
namespace {

// Per-group element offsets of separately allocated weight matrices, handed to the device as a kernel
// argument (no host-to-device copy, so the call stays asynchronous and capturable).
constexpr int kMaxWeightList = 256;
struct WeightOffsets {
    int64_t v[kMaxWeightList];
};
__global__ void gmm_weight_offsets_kernel(const WeightOffsets o, int n, int64_t *__restrict__ dst) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) dst[i] = o.v[i];
}

// ---- schedule ------------------------------------------------------------------------
// One workgroup turns the device-resident group list into the tile table.  Every thread takes a run of consecutive
// groups; the running quantities (group end offsets, entry numbers, slot numbers, split-workspace blocks) come from
// block-wide prefix scans, so the kernel's time does not grow with the number of groups the way a serial walk does.
//
// Entries.  With split_tails the last row tile of a group may be a smaller one (64 or 128 rows, the smallest that
// holds the remainder), so ragged groups do not pay for a whole extra tile.  Normally a group is one entry and the
// small tile stays in the group's tile range, next to the full tiles of the same column panel, so the weight panel
// it reads is being read by its neighbours at the same time.  When the launch has only a few rounds of tiles (fewer
// than tails_last_below tiles in all) the entries come in two passes: first every group's full tiles, then every
// group's small tile as an entry of its own, so that the last, partly filled round is made of the short tiles.
// With a split workspace (split_records != nullptr) the reduction of those last-scheduled small tiles is cut into up
// to kMaxSplit ranges, as many as keep all parts of all tails within one round of the compute units: a small tile of
// a long reduction otherwise runs as long as most of a full tile while a few compute units work and the others wait.
// Each part is an entry that writes fp32 partial sums; gmm_split_reduce_kernel adds them up.
// Split on the reduction dim: a tile's cost is its group's reduction length, so groups with an above-average length
// come first (they start early on every XCD), the short ones fill in after.
struct ScanItem {
    int n0, slots0;      // entries and slots of the first pass
    int n1, slots1;      // ... of the second pass
    int tails, pairs;    // split tails and their (tail, part) blocks of the split workspace
};
__device__ __forceinline__ ScanItem operator+(const ScanItem &a, const ScanItem &b) {
    return ScanItem{a.n0 + b.n0, a.slots0 + b.slots0, a.n1 + b.n1, a.slots1 + b.slots1, a.tails + b.tails, a.pairs + b.pairs};
}

// Exclusive prefix of v over the 256 threads of the workgroup (thread order) and the total; scratch holds 4 values.
template <typename T, typename Op>
__device__ __forceinline__ T block_scan_exclusive(T v, Op op, T identity, T *scratch, T &total) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    T x = v;                                   // inclusive within the wavefront
#pragma unroll
    for (int d = 1; d < 64; d <<= 1) {
        T y;
        static_assert(sizeof(T) % 4 == 0, "scan items are made of 32-bit words");
        const int *src = reinterpret_cast<const int *>(&x);
        int *dst = reinterpret_cast<int *>(&y);
#pragma unroll
        for (int w = 0; w < static_cast<int>(sizeof(T) / 4); ++w) dst[w] = __shfl_up(src[w], d, 64);
        if (lane >= d) x = op(y, x);
    }
    __syncthreads();                           // scratch may still be read from an earlier scan
    if (lane == 63) scratch[wave] = x;
    __syncthreads();
    T base = identity;
    for (int w = 0; w < wave; ++w) base = op(base, scratch[w]);
    total = op(op(scratch[0], scratch[1]), op(scratch[2], scratch[3]));
    // exclusive: everything before this thread = base (+) the lanes before it in its wavefront
    T before;
    {
        const int *src = reinterpret_cast<const int *>(&x);
        int *dst = reinterpret_cast<int *>(&before);
#pragma unroll
        for (int w = 0; w < static_cast<int>(sizeof(T) / 4); ++w) dst[w] = __shfl_up(src[w], 1, 64);
    }
    return lane == 0 ? base : op(base, before);
}

// What one group contributes, and its entries.
struct GroupPlan {
    int row_tiles;       // row tiles of the group (split on rows) / of the output block (split on the reduction dim)
    int tail_rows;       // 64 / 128 if the last row tile is a small one, else 0
    int rem;             // rows of the last row tile
    bool first_pass;     // split on the reduction dim: the group belongs to the first pass
};

__global__ __launch_bounds__(256) void gmm_schedule_kernel(const int64_t *__restrict__ group_list,
                                                           int group_list_type, int group_type, int num_groups,
                                                           int m, int k, int tile_rows, int num_col_tiles,
                                                           int split_tails, int tails_last_below,
                                                           int64_t b_stride_group, int64_t c_stride_group,
                                                           const int64_t *__restrict__ b_offsets, TileTable *table,
                                                           SplitTail *split_records, int split_cols, int split_cus,
                                                           GroupEntry *members, int slot_budget) {
    extern __shared__ int64_t ends[];          // [num_groups] clamped end offset of every group
    __shared__ int64_t scratch64[4];
    __shared__ ScanItem scratch_item[4];
    const int tid = threadIdx.x;
    const int per = (num_groups + 255) >> 8;
    const int g0 = tid * per < num_groups ? tid * per : num_groups;
    const int g1 = g0 + per < num_groups ? g0 + per : num_groups;

    // Group ends.  Cumulative list: end_g = min(m, max(0, list[0..g])); counts: end_g = min(m, sum of the counts so far,
    // negative counts read as 0).  Both are what a walk with "never before the previous end, never past m" gives.
    {
        int64_t run = 0;
        for (int g = g0; g < g1; ++g) {
            int64_t v = group_list[g];
            if (group_list_type == 0) {
                run = v > run ? v : run;
            } else {
                v = v < 0 ? 0 : (v > m ? m : v);
                run += v;
            }
            ends[g] = run;
        }
        int64_t total;
        const int64_t before = group_list_type == 0
            ? block_scan_exclusive(run, [](int64_t a, int64_t b) { return a > b ? a : b; }, int64_t{0}, scratch64, total)
            : block_scan_exclusive(run, [](int64_t a, int64_t b) { return a + b; }, int64_t{0}, scratch64, total);
        for (int g = g0; g < g1; ++g) {
            int64_t e = group_list_type == 0 ? (ends[g] > before ? ends[g] : before) : ends[g] + before;
            ends[g] = e > m ? m : e;
        }
    }
    __syncthreads();

    auto plan_of = [&](int g) {
        const int prev = g > 0 ? static_cast<int>(ends[g - 1]) : 0;
        const int len = static_cast<int>(ends[g]) - prev;              // rows (group_type 0) / reduction length
        GroupPlan p{};
        if (group_type == 0) {
            p.row_tiles = (len + tile_rows - 1) / tile_rows;
            p.rem = len - (p.row_tiles - 1) * tile_rows;
            p.tail_rows = (!split_tails || len <= 0) ? 0 : (p.rem <= 64 ? 64 : (p.rem <= 128 ? 128 : 0));
        } else {
            p.row_tiles = (k + tile_rows - 1) / tile_rows;
            p.rem = k - (p.row_tiles - 1) * tile_rows;
            p.tail_rows = (!split_tails || k <= 0) ? 0 : (p.rem <= 64 ? 64 : (p.rem <= 128 ? 128 : 0));
            p.first_pass = len >= (num_groups > 0 ? m / num_groups : 0);
        }
        return p;
    };
    auto share_of = [&](int row_tiles) { return (row_tiles * num_col_tiles + 7) >> 3; };

    // Launch-wide decisions (split on rows only): do the small tiles go last, and in how many parts.
    bool tails_last = false;
    int split_parts = 1;
    if (group_type == 0 && split_tails) {
        ScanItem mine{};                       // n0: tiles, n1: groups with a small tail
        for (int g = g0; g < g1; ++g) {
            const GroupPlan p = plan_of(g);
            mine.n0 += p.row_tiles * num_col_tiles;
            mine.n1 += p.tail_rows != 0 ? 1 : 0;
        }
        ScanItem all;
        block_scan_exclusive(mine, [](const ScanItem &a, const ScanItem &b) { return a + b; }, ScanItem{}, scratch_item, all);
        const int total = all.n0, tails = all.n1;
        tails_last = total < tails_last_below;
        // Worth splitting only where the small tiles would otherwise end the launch by themselves: the full tiles'
        // last round is complete, or leaves too few compute units free to run the small tiles (about half a full
        // tile's time each) beside it.
        const int tail_tiles = tails * num_col_tiles;
        const int full = total - tail_tiles;
        const int last = full % split_cus;
        const int free_cus = last == 0 ? 0 : split_cus - last;
        if (tails_last && split_records != nullptr && tails > 0 && full > 0 && tail_tiles > 2 * free_cus) {
            split_parts = kSplitCus / tail_tiles;
            if (split_parts > k / kSplitMinRed) split_parts = k / kSplitMinRed;
            if (split_parts > kMaxSplit) split_parts = kMaxSplit;
            if (split_parts < 2) split_parts = 1;
        }
    }
    // parts of a split tail: equal ranges of whole K steps, none empty
    const int steps = (k + BK - 1) / BK;
    const int part_len = split_parts > 1 ? (steps + split_parts - 1) / split_parts * BK : k;
    const int used_parts = split_parts > 1 ? (k + part_len - 1) / part_len : 1;

    // ---- whole groups to single XCDs ----------------------------------------------------------------
    // With many groups an XCD's eighth of a group is only a handful of tiles, and every XCD fetches nearly all of the
    // group's operand panels into its own L2.  Split on rows only (there a group's tiles are its work): the groups are
    // ranked by their tile counts and dealt out by rank; every XCD gets a list of its own and takes all tiles of its
    // groups, so a group's operands are fetched by one XCD only.  Taken when no XCD ends up more than 3 % over the
    // average (the launch's grid allows for 4 %); otherwise every group is cut in eight as usual.
    __shared__ int keys[kMaxListGroups];
    __shared__ int by_rank[kMaxListGroups];
    __shared__ int rank_of[kMaxListGroups];
    __shared__ int asg_xcd[kMaxListGroups];
    __shared__ int asg_pos[kMaxListGroups];
    __shared__ int asg_begin[kMaxListGroups];
    __shared__ int xcd_load[8];
    __shared__ int xcd_count[8];
    __shared__ int lists_ok;
    bool lists = false;
    __shared__ int most_row_tiles;
    if (tid == 0) most_row_tiles = 0;
    __syncthreads();
    const bool lists_wanted = members != nullptr && num_groups >= 16 && num_groups <= kMaxListGroups && !tails_last;
    const int out_tiles = ((k + tile_rows - 1) / tile_rows) * num_col_tiles;     // split on the reduction dim: tiles per group
    if (lists_wanted) {
        int most = 0;
        for (int g = g0; g < g1; ++g) {
            if (group_type == 0) {
                const int rt = plan_of(g).row_tiles;
                keys[g] = rt * num_col_tiles;
                most = rt > most ? rt : most;
            } else {
                const int prev = g > 0 ? static_cast<int>(ends[g - 1]) : 0;
                keys[g] = static_cast<int>(ends[g]) - prev;              // the work of a group's tiles: its reduction length
            }
        }
        if (most > 0) atomicMax(&most_row_tiles, most);
        __syncthreads();
    }
    // Only where it pays.  Split on rows: a group of more than 8 row tiles has eighths of distinct row tiles anyway
    // (every XCD then fetches its own rows of the group and only the weight panels eight times), and measured on a
    // skewed workload whose tiles lie mostly in such groups the lists gain nothing.  Split on the reduction dim: an
    // output block of at most 256 tiles (an eighth of it is then at most one block of 4 x 8).
    if (lists_wanted && (group_type == 0 ? most_row_tiles <= 8 : out_tiles <= 256)) {
        for (int g = g0; g < g1; ++g) {
            const int key = keys[g];
            int rank = 0;
#pragma unroll 8
            for (int h = 0; h < num_groups; ++h) rank += (keys[h] > key || (keys[h] == key && h < g)) ? 1 : 0;
            by_rank[rank] = g;
            rank_of[g] = rank;
        }
        __syncthreads();
        // Dealt out by rank, eight at a time, alternately ascending and descending over the XCDs (rank 0..7 to XCD
        // 0..7, rank 8..15 to XCD 7..0, ...): every group finds its XCD, its place in that XCD's list and the tiles in
        // front of it by itself.  Empty groups are ranked last and get no entry.
        if (tid < 8) {
            xcd_load[tid] = 0;
            xcd_count[tid] = 0;
        }
        __syncthreads();
        for (int g = g0; g < g1; ++g) {
            const int rank = rank_of[g];
            const int round = rank >> 3;
            const int x = (round & 1) ? 7 - (rank & 7) : (rank & 7);
            int begin = round * out_tiles;        // split on the reduction dim: every group has the same tiles
            if (group_type == 0) {
                begin = 0;
                for (int o = 0; o < round; ++o) begin += keys[by_rank[o * 8 + ((o & 1) ? 7 - x : x)]];
            }
            const bool has_entry = group_type == 2 || keys[g] != 0;   // (an empty group's output block is written as zeros)
            asg_xcd[g] = has_entry ? x : -1;
            asg_pos[g] = round;
            asg_begin[g] = begin;
            if (has_entry) {
                atomicAdd(&xcd_load[x], keys[g]);
                atomicAdd(&xcd_count[x], 1);
            }
        }
        __syncthreads();
        if (tid == 0) {
            long long total = 0;
            int max_load = 0;
            for (int q = 0; q < 8; ++q) {
                total += xcd_load[q];
                max_load = xcd_load[q] > max_load ? xcd_load[q] : max_load;
            }
            lists_ok = total > 0 && static_cast<long long>(max_load) * 800 <= total * 103 ? 1 : 0;
            // never more slots than the launch has workgroups for: the tiles beyond would stay unwritten
            int most_groups = 0;
            for (int q = 0; q < 8; ++q) most_groups = xcd_count[q] > most_groups ? xcd_count[q] : most_groups;
            const long long zero_fill = group_type == 0 && ends[num_groups - 1] < m
                ? ((static_cast<long long>((m - static_cast<int>(ends[num_groups - 1]) + tile_rows - 1) / tile_rows) * num_col_tiles + 7) >> 3) : 0;
            const long long need = group_type == 0 ? max_load + zero_fill : static_cast<long long>(most_groups) * out_tiles;
            if (need > slot_budget) lists_ok = 0;
        }
        __syncthreads();
        lists = lists_ok != 0;
    }

    // What every group emits in each pass.
    auto item_of = [&](const GroupPlan &p) {
        ScanItem it{};
        if (group_type == 2) {
            if (p.row_tiles > 0) {
                if (p.first_pass) { it.n0 = 1; it.slots0 = share_of(p.row_tiles); }
                else { it.n1 = 1; it.slots1 = share_of(p.row_tiles); }
            }
        } else if (p.row_tiles > 0) {
            if (!tails_last) {
                it.n0 = 1; it.slots0 = share_of(p.row_tiles);
            } else {
                const int full_tiles = p.tail_rows != 0 ? p.row_tiles - 1 : p.row_tiles;
                if (full_tiles > 0) { it.n0 = 1; it.slots0 = share_of(full_tiles); }
                if (p.tail_rows != 0) {
                    const int parts = split_parts > 1 ? used_parts : 1;
                    it.n1 = parts; it.slots1 = parts * share_of(1);
                    if (split_parts > 1) { it.tails = 1; it.pairs = parts; }
                }
            }
        }
        return it;
    };
    ScanItem mine{};
    for (int g = g0; g < g1; ++g) mine = mine + item_of(plan_of(g));
    ScanItem all;
    ScanItem at = block_scan_exclusive(mine, [](const ScanItem &a, const ScanItem &b) { return a + b; }, ScanItem{}, scratch_item, all);

    const int max_entries = (1 + kMaxSplit) * num_groups + 2;
    auto put = [&](int idx, const GroupEntry &e) {
        if (idx < max_entries) table->entries[idx] = e;
        if (idx < 16) table->begins[idx] = e.tile_begin;
    };
    if (lists) {
        const int stride = num_groups + 1;      // a list may hold nearly every group, and the zero-fill pseudo-group
        for (int g = g0; g < g1; ++g) {
            if (asg_xcd[g] < 0) continue;
            const GroupPlan p = plan_of(g);
            const int prev = g > 0 ? static_cast<int>(ends[g - 1]) : 0;
            GroupEntry f{};
            f.tile_rows = tile_rows;
            if (group_type == 0) {
                f.row_begin = prev;
                f.row_end = static_cast<int>(ends[g]);
                f.red_begin = 0;
                f.red_end = k;
                f.b_off = b_offsets != nullptr ? b_offsets[g] : g * b_stride_group;
            } else {
                f.row_begin = 0;
                f.row_end = k;
                f.red_begin = prev;
                f.red_end = static_cast<int>(ends[g]);
                f.c_off = g * c_stride_group;
            }
            f.num_row_tiles = p.row_tiles;
            f.tail_rows = p.tail_rows;
            f.num_tiles = p.row_tiles * num_col_tiles;
            f.share = f.num_tiles;
            f.whole = 1;
            f.tile_begin = asg_begin[g];
            members[static_cast<int64_t>(asg_xcd[g]) * stride + asg_pos[g]] = f;
        }
        if (tid == 0) {
            int slots = 0;
            for (int q = 0; q < 8; ++q) {
                const int tiles_q = group_type == 0 ? xcd_load[q] : xcd_count[q] * out_tiles;
                slots = tiles_q > slots ? tiles_q : slots;
            }
            int counts[8];
            for (int q = 0; q < 8; ++q) counts[q] = xcd_count[q];
            const int last_end = static_cast<int>(ends[num_groups - 1]);
            if (group_type == 0 && last_end < m) {                 // rows past the last offset: zero-fill, an eighth for every XCD behind its groups
                GroupEntry e{};
                e.row_begin = last_end;
                e.row_end = m;
                e.tile_rows = tile_rows;
                const int len = m - last_end;
                e.num_row_tiles = (len + tile_rows - 1) / tile_rows;
                const int rem = len - (e.num_row_tiles - 1) * tile_rows;
                e.tail_rows = !split_tails ? 0 : (rem <= 64 ? 64 : (rem <= 128 ? 128 : 0));
                e.num_tiles = e.num_row_tiles * num_col_tiles;
                e.share = (e.num_tiles + 7) >> 3;
                int most = 0;
                for (int q = 0; q < 8; ++q) {
                    e.tile_begin = xcd_load[q];
                    members[static_cast<int64_t>(q) * stride + counts[q]] = e;
                    counts[q] += 1;
                    most = xcd_load[q] + e.share > most ? xcd_load[q] + e.share : most;
                }
                slots = most;
            }
            table->slots_per_xcd = slots;
            table->num_entries = 0;
            table->num_split_tails = 0;
            table->lists_off = static_cast<int>(reinterpret_cast<char *>(members) - reinterpret_cast<char *>(table));
            table->list_stride = stride;
            for (int q = 0; q < 8; ++q) table->list_count[q] = counts[q];
            for (int i = 0; i < 8; ++i) table->zeros[i] = 0;
            for (int i = 0; i < 16; ++i) table->begins[i] = 0x7fffffff;
        }
        return;
    }
    for (int g = g0; g < g1; ++g) {
        const GroupPlan p = plan_of(g);
        const ScanItem it = item_of(p);
        const int prev = g > 0 ? static_cast<int>(ends[g - 1]) : 0;
        const int end = static_cast<int>(ends[g]);
        GroupEntry e{};
        e.tile_rows = tile_rows;
        if (group_type == 0) {
            e.row_begin = prev; e.row_end = end; e.red_begin = 0; e.red_end = k;
            e.b_off = b_offsets != nullptr ? b_offsets[g] : g * b_stride_group;
            e.c_off = 0;
        } else {
            e.row_begin = 0; e.row_end = k; e.red_begin = prev; e.red_end = end;
            e.b_off = 0;
            e.c_off = g * c_stride_group;
        }
        if (it.n0 != 0) {                       // first pass: the whole group, or its full tiles
            GroupEntry f = e;
            const bool full_only = group_type == 0 && tails_last && p.tail_rows != 0;
            f.num_row_tiles = full_only ? p.row_tiles - 1 : p.row_tiles;
            f.tail_rows = full_only ? 0 : p.tail_rows;
            if (full_only) f.row_end = f.row_begin + f.num_row_tiles * tile_rows;
            f.num_tiles = f.num_row_tiles * num_col_tiles;
            f.share = (f.num_tiles + 7) >> 3;
            f.tile_begin = at.slots0;
            put(at.n0, f);
        }
        if (it.n1 != 0) {                       // second pass
            GroupEntry f = e;
            if (group_type == 0) {              // the small tile, whole or in parts
                f.row_begin = prev + (p.row_tiles - 1) * tile_rows;
                f.num_row_tiles = 1;
                f.tail_rows = p.tail_rows;
            } else {
                f.num_row_tiles = p.row_tiles;
                f.tail_rows = p.tail_rows;
            }
            f.num_tiles = f.num_row_tiles * num_col_tiles;
            f.share = (f.num_tiles + 7) >> 3;
            if (it.tails != 0) {
                if (at.tails < num_groups) split_records[at.tails] = SplitTail{f.row_begin, p.rem, at.pairs, it.n1};
                for (int s = 0; s < it.n1; ++s) {
                    f.red_begin = s * part_len;
                    f.red_end = f.red_begin + part_len < k ? f.red_begin + part_len : k;
                    f.split = s + 1;
                    f.c_off = (static_cast<int64_t>(at.pairs + s) * kSplitRows - f.row_begin) * split_cols;
                    f.tile_begin = all.slots0 + at.slots1 + s * f.share;
                    put(all.n0 + at.n1 + s, f);
                }
            } else {
                f.tile_begin = all.slots0 + at.slots1;
                put(all.n0 + at.n1, f);
            }
        }
        at = at + it;
    }
    if (tid == 0) {
        int n = all.n0 + all.n1;
        int slots = all.slots0 + all.slots1;
        const int last_end = num_groups > 0 ? static_cast<int>(ends[num_groups - 1]) : 0;
        if (group_type == 0 && last_end < m) {  // rows past the last offset: zero-fill (empty reduction range)
            GroupEntry e{};
            e.row_begin = last_end;
            e.row_end = m;
            e.tile_rows = tile_rows;
            const int len = m - last_end;
            e.num_row_tiles = (len + tile_rows - 1) / tile_rows;
            const int rem = len - (e.num_row_tiles - 1) * tile_rows;
            e.tail_rows = !split_tails ? 0 : (rem <= 64 ? 64 : (rem <= 128 ? 128 : 0));
            e.num_tiles = e.num_row_tiles * num_col_tiles;
            e.share = (e.num_tiles + 7) >> 3;
            e.tile_begin = slots;
            slots += e.share;
            put(n++, e);
        }
        table->slots_per_xcd = slots;
        table->num_entries = n;
        table->num_split_tails = all.tails;
        table->lists_off = 0;
        table->list_stride = 0;
        for (int i = 0; i < 8; ++i) table->zeros[i] = 0;
        for (int i = n; i < 16; ++i) table->begins[i] = 0x7fffffff;
    }
}

// 8 contiguous 16-bit elements starting at p; elements >= nvalid read as zero.
__device__ __forceinline__ v16 load8(const uint16_t *p, int nvalid, bool vec_ok) {
    if (nvalid >= 8 && vec_ok && (reinterpret_cast<uintptr_t>(p) & 15u) == 0) return *reinterpret_cast<const v16 *>(p);
    v16 r = {0u, 0u, 0u, 0u};
    if (nvalid > 0) {
        uint16_t tmp[8];
#pragma unroll
        for (int e = 0; e < 8; ++e) tmp[e] = e < nvalid ? p[e] : static_cast<uint16_t>(0);
        r = *reinterpret_cast<v16 *>(tmp);
    }
    return r;
}

// Operand tile loader.  RED == true: memory is contiguous along the reduction
// dim; RED == false: contiguous along the outer (row of A / col of B) dim.
template <bool RED>
struct TileLoader {
    v16 r[8];

    // outer0/outer_end: first outer index of the tile and the exclusive bound of
    // valid outer indices; red0/red_end likewise for this 64-wide reduction step.
    __device__ __forceinline__ void load(const uint16_t *base, int64_t stride_outer, int64_t stride_red, int outer0,
                                         int outer_end, int red0, int red_end, bool vec_ok) {
        const int tid = threadIdx.x;
        if constexpr (RED) {
            const int ck = tid & 7;
            const int red = red0 + ck * 8;
            const int nvalid = red_end - red;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                const int outer = outer0 + (tid >> 3) + 32 * i;
                const bool ok = outer < outer_end;
                const uint16_t *p = base + static_cast<int64_t>(ok ? outer : outer0) * stride_outer + red;
                r[i] = load8(p, ok ? nvalid : 0, vec_ok);
            }
        } else {
            const int kb = tid & 7;
            const int nb = tid >> 3;
            const int outer = outer0 + nb * 8;
            const int nvalid = outer_end - outer;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                const int red = red0 + kb * 8 + j;
                const bool ok = red < red_end;
                const uint16_t *p = base + static_cast<int64_t>(ok ? red : red0) * stride_red + outer;
                r[j] = load8(p, ok ? nvalid : 0, vec_ok);
            }
        }
    }

    __device__ __forceinline__ void store(char *lds_tile) const {
        const int tid = threadIdx.x;
        if constexpr (RED) {
            const int ck = tid & 7;
            const int row = tid >> 3;
            char *dst = lds_tile + row * 128 + ((ck ^ swz(row)) << 4);
#pragma unroll
            for (int i = 0; i < 8; ++i) *reinterpret_cast<v16 *>(dst + i * 32 * 128) = r[i];
        } else {
            const int kb = tid & 7;
            const int nb = tid >> 3;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                v16 o;
#pragma unroll
                for (int mth = 0; mth < 4; ++mth) {
                    const unsigned lo = r[2 * mth][c >> 1];
                    const unsigned hi = r[2 * mth + 1][c >> 1];
                    o[mth] = (c & 1) ? ((lo >> 16) | (hi & 0xffff0000u)) : ((lo & 0xffffu) | (hi << 16));
                }
                const int row = nb * 8 + c;
                *reinterpret_cast<v16 *>(lds_tile + row * 128 + ((kb ^ swz(row)) << 4)) = o;
            }
        }
    }
};

template <int DT, bool A_RED, bool B_RED, int OUT>
__global__ __launch_bounds__(256) void gmm16_kernel(const GmmArgs p) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const TileCoord tc = locate_tile<false>(p.table);
    if (!tc.valid) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int row0 = tc.e.row_begin + tc.row_tile * tc.e.tile_rows;
    const int row_end = tc.e.row_end;
    const int col0 = tc.col_tile * BN;
    const int col_end = p.cols;
    const int red_begin = tc.e.red_begin, red_end = tc.e.red_end;

    const uint16_t *a_base = static_cast<const uint16_t *>(p.a);
    const uint16_t *b_base = static_cast<const uint16_t *>(p.b) + tc.e.b_off;
    const bool a_vec = p.a_vec_ok != 0, b_vec = p.b_vec_ok != 0;

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // per-lane fragment read offsets (bytes) inside an operand tile
    const int frow = lane & 31;
    const int fsw = swz(frow);
    const int hi = lane >> 5;
    int a_off[4], b_off[4];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
        const int chunk = ((kk * 2 + hi) ^ fsw) << 4;
        a_off[kk] = (wm * 128 + frow) * 128 + chunk;
        b_off[kk] = (wn * 128 + frow) * 128 + chunk;
    }

    TileLoader<A_RED> la;
    TileLoader<B_RED> lb;
    const int nk = (red_end - red_begin + BK - 1) / BK;
    if (nk > 0) {
        la.load(a_base, p.a_stride_row, p.a_stride_red, row0, row_end, red_begin, red_end, a_vec);
        lb.load(b_base, p.b_stride_col, p.b_stride_red, col0, col_end, red_begin, red_end, b_vec);
        la.store(lds);
        lb.store(lds + kTileBytes);
        __syncthreads();
    }
    for (int kt = 0; kt < nk; ++kt) {
        char *sa = lds + (kt & 1) * 2 * kTileBytes;
        char *sb = sa + kTileBytes;
        const bool more = kt + 1 < nk;
        if (more) {
            const int red0 = red_begin + (kt + 1) * BK;
            la.load(a_base, p.a_stride_row, p.a_stride_red, row0, row_end, red0, red_end, a_vec);
            lb.load(b_base, p.b_stride_col, p.b_stride_red, col0, col_end, red0, red_end, b_vec);
        }
#pragma unroll
        for (int kk = 0; kk < 4; ++kk) {
            v16 af[4], bf[4];
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                af[t] = *reinterpret_cast<const v16 *>(sa + a_off[kk] + t * 32 * 128);
                bf[t] = *reinterpret_cast<const v16 *>(sb + b_off[kk] + t * 32 * 128);
            }
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j) acc[i][j] = mfma16<DT>(bf[j], af[i], acc[i][j]);
        }
        if (more) {
            char *na = lds + ((kt + 1) & 1) * 2 * kTileBytes;
            la.store(na);
            lb.store(na + kTileBytes);
        }
        __syncthreads();
    }

    // Epilogue.  acc[i][j][4*q+e] = C[row0 + wm*128 + i*32 + (lane&31)]
    //                                [col0 + wn*128 + j*32 + 8*q + 4*(lane>>5) + e]
    const int64_t ldc = p.c_stride_row;
    const bool c_vec = p.c_vec_ok != 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = row0 + wm * 128 + i * 32 + (lane & 31);
        if (row >= row_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int col = col0 + wn * 128 + j * 32 + 8 * q + 4 * hi;
                if (col >= col_end) continue;
                const int64_t at = tc.e.c_off + static_cast<int64_t>(row) * ldc + col;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * q + e];
                const bool full = c_vec && col + 4 <= col_end;
                if constexpr (OUT == OUT_SAME) {
                    uint16_t *c = static_cast<uint16_t *>(p.c) + at;
                    const bool full8 = full && (reinterpret_cast<uintptr_t>(c) & 7u) == 0;
                    uint16_t h[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) h[e] = DT == MS_BF16 ? BF16::from_float(v[e]) : FP16::from_float(v[e]);
                    if (full8) {
                        *reinterpret_cast<uint2 *>(c) = *reinterpret_cast<uint2 *>(h);
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < col_end) c[e] = h[e];
                    }
                } else {
                    float *c = static_cast<float *>(p.c) + at;
                    if (full && (reinterpret_cast<uintptr_t>(c) & 15u) == 0) {
                        f32x4 o = {v[0], v[1], v[2], v[3]};
                        if constexpr (OUT == ACC_F32) o += *reinterpret_cast<f32x4 *>(c);
                        *reinterpret_cast<f32x4 *>(c) = o;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            if (col + e < col_end) c[e] = (OUT == ACC_F32 ? c[e] : 0.f) + v[e];
                    }
                }
            }
        }
    }
}

// ---- fp32 MFMA kernel ---------------------------------------------------------------------
// v_mfma_f32_32x32x2f32 on square tiles of 64 * TM rows and columns (2 x 2 wavefronts of TM x TM blocks of 32 x 32), K
// steps of 16 (large tile) or 32 (small tile).  Element-wise guarded loads, so any pair of strides goes.  The next K
// step's operands are fetched into registers while the current one is multiplied and then written to the other of two
// LDS buffers: one barrier per step, and the loads have a whole step to arrive.  TM = 2 (128 x 128) for launches with
// tiles enough for every compute unit, TM = 1 (64 x 64) for small ones, which otherwise leave most of the chip idle.
constexpr int kTile32Large = 128, kTile32Small = 64;

template <bool ACC, int TM>
__global__ __launch_bounds__(256) void gmm32_kernel(const GmmArgs p) {
    constexpr int T = 64 * TM;
    constexpr int FK = TM == 1 ? 32 : 16;      // K step: 8 K elements per thread and operand, two 17 KB buffers each
    constexpr int PITCH = T + 4;
    constexpr int PER = T * FK / 256;          // elements per thread, operand and K step
    __shared__ float sa[2][FK][PITCH];
    __shared__ float sb[2][FK][PITCH];
    const TileCoord tc = locate_tile<false>(p.table);
    if (!tc.valid) return;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;
    const int row0 = tc.e.row_begin + tc.row_tile * T;
    const int row_end = tc.e.row_end;
    const int col0 = tc.col_tile * T;
    const int col_end = p.cols;
    const int red_end = tc.e.red_end;
    const float *a_base = static_cast<const float *>(p.a);
    const float *b_base = static_cast<const float *>(p.b) + tc.e.b_off;
    const bool a_red = p.a_stride_red == 1, b_red = p.b_stride_red == 1;

    f32x16 acc[TM][TM];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // element i of this thread: (reduction index kk, outer index r) inside the tile, consecutive threads along the
    // operand's contiguous dim
    auto fetch = [&](float (&ra)[PER], float (&rb)[PER], int red0) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + i * 256;
            {
                const int kk = a_red ? idx % FK : idx / T;
                const int r = a_red ? idx / FK : idx % T;
                const int row = row0 + r, red = red0 + kk;
                ra[i] = (row < row_end && red < red_end)
                            ? a_base[static_cast<int64_t>(row) * p.a_stride_row + static_cast<int64_t>(red) * p.a_stride_red]
                            : 0.f;
            }
            {
                const int kk = b_red ? idx % FK : idx / T;
                const int cc = b_red ? idx / FK : idx % T;
                const int col = col0 + cc, red = red0 + kk;
                rb[i] = (col < col_end && red < red_end)
                            ? b_base[static_cast<int64_t>(red) * p.b_stride_red + static_cast<int64_t>(col) * p.b_stride_col]
                            : 0.f;
            }
        }
    };
    auto stash = [&](int buf, const float (&ra)[PER], const float (&rb)[PER]) {
#pragma unroll
        for (int i = 0; i < PER; ++i) {
            const int idx = tid + i * 256;
            sa[buf][a_red ? idx % FK : idx / T][a_red ? idx / FK : idx % T] = ra[i];
            sb[buf][b_red ? idx % FK : idx / T][b_red ? idx / FK : idx % T] = rb[i];
        }
    };
    auto multiply = [&](int buf) {
#pragma unroll
        for (int ks = 0; ks < FK / 2; ++ks) {
            const int kk = ks * 2 + (lane >> 5);
            float av[TM], bv[TM];
#pragma unroll
            for (int t = 0; t < TM; ++t) {
                av[t] = sa[buf][kk][wm * 32 * TM + t * 32 + (lane & 31)];
                bv[t] = sb[buf][kk][wn * 32 * TM + t * 32 + (lane & 31)];
            }
#pragma unroll
            for (int i = 0; i < TM; ++i)
#pragma unroll
                for (int j = 0; j < TM; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bv[j], av[i], acc[i][j], 0, 0, 0);
        }
    };

    // K step t is multiplied out of LDS buffer t & 1 while step t + 1 is fetched into registers, then written to the
    // other buffer.  (Two steps of fetches in flight instead of one measured the same: at these sizes a step is as long
    // as its dependent MFMAs.)
    float ra[PER], rb[PER];
    const int red_begin = tc.e.red_begin;
    if (red_begin < red_end) {
        fetch(ra, rb, red_begin);
        stash(0, ra, rb);
    }
    __syncthreads();
    int buf = 0;
    for (int red0 = red_begin; red0 < red_end; red0 += FK) {
        const bool more = red0 + FK < red_end;
        if (more) fetch(ra, rb, red0 + FK);
        multiply(buf);
        if (more) stash(buf ^ 1, ra, rb);
        __syncthreads();          // everyone is done with `buf`, and the other buffer is complete
        buf ^= 1;
    }
    float *c_base = static_cast<float *>(p.c) + tc.e.c_off;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        const int row = row0 + wm * 32 * TM + i * 32 + (lane & 31);
        if (row >= row_end) continue;
#pragma unroll
        for (int j = 0; j < TM; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) {
                const int col = col0 + wn * 32 * TM + j * 32 + 8 * (e >> 2) + 4 * (lane >> 5) + (e & 3);
                if (col < col_end) {
                    float *c = c_base + static_cast<int64_t>(row) * p.c_stride_row + col;
                    *c = ACC ? *c + acc[i][j][e] : acc[i][j][e];
                }
            }
    }
}

// ---- host -------------------------------------------------------------------------------
// A launch with fewer than this many rounds of tiles (tiles / compute units) schedules its small tail tiles last.
// Measured with 4, 6, 8 and 12: from 6 on the DeepSeek-share fc1 forward (4.25 rounds) gains 5 %; at 12 the
// Mixtral-shape fc2 dX (8.1 rounds) loses 2.5 %, its tail tiles no longer finding their weight panels in L2.
constexpr int kTailsLastRounds = 6;

// Compute units of the current device (cached per device ordinal; 256 if the query fails).
int current_device_cus() {
    static int cached[64] = {};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 256;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) n = 256;
        cached[dev] = n;
    }
    return cached[dev];
}

constexpr size_t table_bytes(int64_t num_groups) {
    // per group: its full tiles, its tail tile in up to kMaxSplit parts; plus the zero-fill pseudo-group
    return sizeof(TileTable) + static_cast<size_t>((1 + kMaxSplit) * num_groups + 2) * sizeof(GroupEntry);
}
// workspace = tile table, then (8-byte aligned) room for the per-group weight offsets of the list form, then the
// records of the split tails
constexpr size_t offsets_pos(int64_t num_groups) { return (table_bytes(num_groups) + 7) & ~static_cast<size_t>(7); }
constexpr size_t split_records_pos(int64_t num_groups) { return offsets_pos(num_groups) + kMaxWeightList * sizeof(int64_t); }
constexpr size_t members_pos(int64_t num_groups) {
    return split_records_pos(num_groups) + static_cast<size_t>(num_groups) * sizeof(SplitTail);
}
// ... then the eight per-XCD lists of entries (whole groups dealt out to single XCDs): num_groups + 1 entries each
constexpr size_t workspace_need(int64_t num_groups) {
    return members_pos(num_groups) +
           (num_groups >= 16 && num_groups <= kMaxListGroups ? static_cast<size_t>(8 * (num_groups + 1)) * sizeof(GroupEntry) : 0);
}
// ... and, for launches that may split the reduction of their small tail tiles, the fp32 partial sums behind that
constexpr size_t split_ws_pos(int64_t num_groups) { return (workspace_need(num_groups) + 255) & ~static_cast<size_t>(255); }

// Slots (workgroups) per XCD that a launch must provide: no table the schedule kernel can write needs more.
//   common table: every entry rounds its eighth of its tiles up, so an eighth of all tiles plus one slot per entry;
//   a launch that may split its tail tiles has up to kMaxSplit entries per tail and up to kSplitCus more tiles;
//   per-XCD lists, split on rows: the fullest XCD holds at most 1.03 times an eighth of all tiles (the schedule kernel's
//   own balance test) plus its eighth of the zero-fill pseudo-group;
//   per-XCD lists, split on the reduction dim: every group has the same number of output tiles and the XCD with the
//   most groups holds ceil(num_groups / 8) of them, however short their reductions are (an empty group still writes
//   its block of zeros), which exceeds an eighth of all tiles whenever num_groups is not a multiple of 8.
int64_t launch_slots_per_xcd(int group_type, int64_t num_groups, int64_t m, int64_t k, int64_t tile_rows,
                             int64_t num_col_tiles, bool lists, bool split) {
    const int64_t row_tiles_bound = group_type == 0 ? ceil_div(m, tile_rows) + num_groups + 2
                                                    : num_groups * (k / tile_rows + 1);
    const int64_t tiles_bound = row_tiles_bound * num_col_tiles;
    int64_t slots = split ? ceil_div(tiles_bound + kSplitCus, 8) + (1 + kMaxSplit) * num_groups + 2
                          : ceil_div(tiles_bound, 8) + 2 * num_groups + 2;
    if (lists) {
        const int64_t by_lists = group_type == 0
            ? ceil_div(tiles_bound + tiles_bound / 25, 8) + 2 * num_groups + 2
            : ceil_div(num_groups, 8) * ceil_div(k, tile_rows) * num_col_tiles;
        slots = by_lists > slots ? by_lists : slots;
    }
    return slots;
}

// Whether a launch of these sizes can come to split its tail tiles at all (the schedule kernel decides from the
// group list whether it does), and how many bytes of partial sums it may then write: the parts of a launch number at
// most kSplitCus tiles, i.e. kSplitCus / column tiles blocks of kSplitRows x n floats.
bool may_split_tails(int64_t m, int64_t k, int64_t n, int group_type, int dtype, int out_dtype, int accumulate,
                     int num_cus) {
    if (group_type != 0 || dtype == MS_FP32 || out_dtype != dtype || accumulate) return false;
    const int64_t col_tiles = ceil_div(n, BN);
    // (the schedule kernel splits only when at least three quarters of a round of full tiles run in front)
    return k >= 2 * kSplitMinRed && 2 * col_tiles <= kSplitCus && n % 8 == 0 &&
           ceil_div(m, BM) * col_tiles < static_cast<int64_t>(kTailsLastRounds) * num_cus &&
           4 * ceil_div(m, 128) * col_tiles >= 3 * static_cast<int64_t>(num_cus);
}
size_t split_ws_bytes(int64_t n) {
    const int64_t pairs = kSplitCus / ceil_div(n, BN);
    return static_cast<size_t>(pairs) * kSplitRows * static_cast<size_t>(n) * sizeof(float);
}

// y[row, :] of every split tail = the sum of its parts' partial sums (in part order), rounded once.
// grid (num_groups, ceil(n / 2048), 16): block (j, c, z) takes rows z, z + 16, ... of tail j, 8 columns per lane.
template <int DT>
__global__ __launch_bounds__(256) void gmm_split_reduce_kernel(const TileTable *__restrict__ table,
                                                               const SplitTail *__restrict__ tails,
                                                               const float *__restrict__ ws, uint16_t *__restrict__ y,
                                                               int64_t ldy, int n) {
    if (static_cast<int>(blockIdx.x) >= table->num_split_tails) return;
    const SplitTail t = tails[blockIdx.x];
    const int col = (blockIdx.y * 256 + threadIdx.x) * 8;
    if (col >= n) return;
    using DTT = std::conditional_t<DT == MS_BF16, BF16, FP16>;
    for (int r = blockIdx.z; r < t.rows; r += gridDim.z) {
        // all parts requested at once (a part past the last one re-reads part 0 and is left out of the sum)
        f32x4 pl[kMaxSplit], ph[kMaxSplit];
#pragma unroll
        for (int s = 0; s < kMaxSplit; ++s) {
            const float *src = ws + (static_cast<int64_t>(t.pair0 + (s < t.parts ? s : 0)) * kSplitRows + r) * n + col;
            pl[s] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src));
            ph[s] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(src + 4));
        }
        f32x4 lo = pl[0], hi = ph[0];
#pragma unroll
        for (int s = 1; s < kMaxSplit; ++s)
            if (s < t.parts) {
                lo += pl[s];
                hi += ph[s];
            }
        uint16_t o[8];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            o[e] = DTT::from_float(lo[e]);
            o[4 + e] = DTT::from_float(hi[e]);
        }
        *reinterpret_cast<v16 *>(y + static_cast<int64_t>(t.row_begin + r) * ldy + col) = *reinterpret_cast<v16 *>(o);
    }
}

template <int DT, int OUT>
int launch16(hipStream_t stream, const GmmArgs &args, bool a_red, bool b_red, unsigned grid) {
    const void *fn;
    if (a_red && b_red) fn = reinterpret_cast<const void *>(&gmm16_kernel<DT, true, true, OUT>);
    else if (a_red) fn = reinterpret_cast<const void *>(&gmm16_kernel<DT, true, false, OUT>);
    else if (b_red) fn = reinterpret_cast<const void *>(&gmm16_kernel<DT, false, true, OUT>);
    else fn = reinterpret_cast<const void *>(&gmm16_kernel<DT, false, false, OUT>);
    hipError_t e = set_max_dynamic_lds(fn, kLdsBytes16);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm: hipFuncSetAttribute: %s", hipGetErrorString(e));
    GmmArgs copy = args;
    void *kargs[] = {&copy};
    e = hipLaunchKernel(fn, dim3(grid), dim3(256), kargs, kLdsBytes16, stream);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm: launch failed: %s", hipGetErrorString(e));
    return MS_OK;
}

}  // namespace
}  // namespace ms

using namespace ms;

extern "C" int ms_gmm_workspace_size(int64_t num_groups, int64_t m, int group_type, size_t *bytes) {
    (void)m;
    (void)group_type;
    MS_REQUIRE(bytes != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_gmm_workspace_size: bytes is NULL");
    MS_REQUIRE(num_groups >= 1 && num_groups <= kMaxGroups, MS_ERR_UNSUPPORTED,
               "ms_gmm_workspace_size: num_groups %lld outside [1, %d]", (long long)num_groups, kMaxGroups);
    *bytes = (workspace_need(num_groups) + 255) & ~static_cast<size_t>(255);
    return MS_OK;
}

// Workgroups per XCD that ms_gmm launches for a 16-bit problem of these sizes (grid = 8 times that): host arithmetic
// only.  lists / split: whether the launch may deal whole groups out to single XCDs / split the reduction of its tail tiles.
extern "C" int ms_gmm_launch_slots(int64_t num_groups, int64_t m, int64_t k, int64_t n, int group_type, int lists,
                                   int split, int64_t *slots_per_xcd) {
    MS_REQUIRE(slots_per_xcd != nullptr && num_groups >= 1 && num_groups <= kMaxGroups && m >= 0 && k >= 0 && n >= 0 &&
                   (group_type == 0 || group_type == 2),
               MS_ERR_INVALID_ARGUMENT, "ms_gmm_launch_slots: bad arguments");
    *slots_per_xcd = launch_slots_per_xcd(group_type, num_groups, m, k, BM, ceil_div(n, BN), lists != 0, split != 0);
    return MS_OK;
}

// The tile order of the kernels, evaluated on the host (the same function the kernels call).
extern "C" int ms_gmm_tile_order(int num_row_tiles, int num_col_tiles, int index, int *row_tile, int *col_tile) {
    MS_REQUIRE(num_row_tiles >= 1 && num_col_tiles >= 1 && index >= 0 &&
                   static_cast<int64_t>(index) < static_cast<int64_t>(num_row_tiles) * num_col_tiles &&
                   static_cast<int64_t>(num_row_tiles) * num_col_tiles < (1ll << 30) && row_tile != nullptr && col_tile != nullptr,
               MS_ERR_INVALID_ARGUMENT, "ms_gmm_tile_order: bad arguments");
    tile_order(index, num_row_tiles, num_col_tiles, *row_tile, *col_tile);
    return MS_OK;
}

extern "C" int ms_gmm_workspace_size_split(int64_t num_groups, int64_t m, int64_t k, int64_t n, int group_type, int dtype,
                                           int out_dtype, int accumulate, size_t *bytes) {
    if (int rc = ms_gmm_workspace_size(num_groups, m, group_type, bytes)) return rc;
    MS_REQUIRE(m >= 0 && k >= 0 && n >= 0, MS_ERR_INVALID_ARGUMENT, "ms_gmm_workspace_size_split: bad sizes m=%lld k=%lld n=%lld",
               (long long)m, (long long)k, (long long)n);
    if (may_split_tails(m, k, n, group_type, dtype, out_dtype, accumulate, kSplitCus))
        *bytes = (split_ws_pos(num_groups) + split_ws_bytes(n) + 255) & ~static_cast<size_t>(255);
    return MS_OK;
}

// weight_offsets: nullptr for one strided weight tensor, else num_groups element offsets (relative to
// `weight`) of separately allocated per-group matrices; all_weights_aligned16 then says whether every one of
// them starts on a 16-byte boundary.
// Second output of the fused SwiGLU form (n = 2 * ffn weight columns: gate | up).
struct SwigluOut {
    void *act;
    int64_t act_stride_row;
    const void *probs;
    int probs_dtype;
};
// Inputs of the fused SwiGLU backward form (the product is dact [m, ffn]; what is written is d_fc1 [m, 2*ffn]).
struct SwigluGradIn {
    const void *fc1;
    int64_t fc1_stride_row;
    const void *probs;
    int probs_dtype;
    float *partials;
    int partials_per_row;
};

// grad_probs[r] = sum of the row's partial sums, in the probabilities' dtype.  One wavefront per row.
__global__ __launch_bounds__(256) void swiglu_grad_probs_kernel(const float *__restrict__ partials, int per_row, int rows,
                                                                void *__restrict__ grad_probs, int probs_dtype) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6);
    const int lane = threadIdx.x & 63;
    if (row >= rows) return;
    float s = 0.f;
    for (int i = lane; i < per_row; i += 64) s += partials[static_cast<int64_t>(row) * per_row + i];
#pragma unroll
    for (int d = 32; d > 0; d >>= 1) s += __shfl_down(s, d, 64);
    if (lane == 0) store_float_as(grad_probs, row, probs_dtype, s);
}

static int gmm_impl(ms_stream_t stream_, const void *x, int64_t x_stride0, int64_t x_stride1, const void *weight,
                    int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1, void *y, int64_t y_stride_row,
                    const int64_t *group_list, int group_list_type, int group_type, int64_t num_groups, int64_t m,
                    int64_t k, int64_t n, int dtype, int out_dtype, int accumulate, void *workspace,
                    size_t workspace_bytes, const WeightOffsets *weight_offsets, bool all_weights_aligned16,
                    const SwigluOut *swiglu = nullptr, const SwigluGradIn *swiglu_grad = nullptr,
                    bool allow_split = true) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED, "ms_gmm: bad dtype %d", dtype);
    MS_REQUIRE(out_dtype == dtype || out_dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "ms_gmm: out_dtype must equal dtype or be fp32");
    MS_REQUIRE(!accumulate || out_dtype == MS_FP32, MS_ERR_UNSUPPORTED, "ms_gmm: accumulate needs an fp32 output");
    MS_REQUIRE(group_type == 0 || group_type == 2, MS_ERR_UNSUPPORTED, "ms_gmm: group_type must be 0 or 2, got %d", group_type);
    MS_REQUIRE(group_list_type == 0 || group_list_type == 1, MS_ERR_INVALID_ARGUMENT,
               "ms_gmm: group_list_type must be 0 or 1, got %d", group_list_type);
    MS_REQUIRE(num_groups >= 1 && num_groups <= kMaxGroups, MS_ERR_UNSUPPORTED,
               "ms_gmm: num_groups %lld outside [1, %d]", (long long)num_groups, kMaxGroups);
    MS_REQUIRE(m >= 0 && k >= 0 && n >= 0 && m < (1ll << 31) - 512 && k < (1ll << 31) - 512 && n < (1ll << 31) - 512,
               MS_ERR_INVALID_ARGUMENT, "ms_gmm: bad sizes m=%lld k=%lld n=%lld", (long long)m, (long long)k, (long long)n);
    MS_REQUIRE(group_list != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_gmm: group_list is NULL");
    const size_t need = workspace_need(num_groups);
    MS_REQUIRE(workspace != nullptr && workspace_bytes >= need, MS_ERR_WORKSPACE_TOO_SMALL,
               "ms_gmm: workspace %zu < %zu bytes", workspace_bytes, need);
    MS_REQUIRE((reinterpret_cast<uintptr_t>(workspace) & 7u) == 0, MS_ERR_INVALID_ARGUMENT, "ms_gmm: workspace must be 8-byte aligned");

    // Output extent; nothing to do for an empty output.
    const int64_t out_rows = group_type == 0 ? m : k;       // rows per output block
    const int64_t red_total = group_type == 0 ? k : m;
    if (n == 0 || out_rows == 0) return MS_OK;
    MS_REQUIRE(y != nullptr || swiglu != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_gmm: y is NULL");
    MS_REQUIRE(red_total == 0 || (x != nullptr && weight != nullptr), MS_ERR_INVALID_ARGUMENT, "ms_gmm: NULL operand");
    MS_REQUIRE(y_stride_row >= n, MS_ERR_INVALID_ARGUMENT, "ms_gmm: y_stride_row %lld < n %lld", (long long)y_stride_row, (long long)n);

    // x is [rows, red] for both group types ([m,k] / [k,m]); weight is [red, cols].
    const int64_t a_stride_row = x_stride0, a_stride_red = x_stride1;
    const int64_t b_stride_red = w_stride0, b_stride_col = w_stride1;
    const bool a_red = a_stride_red == 1 || red_total <= 1;
    const bool a_row = a_stride_row == 1 || out_rows <= 1;
    const bool b_red = b_stride_red == 1 || red_total <= 1;
    const bool b_col = b_stride_col == 1 || n <= 1;
    MS_REQUIRE(a_red || a_row, MS_ERR_UNSUPPORTED, "ms_gmm: x needs one unit stride (got %lld, %lld)", (long long)x_stride0, (long long)x_stride1);
    MS_REQUIRE(b_red || b_col, MS_ERR_UNSUPPORTED, "ms_gmm: weight needs one unit stride (got %lld, %lld)", (long long)w_stride0, (long long)w_stride1);

    const bool is32 = dtype == MS_FP32;
    const int num_cus = current_device_cus();
    // fp32: the small tile where the large one would not give every compute unit two tiles
    const int64_t large32 = (group_type == 0 ? ceil_div(m, kTile32Large) + num_groups / 2 : num_groups * ceil_div(k, kTile32Large)) *
                            ceil_div(n, kTile32Large);
    const int tile32 = large32 < 2 * num_cus ? kTile32Small : kTile32Large;
    const int tile_rows = is32 ? tile32 : BM;
    const int tile_cols = is32 ? tile32 : BN;
    // fused SwiGLU form: a tile holds 128 gate and the matching 128 up columns, i.e. 128 activation columns
    const int64_t num_col_tiles = swiglu != nullptr ? ceil_div(n / 2, tile_cols / 2) : ceil_div(n, tile_cols);
    const int64_t row_tiles_bound = group_type == 0 ? ceil_div(m, tile_rows) + num_groups + 2
                                                    : num_groups * (k / tile_rows + 1);
    const int64_t tiles_bound = row_tiles_bound * num_col_tiles;
    MS_REQUIRE(tiles_bound < (1ll << 30), MS_ERR_UNSUPPORTED, "ms_gmm: problem too large (%lld tiles)", (long long)tiles_bound);

    TileTable *table = static_cast<TileTable *>(workspace);
    const int64_t c_stride_group = k * y_stride_row;
    int64_t *b_offsets = nullptr;
    if (weight_offsets != nullptr) {
        b_offsets = reinterpret_cast<int64_t *>(static_cast<char *>(workspace) + offsets_pos(num_groups));
        hipLaunchKernelGGL(gmm_weight_offsets_kernel, dim3(1), dim3(kMaxWeightList), 0, stream, *weight_offsets,
                           static_cast<int>(num_groups), b_offsets);
        MS_CHECK_LAUNCH("gmm_weight_offsets_kernel");
    }
    // Splitting the reduction of small tail tiles needs the larger workspace of ms_gmm_workspace_size_split; with the
    // plain one the launch runs unsplit.
    SplitTail *split_records = nullptr;
    float *split_ws = nullptr;
    if (allow_split && swiglu == nullptr && swiglu_grad == nullptr &&
        may_split_tails(m, k, n, group_type, dtype, out_dtype, accumulate, num_cus) &&
        workspace_bytes >= split_ws_pos(num_groups) + split_ws_bytes(n) &&
        (reinterpret_cast<uintptr_t>(workspace) & 15u) == 0) {
        split_records = reinterpret_cast<SplitTail *>(static_cast<char *>(workspace) + split_records_pos(num_groups));
        split_ws = reinterpret_cast<float *>(static_cast<char *>(workspace) + split_ws_pos(num_groups));
    }
    // whole groups to single XCDs (fast kernels only): room for the lists lies in every workspace of 16 to 512 groups
    // (the split on the reduction dim has a kernel variant with that lookup only for the layout of the weight gradient,
    // both operands contiguous along their outer dims)
    GroupEntry *members = num_groups >= 16 && num_groups <= kMaxListGroups &&
                                  (group_type == 0 || (a_stride_row == 1 && b_stride_col == 1 && a_stride_red != 1 && b_stride_red != 1))
        ? reinterpret_cast<GroupEntry *>(static_cast<char *>(workspace) + members_pos(num_groups)) : nullptr;
    const int64_t slots_per_xcd = launch_slots_per_xcd(group_type, num_groups, m, k, tile_rows, num_col_tiles,
                                                       members != nullptr, split_ws != nullptr);
    MS_REQUIRE(slots_per_xcd < (1ll << 27), MS_ERR_UNSUPPORTED, "ms_gmm: problem too large (%lld slots per XCD)",
               (long long)slots_per_xcd);
    auto schedule = [&](int split_tails) -> int {
        hipLaunchKernelGGL(gmm_schedule_kernel, dim3(1), dim3(256), static_cast<size_t>(num_groups) * sizeof(int64_t),
                           stream, group_list, group_list_type, group_type, static_cast<int>(num_groups),
                           static_cast<int>(m), static_cast<int>(k), tile_rows, static_cast<int>(num_col_tiles),
                           split_tails, kTailsLastRounds * num_cus, w_stride_group, c_stride_group, b_offsets, table,
                           split_tails ? split_records : nullptr, static_cast<int>(n), num_cus,
                           split_tails ? members : nullptr, static_cast<int>(slots_per_xcd));
        MS_CHECK_LAUNCH("gmm_schedule_kernel");
        return MS_OK;
    };

    GmmArgs args{};
    args.a = x;
    args.b = weight;
    args.c = y;
    args.table = table;
    args.a_stride_row = a_stride_row;
    args.a_stride_red = a_stride_red;
    args.b_stride_red = b_stride_red;
    args.b_stride_col = b_stride_col;
    args.c_stride_row = y_stride_row;
    args.cols = static_cast<int>(n);
    args.num_col_tiles = static_cast<int>(num_col_tiles);
    const unsigned grid = static_cast<unsigned>(slots_per_xcd * 8);

    if (swiglu != nullptr) {
        args.cols = static_cast<int>(n / 2);
        args.act = swiglu->act;
        args.act_stride_row = swiglu->act_stride_row;
        args.probs = swiglu->probs;
        args.probs_dtype = swiglu->probs_dtype;
    }
    if (is32) {
        MS_REQUIRE(swiglu == nullptr, MS_ERR_UNSUPPORTED, "ms_gmm_swiglu: 16-bit dtypes only");
        if (int rc = schedule(0)) return rc;
        if (tile32 == kTile32Large) {
            if (accumulate) hipLaunchKernelGGL((gmm32_kernel<true, 2>), dim3(grid), dim3(256), 0, stream, args);
            else hipLaunchKernelGGL((gmm32_kernel<false, 2>), dim3(grid), dim3(256), 0, stream, args);
        } else {
            if (accumulate) hipLaunchKernelGGL((gmm32_kernel<true, 1>), dim3(grid), dim3(256), 0, stream, args);
            else hipLaunchKernelGGL((gmm32_kernel<false, 1>), dim3(grid), dim3(256), 0, stream, args);
        }
        MS_CHECK_LAUNCH("gmm32_kernel");
        return MS_OK;
    }

    // 16-byte vector eligibility of each operand.
    const bool use_a_red = a_stride_red == 1;  // prefer the reduction-contiguous reading when both hold
    const bool use_b_red = b_stride_red == 1;
    const int64_t a_other = use_a_red ? a_stride_row : a_stride_red;
    const int64_t b_other = use_b_red ? b_stride_col : b_stride_red;
    args.a_vec_ok = aligned16(x) && a_other % 8 == 0;
    args.b_vec_ok = weight_offsets != nullptr ? (all_weights_aligned16 && b_other % 8 == 0)
                                              : (aligned16(weight) && b_other % 8 == 0 && w_stride_group % 8 == 0);
    const int out_size = out_dtype == MS_FP32 ? 4 : 2;
    args.c_vec_ok = (reinterpret_cast<uintptr_t>(y) % (4 * out_size) == 0) && y_stride_row % 4 == 0 &&
                    (group_type == 0 || c_stride_group % 4 == 0);
    if (swiglu != nullptr)   // 16-byte row stores of both outputs, whole 8-column chunks in each half
        args.c_vec_ok = aligned16(y) && y_stride_row % 8 == 0 && aligned16(swiglu->act) &&
                        swiglu->act_stride_row % 8 == 0 && (n / 2) % 8 == 0;
    if (swiglu_grad != nullptr) {
        args.c_vec_ok = aligned16(y) && y_stride_row % 8 == 0 && aligned16(swiglu_grad->fc1) &&
                        swiglu_grad->fc1_stride_row % 8 == 0 && n % 8 == 0;
        args.fc1 = swiglu_grad->fc1;
        args.fc1_stride_row = swiglu_grad->fc1_stride_row;
        args.probs = swiglu_grad->probs;
        args.probs_dtype = swiglu_grad->probs_dtype;
        args.partials = swiglu_grad->partials;
        args.partials_per_row = swiglu_grad->partials_per_row;
    }
    // A stride of 1 in a dim of extent 1 may come with an arbitrary other stride.
    const bool a_is_red = use_a_red || !a_row;
    const bool b_is_red = use_b_red || !b_col;
    if (!use_a_red && a_stride_row != 1) args.a_vec_ok = 0;
    if (!use_b_red && b_stride_col != 1) args.b_vec_ok = 0;

    const int out = accumulate ? ACC_F32 : (out_dtype == MS_FP32 ? OUT_F32 : OUT_SAME);
    // The fast kernels need 16-byte vector access everywhere: aligned bases, strides in multiples of 8
    // elements, whole 8-element chunks along every contiguous dim, and (for operands contiguous along the
    // reduction dim) reduction ranges that start at multiples of 8, i.e. no split on the reduction dim.
    const bool a_truly_contig = a_is_red ? a_stride_red == 1 : a_stride_row == 1;
    const bool b_truly_contig = b_is_red ? b_stride_red == 1 : b_stride_col == 1;
    bool fast = args.a_vec_ok && args.b_vec_ok && args.c_vec_ok && a_truly_contig && b_truly_contig;
    // An operand that is contiguous along its outer dim is fetched in whole 8-index chunks clamped to the end of the
    // tile's row range, so that range must be the full, 8-aligned extent: for x that only holds when the split is on
    // the reduction dim (with a split on rows the groups' row ranges start and end anywhere).
    if (a_is_red) fast = fast && red_total % 8 == 0 && group_type == 0;
    else fast = fast && group_type == 2 && out_rows % 8 == 0 && out_rows >= 8;
    if (b_is_red) fast = fast && red_total % 8 == 0 && group_type == 0; else fast = fast && n % 8 == 0 && n >= 8;
    // the epilogue writes 16 bytes per lane: 8 columns of a 16-bit output, 4 of an fp32 one
    fast = fast && (out_dtype == MS_FP32 ? n % 4 == 0 && reinterpret_cast<uintptr_t>(y) % 16 == 0
                                         : n % 8 == 0 && aligned16(y) && y_stride_row % 8 == 0);
    // per-lane global offsets are 32-bit byte offsets inside one 256 x 64 operand tile
    const int64_t a_span = a_is_red ? 256 * a_stride_row : 64 * a_stride_red;
    const int64_t b_span = b_is_red ? 256 * b_stride_col : 64 * b_stride_red;
    fast = fast && a_span < (1ll << 30) && b_span < (1ll << 30);
    if (swiglu != nullptr) {
        MS_REQUIRE(fast && a_is_red && !b_is_red, MS_ERR_UNSUPPORTED,
                   "ms_gmm_swiglu: needs the vector-access layout (16-byte aligned operands and outputs, x contiguous "
                   "along k, weight contiguous along its columns, k and ffn multiples of 8)");
        if (int rc = schedule(1)) return rc;
        return launch_gmm16_fast(stream, args, dtype, OUT_SWIGLU, true, false, grid);
    }
    if (swiglu_grad != nullptr) {
        MS_REQUIRE(fast && a_is_red && b_is_red, MS_ERR_UNSUPPORTED,
                   "ms_gmm_swiglu_grad: needs the vector-access layout (16-byte aligned operands and outputs, dy and the "
                   "transposed weight view contiguous along k, k and ffn multiples of 8)");
        if (int rc = schedule(1)) return rc;
        return launch_gmm16_fast(stream, args, dtype, OUT_SWIGLU_GRAD, true, true, grid);
    }
    if (int rc = schedule(fast ? 1 : 0)) return rc;
    if (fast) {
        args.split_ws = split_ws;
        if (int rc = launch_gmm16_fast(stream, args, dtype, out, a_is_red, b_is_red, grid, members != nullptr)) return rc;
        if (split_ws != nullptr) {
            // at most kSplitCus / (2 parts x column tiles) tails are ever split in one launch
            const int64_t max_tails = kSplitCus / (2 * num_col_tiles) < num_groups ? kSplitCus / (2 * num_col_tiles) : num_groups;
            const dim3 rgrid(static_cast<unsigned>(max_tails), static_cast<unsigned>(ceil_div(n, 2048)), 16);
            if (dtype == MS_BF16)
                hipLaunchKernelGGL(gmm_split_reduce_kernel<MS_BF16>, rgrid, dim3(256), 0, stream, table, split_records,
                                   split_ws, static_cast<uint16_t *>(y), y_stride_row, static_cast<int>(n));
            else
                hipLaunchKernelGGL(gmm_split_reduce_kernel<MS_FP16>, rgrid, dim3(256), 0, stream, table, split_records,
                                   split_ws, static_cast<uint16_t *>(y), y_stride_row, static_cast<int>(n));
            MS_CHECK_LAUNCH("gmm_split_reduce_kernel");
        }
        return MS_OK;
    }
    if (dtype == MS_BF16) {
        if (out == OUT_SAME) return launch16<MS_BF16, OUT_SAME>(stream, args, a_is_red, b_is_red, grid);
        if (out == OUT_F32) return launch16<MS_BF16, OUT_F32>(stream, args, a_is_red, b_is_red, grid);
        return launch16<MS_BF16, ACC_F32>(stream, args, a_is_red, b_is_red, grid);
    }
    if (out == OUT_SAME) return launch16<MS_FP16, OUT_SAME>(stream, args, a_is_red, b_is_red, grid);
    if (out == OUT_F32) return launch16<MS_FP16, OUT_F32>(stream, args, a_is_red, b_is_red, grid);
    return launch16<MS_FP16, ACC_F32>(stream, args, a_is_red, b_is_red, grid);
}

extern "C" int ms_gmm(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1, const void *weight,
                      int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1, void *y, int64_t y_stride_row,
                      const int64_t *group_list, int group_list_type, int group_type, int64_t num_groups, int64_t m,
                      int64_t k, int64_t n, int dtype, int out_dtype, int accumulate, void *workspace,
                      size_t workspace_bytes) {
    return gmm_impl(stream, x, x_stride0, x_stride1, weight, w_stride_group, w_stride0, w_stride1, y, y_stride_row,
                    group_list, group_list_type, group_type, num_groups, m, k, n, dtype, out_dtype, accumulate,
                    workspace, workspace_bytes, nullptr, false);
}

// ---- the entry point that allocates nothing -------------------------------------------------------------
// The tile table that ms_gmm takes through its workspace argument lives here in a fixed device array, one copy per
// GPU.  In host code the array's name is only a handle for hipGetSymbolAddress; kernels get the address that call
// returned, looked up once per device.
constexpr int kNoAllocMaxGroups = 1024;
// (the need is largest either for the most groups or for the most groups that may get per-XCD lists)
constexpr size_t kScratchNeed = workspace_need(kNoAllocMaxGroups) > workspace_need(kMaxListGroups)
    ? workspace_need(kNoAllocMaxGroups) : workspace_need(kMaxListGroups);
constexpr size_t kScratchBytes = (kScratchNeed + 255) & ~static_cast<size_t>(255);
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {
constexpr int kMaxDevices = 64;
int scratch_of_current_device(void **out) {
    static std::mutex mu;
    static void *ptrs[kMaxDevices] = {};
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm_noalloc: hipGetDevice: %s", hipGetErrorString(e));
    MS_REQUIRE(dev >= 0 && dev < kMaxDevices, MS_ERR_UNSUPPORTED, "ms_gmm_noalloc: device ordinal %d outside [0, %d)", dev,
               kMaxDevices);
    std::lock_guard<std::mutex> lock(mu);
    if (ptrs[dev] == nullptr) {
        void *p = nullptr;
        e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
        MS_REQUIRE(e == hipSuccess && p != nullptr, MS_ERR_HIP, "ms_gmm_noalloc: hipGetSymbolAddress: %s",
                   hipGetErrorString(e));
        ptrs[dev] = p;
    }
    *out = ptrs[dev];
    return MS_OK;
}
}  // namespace

extern "C" int ms_gmm_noalloc(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1, const void *weight,
                              int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1, void *y, int64_t y_stride_row,
                              const int64_t *group_list, int group_list_type, int group_type, int64_t num_groups,
                              int64_t m, int64_t k, int64_t n, int dtype, int out_dtype, int accumulate) {
    MS_REQUIRE(num_groups >= 1 && num_groups <= kNoAllocMaxGroups, MS_ERR_UNSUPPORTED,
               "ms_gmm_noalloc: num_groups %lld outside [1, %d] (the fixed tile-table buffer holds no more; use ms_gmm "
               "with a caller-provided workspace beyond that)", (long long)num_groups, kNoAllocMaxGroups);
    void *table = nullptr;
    if (int rc = scratch_of_current_device(&table)) return rc;
    return gmm_impl(stream, x, x_stride0, x_stride1, weight, w_stride_group, w_stride0, w_stride1, y, y_stride_row,
                    group_list, group_list_type, group_type, num_groups, m, k, n, dtype, out_dtype, accumulate, table,
                    kScratchBytes, nullptr, false, nullptr, nullptr, /*allow_split=*/false);
}

extern "C" int ms_gmm_swiglu(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1, const void *weight,
                             int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1, void *y, int64_t y_stride_row,
                             void *act, int64_t act_stride_row, const void *probs, int probs_dtype,
                             const int64_t *group_list, int group_list_type, int64_t num_groups, int64_t m, int64_t k,
                             int64_t ffn, int dtype, void *workspace, size_t workspace_bytes) {
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16, MS_ERR_UNSUPPORTED, "ms_gmm_swiglu: dtype must be bf16 or fp16");
    MS_REQUIRE(ffn >= 0 && ffn < (1ll << 30), MS_ERR_INVALID_ARGUMENT, "ms_gmm_swiglu: bad ffn %lld", (long long)ffn);
    MS_REQUIRE(act != nullptr || m == 0 || ffn == 0, MS_ERR_INVALID_ARGUMENT, "ms_gmm_swiglu: act is NULL");
    MS_REQUIRE(act_stride_row >= ffn, MS_ERR_INVALID_ARGUMENT, "ms_gmm_swiglu: act_stride_row %lld < ffn %lld",
               (long long)act_stride_row, (long long)ffn);
    MS_REQUIRE(probs == nullptr || probs_dtype == MS_BF16 || probs_dtype == MS_FP16 || probs_dtype == MS_FP32,
               MS_ERR_UNSUPPORTED, "ms_gmm_swiglu: probs dtype %d is not one of bf16/fp16/fp32", probs_dtype);
    const SwigluOut extra{act, act_stride_row, probs, probs_dtype};
    return gmm_impl(stream, x, x_stride0, x_stride1, weight, w_stride_group, w_stride0, w_stride1, y,
                    y != nullptr ? y_stride_row : 2 * ffn, group_list, group_list_type, /*group_type=*/0, num_groups, m, k,
                    2 * ffn, dtype, dtype, /*accumulate=*/0, workspace, workspace_bytes, nullptr, false, &extra);
}

namespace {
int64_t swiglu_partials_per_row(int64_t ffn) { return (ffn + 63) / 64; }
size_t swiglu_grad_partials_pos(int64_t num_groups) { return (workspace_need(num_groups) + 255) & ~static_cast<size_t>(255); }
}  // namespace

extern "C" int ms_gmm_swiglu_grad_workspace_size(int64_t num_groups, int64_t m, int64_t ffn, size_t *bytes) {
    MS_REQUIRE(bytes != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_gmm_swiglu_grad_workspace_size: bytes is NULL");
    MS_REQUIRE(num_groups >= 1 && num_groups <= kMaxGroups && m >= 0 && ffn >= 0, MS_ERR_INVALID_ARGUMENT,
               "ms_gmm_swiglu_grad_workspace_size: bad sizes");
    *bytes = swiglu_grad_partials_pos(num_groups) +
             ((static_cast<size_t>(m) * swiglu_partials_per_row(ffn) * sizeof(float) + 255) & ~static_cast<size_t>(255));
    return MS_OK;
}

extern "C" int ms_gmm_swiglu_grad(ms_stream_t stream, const void *dy, int64_t dy_stride0, int64_t dy_stride1,
                                  const void *weight, int64_t w_stride_group, int64_t w_stride0, int64_t w_stride1,
                                  const void *fc1, int64_t fc1_stride_row, const void *probs, int probs_dtype,
                                  void *d_fc1, int64_t d_fc1_stride_row, void *grad_probs, const int64_t *group_list,
                                  int group_list_type, int64_t num_groups, int64_t m, int64_t k, int64_t ffn, int dtype,
                                  void *workspace, size_t workspace_bytes) {
    const char *fn = "ms_gmm_swiglu_grad";
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16, MS_ERR_UNSUPPORTED, "%s: dtype must be bf16 or fp16", fn);
    MS_REQUIRE(ffn >= 0 && ffn < (1ll << 30) && m >= 0, MS_ERR_INVALID_ARGUMENT, "%s: bad sizes", fn);
    MS_REQUIRE(num_groups >= 1 && num_groups <= kMaxGroups, MS_ERR_UNSUPPORTED, "%s: num_groups %lld outside [1, %d]", fn,
               (long long)num_groups, kMaxGroups);
    MS_REQUIRE((probs == nullptr) == (grad_probs == nullptr), MS_ERR_INVALID_ARGUMENT,
               "%s: probs and grad_probs must be given together", fn);
    MS_REQUIRE(probs == nullptr || probs_dtype == MS_BF16 || probs_dtype == MS_FP16 || probs_dtype == MS_FP32,
               MS_ERR_UNSUPPORTED, "%s: probs dtype %d is not one of bf16/fp16/fp32", fn, probs_dtype);
    if (m == 0 || ffn == 0) return MS_OK;
    MS_REQUIRE(fc1 != nullptr && d_fc1 != nullptr, MS_ERR_INVALID_ARGUMENT, "%s: NULL tensor pointer", fn);
    MS_REQUIRE(fc1_stride_row >= 2 * ffn && d_fc1_stride_row >= 2 * ffn, MS_ERR_INVALID_ARGUMENT,
               "%s: fc1 / d_fc1 row strides must be at least 2*ffn", fn);
    size_t need = 0;
    if (int rc = ms_gmm_swiglu_grad_workspace_size(num_groups, m, ffn, &need)) return rc;
    MS_REQUIRE(workspace != nullptr && workspace_bytes >= need, MS_ERR_WORKSPACE_TOO_SMALL, "%s: workspace %zu < %zu bytes",
               fn, workspace_bytes, need);
    const int per_row = static_cast<int>(swiglu_partials_per_row(ffn));
    float *partials = grad_probs != nullptr
        ? reinterpret_cast<float *>(static_cast<char *>(workspace) + swiglu_grad_partials_pos(num_groups)) : nullptr;
    const SwigluGradIn extra{fc1, fc1_stride_row, probs, probs_dtype, partials, per_row};
    if (int rc = gmm_impl(stream, dy, dy_stride0, dy_stride1, weight, w_stride_group, w_stride0, w_stride1, d_fc1,
                          d_fc1_stride_row, group_list, group_list_type, /*group_type=*/0, num_groups, m, k, ffn, dtype,
                          dtype, /*accumulate=*/0, workspace, workspace_bytes, nullptr, false, nullptr, &extra))
        return rc;
    if (grad_probs != nullptr) {
        hipLaunchKernelGGL(swiglu_grad_probs_kernel, dim3(static_cast<unsigned>(ceil_div(m, 4))), dim3(256), 0,
                           static_cast<hipStream_t>(stream), partials, per_row, static_cast<int>(m), grad_probs, probs_dtype);
        MS_CHECK_LAUNCH("swiglu_grad_probs_kernel");
    }
    return MS_OK;
}

extern "C" int ms_gmm_weight_list(ms_stream_t stream, const void *x, int64_t x_stride0, int64_t x_stride1,
                                  const void *const *weights, int64_t w_stride0, int64_t w_stride1, void *y,
                                  int64_t y_stride_row, const int64_t *group_list, int group_list_type,
                                  int64_t num_groups, int64_t m, int64_t k, int64_t n, int dtype, int out_dtype,
                                  void *workspace, size_t workspace_bytes) {
    MS_REQUIRE(num_groups >= 1 && num_groups <= kMaxWeightList, MS_ERR_UNSUPPORTED,
               "ms_gmm_weight_list: num_groups %lld outside [1, %d] (stack the weights and use ms_gmm beyond that)",
               (long long)num_groups, kMaxWeightList);
    MS_REQUIRE(weights != nullptr, MS_ERR_INVALID_ARGUMENT, "ms_gmm_weight_list: weights is NULL");
    MS_REQUIRE(dtype == MS_BF16 || dtype == MS_FP16 || dtype == MS_FP32, MS_ERR_UNSUPPORTED,
               "ms_gmm_weight_list: bad dtype %d", dtype);
    const int64_t elem = dtype == MS_FP32 ? 4 : 2;
    WeightOffsets off{};
    bool aligned = true;
    for (int64_t g = 0; g < num_groups; ++g) {
        MS_REQUIRE(weights[g] != nullptr || k == 0 || n == 0, MS_ERR_INVALID_ARGUMENT,
                   "ms_gmm_weight_list: weights[%lld] is NULL", (long long)g);
        const int64_t delta = static_cast<const char *>(weights[g]) - static_cast<const char *>(weights[0]);
        MS_REQUIRE(delta % elem == 0, MS_ERR_INVALID_ARGUMENT,
                   "ms_gmm_weight_list: weights[%lld] is not element-aligned relative to weights[0]", (long long)g);
        off.v[g] = delta / elem;
        aligned = aligned && aligned16(weights[g]);
    }
    return gmm_impl(stream, x, x_stride0, x_stride1, weights[0], 0, w_stride0, w_stride1, y, y_stride_row, group_list,
                    group_list_type, /*group_type=*/0, num_groups, m, k, n, dtype, out_dtype, /*accumulate=*/0,
                    workspace, workspace_bytes, &off, aligned);
}
