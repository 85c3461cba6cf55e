// Declarations shared by the grouped-matmul translation units.
#pragma once

#include "common.h"

namespace ms {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

constexpr int kMaxGroups = 4096;

struct GroupEntry {
    int row_begin, row_end;  // output rows of the group
    int red_begin, red_end;  // reduction range of the group
    int tile_begin;          // first slot of this group in every XCD's slot sequence
    int num_row_tiles;
    int tile_rows;           // rows per full tile
    int tail_rows;           // rows of the group's last row tile if it is a smaller one (64 / 128), else 0
    int num_tiles;           // num_row_tiles * column tiles
    int share;               // ceil(num_tiles / 8): tiles of this group handled by each XCD
    int split;               // 0, or 1 + the part number of a small tail tile whose reduction is split: such a
                             // tile writes fp32 partial sums to the split workspace (c_off then points there)
    int whole;               // entry of an XCD's own list: 1 = that XCD takes all tiles of the group, 0 = its eighth
    int64_t b_off;           // element offset of the group's weight block
    int64_t c_off;           // element offset of the group's output block
};

// One small tail tile row whose reduction was split into `parts` ranges: the partial sums of part s and local row r
// are row (pair0 + s) * kSplitRows + r of the split workspace ([.., cols] fp32).
struct SplitTail {
    int row_begin, rows;
    int pair0, parts;
};
constexpr int kSplitRows = 128;          // rows reserved per (tail, part) pair: the largest small tile
constexpr int kMaxSplit = 4;             // most parts a reduction is split into
constexpr int kSplitCus = 256;           // a launch's split parts never number more than this (one round of MI355X's CUs)
constexpr int kSplitMinRed = 2048;       // shortest reduction range worth a part of its own
constexpr int kMaxListGroups = 256;      // most groups that may be dealt out whole to single XCDs (ranked by counting,
                                         // dealt out by one thread)

struct TileTable {
    int slots_per_xcd;       // sum of the entries' shares
    int num_entries;
    int num_split_tails;     // tail tile rows whose reduction was split (entries of the SplitTail array in use)
    int lists_off;           // 0, or the byte offset from the table to eight lists of entries, one per XCD (whole groups
                             // dealt out to single XCDs); `entries` is then unused
    int list_stride;         // entries reserved per list
    int pad[3];
    int zeros[8];            // always zero: source of out-of-range operand chunks (holds an aligned 16-byte block)
    int begins[16];          // tile_begin of the first 16 entries (INT_MAX past the last): one load finds the entry
    int list_count[8];       // entries in use in every XCD's list
    GroupEntry entries[1];
};

struct GmmArgs {
    const void *a;
    const void *b;
    void *c;
    const TileTable *table;
    int64_t a_stride_row, a_stride_red;
    int64_t b_stride_red, b_stride_col;
    int64_t c_stride_row;
    int cols;          // n (fused SwiGLU form: the number of activation columns, ffn = n / 2)
    int num_col_tiles;
    int a_vec_ok, b_vec_ok, c_vec_ok;
    // fused SwiGLU form only (OUT_SWIGLU): second output and the per-row factor
    void *act;                 // [rows, cols] activation output, same dtype
    int64_t act_stride_row;
    const void *probs;         // optional per-row probability
    int probs_dtype;
    // fused SwiGLU backward form only (OUT_SWIGLU_GRAD): c is d_fc1 [rows, 2*cols]
    const void *fc1;           // [rows, 2*cols] saved output of the first matmul (gate | up)
    int64_t fc1_stride_row;
    float *partials;           // [rows, partials_per_row] row sums of dact * silu(gate) * up per 64 columns, or NULL
    int partials_per_row;
    // split tail tiles only (OUT_SAME): fp32 partial sums, rows of `cols` floats
    float *split_ws;
};

struct TileCoord {
    GroupEntry e;
    int row_tile, col_tile;
    int tile_rows;           // rows of this tile (the entry's tile_rows, or its tail_rows for the last row tile)
    bool valid;
};

// Tile order inside a group of R row tiles x C column panels: the r-th tile the kernels take.  Column panels in sets of
// 8, row tiles in sets of 4, row-tile-fastest inside such a 4 x 8 block.  The 32 compute units of an XCD then work on
// one block at a time and fetch 4 + 8 operand panels for 32 tiles; with many row tiles (the weight gradient: hidden /
// 256 of them) plain row-tile-fastest order would have them on 16 x 2 tiles and fetch 18.  Up to 4 row tiles per group
// the two orders are the same.  A single row tile left over after the blocks of 4 (a group of 5 or 9 row tiles:
// typically the small tail tile of a ragged group) joins the last block instead of forming one of its own, so it runs
// beside the tiles whose column panels it shares (measured: 0.2 to 0.4 % per layer step).
__host__ __device__ __forceinline__ void tile_order(int r, int R, int C, int &row_tile, int &col_tile) {
    constexpr int BR = 4, BC = 8;      // measured against 8 x 4, 8 x 8, 2 x 16 and 4 x 16: the fastest for all three products
    const int cg = r / (BC * R);
    const int rem = r - cg * BC * R;
    const int wc = C - BC * cg < BC ? C - BC * cg : BC;    // column panels in this set
    int nb = (R + BR - 1) / BR;
    if (R > BR && R % BR == 1) nb -= 1;                     // a single left-over row tile joins the block before it
    int rb = rem / (BR * wc);
    rb = rb > nb - 1 ? nb - 1 : rb;
    const int rem2 = rem - rb * BR * wc;
    const int hr = rb == nb - 1 ? R - BR * rb : BR;        // row tiles in this block
    const int lc = rem2 / hr;
    col_tile = BC * cg + lc;
    row_tile = BR * rb + (rem2 - lc * hr);
}

// Map this workgroup to its tile.  Workgroup b runs on XCD b % 8 (round-robin dispatch) and takes slot
// b / 8 of that XCD's slot sequence.  Normally every XCD walks the groups in the same order and owns one contiguous
// eighth of each group's tiles (in the blocked order above), so concurrently running
// workgroups of an XCD share operand panels in that XCD's L2, and every XCD gets an equal part of every
// group however unequal the groups are.  With many groups the schedule may instead deal whole groups out to single
// XCDs (every XCD then has a list of its own): a group's operands are fetched into one L2 instead of eight.
// LISTS: the kernel may meet per-XCD lists (the fast kernels of the split on rows); the others are compiled without that
// path, which costs the weight-gradient kernel 0.3 us per tile at its start when it is merely present.
template <bool LISTS>
__device__ __forceinline__ TileCoord locate_tile(const TileTable *table) {
    TileCoord tc;
    tc.valid = false;
    const int xcd = blockIdx.x & 7;
    const int slot = blockIdx.x >> 3;
    if (slot >= table->slots_per_xcd) return tc;
    if (LISTS && table->num_entries == 0) {     // per-XCD lists (the common table is empty then); no further header
                                                // field is read on the way to the common case
        const GroupEntry *list = reinterpret_cast<const GroupEntry *>(reinterpret_cast<const char *>(table) + table->lists_off) +
                                 static_cast<int64_t>(xcd) * table->list_stride;
        int lo = 0, hi = table->list_count[xcd];
        if (hi == 0) return tc;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (list[mid].tile_begin <= slot) lo = mid; else hi = mid;
        }
        tc.e = list[lo];
        const int r = slot - tc.e.tile_begin + (tc.e.whole != 0 ? 0 : xcd * tc.e.share);
        if (r >= tc.e.num_tiles || (tc.e.whole == 0 && slot - tc.e.tile_begin >= tc.e.share)) return tc;
        tile_order(r, tc.e.num_row_tiles, tc.e.num_tiles / tc.e.num_row_tiles, tc.row_tile, tc.col_tile);
        tc.tile_rows = (tc.e.tail_rows != 0 && tc.row_tile == tc.e.num_row_tiles - 1) ? tc.e.tail_rows : tc.e.tile_rows;
        tc.valid = true;
        return tc;
    }
    // last entry with tile_begin <= slot.  Up to 16 entries (8 experts with their tail tiles) their begins lie in the
    // table's header and are fetched at once, instead of one dependent load per step of a binary search.
    int lo = 0;
    if (table->num_entries <= 16) {
#pragma unroll
        for (int i = 1; i < 16; ++i) lo += table->begins[i] <= slot ? 1 : 0;
    } else {
        int hi = table->num_entries;
        while (hi - lo > 1) {
            const int mid = (lo + hi) >> 1;
            if (table->entries[mid].tile_begin <= slot) lo = mid; else hi = mid;
        }
    }
    tc.e = table->entries[lo];
    const int r = xcd * tc.e.share + (slot - tc.e.tile_begin);
    if (r >= tc.e.num_tiles) return tc;
    tile_order(r, tc.e.num_row_tiles, tc.e.num_tiles / tc.e.num_row_tiles, tc.row_tile, tc.col_tile);
    tc.tile_rows = (tc.e.tail_rows != 0 && tc.row_tile == tc.e.num_row_tiles - 1) ? tc.e.tail_rows : tc.e.tile_rows;
    tc.valid = true;
    return tc;
}

constexpr int BM = 256, BN = 256, BK = 64;
constexpr int kTileBytes = BM * BK * 2;                 // 32 KB per operand per stage
constexpr int kLdsBytes16 = 4 * kTileBytes;             // A,B x 2 stages = 128 KB

enum OutMode { OUT_SAME = 0, OUT_F32 = 1, ACC_F32 = 2, OUT_SWIGLU = 3, OUT_SWIGLU_GRAD = 4 };

template <int DT>
__device__ __forceinline__ f32x16 mfma16(v16 a, v16 b, f32x16 c) {
    if constexpr (DT == MS_BF16) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c,
                                                       0, 0, 0);
    } else {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a), __builtin_bit_cast(f16x8, b), c, 0,
                                                      0, 0);
    }
}

// LDS swizzle: 16-byte chunk position of (row, chunk) inside the row's 128 bytes.
__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }


// Fast 16-bit kernels (gmm_fast.hip).  Returns MS_OK after launching, or -1 if
// this problem does not meet the fast kernels' alignment conditions.
// lists: the table may come as per-XCD lists (only asked of the weight-gradient product, whose common kernel is compiled
// without that lookup; the kernels of the split on rows always have it).
int launch_gmm16_fast(hipStream_t stream, const GmmArgs &args, int dtype, int out_mode, bool a_red, bool b_red,
                      unsigned grid, bool lists = false);

}  // namespace ms
