// Fast path of the 16-bit grouped matmul for gfx950: 256x256x64 macro tile per
// 256-thread workgroup (2x2 wavefronts, 128x128 per wavefront = 4x4
// v_mfma_f32_32x32x16), for problems whose pointers and strides allow 16-byte
// vector access everywhere.  All edge handling is branch-free (clamped addresses,
// zero masks on the reduction tail).  The last row tile of a group may be a
// 128x256 or 64x256 tile (1x4 wavefronts of 128x64 / 64x64) so that ragged
// groups do not pay for a full 256-row tile; the tile table says which.
//
// LDS layout per operand tile
//   * operand contiguous along the reduction dim in memory ("RED"): stored as
//     [outer][64 reduction] rows of 128 bytes with an XOR swizzle of the 16-byte
//     chunks; MFMA fragments are read with ds_read_b128 (bank-conflict free).
//   * operand contiguous along the outer dim (row of A / column of B): stored as it
//     lies in memory, [64 reduction][256 outer] with a row pitch of 576 bytes, and the
//     MFMA fragments (8 consecutive reduction values per lane) are produced by the
//     transposing LDS read ds_read_b64_tr_b16.  No register transposition, and the
//     global loads stay fully coalesced (32 lanes x 16 bytes per memory row).
//
// K loop, software-pipelined by hand so that global loads are in flight all the time:
//   registers hold tile kt+1 (loaded one K step ago), LDS stage `cur` holds tile kt.
//   step kt, phase p = 0..3 (one 16-wide slice of the 64-wide K step each):
//       store part p of tile kt+1 from registers to LDS stage `nxt`
//       issue the global loads of part p of tile kt+2 into the same registers
//       read the MFMA fragments of slice p+1 from LDS stage `cur`
//       16 MFMAs on the fragments of slice p
//   (parts: loads 0-3 / 4-7 of A, loads 0-3 / 4-7 of B, of each lane's eight per operand)
//   in phase 3 a workgroup barrier sits between the two halves of the MFMAs; after it
//   the fragments of slice 0 of tile kt+1 are read from stage `nxt`.
// Every load therefore has a full K step (64 MFMAs per wavefront) to arrive, and the
// vector memory path sees a steady request stream instead of one burst per step.
#include <type_traits>
#include <utility>

#include "gmm_common.h"

#ifdef MS_TRACE_TILES
// Diagnostic build only (python -m mindspeed_amd.build --trace): every workgroup of the fast kernels records when it
// started, found its tile, had its first operands in LDS, left the K loop and finished (100 MHz wall clock), plus the
// compute unit it ran on; ms_trace_read copies the records of the last launches out.  The record of workgroup b is
// slot b % kTraceSlots, so a launch with more workgroups than that overwrites its own early records.
namespace ms {
constexpr int kTraceSlots = 16384;
__device__ long long g_tile_trace[kTraceSlots * 8];
}  // namespace ms
#define MS_TRACE(i) do { if (threadIdx.x == 0) ms::g_tile_trace[(blockIdx.x % ms::kTraceSlots) * 8 + (i)] = wall_clock64(); } while (0)
#else
#define MS_TRACE(i)
#endif

namespace ms {
namespace {

// Instruction-class masks of __builtin_amdgcn_sched_group_barrier.
constexpr int SG_MFMA = 0x008, SG_VMEM_RD = 0x020, SG_DS_RD = 0x100, SG_DS_WR = 0x200;

template <int MASK, int N, int ID>
__device__ __forceinline__ void sg() {
    if constexpr (N > 0) __builtin_amdgcn_sched_group_barrier(MASK, N, ID);
}

// Bytes of one operand tile in LDS.  RED: [ROWS outer][64 reduction] x 2 bytes.  !RED: [64 reduction][ROWS outer]
// x 2 bytes with 64 bytes of padding per row (pitch mod 256 == 64 keeps the transposing reads conflict-free).
template <bool RED, int ROWS>
constexpr int tile_bytes() { return RED ? ROWS * 128 : 64 * (ROWS * 2 + 64); }
constexpr int kRedTileBytes = tile_bytes<true, 256>();
constexpr int kOuterTileBytes = tile_bytes<false, 256>();

constexpr int kStagePitch = 264;                          // epilogue staging: 128 x 2 bytes + 8 bytes pad
constexpr int kStagePerWave = 128 * kStagePitch;          // one 128 x 128 16-bit block per wavefront
constexpr int kStageBytes = 4 * kStagePerWave;

typedef short s16x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint2 lds_read_tr(const char *p) {
    const s16x4 v = __builtin_amdgcn_ds_read_tr16_b64_v4i16(
        (__attribute__((address_space(3))) s16x4 *)(p));
    return __builtin_bit_cast(uint2, v);
}

// One operand of the macro tile (ROWS outer indices x 64 reduction indices):
// global -> registers -> LDS, and LDS -> MFMA fragments.
template <bool RED, int ROWS>
struct Operand {
    static constexpr int NL = ROWS / 32;          // 16-byte loads per lane per K step (8, 4 or 2)
    static constexpr int PITCH = ROWS * 2 + 64;   // !RED: bytes per reduction row in LDS
    static constexpr int CP = ROWS / 8;           // !RED: 16-byte chunks per reduction row
    static constexpr int RP = 256 / CP;           // !RED: reduction rows covered by one load of the workgroup
    unsigned off[NL];   // per-lane global byte offsets of the loads, relative to the tile's base pointer
    unsigned off0;      // !RED: offset of (reduction index 0, this lane's outer chunk), always valid
    unsigned st_off;    // byte offset of this lane's first LDS store inside the tile
    unsigned frag_off;  // byte offset of this lane's fragment reads inside the tile
    v16 r[NL];

    // outer0: first outer index of the tile; outer_last: clamp bound (RED: last valid outer index,
    // !RED: last valid start of an 8-wide chunk); wave_outer: this wavefront's first outer index in the tile.
    // split (only for !RED, fused SwiGLU form): the second half of the tile's outer indices lies `split`
    // elements further on in memory than the first half's continuation would (gate columns c0 .. c0+127 and
    // up columns ffn+c0 .. ffn+c0+127 side by side in one tile: split = ffn - ROWS/2), with the clamp bound
    // moved along by ffn.
    __device__ __forceinline__ void init(int64_t stride_outer, int64_t stride_red, int outer0, int outer_last,
                                         int wave_outer, int split = 0, int split_last = 0) {
        const int tid = threadIdx.x;
        const int lane = tid & 63;
        if constexpr (RED) {
            const int ck = tid & 7;
            const int row = tid >> 3;
#pragma unroll
            for (int i = 0; i < NL; ++i) {
                int outer = outer0 + row + 32 * i;
                outer = outer > outer_last ? outer_last : outer;
                off[i] = static_cast<unsigned>((static_cast<int64_t>(outer - outer0) * stride_outer + ck * 8) * 2);
            }
            off0 = 0;
            st_off = row * 128 + ((ck ^ swz(row)) << 4);
            const int frow = lane & 31;
            frag_off = (wave_outer + frow) * 128 + (((lane >> 5) ^ swz(frow)) << 4);
        } else {
            const int chunk = tid % CP;   // 16-byte chunk along the outer dim
            const int rrow = tid / CP;    // reduction row within one load of the workgroup
            const bool second = chunk >= CP / 2;
            int outer = outer0 + chunk * 8 + (second ? split : 0);
            const int last = outer_last + (second ? split_last : 0);
            outer = outer > last ? last : outer;
#pragma unroll
            for (int i = 0; i < NL; ++i)
                off[i] = static_cast<unsigned>((static_cast<int64_t>(i * RP + rrow) * stride_red + (outer - outer0)) * 2);
            off0 = static_cast<unsigned>((outer - outer0) * 2);
            st_off = rrow * PITCH + chunk * 16;
            // transposing read: in each group of 16 lanes, lane L supplies the 4-element segment at
            // (reduction L/4, outer 4*(L%4)) and receives reduction 0..3 of outer L.
            const int l16 = lane & 15;
            const int red = 8 * (lane >> 5) + (l16 >> 2);
            const int out = wave_outer + 16 * ((lane >> 4) & 1) + 4 * (l16 & 3);
            frag_off = red * PITCH + out * 2;
        }
    }

    // base: pointer to element (outer0, red0) of the tile.  Loads i = h*NL/2 .. (h+1)*NL/2 - 1 of this lane.
    // TAIL: the tile may cross red_end, reduction indices >= nvalid (relative to red0) read as zero.
    template <bool TAIL>
    __device__ __forceinline__ void load_half(const char *base, int nvalid, int h) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = h * (NL / 2); i < (h + 1) * (NL / 2); ++i) {
            if constexpr (!TAIL) {
                r[i] = *reinterpret_cast<const v16 *>(base + off[i]);
            } else {
                // RED: one chunk of 8 reduction indices per lane (whole or nothing: the reduction extent is a
                // multiple of 8 on this path); !RED: one reduction index per load.  Masked-out lanes read a
                // valid address (chunk 0 / reduction index 0) instead.
                const int q = tid & 7;
                const bool ok = RED ? (q * 8 < nvalid) : (i * RP + tid / CP < nvalid);
                const unsigned o = ok ? off[i] : (RED ? off[i] - q * 16 : off0);
                const v16 v = *reinterpret_cast<const v16 *>(base + o);
                const v16 z = {0u, 0u, 0u, 0u};
                r[i] = ok ? v : z;
            }
        }
    }

    __device__ __forceinline__ void store_half(char *tile, int h) const {
#pragma unroll
        for (int i = h * (NL / 2); i < (h + 1) * (NL / 2); ++i) {
            if constexpr (RED) *reinterpret_cast<v16 *>(tile + st_off + i * 32 * 128) = r[i];
            else *reinterpret_cast<v16 *>(tile + st_off + i * RP * PITCH) = r[i];
        }
    }

    // Fragment t (32 outer indices) of K slice kk (16 reduction indices): 8 consecutive reduction values
    // of outer index (lane & 31), reduction half (lane >> 5).
    __device__ __forceinline__ v16 frag(const char *tile, int kk, int t) const {
        if constexpr (RED) {
            return *reinterpret_cast<const v16 *>(tile + (frag_off ^ ((kk * 2) << 4)) + t * 32 * 128);
        } else {
            const char *p = tile + frag_off + kk * 16 * PITCH + t * 64;
            const uint2 lo = lds_read_tr(p);
            const uint2 hi = lds_read_tr(p + 4 * PITCH);
            return v16{lo.x, lo.y, hi.x, hi.y};
        }
    }
};

// sched_group_barrier sequence for one phase: NM MFMAs with NRD LDS reads, NWR LDS writes and NLD global
// loads spread evenly between them.
constexpr int share(int total, int slots, int g) { return total * (g + 1) / slots - total * g / slots; }

template <int NM, int NRD, int NWR, int NLD, int ID, int... G>
__device__ __forceinline__ void interleave(std::integer_sequence<int, G...>) {
    ((sg<SG_DS_RD, share(NRD, NM, G), ID>(), sg<SG_DS_WR, share(NWR, NM, G), ID>(),
      sg<SG_VMEM_RD, share(NLD, NM, G), ID>(), sg<SG_MFMA, 1, ID>()),
     ...);
}

// ---- ring-buffered variant of the 256-row tile: global -> LDS transfers without a register stage ----------
//
// global_load_lds_dwordx4 moves 16 bytes per lane from per-lane global addresses straight into LDS, where one
// wavefront's 64 lanes fill 1 KB of consecutive bytes.  The LDS position of a lane is therefore fixed and the
// bank-conflict-avoiding swizzle is applied on the global side: the lane that owns LDS chunk c of a row
// fetches the memory chunk that the swizzle maps to c.  With no staging registers and no LDS store
// instructions the K loop can keep several tiles in flight: a ring of kRing stages of 32 reduction indices
// (16 KB per operand), tile kt+4 being requested while tile kt is multiplied, so every transfer has more than
// three K steps to arrive.
//   RED operand:  [256 outer][32 reduction], 64-byte rows, chunk c of row r holds memory chunk c ^ ((r >> 2) & 3)
//   !RED operand: [32 reduction][256 outer], 512-byte rows, chunk c of row r holds memory chunk c ^ ((r & 3) << 2)
// (the first keeps 16 consecutive rows of one chunk column on 16 different bank groups for ds_read_b128, the
// second keeps the four rows of one ds_read_b64_tr_b16 group on four different 64-byte bank groups).
constexpr int KS = 32;                        // reduction indices per ring stage
constexpr int kRing = 5;
constexpr int kRingTile = 256 * KS * 2;       // bytes of one operand in one stage
constexpr int kRingStage = 2 * kRingTile;
constexpr int kRingBytes = kRing * kRingStage;
constexpr int kXfers = kRingTile / 4 / 1024;  // 1 KB transfers per wavefront, operand and stage (4)

constexpr int waitcnt_imm(int vm, int lgkm) { return (vm & 15) | ((vm >> 4) << 14) | (7 << 4) | (lgkm << 8); }

using global_cptr = const char __attribute__((address_space(1))) *;
using lds_ptr = char __attribute__((address_space(3))) *;

template <bool RED>
struct RingOperand {
    unsigned off[kXfers];   // per-lane global byte offsets of this wavefront's transfers, relative to the tile base
    int key[kXfers];        // reduction index (relative to the tile) whose validity decides transfer i of this lane
    unsigned frag_off;      // byte offset of this lane's fragment reads inside the operand tile
    unsigned tsel[4];       // !RED: swizzled 64-byte column-group offset of fragment t

    __device__ __forceinline__ void init(int64_t stride_outer, int64_t stride_red, int outer0, int outer_last,
                                         int wave_outer, int wave) {
        const int lane = threadIdx.x & 63;
        if constexpr (RED) {
            const int cg = (lane & 3) ^ ((lane >> 4) & 3);   // memory chunk of this lane: c ^ ((row >> 2) & 3)
#pragma unroll
            for (int i = 0; i < kXfers; ++i) {
                const int row = (wave * kXfers + i) * 16 + (lane >> 2);
                int outer = outer0 + row;
                outer = outer > outer_last ? outer_last : outer;
                off[i] = static_cast<unsigned>((static_cast<int64_t>(outer - outer0) * stride_outer + cg * 8) * 2);
                key[i] = cg * 8;
            }
            const int frow = lane & 31;
            frag_off = (wave_outer + frow) * 64 + (((lane >> 5) ^ ((frow >> 2) & 3)) << 4);
#pragma unroll
            for (int t = 0; t < 4; ++t) tsel[t] = 0;
        } else {
#pragma unroll
            for (int i = 0; i < kXfers; ++i) {
                const int rr = (wave * kXfers + i) * 2 + (lane >> 5);
                const int cg = (lane & 31) ^ ((rr & 3) << 2);
                int outer = outer0 + cg * 8;
                outer = outer > outer_last ? outer_last : outer;
                off[i] = static_cast<unsigned>((static_cast<int64_t>(rr) * stride_red + (outer - outer0)) * 2);
                key[i] = rr;
            }
            // transposing read: in each group of 16 lanes, lane L supplies the 4-element segment at
            // (reduction L/4, outer 4*(L%4)) and receives reduction 0..3 of outer L.
            const int l16 = lane & 15;
            const int sw = l16 >> 2;
            const int red = 8 * (lane >> 5) + sw;
            frag_off = red * 512 + wave_outer * 2 + 32 * ((lane >> 4) & 1) + 8 * (l16 & 3);
#pragma unroll
            for (int t = 0; t < 4; ++t) tsel[t] = (t ^ sw) << 6;
        }
    }

    // Request transfer i of this wavefront's part of one tile.  base: pointer to element (outer0, first
    // reduction index of the tile), uniform; dst: LDS byte address of this wavefront's part of the operand's
    // stage; nvalid: reduction indices of the tile that lie inside the group (<= 0 for a tile past the end,
    // >= KS for a whole one).  Lanes whose data lies outside fetch from a block of zeros instead, so every
    // tile costs the same number of transfers whatever it holds: the wait counters of the K loop rely on that.
    // Written as inline assembly on purpose: the compiler then does not know that LDS is being written
    // behind its back and leaves all waiting on these transfers to the explicit s_waitcnt of the K loop
    // (it would otherwise drain them before every transposing LDS read).  M0 carries the LDS address (declared as clobbered).
    __device__ __forceinline__ void request(int i, const char *base, unsigned dst, int nvalid, const char *zeros) const {
        const char *src = key[i] < nvalid ? base + off[i] : zeros;
        asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off"
                     :: "s"(dst + i * 1024), "v"(src) : "memory", "m0");
    }

    // Fragment t of 16-wide slice kk of the tile at `tile`.
    __device__ __forceinline__ v16 frag(const char *tile, int kk, int t) const {
        if constexpr (RED) {
            return *reinterpret_cast<const v16 *>(tile + (frag_off ^ (kk << 5)) + t * 32 * 64);
        } else {
            const char *p = tile + frag_off + tsel[t] + kk * 16 * 512;
            const uint2 lo = lds_read_tr(p);
            const uint2 hi = lds_read_tr(p + 4 * 512);
            return v16{lo.x, lo.y, hi.x, hi.y};
        }
    }
};

// Which operand layouts take the ring: both operands contiguous along their outer dim (the weight-gradient
// product x^T dy).  There every transfer covers whole 512-byte memory rows, and the register-staged loop is
// at its slowest because both operands go through the slower transposing reads on top of the LDS stores.
// An operand contiguous along the reduction dim would be fetched as 64-byte half lines (32 reduction
// indices per stage), which doubles its request count at L2; measured, those products run a few percent
// slower on the ring than on the register-staged loop, so they stay there.
template <bool A_RED, bool B_RED>
constexpr bool use_ring() { return !A_RED && !B_RED; }

template <int DT, bool A_RED, bool B_RED>
__device__ __forceinline__ void ring_k_loop(const GmmArgs &p, const TileCoord &tc, char *lds, int row0, int col0,
                                            f32x16 (&acc)[4][4]) {
    constexpr int TM = 4, TN = 4;
    const int tid = threadIdx.x;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = wave >> 1, wn = wave & 1;
    const int red_begin = tc.e.red_begin;
    const int red_len = tc.e.red_end - red_begin;
    const int nk = (red_len + KS - 1) / KS;
    if (nk <= 0) return;

    RingOperand<A_RED> la;
    RingOperand<B_RED> lb;
    la.init(p.a_stride_row, p.a_stride_red, row0, A_RED ? tc.e.row_end - 1 : tc.e.row_end - 8, wm * 128, wave);
    lb.init(p.b_stride_col, p.b_stride_red, col0, B_RED ? p.cols - 1 : p.cols - 8, wn * 128, wave);
    const char *a_ptr = static_cast<const char *>(p.a) +
                        (static_cast<int64_t>(row0) * p.a_stride_row + static_cast<int64_t>(red_begin) * p.a_stride_red) * 2;
    const char *b_ptr = static_cast<const char *>(p.b) +
                        (tc.e.b_off + static_cast<int64_t>(col0) * p.b_stride_col +
                         static_cast<int64_t>(red_begin) * p.b_stride_red) * 2;
    const int64_t a_step = p.a_stride_red * KS * 2;
    const int64_t b_step = p.b_stride_red * KS * 2;
    const char *zeros = reinterpret_cast<const char *>((reinterpret_cast<uintptr_t>(p.table->zeros) + 15) & ~uintptr_t(15));

    const unsigned lds0 = static_cast<unsigned>(reinterpret_cast<uintptr_t>((lds_ptr)lds));
    // Tiles are requested in order, one per K step plus kRing - 1 up front, and the sequence simply runs on
    // past the last tile (all-zero tiles that nobody multiplies): the number of transfers in flight is then the
    // same at every step and one wait count serves the whole loop.
    int left = red_len;        // reduction indices from the next requested tile's start to the group's end
    int issue_stage = 0;       // ring stage of the next request
    // transfer g = 0..7 of the next tile: 0-3 operand A, 4-7 operand B
    auto request_part = [&](int g) {
        const unsigned dst = lds0 + issue_stage * kRingStage + wave * (kXfers * 1024);
        if (g < kXfers) la.request(g, a_ptr, dst, left, zeros);
        else lb.request(g - kXfers, b_ptr, dst + kRingTile, left, zeros);
    };
    auto request_done = [&]() {
        a_ptr += a_step;
        b_ptr += b_step;
        left -= KS;
        issue_stage = issue_stage + 1 == kRing ? 0 : issue_stage + 1;
    };

    v16 af[2][TM], bf[2][TN];
    auto read_frags = [&](const char *stage, int set, int kk) {
#pragma unroll
        for (int t = 0; t < TM; ++t) af[set][t] = la.frag(stage, kk, t);
#pragma unroll
        for (int t = 0; t < TN; ++t) bf[set][t] = lb.frag(stage + kRingTile, kk, t);
    };
    auto mfmas = [&](int set, int i0, int i1) {
#pragma unroll
        for (int i = i0; i < i1; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j) acc[i][j] = mfma16<DT>(bf[set][j], af[set][i], acc[i][j]);
    };
    // Wait until only the kRing - 2 most recently requested tiles (2 * kXfers transfers each) are still in
    // flight, and for this wavefront's LDS reads; then meet the other wavefronts.
    auto arrive = [&]() {
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((kRing - 2) * 2 * kXfers, 0));
        __builtin_amdgcn_s_barrier();
    };

    for (int t = 0; t < kRing - 1; ++t) {
#pragma unroll
        for (int g = 0; g < 2 * kXfers; ++g) request_part(g);
        request_done();
    }
    arrive();
    MS_TRACE(3);
    read_frags(lds, 0, 0);
    __builtin_amdgcn_sched_barrier(0);

    constexpr int NM = TM * TN;
    constexpr int NRD = (A_RED ? TM : 2 * TM) + (B_RED ? TN : 2 * TN);
    int cur_stage = 0;
    // One K step of 32 reduction indices = two 16-wide slices.
    for (int kt = 0; kt < nk; ++kt) {
        const char *cur = lds + cur_stage * kRingStage;
        cur_stage = cur_stage + 1 == kRing ? 0 : cur_stage + 1;
        const char *nxt = lds + cur_stage * kRingStage;
        // The eight transfer requests for tile kt + kRing - 1 go into the stage that tile kt - 1 occupied (free: every
        // wavefront finished reading it before the barrier of the previous step) and are spread over the whole step,
        // four in slice 0, two before and two after the barrier of slice 1: an even request stream measured 1 %
        // faster than all eight in slice 0, and all eight in one burst 4 % slower.
        // slice 0: eight groups of { a request (every other group), the slice-1 fragments of one 32-row block of each
        // operand (first four groups), two MFMAs }
#pragma unroll
        for (int g = 0; g < 8; ++g) {
            if ((g & 1) == 0) request_part(g >> 1);
            if (g < 4) {
                af[1][g] = la.frag(cur, 1, g);
                bf[1][g] = lb.frag(cur + kRingTile, 1, g);
            }
#pragma unroll
            for (int u = 2 * g; u < 2 * g + 2; ++u)
                acc[u / TN][u % TN] = mfma16<DT>(bf[0][u % TN], af[0][u / TN], acc[u / TN][u % TN]);
            __builtin_amdgcn_sched_barrier(0);
        }
        // slice 1: the barrier sits between the two halves of its MFMAs; after it tile kt + 1 is complete
        // in LDS (after the last step that is an all-zero tile, read and never used).  Six of this step's eight
        // requests have been issued when the barrier's wait is reached, so it allows two fewer in flight.
        request_part(4);
        mfmas(1, 0, 1);
        __builtin_amdgcn_sched_barrier(0);
        request_part(5);
        mfmas(1, 1, TM / 2);
        __builtin_amdgcn_sched_barrier(0);
        __builtin_amdgcn_s_waitcnt(waitcnt_imm((kRing - 2) * 2 * kXfers - 2, 0));
        __builtin_amdgcn_s_barrier();
        request_part(6);
        request_part(7);
        request_done();
        read_frags(nxt, 0, 0);
        mfmas(1, TM / 2, TM);
        interleave<NM / 2, NRD, 0, 0, 1>(std::make_integer_sequence<int, NM / 2>{});
        __builtin_amdgcn_sched_barrier(0);
    }
    // the transfers of the trailing all-zero tiles must have landed before the stages are reused
    __builtin_amdgcn_s_waitcnt(waitcnt_imm(0, 0));
}

// One macro tile of TBM x 256 outputs.  TBM = 256: 2x2 wavefronts of 128x128; TBM = 128 / 64: 1x4 wavefronts
// of 128x64 / 64x64.
template <int DT, bool A_RED, bool B_RED, int OUT, int TBM>
__device__ __forceinline__ void gmm16_tile(const GmmArgs &p, const TileCoord &tc, char *lds) {
    constexpr int WAVES_M = TBM == 256 ? 2 : 1;
    constexpr int WAVES_N = 4 / WAVES_M;
    constexpr int TM = TBM / WAVES_M / 32;      // 32-row MFMA blocks per wavefront
    constexpr int TN = BN / WAVES_N / 32;       // 32-column MFMA blocks per wavefront
    constexpr int A_BYTES = tile_bytes<A_RED, TBM>();
    constexpr int STAGE = A_BYTES + tile_bytes<B_RED, BN>();

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave / WAVES_N, wn = wave % WAVES_N;
    const int hi = lane >> 5;

    const int row0 = tc.e.row_begin + tc.row_tile * BM;   // all but the last row tile of a group are full
    const int row_end = tc.e.row_end;
    constexpr bool SWIGLU = OUT == OUT_SWIGLU;
    constexpr int HALF = BN / 2;                          // activation columns per tile in the fused form
    const int col0 = tc.col_tile * (SWIGLU ? HALF : BN);  // fused: first activation (= gate) column
    const int col_end = p.cols;
    const int red_begin = tc.e.red_begin, red_end = tc.e.red_end;

    f32x16 acc[TM][TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    if constexpr (TBM == 256 && use_ring<A_RED, B_RED>()) {
        ring_k_loop<DT, A_RED, B_RED>(p, tc, lds, row0, col0, acc);
    } else {
        Operand<A_RED, TBM> la;
        Operand<B_RED, BN> lb;
        la.init(p.a_stride_row, p.a_stride_red, row0, A_RED ? row_end - 1 : row_end - 8, wm * TM * 32);
        if constexpr (SWIGLU) {
            static_assert(!SWIGLU || !B_RED, "the fused SwiGLU form reads the weight along its columns");
            lb.init(p.b_stride_col, p.b_stride_red, col0, col_end - 8, wn * TN * 32, col_end - HALF, col_end);
        } else {
            lb.init(p.b_stride_col, p.b_stride_red, col0, B_RED ? col_end - 1 : col_end - 8, wn * TN * 32);
        }
        // uniform base pointers of element (outer0, red_begin); advanced by one K step per iteration
        const char *a_ptr = static_cast<const char *>(p.a) +
                            (static_cast<int64_t>(row0) * p.a_stride_row + static_cast<int64_t>(red_begin) * p.a_stride_red) * 2;
        const char *b_ptr = static_cast<const char *>(p.b) +
                            (tc.e.b_off + static_cast<int64_t>(col0) * p.b_stride_col +
                             static_cast<int64_t>(red_begin) * p.b_stride_red) * 2;
        const int64_t a_step = p.a_stride_red * BK * 2;
        const int64_t b_step = p.b_stride_red * BK * 2;

        const int red_len = red_end - red_begin;
        const int nk = (red_len + BK - 1) / BK;

        v16 af[2][TM], bf[2][TN];
        auto read_frags = [&](const char *stage, int set, int kk) {
#pragma unroll
            for (int t = 0; t < TM; ++t) af[set][t] = la.frag(stage, kk, t);
#pragma unroll
            for (int t = 0; t < TN; ++t) bf[set][t] = lb.frag(stage + A_BYTES, kk, t);
        };
        auto mfmas = [&](int set, int i0, int i1) {
#pragma unroll
            for (int i = i0; i < i1; ++i)
#pragma unroll
                for (int j = 0; j < TN; ++j) acc[i][j] = mfma16<DT>(bf[set][j], af[set][i], acc[i][j]);
        };
        // part p of a tile: p = 0,1 -> A halves, p = 2,3 -> B halves
        auto load_part = [&](auto tail_c, int part, int nvalid) {
            constexpr bool TAIL = decltype(tail_c)::value;
            if (part < 2) la.template load_half<TAIL>(a_ptr, nvalid, part);
            else lb.template load_half<TAIL>(b_ptr, nvalid, part - 2);
        };
        auto store_part = [&](char *stage, int part) {
            if (part < 2) la.store_half(stage, part);
            else lb.store_half(stage + A_BYTES, part - 2);
        };
        auto lds_barrier = [&]() {
            __builtin_amdgcn_s_waitcnt(0xC07F);   // lgkmcnt(0) only: global loads stay in flight
            __builtin_amdgcn_s_barrier();
        };

        if (nk > 0) {
            // tile 0 -> LDS stage 0; tile 1 -> registers.  Both use the masked loads (whose results are
            // consumed at once), so no load is outstanding when the steady-state loop is entered and the
            // loop's own issue order alone decides how long each of its waits has to be.
#pragma unroll
            for (int part = 0; part < 4; ++part) load_part(std::true_type{}, part, red_len);
#pragma unroll
            for (int part = 0; part < 4; ++part) store_part(lds, part);
            if (nk > 1) {
                a_ptr += a_step;
                b_ptr += b_step;
#pragma unroll
                for (int part = 0; part < 4; ++part) load_part(std::true_type{}, part, red_len - BK);
            }
            lds_barrier();
            MS_TRACE(3);
            read_frags(lds, 0, 0);
        }

        // instruction counts of one phase (one 16-wide K slice)
        constexpr int NM = TM * TN;                                        // MFMAs
        constexpr int NRD = (A_RED ? TM : 2 * TM) + (B_RED ? TN : 2 * TN); // LDS fragment reads
        constexpr int NLA = Operand<A_RED, TBM>::NL / 2;                   // loads / stores of an A part
        constexpr int NLB = Operand<B_RED, BN>::NL / 2;                    // ... of a B part

        int kt = 0;
        // HAS1: tile kt+1 exists (it is in registers); HAS2: tile kt+2 exists; tail2_c: tile kt+2 is the last one.
        auto k_step = [&](auto has1_c, auto has2_c, auto tail2_c) {
            constexpr bool HAS1 = decltype(has1_c)::value;
            constexpr bool HAS2 = decltype(has2_c)::value;
            const char *cur = lds + (kt & 1) * STAGE;
            char *nxt = lds + ((kt + 1) & 1) * STAGE;
            if constexpr (HAS2) {
                a_ptr += a_step;
                b_ptr += b_step;
            }
            const int left2 = red_len - (kt + 2) * BK;
#pragma unroll
            for (int kk = 0; kk < 4; ++kk) {
                const int set = kk & 1;
                if constexpr (HAS1) store_part(nxt, kk);
                if constexpr (HAS2) load_part(tail2_c, kk, left2);
                if (kk < 2) {
                    read_frags(cur, set ^ 1, kk + 1);
                    mfmas(set, 0, TM);
                    interleave<NM, NRD, HAS1 ? NLA : 0, HAS2 ? NLA : 0, 0>(std::make_integer_sequence<int, NM>{});
                    __builtin_amdgcn_sched_barrier(0);
                } else if (kk == 2) {
                    read_frags(cur, set ^ 1, kk + 1);
                    mfmas(set, 0, TM);
                    interleave<NM, NRD, HAS1 ? NLB : 0, HAS2 ? NLB : 0, 0>(std::make_integer_sequence<int, NM>{});
                    __builtin_amdgcn_sched_barrier(0);
                } else {
                    mfmas(set, 0, TM / 2);
                    interleave<NM / 2, 0, HAS1 ? NLB : 0, HAS2 ? NLB : 0, 0>(std::make_integer_sequence<int, NM / 2>{});
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (HAS1) {
                        lds_barrier();
                        read_frags(nxt, 0, 0);
                    }
                    mfmas(set, TM / 2, TM);
                    if constexpr (HAS1) interleave<NM / 2, NRD, 0, 0, 1>(std::make_integer_sequence<int, NM / 2>{});
                    __builtin_amdgcn_sched_barrier(0);
                }
            }
        };
        for (; kt + 3 < nk; ++kt) k_step(std::true_type{}, std::true_type{}, std::false_type{});
        if (kt + 3 == nk) { k_step(std::true_type{}, std::true_type{}, std::true_type{}); ++kt; }
        if (kt + 2 == nk) { k_step(std::true_type{}, std::false_type{}, std::false_type{}); ++kt; }
        if (kt + 1 == nk) { k_step(std::false_type{}, std::false_type{}, std::false_type{}); ++kt; }
    }

    // Epilogue.  acc[i][j][4*q+e] = C[row0 + wm*TM*32 + i*32 + (lane&31)]
    //                                [col0 + wn*TN*32 + j*32 + 8*q + 4*(lane>>5) + e]
    MS_TRACE(4);
    const int64_t ldc = p.c_stride_row;
    constexpr int WR = TM * 32, WC = TN * 32;       // this wavefront's block of the tile
    if constexpr (OUT == OUT_SAME || OUT == OUT_SWIGLU || OUT == OUT_SWIGLU_GRAD) {
        // 16-bit output: each wavefront stages its block in its own LDS region (row pitch WC*2 + 8 bytes:
        // conflict-free for the 8-byte column-slice writes and the row reads) and writes it out as 16 bytes
        // per lane, WC*2 contiguous bytes per row.
        constexpr int SP = WC * 2 + 8;
        static_assert(WR * SP <= kStagePerWave, "staging region too small");
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();          // every wavefront is done reading the operand stages
        char *stg = lds + wave * kStagePerWave;
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    uint16_t h[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        h[e] = DT == MS_BF16 ? BF16::from_float(acc[i][j][4 * q + e]) : FP16::from_float(acc[i][j][4 * q + e]);
                    *reinterpret_cast<uint2 *>(stg + (i * 32 + (lane & 31)) * SP + (j * 32 + 8 * q + 4 * hi) * 2) =
                        *reinterpret_cast<uint2 *>(h);
                }
        __builtin_amdgcn_s_waitcnt(0xC07F);    // own writes only: the region is private to this wavefront
        constexpr int LPR = WC / 8;            // lanes per row (8 columns = 16 bytes each)
        constexpr int RPP = 64 / LPR;          // rows per pass
        const int chunk = lane % LPR;
        // Fused form: the wavefronts of the first half of the tile's columns hold gate columns, their
        // partners (same rows, other half) the matching up columns, ffn further on in the output row.
        constexpr int GATE_WAVES = WAVES_N / 2;
        const bool up_half = SWIGLU && wn >= GATE_WAVES;
        const int acol = col0 + (SWIGLU ? wn % GATE_WAVES : wn) * WC + chunk * 8;   // activation column
        const int col = SWIGLU ? acol + (up_half ? col_end : 0) : acol;
        const bool col_ok = acol < col_end;    // cols is a multiple of 8 on this path
        if constexpr (OUT == OUT_SWIGLU_GRAD) {
            // The staged block is dact = dY @ W2^T (rounded, as the stand-alone matmul would store it); what is
            // written is d_fc1 = SwiGLU backward of it on the saved fc1 output, the same arithmetic as the
            // stand-alone kernel, and per 64 columns the row sums that make up the probabilities' gradient.
            using DTT = std::conditional_t<DT == MS_BF16, BF16, FP16>;
            const uint16_t *fbase = static_cast<const uint16_t *>(p.fc1) + acol;
            uint16_t *dbase = static_cast<uint16_t *>(p.c) + acol;
#pragma unroll 2
            for (int pass = 0; pass < WR / RPP; ++pass) {
                const int r = pass * RPP + lane / LPR;
                const int row = row0 + wm * WR + r;
                const bool ok = col_ok && row < row_end;
                uint16_t d[8], g[8], u[8], og[8], ou[8];
                *reinterpret_cast<uint2 *>(d) = *reinterpret_cast<const uint2 *>(stg + r * SP + chunk * 16);
                *reinterpret_cast<uint2 *>(d + 4) = *reinterpret_cast<const uint2 *>(stg + r * SP + chunk * 16 + 8);
                float dot = 0.f;
                if (ok) {
                    const uint16_t *fg = fbase + static_cast<int64_t>(row) * p.fc1_stride_row;
                    *reinterpret_cast<v16 *>(g) = *reinterpret_cast<const v16 *>(fg);
                    *reinterpret_cast<v16 *>(u) = *reinterpret_cast<const v16 *>(fg + col_end);
                    const float pr = p.probs != nullptr ? load_scalar_as_float(p.probs, row, p.probs_dtype) : 1.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float gf = DTT::to_float(g[e]), uf = DTT::to_float(u[e]), df = DTT::to_float(d[e]);
                        const float sig = 1.f / (1.f + __expf(-gf));
                        const float act = gf * sig;
                        dot = fmaf(df, act * uf, dot);
                        const float dp = df * pr;
                        og[e] = DTT::from_float(dp * uf * (sig * (1.f + gf * (1.f - sig))));
                        ou[e] = DTT::from_float(dp * act);
                    }
                    uint16_t *dg = dbase + static_cast<int64_t>(row) * ldc;
                    *reinterpret_cast<v16 *>(dg) = *reinterpret_cast<v16 *>(og);
                    *reinterpret_cast<v16 *>(dg + col_end) = *reinterpret_cast<v16 *>(ou);
                }
                if (p.partials != nullptr) {
                    // 8 lanes = 64 columns: one partial sum per row and 64-column block
                    dot += __shfl_xor(dot, 1, 64);
                    dot += __shfl_xor(dot, 2, 64);
                    dot += __shfl_xor(dot, 4, 64);
                    if ((chunk & 7) == 0 && ok)
                        p.partials[static_cast<int64_t>(row) * p.partials_per_row + (acol >> 6)] = dot;
                }
            }
        } else if (!SWIGLU || p.c != nullptr) {
            uint16_t *cbase = static_cast<uint16_t *>(p.c) + tc.e.c_off + col;
#pragma unroll 4
            for (int pass = 0; pass < WR / RPP; ++pass) {
                const int r = pass * RPP + lane / LPR;
                const int row = row0 + wm * WR + r;
                const uint2 lo = *reinterpret_cast<const uint2 *>(stg + r * SP + chunk * 16);
                const uint2 hi2 = *reinterpret_cast<const uint2 *>(stg + r * SP + chunk * 16 + 8);
                if (col_ok && row < row_end)
                    *reinterpret_cast<v16 *>(cbase + static_cast<int64_t>(row) * ldc) = v16{lo.x, lo.y, hi2.x, hi2.y};
            }
        }
        if constexpr (SWIGLU) {
            // act = silu(gate) * up * prob from the staged (already rounded) values, exactly what the
            // stand-alone SwiGLU kernel computes from the stored fc1 output.  Each wavefront of a pair
            // takes half of the rows.
            using DTT = std::conditional_t<DT == MS_BF16, BF16, FP16>;
            __builtin_amdgcn_s_waitcnt(0xC07F);
            __builtin_amdgcn_s_barrier();      // the partner's block is staged
            const char *gstg = lds + (wm * WAVES_N + wn % GATE_WAVES) * kStagePerWave;
            const char *ustg = gstg + GATE_WAVES * kStagePerWave;
            const int rbase = up_half ? WR / 2 : 0;
            uint16_t *abase = static_cast<uint16_t *>(p.act) + acol;
#pragma unroll 4
            for (int pass = 0; pass < WR / 2 / RPP; ++pass) {
                const int r = rbase + pass * RPP + lane / LPR;
                const int row = row0 + wm * WR + r;
                uint16_t g[8], u[8], o[8];
                *reinterpret_cast<uint2 *>(g) = *reinterpret_cast<const uint2 *>(gstg + r * SP + chunk * 16);
                *reinterpret_cast<uint2 *>(g + 4) = *reinterpret_cast<const uint2 *>(gstg + r * SP + chunk * 16 + 8);
                *reinterpret_cast<uint2 *>(u) = *reinterpret_cast<const uint2 *>(ustg + r * SP + chunk * 16);
                *reinterpret_cast<uint2 *>(u + 4) = *reinterpret_cast<const uint2 *>(ustg + r * SP + chunk * 16 + 8);
                if (col_ok && row < row_end) {
                    const float pr = p.probs != nullptr ? load_scalar_as_float(p.probs, row, p.probs_dtype) : 1.f;
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float gf = DTT::to_float(g[e]);
                        o[e] = DTT::from_float(gf * (1.f / (1.f + __expf(-gf))) * DTT::to_float(u[e]) * pr);
                    }
                    *reinterpret_cast<v16 *>(abase + static_cast<int64_t>(row) * p.act_stride_row) = *reinterpret_cast<v16 *>(o);
                }
            }
        }
    } else {
        // fp32 output or fp32 `+=`: an accumulator register holds four consecutive columns of one row, so written
        // straight from the registers one instruction would touch 32 rows with 32 bytes each.  Instead each
        // wavefront stages one 32-row strip of its block at a time in its own LDS region (row pitch WC + 4
        // floats) and moves it as whole row segments: WC * 4 contiguous bytes per row, 16 bytes per lane.
        constexpr int SPF = WC + 4;              // floats per staged row
        static_assert(32 * SPF * 4 <= kStagePerWave, "staging region too small");
        __builtin_amdgcn_s_waitcnt(0xC07F);
        __builtin_amdgcn_s_barrier();          // every wavefront is done reading the operand stages
        float *stg = reinterpret_cast<float *>(lds + wave * kStagePerWave);
        constexpr int LPR = WC / 4;            // lanes per row (4 columns = 16 bytes each)
        constexpr int RPP = 64 / LPR;          // rows per pass
        const int c4 = (lane % LPR) * 4;
        const int col = col0 + wn * WC + c4;
        const bool col_ok = col < col_end;     // cols is a multiple of 4 on this path
        float *cbase = static_cast<float *>(p.c) + tc.e.c_off + col;
        const float *lbase = static_cast<const float *>(p.c) + tc.e.c_off + (col_ok ? col : col_end - 4);   // always inside the row
        constexpr int NP = 32 / RPP;           // passes per strip
        // `+=`: the old values of strip i + 1 are requested while strip i is staged and written, from clamped
        // (always valid) addresses, so that a whole strip's loads are in flight at a time
        f32x4 old[2][NP];
        auto load_old = [&](f32x4 (&dst)[NP], int i) {
#pragma unroll
            for (int pass = 0; pass < NP; ++pass) {
                int row = row0 + wm * WR + i * 32 + pass * RPP + lane / LPR;
                row = row < row_end ? row : row_end - 1;
                dst[pass] = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(lbase + static_cast<int64_t>(row) * ldc));
            }
        };
        if constexpr (OUT == ACC_F32) load_old(old[0], 0);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
                for (int q = 0; q < 4; ++q) {
                    const f32x4 o = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
                    *reinterpret_cast<f32x4 *>(stg + (lane & 31) * SPF + j * 32 + 8 * q + 4 * hi) = o;
                }
            if constexpr (OUT == ACC_F32) {
                if (i + 1 < TM) load_old(old[(i + 1) & 1], i + 1);
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);    // own writes only: the region is private to this wavefront
#pragma unroll
            for (int pass = 0; pass < NP; ++pass) {
                const int r = pass * RPP + lane / LPR;
                const int row = row0 + wm * WR + i * 32 + r;
                f32x4 o = *reinterpret_cast<const f32x4 *>(stg + r * SPF + c4);
                if constexpr (OUT == ACC_F32) o += old[i & 1][pass];
                if (col_ok && row < row_end) __builtin_nontemporal_store(o, reinterpret_cast<f32x4 *>(cbase + static_cast<int64_t>(row) * ldc));
            }
            __builtin_amdgcn_s_waitcnt(0xC07F);    // the strip has been read before the next one overwrites it
        }
    }
}

// LISTS: the launch may come with per-XCD lists of entries.  Always so for the split on rows (A_RED); the weight-gradient
// product has a variant of its own for launches of many groups, so that the common one does not carry that lookup.
template <int DT, bool A_RED, bool B_RED, int OUT, bool LISTS = A_RED>
__global__ __launch_bounds__(256) void gmm16_fast_kernel(const GmmArgs p) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    MS_TRACE(1);
    const TileCoord tc = locate_tile<LISTS>(p.table);
    if (!tc.valid) return;
    MS_TRACE(2);
    if (tc.tile_rows == 256) {
        gmm16_tile<DT, A_RED, B_RED, OUT, 256>(p, tc, lds);
    } else if (OUT == OUT_SAME && A_RED && tc.e.split != 0) {
        // one part of a small tail tile whose reduction is split: fp32 partial sums into the split workspace
        // (rows of `cols` floats; the entry's c_off leads to this part's block)
        GmmArgs q = p;
        q.c = p.split_ws;
        q.c_stride_row = p.cols;
        if (tc.tile_rows == 128) gmm16_tile<DT, A_RED, B_RED, OUT_F32, 128>(q, tc, lds);
        else gmm16_tile<DT, A_RED, B_RED, OUT_F32, 64>(q, tc, lds);
    } else if (tc.tile_rows == 128) {
        gmm16_tile<DT, A_RED, B_RED, OUT, 128>(p, tc, lds);
    } else {
        gmm16_tile<DT, A_RED, B_RED, OUT, 64>(p, tc, lds);
    }
#ifdef MS_TRACE_TILES
    if (threadIdx.x == 0) {
        unsigned hw_id, xcc_id;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw_id));
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc_id));
        long long *rec = g_tile_trace + (blockIdx.x % kTraceSlots) * 8;
        rec[0] = (static_cast<long long>(xcc_id & 0xf) << 32) | ((hw_id >> 8) & 0xff) | (1ll << 40);   // XCC, CU/SH/SE bits, "valid"
        rec[5] = wall_clock64();
        rec[6] = tc.tile_rows;
    }
#endif
}

template <int DT, int OUT>
int launch_fast(hipStream_t stream, const GmmArgs &args, bool a_red, bool b_red, unsigned grid, bool lists) {
    const void *fn;
    if constexpr (OUT == OUT_SWIGLU) {
        MS_REQUIRE(a_red && !b_red, MS_ERR_UNSUPPORTED, "ms_gmm_swiglu: operand layout not supported");
        fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, true, false, OUT>);
    } else if constexpr (OUT == OUT_SWIGLU_GRAD) {
        MS_REQUIRE(a_red && b_red, MS_ERR_UNSUPPORTED, "ms_gmm_swiglu_grad: operand layout not supported");
        fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, true, true, OUT>);
    } else if (a_red && b_red) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, true, true, OUT>);
    else if (a_red) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, true, false, OUT>);
    else if (b_red) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, false, true, OUT>);
    else if (lists) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, false, false, OUT, true>);
    else fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, false, false, OUT>);
    int lds_bytes = 2 * ((a_red ? kRedTileBytes : kOuterTileBytes) + (b_red ? kRedTileBytes : kOuterTileBytes));
    if ((OUT == OUT_SAME || OUT == OUT_SWIGLU || OUT == OUT_SWIGLU_GRAD) && lds_bytes < kStageBytes) lds_bytes = kStageBytes;
    if (!a_red && !b_red && lds_bytes < kRingBytes) lds_bytes = kRingBytes;   // use_ring<false, false>()
    hipError_t e = set_max_dynamic_lds(fn, lds_bytes);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm: hipFuncSetAttribute: %s", hipGetErrorString(e));
    GmmArgs copy = args;
    void *kargs[] = {&copy};
    e = hipLaunchKernel(fn, dim3(grid), dim3(256), kargs, lds_bytes, stream);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm: launch failed: %s", hipGetErrorString(e));
    return MS_OK;
}

}  // namespace

int launch_gmm16_fast(hipStream_t stream, const GmmArgs &args, int dtype, int out_mode, bool a_red, bool b_red,
                      unsigned grid, bool lists) {
    if (out_mode == OUT_SWIGLU) {
        if (dtype == MS_BF16) return launch_fast<MS_BF16, OUT_SWIGLU>(stream, args, a_red, b_red, grid, lists);
        return launch_fast<MS_FP16, OUT_SWIGLU>(stream, args, a_red, b_red, grid, lists);
    }
    if (out_mode == OUT_SWIGLU_GRAD) {
        if (dtype == MS_BF16) return launch_fast<MS_BF16, OUT_SWIGLU_GRAD>(stream, args, a_red, b_red, grid, lists);
        return launch_fast<MS_FP16, OUT_SWIGLU_GRAD>(stream, args, a_red, b_red, grid, lists);
    }
    if (dtype == MS_BF16) {
        if (out_mode == OUT_SAME) return launch_fast<MS_BF16, OUT_SAME>(stream, args, a_red, b_red, grid, lists);
        if (out_mode == OUT_F32) return launch_fast<MS_BF16, OUT_F32>(stream, args, a_red, b_red, grid, lists);
        return launch_fast<MS_BF16, ACC_F32>(stream, args, a_red, b_red, grid, lists);
    }
    if (out_mode == OUT_SAME) return launch_fast<MS_FP16, OUT_SAME>(stream, args, a_red, b_red, grid, lists);
    if (out_mode == OUT_F32) return launch_fast<MS_FP16, OUT_F32>(stream, args, a_red, b_red, grid, lists);
    return launch_fast<MS_FP16, ACC_F32>(stream, args, a_red, b_red, grid, lists);
}

}  // namespace ms

#ifdef MS_TRACE_TILES
// Diagnostic builds only: ms_trace_clear zeroes the tile trace (call it before the launch to be looked at: records of
// earlier, larger launches would otherwise remain), ms_trace_read copies its first n values (8 per record) to host memory.
extern "C" int ms_trace_clear(void) {
    static long long zeros[ms::kTraceSlots * 8];
    if (hipDeviceSynchronize() != hipSuccess) return MS_ERR_HIP;
    return hipMemcpyToSymbol(HIP_SYMBOL(ms::g_tile_trace), zeros, sizeof(zeros)) == hipSuccess ? MS_OK : MS_ERR_HIP;
}

extern "C" int ms_trace_read(long long *host, int n) {
    if (n < 0 || n > ms::kTraceSlots * 8) return MS_ERR_INVALID_ARGUMENT;
    return hipMemcpyFromSymbol(host, HIP_SYMBOL(ms::g_tile_trace), sizeof(long long) * n) == hipSuccess ? MS_OK : MS_ERR_HIP;
}
#endif
