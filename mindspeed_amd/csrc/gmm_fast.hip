// Fast path of the 16-bit grouped matmul for gfx950: same 256x256x64 macro tile and
// LDS layout as the generic kernel, but for problems whose pointers and strides
// allow 16-byte vector access everywhere.  All edge handling is branch-free
// (clamped addresses, zero masks on the reduction tail), global loads use a
// uniform 64-bit tile base plus per-lane 32-bit offsets, and the K loop is
// software-pipelined by hand so that global loads are in flight all the time:
//
//   registers hold tile kt+1 (loaded one K step ago), LDS stage `cur` holds tile kt.
//   step kt, phase p = 0..3 (one 16-wide slice of the 64-wide K step each):
//       store part p of tile kt+1 from registers to LDS stage `nxt`
//       issue the global loads of part p of tile kt+2 into the same registers
//       read the MFMA fragments of slice p+1 from LDS stage `cur`
//       16 MFMAs on the fragments of slice p
//   (parts: A rows/ks 0-3, A 4-7, B 0-3, B 4-7 of each lane's eight 16-byte loads)
//   in phase 3 a workgroup barrier sits between the two halves of the MFMAs; after it
//   the fragments of slice 0 of tile kt+1 are read from stage `nxt`.
//
// Every load therefore has a full K step (64 MFMAs per wavefront) to arrive, and the
// vector memory path sees a steady request stream instead of one burst per step.
#include <type_traits>

#include "gmm_common.h"

namespace ms {
namespace {

// Instruction-class masks of __builtin_amdgcn_sched_group_barrier.
constexpr int SG_MFMA = 0x008, SG_VMEM_RD = 0x020, SG_DS_RD = 0x100, SG_DS_WR = 0x200;

template <int MASK, int N, int ID>
__device__ __forceinline__ void sg() {
    __builtin_amdgcn_sched_group_barrier(MASK, N, ID);
}

// Per-lane global offsets (bytes, relative to the tile's uniform base pointer) of the
// 8 sixteen-byte loads this lane issues per K step.
template <bool RED>
struct FastLoader {
    unsigned off[8];
    unsigned off0;     // !RED: offset of (reduction index 0, this lane's outer chunk), always valid
    unsigned lds_off;  // byte offset of this lane's first LDS store inside an operand tile
    v16 r[8];

    // outer0: first outer index of the tile, outer_last: last valid outer index (clamp bound,
    // for !RED the last valid start of an 8-wide chunk), strides in elements.
    __device__ __forceinline__ void init(int64_t stride_outer, int64_t stride_red, int outer0, int outer_last) {
        const int tid = threadIdx.x;
        if constexpr (RED) {
            const int ck = tid & 7;
            const int row = tid >> 3;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                int outer = outer0 + row + 32 * i;
                outer = outer > outer_last ? outer_last : outer;
                off[i] = static_cast<unsigned>((static_cast<int64_t>(outer - outer0) * stride_outer + ck * 8) * 2);
            }
            off0 = 0;
            lds_off = row * 128 + ((ck ^ swz(row)) << 4);
        } else {
            const int kb = tid & 7;
            const int nb = tid >> 3;
            int outer = outer0 + nb * 8;
            outer = outer > outer_last ? outer_last : outer;
#pragma unroll
            for (int j = 0; j < 8; ++j)
                off[j] = static_cast<unsigned>((static_cast<int64_t>(kb * 8 + j) * stride_red + (outer - outer0)) * 2);
            off0 = static_cast<unsigned>((outer - outer0) * 2);
            lds_off = 0;
        }
    }

    // base: pointer to element (outer0, red0) of the tile.  Loads i = 4h..4h+3 of this lane.
    // TAIL: the tile may cross red_end, reduction indices >= nvalid (relative to red0) read as zero.
    template <bool TAIL>
    __device__ __forceinline__ void load_half(const char *base, int nvalid, int h) {
        const int tid = threadIdx.x;
#pragma unroll
        for (int i = 4 * h; i < 4 * h + 4; ++i) {
            if constexpr (!TAIL) {
                r[i] = *reinterpret_cast<const v16 *>(base + off[i]);
            } else {
                // RED: one chunk of 8 reduction indices per lane (whole or nothing: the reduction
                // extent is a multiple of 8 on this path); !RED: one reduction index per load.
                // Masked-out lanes read a valid address (chunk 0 / reduction index 0) instead.
                const int q = tid & 7;
                const bool ok = RED ? (q * 8 < nvalid) : (q * 8 + i < nvalid);
                const unsigned o = ok ? off[i] : (RED ? off[i] - q * 16 : off0);
                const v16 v = *reinterpret_cast<const v16 *>(base + o);
                const v16 z = {0u, 0u, 0u, 0u};
                r[i] = ok ? v : z;
            }
        }
    }

    __device__ __forceinline__ void store_half(char *lds_tile, int h) const {
        if constexpr (RED) {
#pragma unroll
            for (int i = 4 * h; i < 4 * h + 4; ++i) *reinterpret_cast<v16 *>(lds_tile + lds_off + i * 32 * 128) = r[i];
        } else {
            // 4 (reduction) x 8 (outer) block -> for each outer index 4 reduction values = 8 bytes
            const int tid = threadIdx.x;
            const int kb = tid & 7;
            const int nb = tid >> 3;
#pragma unroll
            for (int c = 0; c < 8; ++c) {
                uint2 o;
                // bytes of {hi:lo}: low halves -> 0x05040100, high halves -> 0x07060302
                const unsigned sel = (c & 1) ? 0x07060302u : 0x05040100u;
                o.x = __builtin_amdgcn_perm(r[4 * h + 1][c >> 1], r[4 * h][c >> 1], sel);
                o.y = __builtin_amdgcn_perm(r[4 * h + 3][c >> 1], r[4 * h + 2][c >> 1], sel);
                const int row = nb * 8 + c;
                *reinterpret_cast<uint2 *>(lds_tile + row * 128 + ((kb ^ swz(row)) << 4) + h * 8) = o;
            }
        }
    }
};

template <int DT, bool A_RED, bool B_RED, int OUT>
__global__ __launch_bounds__(256) void gmm16_fast_kernel(const GmmArgs p) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const TileCoord tc = locate_tile(p.table);
    if (!tc.valid) return;

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wm = wave >> 1, wn = wave & 1;

    const int row0 = tc.e.row_begin + tc.row_tile * BM;
    const int row_end = tc.e.row_end;
    const int col0 = tc.col_tile * BN;
    const int col_end = p.cols;
    const int red_begin = tc.e.red_begin, red_end = tc.e.red_end;

    f32x16 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

    // per-lane fragment read offsets (bytes) inside an operand tile
    const int frow = lane & 31;
    const int hi = lane >> 5;
    const int fbase = frow * 128 + ((hi ^ swz(frow)) << 4);   // chunk (kk*2+hi)^swz = (kk*2) ^ (hi^swz)
    const int a_frag = wm * 128 * 128 + fbase;
    const int b_frag = wn * 128 * 128 + fbase;

    FastLoader<A_RED> la;
    FastLoader<B_RED> lb;
    la.init(p.a_stride_row, p.a_stride_red, row0, A_RED ? row_end - 1 : row_end - 8);
    lb.init(p.b_stride_col, p.b_stride_red, col0, B_RED ? col_end - 1 : col_end - 8);
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

    v16 af[2][4], bf[2][4];
    auto read_frags = [&](const char *stage, int set, int kk) {
        const int koff = (kk * 2) << 4;   // XOR term of the fragment's chunk
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            af[set][t] = *reinterpret_cast<const v16 *>(stage + (a_frag ^ koff) + t * 32 * 128);
            bf[set][t] = *reinterpret_cast<const v16 *>(stage + kTileBytes + (b_frag ^ koff) + t * 32 * 128);
        }
    };
    auto mfmas = [&](int set, int i0, int i1) {
#pragma unroll
        for (int i = i0; i < i1; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = mfma16<DT>(bf[set][j], af[set][i], acc[i][j]);
    };
    // part p of a tile: p = 0,1 -> A halves, p = 2,3 -> B halves
    auto load_part = [&](auto tail_c, int p, int nvalid) {
        constexpr bool TAIL = decltype(tail_c)::value;
        if (p < 2) la.template load_half<TAIL>(a_ptr, nvalid, p);
        else lb.template load_half<TAIL>(b_ptr, nvalid, p - 2);
    };
    auto store_part = [&](char *stage, int p) {
        if (p < 2) la.store_half(stage, p);
        else lb.store_half(stage + kTileBytes, p - 2);
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
        for (int p = 0; p < 4; ++p) load_part(std::true_type{}, p, red_len);
#pragma unroll
        for (int p = 0; p < 4; ++p) store_part(lds, p);
        if (nk > 1) {
            a_ptr += a_step;
            b_ptr += b_step;
#pragma unroll
            for (int p = 0; p < 4; ++p) load_part(std::true_type{}, p, red_len - BK);
        }
        lds_barrier();
        read_frags(lds, 0, 0);
    }

    int kt = 0;
    // HAS1: tile kt+1 exists (it is in registers); HAS2: tile kt+2 exists; TAIL2: tile kt+2 is the last one.
    auto k_step = [&](auto has1_c, auto has2_c, auto tail2_c) {
        constexpr bool HAS1 = decltype(has1_c)::value;
        constexpr bool HAS2 = decltype(has2_c)::value;
        const char *cur = lds + (kt & 1) * 2 * kTileBytes;
        char *nxt = lds + ((kt + 1) & 1) * 2 * kTileBytes;
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
            if (kk < 3) {
                read_frags(cur, set ^ 1, kk + 1);
                mfmas(set, 0, 4);
#pragma unroll
                for (int g = 0; g < 8; ++g) {
                    sg<SG_DS_RD, 1, 0>();
                    sg<SG_MFMA, 1, 0>();
                    if (HAS1 && g < 4) sg<SG_DS_WR, (A_RED && B_RED) ? 1 : 2, 0>();
                    if (HAS2 && g >= 4) sg<SG_VMEM_RD, 1, 0>();
                    sg<SG_MFMA, 1, 0>();
                }
                __builtin_amdgcn_sched_barrier(0);
            } else {
                mfmas(set, 0, 2);
                if constexpr (HAS1) {
#pragma unroll
                    for (int g = 0; g < 4; ++g) {
                        sg<SG_DS_WR, (A_RED && B_RED) ? 1 : 2, 0>();
                        sg<SG_MFMA, 1, 0>();
                        if (HAS2) sg<SG_VMEM_RD, 1, 0>();
                        sg<SG_MFMA, 1, 0>();
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (HAS1) {
                    lds_barrier();
                    read_frags(nxt, 0, 0);
                }
                mfmas(set, 2, 4);
                if constexpr (HAS1) {
#pragma unroll
                    for (int g = 0; g < 8; ++g) {
                        sg<SG_DS_RD, 1, 1>();
                        sg<SG_MFMA, 1, 1>();
                    }
                }
                __builtin_amdgcn_sched_barrier(0);
            }
        }
    };
    for (; kt + 3 < nk; ++kt) k_step(std::true_type{}, std::true_type{}, std::false_type{});
    if (kt + 3 == nk) { k_step(std::true_type{}, std::true_type{}, std::true_type{}); ++kt; }
    if (kt + 2 == nk) { k_step(std::true_type{}, std::false_type{}, std::false_type{}); ++kt; }
    if (kt + 1 == nk) { k_step(std::false_type{}, std::false_type{}, std::false_type{}); ++kt; }

    // Epilogue.  acc[i][j][4*q+e] = C[row0 + wm*128 + i*32 + (lane&31)]
    //                                [col0 + wn*128 + j*32 + 8*q + 4*(lane>>5) + e]
    const int64_t ldc = p.c_stride_row;
    const bool full_cols = col0 + BN <= col_end;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int row = row0 + wm * 128 + i * 32 + (lane & 31);
        if (row >= row_end) continue;
#pragma unroll
        for (int j = 0; j < 4; ++j) {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int col = col0 + wn * 128 + j * 32 + 8 * q + 4 * hi;
                if (!full_cols && col >= col_end) continue;   // cols is a multiple of 4 on this path
                const int64_t at = tc.e.c_off + static_cast<int64_t>(row) * ldc + col;
                float v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = acc[i][j][4 * q + e];
                if constexpr (OUT == OUT_SAME) {
                    uint16_t h[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) h[e] = DT == MS_BF16 ? BF16::from_float(v[e]) : FP16::from_float(v[e]);
                    *reinterpret_cast<uint2 *>(static_cast<uint16_t *>(p.c) + at) = *reinterpret_cast<uint2 *>(h);
                } else {
                    float *c = static_cast<float *>(p.c) + at;
                    f32x4 o = {v[0], v[1], v[2], v[3]};
                    if constexpr (OUT == ACC_F32) o += *reinterpret_cast<f32x4 *>(c);
                    *reinterpret_cast<f32x4 *>(c) = o;
                }
            }
        }
    }
}

template <int DT, int OUT>
int launch_fast(hipStream_t stream, const GmmArgs &args, bool a_red, bool b_red, unsigned grid) {
    const void *fn;
    if (a_red && b_red) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, true, true, OUT>);
    else if (a_red) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, true, false, OUT>);
    else if (b_red) fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, false, true, OUT>);
    else fn = reinterpret_cast<const void *>(&gmm16_fast_kernel<DT, false, false, OUT>);
    hipError_t e = hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBytes16);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm: hipFuncSetAttribute: %s", hipGetErrorString(e));
    GmmArgs copy = args;
    void *kargs[] = {&copy};
    e = hipLaunchKernel(fn, dim3(grid), dim3(256), kargs, kLdsBytes16, stream);
    MS_REQUIRE(e == hipSuccess, MS_ERR_HIP, "ms_gmm: launch failed: %s", hipGetErrorString(e));
    return MS_OK;
}

}  // namespace

int launch_gmm16_fast(hipStream_t stream, const GmmArgs &args, int dtype, int out_mode, bool a_red, bool b_red,
                      unsigned grid) {
    if (dtype == MS_BF16) {
        if (out_mode == OUT_SAME) return launch_fast<MS_BF16, OUT_SAME>(stream, args, a_red, b_red, grid);
        if (out_mode == OUT_F32) return launch_fast<MS_BF16, OUT_F32>(stream, args, a_red, b_red, grid);
        return launch_fast<MS_BF16, ACC_F32>(stream, args, a_red, b_red, grid);
    }
    if (out_mode == OUT_SAME) return launch_fast<MS_FP16, OUT_SAME>(stream, args, a_red, b_red, grid);
    if (out_mode == OUT_F32) return launch_fast<MS_FP16, OUT_F32>(stream, args, a_red, b_red, grid);
    return launch_fast<MS_FP16, ACC_F32>(stream, args, a_red, b_red, grid);
}

}  // namespace ms
