// Hardware probe: what one memory instruction costs the MFMA pipe of the wavefront that issues it.  One workgroup of
// four wavefronts (one per SIMD, as in the grouped-matmul kernels) runs 2048 clocks' worth of independent MFMAs per
// loop iteration, with 16 (or 32) instructions of one kind spread evenly between them, in exact program order
// (everything is volatile inline assembly); the extra clocks per iteration over the MFMAs alone, divided by the number
// of instructions, is the cost.  Kinds: 16-byte global loads with 64-bit and with base + 32-bit addressing, the
// global -> LDS forms of both, buffer loads, 16- and 8-byte LDS stores, plain VALU operations; for both bf16 MFMA shapes.
// Build and run: python -m mindspeed_amd.probes run issue_cost
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef int i4 __attribute__((ext_vector_type(4)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));

template <int KIND, int NL, int MF, int WAVES>   // MF: 0 = 16x16x32, 1 = 32x32x16; WAVES: 4 (one per SIMD) or 8 (two per SIMD, half the MFMAs each)
__global__ __launch_bounds__(WAVES * 64) void mix(long long *out, const u4 *g, int iters) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    for (int i = threadIdx.x; i < 131072 / 4; i += blockDim.x) reinterpret_cast<int *>(lds)[i] = 0;
    __syncthreads();
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    constexpr int NACC = WAVES == 4 ? 64 : 32;
    f4 acc[NACC];
#pragma unroll
    for (int i = 0; i < NACC; ++i) { acc[i] = f4{0, 0, 0, 0}; asm volatile("" : "+a"(acc[i])); }
    u4 fa = {0, 0, 0, 0}, fb = {0, 0, 0, 0};
    asm volatile("" : "+v"(fa), "+v"(fb));
    u4 rg[NL ? NL : 1];
    const u4 *gp = g + threadIdx.x;
    const unsigned voff = threadIdx.x * 16;
    i4 rsrc;
    rsrc[0] = (int)(unsigned)(uintptr_t)g; rsrc[1] = (int)(unsigned)((uintptr_t)g >> 32); rsrc[2] = 1 << 20; rsrc[3] = 0x00020000;
    rsrc[0] = __builtin_amdgcn_readfirstlane(rsrc[0]); rsrc[1] = __builtin_amdgcn_readfirstlane(rsrc[1]);
    rsrc[2] = __builtin_amdgcn_readfirstlane(rsrc[2]); rsrc[3] = __builtin_amdgcn_readfirstlane(rsrc[3]);
    const unsigned ldsbase = (wave & 3) * 16384;
    unsigned sink = 0;
    constexpr int NM = (MF ? 64 : 128) * 4 / WAVES;
    long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < NM; ++u) {
            if constexpr (MF == 0) asm volatile("v_mfma_f32_16x16x32_bf16 %0, %1, %2, %0" : "+a"(acc[u & (NACC - 1)]) : "v"(fa), "v"(fb));
            else asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+a"(*reinterpret_cast<__attribute__((ext_vector_type(16))) float *>(&acc[(u & (NACC / 4 - 1)) * 4])) : "v"(fa), "v"(fb));
            if constexpr (KIND == 11 || KIND == 12) {
                // the same loads in four (KIND 11) or two (KIND 12) back-to-back bursts instead of one at a time
                constexpr int B = KIND == 11 ? 4 : 2;
                if (u % (NM / B) == 1) {
#pragma unroll
                    for (int j = 0; j < NL / B; ++j) {
                        const int i = (u / (NM / B)) * (NL / B) + j;
                        asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(rg[i]) : "v"(gp + i * 256));
                    }
                }
            } else if (NL > 0 && u % (NM / (NL ? NL : 1)) == 1) {
                const int i = u / (NM / (NL ? NL : 1));
                if constexpr (KIND == 1) asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(rg[i]) : "v"(gp + i * 256));
                if constexpr (KIND == 2) asm volatile("global_load_dwordx4 %0, %1, %2" : "=v"(rg[i]) : "v"(voff + i * 4096), "s"(g));
                if constexpr (KIND == 3) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(ldsbase + i * 1024), "v"(gp + i * 256) : "memory", "m0");
                if constexpr (KIND == 4) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2" :: "s"(ldsbase + i * 1024), "v"(voff + i * 4096), "s"(g) : "memory", "m0");
                if constexpr (KIND == 5) asm volatile("buffer_load_dwordx4 %0, %1, %2, 0 offen" : "=v"(rg[i]) : "v"(voff + i * 4096), "s"(rsrc));
                if constexpr (KIND == 6) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, 0 offen lds" :: "s"(ldsbase + i * 1024), "v"(voff + i * 4096), "s"(rsrc) : "memory", "m0");
                if constexpr (KIND == 7) asm volatile("ds_write_b128 %0, %1" :: "v"(voff + i * 1024), "v"(fa) : "memory");
                if constexpr (KIND == 8) asm volatile("ds_write_b64 %0, %1" :: "v"(voff + i * 1024), "v"(*reinterpret_cast<__attribute__((ext_vector_type(2))) unsigned *>(&fa)) : "memory");
                if constexpr (KIND == 9) asm volatile("v_add_u32 %0, %0, %1\n" : "+v"(sink) : "v"(voff));
                if constexpr (KIND == 13) asm volatile("ds_read_b128 %0, %1" : "=v"(rg[i]) : "v"(voff + (i % 16) * 1024));
                if constexpr (KIND == 14) {
                    u2 t;
                    asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(t) : "v"(voff / 2 + (i % 16) * 512));
                    rg[i][0] = t[0]; rg[i][1] = t[1];
                }
            }
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
        if constexpr (KIND == 1 || KIND == 2 || KIND == 5 || KIND == 11 || KIND == 12 || KIND == 13 || KIND == 14) { for (int i = 0; i < NL; ++i) sink ^= rg[i][0]; }
    }
    long long t1 = clock64();
    float s = 0;
#pragma unroll
    for (int i = 0; i < NACC; ++i) s += acc[i][0];
    if (sink == 0x12345678u || s == 1.2345f) out[1] = sink;
    // the slowest wavefront counts (with two per SIMD the older one is served first and finishes early)
    if ((threadIdx.x & 63) == 0 && blockIdx.x == 0) atomicMax(reinterpret_cast<unsigned long long *>(out), static_cast<unsigned long long>(t1 - t0));
}
template <int KIND, int NL, int MF, int WAVES = 4> void run(const char *name, long long *o, const u4 *g) {
    const int iters = 2000;
    (void)hipFuncSetAttribute((const void *)mix<KIND, NL, MF, WAVES>, hipFuncAttributeMaxDynamicSharedMemorySize, 131072);
    long long r[2] = {0, 0};
    (void)hipMemset(o, 0, 16);
    hipLaunchKernelGGL((mix<KIND, NL, MF, WAVES>), dim3(1), dim3(WAVES * 64), 131072, 0, o, g, iters);
    (void)hipDeviceSynchronize();
    (void)hipMemcpy(r, o, 16, hipMemcpyDeviceToHost);
    // per SIMD and iteration: 2048 clocks of MFMAs and, with 8 wavefronts, twice the memory instructions
    const int per_simd = (NL ? NL : 1) * WAVES / 4;
    printf("%-72s clk per K-step %8.1f  extra per op %6.2f\n", name, (double)r[0] / iters, ((double)r[0] / iters - 2073.0) / per_simd);
}
int main() {
    long long *o; u4 *g; (void)hipMalloc(&o, 64); (void)hipMalloc(&g, 1 << 20); (void)hipMemset(g, 0, 1 << 20);
    run<1, 16, 0>("16x16x32: global_load_dwordx4 v, v64, off", o, g);
    run<2, 16, 0>("16x16x32: global_load_dwordx4 v, v32, s[base]", o, g);
    run<3, 16, 0>("16x16x32: m0 + global_load_lds_dwordx4 v64, off", o, g);
    run<4, 16, 0>("16x16x32: m0 + global_load_lds_dwordx4 v32, s[base]", o, g);
    run<5, 16, 0>("16x16x32: buffer_load_dwordx4 v, v32, s[rsrc] offen", o, g);
    run<6, 16, 0>("16x16x32: m0 + buffer_load_dwordx4 v32, s[rsrc] offen lds", o, g);
    run<7, 16, 0>("16x16x32: ds_write_b128", o, g);
    run<8, 32, 0>("16x16x32: ds_write_b64 x32", o, g);
    run<9, 32, 0>("16x16x32: 32 VALU ops", o, g);
    run<1, 16, 1>("32x32x16: global_load_dwordx4 v, v64, off", o, g);
    run<3, 16, 1>("32x32x16: m0 + global_load_lds_dwordx4 v64, off", o, g);
    run<7, 16, 1>("32x32x16: ds_write_b128", o, g);
    run<0, 0, 1>("32x32x16: MFMA only", o, g);
    run<13, 16, 1>("32x32x16: ds_read_b128", o, g);
    run<14, 32, 1>("32x32x16: ds_read_b64_tr_b16 x32", o, g);
    run<13, 16, 0>("16x16x32: ds_read_b128", o, g);
    run<14, 32, 0>("16x16x32: ds_read_b64_tr_b16 x32", o, g);
    run<11, 16, 1>("32x32x16: global_load_dwordx4, four bursts of four", o, g);
    run<12, 16, 1>("32x32x16: global_load_dwordx4, two bursts of eight", o, g);
    run<11, 16, 0>("16x16x32: global_load_dwordx4, four bursts of four", o, g);
    // two wavefronts per SIMD, each with half the MFMAs and the same number of memory instructions as above
    // (so twice as many per SIMD): does the other wavefront's MFMA stream hide them?
    run<0, 0, 1, 8>("32x32x16, 8 wavefronts: MFMA only", o, g);
    run<1, 16, 1, 8>("32x32x16, 8 wavefronts: global_load_dwordx4 v, v64, off", o, g);
    run<3, 16, 1, 8>("32x32x16, 8 wavefronts: m0 + global_load_lds_dwordx4 v64, off", o, g);
    run<7, 16, 1, 8>("32x32x16, 8 wavefronts: ds_write_b128", o, g);
    run<0, 0, 0, 8>("16x16x32, 8 wavefronts: MFMA only", o, g);
    run<1, 16, 0, 8>("16x16x32, 8 wavefronts: global_load_dwordx4 v, v64, off", o, g);
    run<3, 16, 0, 8>("16x16x32, 8 wavefronts: m0 + global_load_lds_dwordx4 v64, off", o, g);
    run<7, 16, 0, 8>("16x16x32, 8 wavefronts: ds_write_b128", o, g);
    return 0;
}
