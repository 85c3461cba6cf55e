// Hardware probe: LDS throughput of one compute unit by instruction form and number of wavefronts.
// Reads: ds_read_b32 / b64 / b128 and the transposing ds_read_b64_tr_b16, 16 independent reads in flight per wavefront;
// writes: ds_write_b32 / b64 / b96 / b128, the two-address forms, and the global -> LDS transfer, 8 in flight.
// Prints clocks per wavefront-instruction and bytes per clock for the whole compute unit; conflict-free addresses.
// Build and run: python -m mindspeed_amd.probes run lds_rates
#include <hip/hip_runtime.h>
#include <stdio.h>
typedef unsigned u4 __attribute__((ext_vector_type(4)));
typedef unsigned u2 __attribute__((ext_vector_type(2)));
typedef unsigned u3 __attribute__((ext_vector_type(3)));

template <int W>   // W: 4, 8, 16 bytes; 9 = transposing 8-byte read
__global__ void rd(long long *out, int iters, int stride) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    for (int i = threadIdx.x; i < 65536 / 4; i += blockDim.x) reinterpret_cast<int *>(lds)[i] = i;
    __syncthreads();
    const int lane = threadIdx.x & 63;
    unsigned a = lane * stride;
    u4 r[16];
    unsigned sink = 0;
    long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 16; ++u) {
            if constexpr (W == 16) asm volatile("ds_read_b128 %0, %1" : "=v"(r[u]) : "v"(a + u * 2048));
            else if constexpr (W == 8) { u2 t; asm volatile("ds_read_b64 %0, %1" : "=v"(t) : "v"(a + u * 2048)); r[u][0] = t[0]; r[u][1] = t[1]; }
            else if constexpr (W == 9) { u2 t; asm volatile("ds_read_b64_tr_b16 %0, %1" : "=v"(t) : "v"(a + u * 2048)); r[u][0] = t[0]; r[u][1] = t[1]; }
            else { unsigned t; asm volatile("ds_read_b32 %0, %1" : "=v"(t) : "v"(a + u * 2048)); r[u][0] = t; }
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
        for (int u = 0; u < 16; ++u) sink ^= r[u][0];
    }
    long long t1 = clock64();
    if (sink == 0x12345678u) out[1] = sink;
    if (threadIdx.x == 0) out[0] = t1 - t0;
}
template <int W> void run_read(const char *name, int bytes, long long *o) {
    const int iters = 4000;
    for (int si = 0; si < (bytes == 16 ? 1 : 2); ++si) {
        int stride = si ? 16 : bytes;
        for (int threads : {64, 128, 256, 512}) {
            long long r[2] = {0, 0};
            hipLaunchKernelGGL(rd<W>, dim3(1), dim3(threads), 65536, 0, o, iters, stride); (void)hipDeviceSynchronize();
            (void)hipMemcpy(r, o, 16, hipMemcpyDeviceToHost);
            double per = (double)r[0] / (iters * 16);
            printf("%-22s lane stride %2d B  waves %d  clk per wave-instr %7.2f  CU bytes/clk %7.1f\n", name, stride, threads / 64, per,
                   (threads / 64) * 64.0 * bytes / per);
        }
    }
}

template <int W>
__global__ void wr(long long *out, const u4 *g, int iters, int stride) {
    extern __shared__ __attribute__((aligned(16))) char lds[];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    unsigned a = (wave * 8192 + lane * stride) & 65535;
    u4 v = {1, 2, 3, (unsigned)lane};
    asm volatile("" : "+v"(v));
    u2 vhi = {v[2], v[3]};
    asm volatile("" : "+v"(vhi));
    const u4 *gp = g + threadIdx.x;
    long long t0 = clock64();
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            if constexpr (W == 16) asm volatile("ds_write_b128 %0, %1" :: "v"(a + u * 1024), "v"(v) : "memory");
            if constexpr (W == 12) asm volatile("ds_write_b96 %0, %1" :: "v"(a + u * 1024), "v"(*reinterpret_cast<u3 *>(&v)) : "memory");
            if constexpr (W == 8) asm volatile("ds_write_b64 %0, %1" :: "v"(a + u * 512), "v"(*reinterpret_cast<u2 *>(&v)) : "memory");
            if constexpr (W == 4) asm volatile("ds_write_b32 %0, %1" :: "v"(a + u * 256), "v"(v[0]) : "memory");
            if constexpr (W == 17) asm volatile("ds_write2_b64 %0, %1, %2 offset1:1" :: "v"(a + u * 1024), "v"(*reinterpret_cast<u2 *>(&v)), "v"(vhi) : "memory");
            if constexpr (W == 18) asm volatile("ds_write2st64_b64 %0, %1, %2 offset1:1" :: "v"((a & ~1023u) / 2 + (lane * 8) + u * 1024), "v"(*reinterpret_cast<u2 *>(&v)), "v"(vhi) : "memory");
            if constexpr (W == 20) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" :: "s"(wave * 8192 + u * 1024), "v"(gp + u * 256) : "memory", "m0");
            if constexpr (W == 21) asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" :: "s"(wave * 8192 + u * 256), "v"(reinterpret_cast<const unsigned *>(g) + threadIdx.x + u * 256) : "memory", "m0");
        }
        asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    }
    long long t1 = clock64();
    if (threadIdx.x == 0) out[0] = t1 - t0;
    if (lds[threadIdx.x] == 77 && iters < 0) out[1] = 1;
}
template <int W> void run_write(const char *name, int bytes, long long *o, const u4 *g, int stride) {
    const int iters = 4000;
    for (int threads : {64, 256, 512}) {
        long long r[2] = {0, 0};
        hipLaunchKernelGGL(wr<W>, dim3(1), dim3(threads), 65536, 0, o, g, iters, stride); (void)hipDeviceSynchronize();
        (void)hipMemcpy(r, o, 16, hipMemcpyDeviceToHost);
        double per = (double)r[0] / (iters * 8);
        printf("%-34s lane stride %3d B  waves %d  clk per wave-instr %7.2f  CU bytes/clk %7.1f\n", name, stride, threads / 64, per,
               (threads / 64) * 64.0 * bytes / per);
    }
}
int main() {
    long long *o; u4 *g; (void)hipMalloc(&o, 64); (void)hipMalloc(&g, 1 << 20); (void)hipMemset(g, 0, 1 << 20);
    run_read<4>("ds_read_b32", 4, o);
    run_read<8>("ds_read_b64", 8, o);
    run_read<9>("ds_read_b64_tr_b16", 8, o);
    run_read<16>("ds_read_b128", 16, o);
    run_write<4>("ds_write_b32", 4, o, g, 4);
    run_write<8>("ds_write_b64", 8, o, g, 8);
    run_write<12>("ds_write_b96", 12, o, g, 16);
    run_write<16>("ds_write_b128", 16, o, g, 16);
    run_write<17>("ds_write2_b64 (adjacent)", 16, o, g, 16);
    run_write<18>("ds_write2st64_b64 (512 B apart)", 16, o, g, 8);
    run_write<20>("global_load_lds_dwordx4", 16, o, g, 16);
    run_write<21>("global_load_lds_dword", 4, o, g, 4);
    return 0;
}
