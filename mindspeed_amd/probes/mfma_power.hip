// Hardware probe: pure MFMA loops (no memory traffic) on random and on all-zero register data, for the two bf16 MFMA
// shapes v_mfma_f32_32x32x16_bf16 and v_mfma_f32_16x16x32_bf16: rate, board power and shader clock, four seconds each.
// Shows how far the matrix cores alone get before the board's power limit pulls the clock down, and that the limit
// depends on the operand values.  Power and clock come from the amdgpu hwmon / sysfs files (read-only).
// Build and run: python -m mindspeed_amd.probes run mfma_power
// With arguments `quick SECONDS` only the 32x32x16 loop on random data runs, for that long (what a benchmark calls to
// read the board it is running on).
#include <hip/hip_runtime.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>
#include <thread>
#include <atomic>
#include <vector>
#include <chrono>
#include <glob.h>
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned v16 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void k32(const v16 *src, float *out, int iters) {
    v16 a[2][4], b[2][4];
    const int t = threadIdx.x + blockIdx.x * 256;
    for (int s = 0; s < 2; ++s) for (int i = 0; i < 4; ++i) { a[s][i] = src[(t * 16 + s * 8 + i) & 65535]; b[s][i] = src[(t * 16 + s * 8 + 4 + i) & 65535]; }
    f32x16 acc[4][4];
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int s = 0; s < 2; ++s)
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int j = 0; j < 4; ++j)
                    acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, b[s][j]), __builtin_bit_cast(bf16x8, a[s][i]), acc[i][j], 0, 0, 0);
    }
    float r = 0.f;
    for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) for (int e = 0; e < 16; ++e) r += acc[i][j][e];
    if (r == 123.456f) out[t] = r;
}

__global__ __launch_bounds__(256) void k16(const v16 *src, float *out, int iters) {
    v16 a[8], b[8];
    const int t = threadIdx.x + blockIdx.x * 256;
    for (int i = 0; i < 8; ++i) { a[i] = src[(t * 16 + i) & 65535]; b[i] = src[(t * 16 + 8 + i) & 65535]; }
    f32x4 acc[8][8];
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int e = 0; e < 4; ++e) acc[i][j][e] = 0.f;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 8; ++j)
                acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, b[j]), __builtin_bit_cast(bf16x8, a[i]), acc[i][j], 0, 0, 0);
    }
    float r = 0.f;
    for (int i = 0; i < 8; ++i) for (int j = 0; j < 8; ++j) for (int e = 0; e < 4; ++e) r += acc[i][j][e];
    if (r == 123.456f) out[t] = r;
}

static std::string hwmon;
static double read_num(const std::string &p) { FILE *f = fopen(p.c_str(), "r"); if (!f) return -1; double v = -1; if (fscanf(f, "%lf", &v) != 1) v = -1; fclose(f); return v; }
static int read_sclk() {
    std::string p = hwmon.substr(0, hwmon.find("/hwmon")) + "/pp_dpm_sclk";
    FILE *f = fopen(p.c_str(), "r"); if (!f) return -1; char line[128]; int mhz = -1;
    while (fgets(line, sizeof line, f)) if (strchr(line, '*')) { char *c = strchr(line, ':'); if (c) mhz = atoi(c + 1); }
    fclose(f); return mhz;
}

int main(int argc, char **argv) {
    glob_t g; if (glob("/sys/class/drm/card*/device/hwmon/hwmon*", 0, nullptr, &g) == 0 && g.gl_pathc) hwmon = g.gl_pathv[0];
    const bool quick = argc >= 2 && strcmp(argv[1], "quick") == 0;
    const double seconds = quick && argc >= 3 ? atof(argv[2]) : 4.0;
    const int n = 65536;
    std::vector<unsigned> h(n * 4);
    v16 *src; float *out;
    (void)hipMalloc(&src, n * 16); (void)hipMalloc(&out, 1 << 22);
    for (int mode = 0; mode < (quick ? 1 : 2); ++mode) {   // 0: random bf16 values ~N(0,1)-like bit patterns, 1: zeros
        srand(1);
        for (auto &w : h) {
            if (mode == 1) { w = 0; continue; }
            auto rb = [] { float f = ((rand() % 2001) - 1000) / 500.0f; unsigned u; memcpy(&u, &f, 4); return (u >> 16) | (rand() & 0); };
            w = rb() | (rb() << 16);
        }
        (void)hipMemcpy(src, h.data(), n * 16, hipMemcpyHostToDevice);
        for (int which = 0; which < (quick ? 1 : 2); ++which) {
            const int iters = (which == 0 ? 20000 : 10000) / (quick ? 8 : 1);   // same flops per launch: 32 x 32768 vs 64 x 16384 per iteration
            const double flops_per_launch = 1024.0 * 4 * (which == 0 ? 32.0 * 32768 : 64.0 * 16384) * iters;
            auto launch = [&] { if (which == 0) hipLaunchKernelGGL(k32, dim3(1024), dim3(256), 0, 0, src, out, iters); else hipLaunchKernelGGL(k16, dim3(1024), dim3(256), 0, 0, src, out, iters); };
            launch(); (void)hipDeviceSynchronize();
            std::atomic<bool> stop{false}; std::vector<double> w; std::vector<int> mhz;
            std::thread th([&] { while (!stop) { w.push_back(read_num(hwmon + "/power1_input") / 1e6); mhz.push_back(read_sclk()); std::this_thread::sleep_for(std::chrono::milliseconds(quick ? 50 : 200)); } });
            hipEvent_t e0, e1; (void)hipEventCreate(&e0); (void)hipEventCreate(&e1);
            auto t0 = std::chrono::steady_clock::now(); int launches = 0;
            (void)hipEventRecord(e0, 0);
            while (std::chrono::duration<double>(std::chrono::steady_clock::now() - t0).count() < seconds) { launch(); (void)hipDeviceSynchronize(); ++launches; }
            (void)hipEventRecord(e1, 0); (void)hipEventSynchronize(e1);
            stop = true; th.join();
            float ms; (void)hipEventElapsedTime(&ms, e0, e1);
            double aw = 0, am = 0; int c = 0; for (size_t i = w.size() / 4; i < w.size(); ++i) { aw += w[i]; am += mhz[i]; ++c; }
            printf("%s %s: %.1f TFLOP/s  %.0f W  %.0f MHz  (%d launches, %.2f ms each)\n", which == 0 ? "32x32x16" : "16x16x32", mode == 0 ? "random" : "zeros",
                   flops_per_launch * launches / ms / 1e9, aw / c, am / c, launches, ms / launches);
            fflush(stdout);
        }
    }
    return 0;
}
