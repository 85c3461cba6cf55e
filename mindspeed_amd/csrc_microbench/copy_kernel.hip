// Measurement helper, not part of the product library: a plain device copy kernel (16-byte vectors, grid-stride).
// The microbenchmarks use it as the reference point "what a copy of this size reaches on this board", and the
// profiler-counter tooling calibrates FETCH_SIZE / WRITE_SIZE against a transfer of known size with it.
// Built into libmindspeed_amd_microbench.so by python -m mindspeed_amd.build --microbench.
#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace {
typedef unsigned v16 __attribute__((ext_vector_type(4)));

__global__ __launch_bounds__(256) void copy_bytes_kernel(const v16 *__restrict__ src, v16 *__restrict__ dst, size_t nvec) {
    for (size_t i = blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x; i < nvec;
         i += static_cast<size_t>(gridDim.x) * blockDim.x)
        dst[i] = src[i];
}
__global__ void copy_tail_kernel(const unsigned char *src, unsigned char *dst, size_t begin, size_t end) {
    const size_t i = begin + blockIdx.x * static_cast<size_t>(blockDim.x) + threadIdx.x;
    if (i < end) dst[i] = src[i];
}
}  // namespace

// Returns 0 on success, 1 for a NULL pointer, 2 for a launch error.
extern "C" int mb_copy_bytes(void *stream_, const void *src, void *dst, size_t bytes) {
    hipStream_t stream = static_cast<hipStream_t>(stream_);
    if (bytes == 0) return 0;
    if (src == nullptr || dst == nullptr) return 1;
    const bool aligned = (reinterpret_cast<uintptr_t>(src) & 15u) == 0 && (reinterpret_cast<uintptr_t>(dst) & 15u) == 0;
    const size_t nvec = aligned ? bytes / 16 : 0;
    if (nvec) {
        size_t blocks = (nvec + 255) / 256;
        if (blocks > 256 * 32) blocks = 256 * 32;
        hipLaunchKernelGGL(copy_bytes_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0, stream,
                           static_cast<const v16 *>(src), static_cast<v16 *>(dst), nvec);
        if (hipGetLastError() != hipSuccess) return 2;
    }
    const size_t done = nvec * 16;
    if (done < bytes) {
        const size_t rest = bytes - done;
        hipLaunchKernelGGL(copy_tail_kernel, dim3(static_cast<unsigned>((rest + 255) / 256)), dim3(256), 0, stream,
                           static_cast<const unsigned char *>(src), static_cast<unsigned char *>(dst), done, bytes);
        if (hipGetLastError() != hipSuccess) return 2;
    }
    return 0;
}
