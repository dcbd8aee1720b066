// Measurement probes for the benchmark (libdsv3probe.so): kernels of known traffic / arithmetic that give the
// ceilings this GPU sustains -- a read stream, a copy, an fp8 MFMA loop and an empty launch.  They are not part of
// libdsv3fp8.so and nothing in the product path calls them.
#include <hip/hip_runtime.h>
#include <stdint.h>

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));
typedef float v4f __attribute__((ext_vector_type(4)));

namespace {

constexpr int kThreads = 256, kUnroll = 8;                 // 8 x 16 bytes in flight per lane

// Every workgroup reads one contiguous slab of kThreads * kUnroll * 16 bytes per step; the xor of what it read is
// written only if it equals a value that random data does not produce, so the loads cannot be dropped.
__global__ __launch_bounds__(kThreads) void read_stream_kernel(const v4i* __restrict__ src, size_t n16, int* sink) {
    const size_t per_step = (size_t)kThreads * kUnroll;
    v4i acc = {0, 0, 0, 0};
    for (size_t base = (size_t)blockIdx.x * per_step; base < n16; base += (size_t)gridDim.x * per_step) {
        v4i v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + (size_t)u * kThreads + threadIdx.x;
            v[u] = i < n16 ? __builtin_nontemporal_load(src + i) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) acc ^= v[u];
    }
    if ((acc[0] ^ acc[1] ^ acc[2] ^ acc[3]) == 0x5eed1234) sink[blockIdx.x] = acc[0];
}

__global__ __launch_bounds__(kThreads) void copy_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, size_t n16) {
    const size_t per_step = (size_t)kThreads * kUnroll;
    for (size_t base = (size_t)blockIdx.x * per_step; base < n16; base += (size_t)gridDim.x * per_step) {
        v4i v[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + (size_t)u * kThreads + threadIdx.x;
            v[u] = i < n16 ? __builtin_nontemporal_load(src + i) : (v4i){0, 0, 0, 0};
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const size_t i = base + (size_t)u * kThreads + threadIdx.x;
            if (i < n16) __builtin_nontemporal_store(v[u], dst + i);
        }
    }
}

// 8 wavefronts per compute unit, 16 independent accumulator tiles each, nothing but v_mfma_f32_16x16x128_f8f6f4 on
// registers: the fp8 matrix rate the chip sustains under its power limit.  Operands are pseudo-random bytes.
__global__ __launch_bounds__(512, 1) void mfma_kernel(int iters, float* sink) {
    const int lane = threadIdx.x & 63;
    v8i a, b;
    for (int i = 0; i < 8; ++i) {
        a[i] = (int)((lane * 2654435761u + i * 40503u + blockIdx.x * 97u) | 0x01010101u) & 0x7b7b7b7b;
        b[i] = (int)((lane * 2246822519u + i * 3266489917u) | 0x01010101u) & 0x7b7b7b7b;
    }
    v4f acc[16];
    for (int i = 0; i < 16; ++i) acc[i] = (v4f){0.f, 0.f, 0.f, 0.f};
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int t = 0; t < 16; ++t)
            acc[t] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[t], 0, 0, 0, 0, 0, 0);
    }
    float r = 0.f;
    for (int i = 0; i < 16; ++i) r += acc[i][0] + acc[i][1] + acc[i][2] + acc[i][3];
    if (r == 12345.678f) sink[blockIdx.x] = r;
}

__global__ void null_kernel() {}

int status() { return hipGetLastError() == hipSuccess ? 0 : 1; }

}  // namespace

extern "C" {

// grid 0: one resident round of workgroups sized to the device (256 CUs x 8)
int dsv3_probe_read_stream(const void* src, size_t bytes, int* sink, int grid, void* stream) {
    const size_t n16 = bytes / 16;
    if (!src || !sink || n16 == 0) return 2;
    const size_t steps = (n16 + (size_t)kThreads * kUnroll - 1) / ((size_t)kThreads * kUnroll);
    size_t g = grid > 0 ? (size_t)grid : 2048;
    if (g > steps) g = steps;
    hipLaunchKernelGGL(read_stream_kernel, dim3((unsigned)g), dim3(kThreads), 0, (hipStream_t)stream, (const v4i*)src, n16, sink);
    return status();
}

int dsv3_probe_copy(const void* src, void* dst, size_t bytes, int grid, void* stream) {
    const size_t n16 = bytes / 16;
    if (!src || !dst || n16 == 0) return 2;
    const size_t steps = (n16 + (size_t)kThreads * kUnroll - 1) / ((size_t)kThreads * kUnroll);
    size_t g = grid > 0 ? (size_t)grid : 2048;
    if (g > steps) g = steps;
    hipLaunchKernelGGL(copy_kernel, dim3((unsigned)g), dim3(kThreads), 0, (hipStream_t)stream, (const v4i*)src, (v4i*)dst, n16);
    return status();
}

// flops of one launch: 256 workgroups x 8 wavefronts x iters x 16 x 65536
int dsv3_probe_mfma(int iters, float* sink, void* stream) {
    if (!sink || iters <= 0) return 2;
    hipLaunchKernelGGL(mfma_kernel, dim3(256), dim3(512), 0, (hipStream_t)stream, iters, sink);
    return status();
}
double dsv3_probe_mfma_flops(int iters) { return 256.0 * 8.0 * iters * 16.0 * 65536.0; }

int dsv3_probe_null(void* stream) {
    hipLaunchKernelGGL(null_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream);
    return status();
}

}  // extern "C"
