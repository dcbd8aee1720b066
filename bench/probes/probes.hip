// Measurement probes for the benchmark (libdsv3probe.so): kernels of known traffic / arithmetic that give the
// ceilings this GPU sustains -- a read stream, a copy, read/write mixes, fp8 MFMA loops (registers only, and with a
// GEMM step's operand traffic) and an empty launch.  They are not part of libdsv3fp8.so and nothing in the product
// path calls them.
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <type_traits>

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

// Streams with the read : write mix of the quantisation kernels: every lane reads RD 16-byte pieces and writes WR
// (act_quant and weight_quant read two bytes per byte written, weight_dequant writes two per byte read).
template <int RD, int WR>
__global__ __launch_bounds__(kThreads) void mix_kernel(const v4i* __restrict__ src, v4i* __restrict__ dst, size_t steps) {
    constexpr int U = 4;
    for (size_t st = blockIdx.x; st < steps; st += gridDim.x) {
        v4i v[U][RD];
#pragma unroll
        for (int u = 0; u < U; ++u)
#pragma unroll
            for (int r = 0; r < RD; ++r)
                v[u][r] = __builtin_nontemporal_load(src + ((st * U + u) * RD + r) * kThreads + threadIdx.x);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            v4i x = v[u][0];
#pragma unroll
            for (int r = 1; r < RD; ++r) x ^= v[u][r];
#pragma unroll
            for (int w = 0; w < WR; ++w)
                __builtin_nontemporal_store(x + (v4i){w, w, w, w}, dst + ((st * U + u) * WR + w) * kThreads + threadIdx.x);
        }
    }
}

// 8 wavefronts per compute unit, nothing but fp8 matrix instructions on registers: the fp8 matrix rate the chip
// sustains under its power limit.  SHAPE 16: v_mfma_f32_16x16x128_f8f6f4 (one instruction = one 128-wide scale block),
// 4 x 4 tiles per wavefront; SHAPE 32: v_mfma_f32_32x32x64_f8f6f4, two chained instructions per scale block (the
// second accumulates onto the first), 2 x 2 tiles per wavefront -- the same flops per step and per cycle, half the
// operand-register reads per flop.
// ORDER 0: one operand pair for all tiles (the operand buses do not toggle between instructions: the most the matrix
// cores issue).  ORDER 1: different fragments of random bytes, consecutive instructions share their A operand
// (what a GEMM's loop nest issues).  ORDER 2: the same fragments in an order in which consecutive instructions
// share neither operand.
// FOLD false: products accumulate inside the matrix core (what a GEMM with power-of-two scales issues).  FOLD true:
// every raw product is folded into its binary32 accumulator by one FMA per element (what binary32 block scales need:
// 4 per 16 x 16 x 128 product, 16 per 32 x 32 x 128 product), one product behind the matrix instructions.
typedef float v16f __attribute__((ext_vector_type(16)));
template <int SHAPE, int ORDER, bool FOLD>
__global__ __launch_bounds__(512, 1) void mfma_kernel(int iters, const int* __restrict__ rnd, float* sink) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    v8i a[4], b[4];                                                   // SHAPE 32: [tile * 2 + K half]
    for (int f = 0; f < 4; ++f)
        for (int i = 0; i < 8; ++i) {
            const unsigned idx = (((blockIdx.x * 8 + wave) * 64 + lane) * 64 + f * 8 + i) & 0xfffff;
            a[f][i] = rnd[idx] & 0x7b7b7b7b;                              // no NaN codes
            b[f][i] = rnd[(idx + 32) & 0xfffff] & (int)0xfbfbfbfb;
        }
    if (ORDER == 0) for (int f = 1; f < 4; ++f) { a[f] = a[0]; b[f] = b[0]; }
    const float sc = 1.0f + lane * 1e-7f;
    float r = 0.f;
    if constexpr (SHAPE == 16) {
        v4f acc[4][4];
        for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) acc[i][j] = (v4f){0.f, 0.f, 0.f, 0.f};
        v4f prev = {0.f, 0.f, 0.f, 0.f};
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 4; ++i)
#pragma unroll
                for (int jj = 0; jj < 4; ++jj) {
                    // ORDER 2 walks the diagonals: (0,0) (1,1) (2,2) (3,3) (0,1) (1,2) ...
                    const int ti = ORDER == 2 ? jj : i, tj = ORDER == 2 ? (jj + i) & 3 : jj;
                    if (FOLD) {
                        const v4f z = {0.f, 0.f, 0.f, 0.f};
                        const v4f p = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[ti], b[tj], z, 0, 0, 0, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 4; ++e) acc[ti][tj][e] = __builtin_fmaf(prev[e], sc, acc[ti][tj][e]);
                        prev = p;
                    } else {
                        acc[ti][tj] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[ti], b[tj], acc[ti][tj], 0, 0, 0, 0, 0, 0);
                    }
                }
        }
        r = prev[0];
        for (int i = 0; i < 4; ++i) for (int j = 0; j < 4; ++j) r += acc[i][j][0] + acc[i][j][1] + acc[i][j][2] + acc[i][j][3];
    } else {
        v16f acc[2][2], prev;
        for (int e = 0; e < 16; ++e) { prev[e] = 0.f; for (int i = 0; i < 2; ++i) for (int j = 0; j < 2; ++j) acc[i][j][e] = 0.f; }
        for (int it = 0; it < iters; ++it) {
#pragma unroll
            for (int i = 0; i < 2; ++i)
#pragma unroll
                for (int j = 0; j < 2; ++j) {
                    if (FOLD) {
                        v16f p;
#pragma unroll
                        for (int e = 0; e < 16; ++e) p[e] = 0.f;
                        p = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i * 2], b[j * 2], p, 0, 0, 0, 0, 0, 0);
                        p = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i * 2 + 1], b[j * 2 + 1], p, 0, 0, 0, 0, 0, 0);
#pragma unroll
                        for (int e = 0; e < 16; ++e) acc[i][j][e] = __builtin_fmaf(prev[e], sc, acc[i][j][e]);
                        prev = p;
                    } else {
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i * 2], b[j * 2], acc[i][j], 0, 0, 0, 0, 0, 0);
                        acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[i * 2 + 1], b[j * 2 + 1], acc[i][j], 0, 0, 0, 0, 0, 0);
                    }
                }
        }
        r = prev[0];
        for (int i = 0; i < 2; ++i) for (int j = 0; j < 2; ++j) for (int e = 0; e < 16; ++e) r += acc[i][j][e];
    }
    if (r == 12345.678f) sink[blockIdx.x] = r;
}

// The loops above inside the operand traffic of a 256 x 256 x 128 GEMM step, with no synchronisation at all: per step
// (16 products of 16 x 16 x 128, or 4 of 32 x 32 x 128) every wavefront copies 4 KiB of an L2-resident 2 MiB window
// into LDS with the direct-to-LDS load (32 KiB per compute unit and 128 small products, as a 256 x 256 tile moves) and
// reads six 2 KiB fragments (two of A, four of B) from LDS into the operand registers (12 KiB, as a 64 x 128 wavefront
// tile reads), one step ahead of the products that use them.  Nothing waits on a barrier and the copied bytes are
// never consumed, so this is what the chip sustains for the GEMM's mix of matrix instructions, fold (FOLD) and data
// movement when every overlap is perfect.
template <int SHAPE, bool FOLD>
__global__ __launch_bounds__(512, 1) void mfma_traffic_kernel(int iters, const int* __restrict__ rnd, float* sink) {
    extern __shared__ __align__(16) unsigned char lds[];               // 64 KiB of fragments | 64 KiB landing area
    const int lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    v4i* frag = (v4i*)lds;
    for (int i = 0; i < 8; ++i) {
        const unsigned idx = ((blockIdx.x * 4096 + threadIdx.x * 8 + i) * 4) & 0xffffc;
        v4i v = *(const v4i*)(rnd + idx);
        for (int e = 0; e < 4; ++e) v[e] &= 0x7b7b7b7b;                // no NaN codes
        frag[threadIdx.x * 8 + i] = v;
    }
    __syncthreads();
    auto load = [&](int f) {                                           // fragment f of 32: lane l's two 16-byte halves
        const v4i lo = frag[(f & 31) * 128 + lane], hi = frag[(f & 31) * 128 + 64 + lane];
        return (v8i){lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
    };
    // Two register sets of A and of B fragments: a step multiplies out of one while the reads for the next step
    // land in the other (B: four new fragments per step; A: two per step, a new set of four every second step).
    // (SHAPE 32 has room for one set of B fragments only -- its raw products take 32 registers where SHAPE 16 needs
    // 8 --: a fragment pair is read again as soon as the last product of the step that uses it has been issued.)
    constexpr int NB = SHAPE == 16 ? 2 : 1;
    v8i a[2][4], b[NB][4];
    for (int f = 0; f < 4; ++f) { a[0][f] = load(wave + f); a[1][f] = load(wave + 8 + f); b[0][f] = load(wave + 4 + f); }
    constexpr int NT = SHAPE == 16 ? 16 : 4, NE = SHAPE == 16 ? 4 : 16;
    float acc[NT][NE], prev[NE];
    for (int t = 0; t < NT; ++t) for (int e = 0; e < NE; ++e) acc[t][e] = 0.f;
    for (int e = 0; e < NE; ++e) prev[e] = 0.f;
    const float sc = 1.0f + lane * 1e-7f;
    const uint32_t land = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)lds + 65536u + wave * 4096u;
    auto step = [&](int it, auto phase) {
        constexpr int P = decltype(phase)::value, BC = P & 1, AC = P >> 1;
        const unsigned char* src = (const unsigned char*)rnd + (size_t)(((it * 8 + wave + blockIdx.x * 3) * 4) & 2047) * 1024;
#pragma unroll
        for (int c = 0; c < 4; ++c)
            asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
                         :: "v"(lane * 16u), "s"(src + c * 1024), "s"(land + BC * 32768u + c * 1024u) : "memory", "m0");
        if constexpr (NB == 2) {
#pragma unroll
            for (int j = 0; j < 4; ++j) b[BC ^ 1][j] = load(it * 6 + wave + j);
        }
        a[AC ^ 1][BC * 2] = load(it * 6 + wave + 4);
        a[AC ^ 1][BC * 2 + 1] = load(it * 6 + wave + 5);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < NT; ++t) {
            float p[NE];
            if constexpr (SHAPE == 16) {
                v4f c;
#pragma unroll
                for (int e = 0; e < 4; ++e) c[e] = FOLD ? 0.f : acc[t][e];
                c = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a[AC][t >> 2], b[BC][t & 3], c, 0, 0, 0, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 4; ++e) p[e] = c[e];
            } else {
                v16f c;
#pragma unroll
                for (int e = 0; e < 16; ++e) c[e] = FOLD ? 0.f : acc[t][e];
                c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[AC][(t >> 1) * 2], b[0][(t & 1) * 2], c, 0, 0, 0, 0, 0, 0);
                c = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(a[AC][(t >> 1) * 2 + 1], b[0][(t & 1) * 2 + 1], c, 0, 0, 0, 0, 0, 0);
#pragma unroll
                for (int e = 0; e < 16; ++e) p[e] = c[e];
                if (t >= 2) {                                         // this B pair's last use of the step
                    b[0][(t & 1) * 2] = load(it * 6 + wave + (t & 1) * 2);
                    b[0][(t & 1) * 2 + 1] = load(it * 6 + wave + (t & 1) * 2 + 1);
                }
            }
            if (FOLD) {
#pragma unroll
                for (int e = 0; e < NE; ++e) { acc[t][e] = __builtin_fmaf(prev[e], sc, acc[t][e]); prev[e] = p[e]; }
            } else {
#pragma unroll
                for (int e = 0; e < NE; ++e) acc[t][e] = p[e];
            }
        }
        asm volatile("s_waitcnt vmcnt(8)" ::: "memory");               // at most two steps of copies in flight
        __builtin_amdgcn_sched_barrier(0);
    };
    for (int it = 0; it < iters; it += 4) {                            // iters is a multiple of four
        step(it, std::integral_constant<int, 0>{});
        step(it + 1, std::integral_constant<int, 1>{});
        step(it + 2, std::integral_constant<int, 2>{});
        step(it + 3, std::integral_constant<int, 3>{});
    }
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    float r = prev[0];
    for (int t = 0; t < NT; ++t) for (int e = 0; e < NE; ++e) r += acc[t][e];
    if (r == 12345.678f) sink[blockIdx.x] = r;
}

__global__ void null_kernel() {}

int status() { return hipGetLastError() == hipSuccess ? 0 : 1; }

template <typename KernelT>
int launch_traffic(KernelT kernel, bool& lds_set, int iters, const void* rnd, float* sink, void* stream) {
    if (!lds_set) {                                                     // 128 KiB of dynamic LDS needs the attribute once
        if (hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 131072) != hipSuccess) return 1;
        lds_set = true;
    }
    hipLaunchKernelGGL(kernel, dim3(256), dim3(512), 131072, (hipStream_t)stream, iters, (const int*)rnd, sink);
    return status();
}

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

// reads rd and writes wr 16-byte pieces per lane and step (rd : wr = 2 : 1 or 1 : 2); bytes_read is rounded down to
// whole steps and returned through *done_read (bytes written = that * wr / rd)
int dsv3_probe_mix(const void* src, void* dst, size_t bytes_read, int rd, int wr, size_t* done_read, void* stream) {
    if (!src || !dst || !((rd == 2 && wr == 1) || (rd == 1 && wr == 2))) return 2;
    const size_t per_step = (size_t)kThreads * 4 * rd * 16;
    const size_t steps = bytes_read / per_step;
    if (steps == 0) return 2;
    if (done_read) *done_read = steps * per_step;
    const unsigned g = (unsigned)(steps < 4096 ? steps : 4096);
    if (rd == 2) hipLaunchKernelGGL((mix_kernel<2, 1>), dim3(g), dim3(kThreads), 0, (hipStream_t)stream, (const v4i*)src, (v4i*)dst, steps);
    else         hipLaunchKernelGGL((mix_kernel<1, 2>), dim3(g), dim3(kThreads), 0, (hipStream_t)stream, (const v4i*)src, (v4i*)dst, steps);
    return status();
}

// flops of one launch: 256 workgroups x 8 wavefronts x iters x 16 x 65536.  rnd: 4 MiB of random bytes.
// 16 x 16 x 128 instructions:
//   mode 0: constant operands, 1: changing random operands, 2: changing operands + the fold's four FMAs,
//   3: mode 2 with a GEMM step's copies into LDS and fragment reads from LDS around it, 4: mode 1 with that traffic
//   (the ceiling of power-of-two scales), 8: mode 2 in an order that shares no operand between consecutive instructions
// 32 x 32 x 64 instructions (two per 128-wide scale block): mode 5: changing operands, 6: + fold, 7: + fold + traffic
int dsv3_probe_mfma(int iters, int mode, const void* rnd, float* sink, void* stream) {
    const bool traffic = mode == 3 || mode == 4 || mode == 7;
    if (!sink || !rnd || iters <= 0 || mode < 0 || mode > 8 || (traffic && iters % 4)) return 2;
    static bool set3 = false, set4 = false, set7 = false;
#define DSV3_PROBE(S_, O_, F_) hipLaunchKernelGGL((mfma_kernel<S_, O_, F_>), dim3(256), dim3(512), 0, (hipStream_t)stream, iters, (const int*)rnd, sink)
    switch (mode) {
        case 0: DSV3_PROBE(16, 0, false); break;
        case 1: DSV3_PROBE(16, 1, false); break;
        case 2: DSV3_PROBE(16, 1, true); break;
        case 3: return launch_traffic(mfma_traffic_kernel<16, true>, set3, iters, rnd, sink, stream);
        case 4: return launch_traffic(mfma_traffic_kernel<16, false>, set4, iters, rnd, sink, stream);
        case 5: DSV3_PROBE(32, 1, false); break;
        case 6: DSV3_PROBE(32, 1, true); break;
        case 7: return launch_traffic(mfma_traffic_kernel<32, true>, set7, iters, rnd, sink, stream);
        case 8: DSV3_PROBE(16, 2, true); break;
    }
#undef DSV3_PROBE
    return status();
}
double dsv3_probe_mfma_flops(int iters) { return 256.0 * 8.0 * iters * 16.0 * 65536.0; }

int dsv3_probe_null(void* stream) {
    hipLaunchKernelGGL(null_kernel, dim3(1), dim3(64), 0, (hipStream_t)stream);
    return status();
}

}  // extern "C"
