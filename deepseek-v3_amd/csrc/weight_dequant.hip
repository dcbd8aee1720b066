// weight_dequant for gfx950: y[i,j] = out( f32(x[i,j]) * s[i/B, j/B] )
// (reference: inference/kernel.py:60-86).
//
// Bandwidth-bound stream kernel; two thirds of the traffic are writes (1 byte in, 2 bytes out per element for
// bf16), so the layout is chosen for the stores.  Vector path (B == 128, n % 8 == 0): a lane converts 8
// consecutive fp8 bytes of one row (one 8-byte load) into 8 outputs and writes them with ONE 16-byte store, so
// a wavefront's store instruction covers 1 KiB of contiguous output.  A wavefront spans 512 columns of a row,
// the four wavefronts of a workgroup take different rows, and each lane walks kRows rows of the same 128-row
// block so the tile scale is fetched once per lane.  No integer division anywhere.  A scalar kernel covers every
// other shape.
#include "common.hpp"

namespace dsv3 {
namespace {

constexpr int kRows = 8;   // rows per lane -> independent 8-byte loads in flight
constexpr int kWavesY = 4;

template <int YD> struct Store8;   // writes 8 consecutive outputs
template <> struct Store8<DSV3_BF16> {
    static __device__ __forceinline__ void put(void* y, int64_t elem, const float (&f)[8]) {
        v4u a;
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = pack_bf16(f[2 * i], f[2 * i + 1]);
        __builtin_nontemporal_store(a, (v4u*)((uint16_t*)y + elem));
    }
};
template <> struct Store8<DSV3_F16> {
    static __device__ __forceinline__ void put(void* y, int64_t elem, const float (&f)[8]) {
        v4u a;
#pragma unroll
        for (int i = 0; i < 4; ++i) a[i] = pack_f16(f[2 * i], f[2 * i + 1]);
        __builtin_nontemporal_store(a, (v4u*)((uint16_t*)y + elem));
    }
};
template <> struct Store8<DSV3_F32> {
    static __device__ __forceinline__ void put(void* y, int64_t elem, const float (&f)[8]) {
        v4f* p = (v4f*)((float*)y + elem);
        v4f lo = { f[0], f[1], f[2], f[3] }, hi = { f[4], f[5], f[6], f[7] };
        __builtin_nontemporal_store(lo, p);
        __builtin_nontemporal_store(hi, p + 1);
    }
};

template <int YD>
__global__ __launch_bounds__(kWave * kWavesY) void weight_dequant_vec_kernel(
        const v2u* __restrict__ x, const float* __restrict__ s, void* __restrict__ y,
        int64_t m, int n8, int sn) {
    const int col8 = blockIdx.x * kWave + threadIdx.x;           // 8-byte chunk within the row
    const int64_t row0 = ((int64_t)blockIdx.y * kWavesY + threadIdx.y) * kRows;
    if (col8 >= n8 || row0 >= m) return;
    const float sc = s[(row0 >> 7) * sn + (col8 >> 4)];
    v2u v[kRows];
#pragma unroll
    for (int r = 0; r < kRows; ++r)
        if (row0 + r < m) v[r] = __builtin_nontemporal_load(x + (row0 + r) * n8 + col8);
#pragma unroll
    for (int r = 0; r < kRows; ++r) {
        if (row0 + r >= m) break;
        float f[8];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
            v2f lo = fp8x2_lo_to_f32(v[r][i]), hi = fp8x2_hi_to_f32(v[r][i]);
            f[4 * i] = lo.x * sc; f[4 * i + 1] = lo.y * sc; f[4 * i + 2] = hi.x * sc; f[4 * i + 3] = hi.y * sc;
        }
        Store8<YD>::put(y, ((row0 + r) * n8 + col8) * 8, f);
    }
}

template <int YD>
__global__ __launch_bounds__(256) void weight_dequant_scalar_kernel(
        const uint8_t* __restrict__ x, const float* __restrict__ s, typename OutT<YD>::type* __restrict__ y,
        int64_t row_base, int64_t n, int block, int64_t sn) {
    const int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t row = row_base + blockIdx.y;
    if (col >= n) return;
    const float sc = s[(row / block) * sn + col / block];
    const uint32_t b = x[row * n + col];
    y[row * n + col] = cvt_out<YD>(fp8x2_lo_to_f32(b).x * sc);
}

template <int YD>
int launch(const void* x, const float* s, void* y, int64_t m, int64_t n, int block, hipStream_t stream) {
    const int64_t sn = (n + block - 1) / block;
    const bool vec = block == 128 && n % 8 == 0 && n / 8 < (1ll << 30) &&
                     ((uintptr_t)x % 8 == 0) && ((uintptr_t)y % 16 == 0);
    if (vec) {
        const int n8 = (int)(n / 8);
        const int64_t gy = (m + kWavesY * kRows - 1) / (kWavesY * kRows);
        const int64_t gx = (n8 + kWave - 1) / kWave;
        if (gy > 65535) {
            // grid.y is limited to 16 bits: walk the rows in slabs of 65528 workgroups (a multiple of 128 rows,
            // so that every slab starts on a scale-block boundary)
            const int64_t slab_rows = 65528ll * kWavesY * kRows;
            for (int64_t r = 0; r < m; r += slab_rows) {
                const int64_t mr = (m - r < slab_rows) ? m - r : slab_rows;
                const int64_t g = (mr + kWavesY * kRows - 1) / (kWavesY * kRows);
                hipLaunchKernelGGL((weight_dequant_vec_kernel<YD>), dim3((unsigned)gx, (unsigned)g), dim3(kWave, kWavesY), 0, stream,
                                   (const v2u*)x + r * n8, s + (r / 128) * sn,
                                   (void*)((char*)y + r * n * OutT<YD>::bytes), mr, n8, (int)sn);
            }
        } else {
            hipLaunchKernelGGL((weight_dequant_vec_kernel<YD>), dim3((unsigned)gx, (unsigned)gy), dim3(kWave, kWavesY), 0, stream,
                               (const v2u*)x, s, y, m, n8, (int)sn);
        }
    } else {
        const int64_t gx = (n + 255) / 256;
        if (gx > 0x7fffffff) return DSV3_ERR_BAD_SHAPE;
        for (int64_t r = 0; r < m; r += 65535) {
            const int64_t mr = (m - r < 65535) ? m - r : 65535;   // grid.y is limited to 16 bits
            hipLaunchKernelGGL((weight_dequant_scalar_kernel<YD>), dim3((unsigned)gx, (unsigned)mr), dim3(256), 0, stream,
                               (const uint8_t*)x, s, (typename OutT<YD>::type*)y, r, n, block, sn);
        }
    }
    return launch_status();
}

}  // namespace

int launch_weight_dequant(const void* x, const float* s, void* y, int y_dtype,
                          int64_t m, int64_t n, int block_size, hipStream_t stream) {
    switch (y_dtype) {
        case DSV3_BF16: return launch<DSV3_BF16>(x, s, y, m, n, block_size, stream);
        case DSV3_F16:  return launch<DSV3_F16>(x, s, y, m, n, block_size, stream);
        case DSV3_F32:  return launch<DSV3_F32>(x, s, y, m, n, block_size, stream);
        default: return DSV3_ERR_BAD_DTYPE;
    }
}

}  // namespace dsv3
