// fp8_gemm for decode shapes with a wide enough N: producer / consumer weight-streaming kernel
// (reference arithmetic: inference/kernel.py:145-172).
//
// A workgroup is five or nine wavefronts.  Four or eight CONSUMERS each own a 16-row strip of b (64 or 128 rows per
// workgroup, inside one 128-row block of weight scales) and walk
// the workgroup's K range; their weights go straight from global memory into the MFMA register layout through a
// ring of NPF K blocks whose loads and waits are written out explicitly (inline asm), so that exactly NPF-1
// blocks stay in flight behind the one being multiplied.  The fifth wavefront is the PRODUCER: it copies the
// activations the consumers share (chunks of KC K blocks x 16*MT rows, plus their scales) into double-buffered
// LDS with global_load_lds_dwordx4.  Keeping the two streams in different wavefronts matters because vector
// loads retire in issue order per wavefront: an activation load in a consumer's queue would force its weight
// ring to drain at every chunk boundary.  One fence-free workgroup barrier per chunk hands a filled buffer to
// the consumers and an emptied one back to the producer.
#include "common.hpp"
#include <type_traits>

namespace dsv3 {
namespace stream {

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

constexpr int kMaxConsumers = 8;          // consumer wavefronts per workgroup: 4 or 8, chosen per launch (blockDim.x / 64 - 1)
constexpr int kThreads = (kMaxConsumers + 1) * kWave;

__device__ __forceinline__ int swz(int row) { return (row & 7) ^ ((row >> 3) & 1); }

__device__ __forceinline__ v8i join(v4i lo, v4i hi) {
    v8i r = { lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3] };
    return r;
}

// lo = what the lane loaded from rows 0..7 of the strip, hi = from rows 8..15 (each load instruction fetches
// 8 rows x 128 contiguous bytes: lanes with (lane&15) < 8 the first 64 bytes of a row, the others the last 64).
// The halves that belong to the lane 8 positions away are exchanged with DPP row rotates.
__device__ __forceinline__ v8i untangle(v4i a, v4i b) {
    v8i r;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        r[i]     = __builtin_amdgcn_update_dpp(a[i], b[i], 0x128, 0xf, 0xc, false);
        r[4 + i] = __builtin_amdgcn_update_dpp(b[i], a[i], 0x128, 0xf, 0x3, false);
    }
    return r;
}

// Workgroup barrier without the memory fence of __syncthreads() (that fence waits for every vector load in
// flight, i.e. for the whole weight ring).  LDS traffic of this wavefront is complete first.
__device__ __forceinline__ void wg_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// 16-byte non-temporal load from (scalar base + 32-bit lane offset + immediate): no 64-bit address VGPRs
#define DSV3_GLOAD(dst, voff, sbase, imm) \
    asm volatile("global_load_dwordx4 %0, %1, %2 offset:" #imm " nt" : "=v"(dst) : "v"(voff), "s"(sbase) : "memory")
// wait until at most n vector loads of this wavefront are outstanding; the ring slot is threaded through the
// statement so that its consumers cannot be scheduled ahead of the wait
#define DSV3_WAIT(n, lo, hi) asm volatile("s_waitcnt vmcnt(" #n ")" : "+v"(lo), "+v"(hi) :: "memory")

template <int N> struct WaitFor;   // vmcnt(N) with N a compile-time number of K blocks x 2 loads
#define DSV3_WAITFOR(N_) template <> struct WaitFor<N_> { static __device__ __forceinline__ void on(v4i& lo, v4i& hi) { DSV3_WAIT(N_, lo, hi); } };
DSV3_WAITFOR(0) DSV3_WAITFOR(2) DSV3_WAITFOR(4) DSV3_WAITFOR(6) DSV3_WAITFOR(8) DSV3_WAITFOR(10) DSV3_WAITFOR(12) DSV3_WAITFOR(14)
#undef DSV3_WAITFOR

// MT: 16-row activation sub-tiles (M <= 16*MT); NPF: ring depth in K blocks (divides the workgroup's K range);
// KC: K blocks per activation chunk (divides NPF or is a multiple of it -- only has to divide the K range).
template <int MT, int NPF, int KC>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(4, 4))) void fp8_gemm_stream_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        void* __restrict__ out, int out_dtype,      // F32 slabs [gridDim.y][M][N] when gridDim.y > 1, else c
        int M, int N, int K, int nkb) {             // nkb: K blocks per workgroup, a multiple of NPF and of KC
    constexpr int ROWS = 16 * MT;
    constexpr int CHUNK_BYTES = KC * ROWS * 128;
    constexpr int DMA = CHUNK_BYTES / 1024;                // 1 KiB global_load_lds instructions per chunk
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    float* lds_s = (float*)(lds + 2 * CHUNK_BYTES);        // [2][KC*ROWS]: a_s * b_s

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KB = K >> 7;
    const int kb0 = blockIdx.y * nkb;
    const int nchunks = nkb / KC;

    const int consumers = (int)(blockDim.x >> 6) - 1, group_rows = consumers * 16;
    if (wave == consumers) {
        // ------------------------------------------------------------------ producer
        const float* bs_src = b_s + (size_t)min((int)(blockIdx.x * group_rows) >> 7, (N - 1) >> 7) * KB + kb0;
        for (int c = 0; c < nchunks; ++c) {
            const int buf = c & 1;
#pragma unroll
            for (int i = 0; i < DMA; ++i) {
                const int R = i * 8 + (lane >> 3);                     // slab row = kbl*ROWS + m
                const int m = min(R % ROWS, M - 1), kb = c * KC + R / ROWS;
                const uint8_t* src = a + (size_t)m * K + (size_t)(kb0 + kb) * 128 + (((lane & 7) ^ swz(R)) * 16);
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + buf * CHUNK_BYTES + i * 1024), 16, 0, 0);
            }
            for (int idx = lane; idx < KC * ROWS; idx += kWave) {
                const int m = min(idx % ROWS, M - 1), kb = c * KC + idx / ROWS;
                lds_s[buf * (KC * ROWS) + idx] = a_s[(size_t)m * KB + kb0 + kb] * bs_src[kb];
            }
            __builtin_amdgcn_s_waitcnt(0x0f70);                        // vmcnt(0): the chunk has landed
            wg_barrier();                                              // barrier #c: chunk c is ready, chunk c-1 is consumed
        }
        return;
    }

    // ---------------------------------------------------------------------- consumers
    const int fr = lane & 15, fq = lane >> 4;
    const int n0 = blockIdx.x * group_rows + wave * 16;
    // lane offsets of its two rows (strip rows fr&7 and (fr&7)+8, clamped to the last row of b) from b, < 2^32
    const uint32_t off_lo = (uint32_t)min(n0 + (fr & 7), N - 1) * (uint32_t)K + (fr >> 3) * 64 + fq * 16;
    const uint32_t off_hi = (uint32_t)min(n0 + (fr & 7) + 8, N - 1) * (uint32_t)K + (fr >> 3) * 64 + fq * 16;
    const uint8_t* wbase = b + (size_t)kb0 * 128;          // wavefront-uniform: K block kb0 of row 0

    v4i wlo[NPF], whi[NPF];
#define DSV3_FETCH(P_, BASE_) if (P_ < NPF) { DSV3_GLOAD(wlo[P_ < NPF ? P_ : 0], off_lo, BASE_, P_ * 128); DSV3_GLOAD(whi[P_ < NPF ? P_ : 0], off_hi, BASE_, P_ * 128); }
    DSV3_FETCH(0, wbase) DSV3_FETCH(1, wbase) DSV3_FETCH(2, wbase) DSV3_FETCH(3, wbase)
    DSV3_FETCH(4, wbase) DSV3_FETCH(5, wbase) DSV3_FETCH(6, wbase) DSV3_FETCH(7, wbase)

    v4f acc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[j] = (v4f){0.f, 0.f, 0.f, 0.f};

    // one K block: wait for ring slot p (LEFT = blocks issued after it that may stay in flight), multiply
    auto step = [&](auto left_tag, int p_, v4i& lo, v4i& hi, int kbl) {
        (void)p_;
        constexpr int LEFT = decltype(left_tag)::value;
        WaitFor<2 * LEFT>::on(lo, hi);
        const v8i wf = untangle(lo, hi);
        const int c = kbl / KC, t = kbl % KC;
        const uint8_t* act = lds + (c & 1) * CHUNK_BYTES;
        const float* sc_base = lds_s + (c & 1) * (KC * ROWS);
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            const int R = t * ROWS + j * 16 + fr, fx = swz(R);
            const uint8_t* r = act + R * 128;
            const v8i af = join(*(const v4i*)(r + ((fq ^ fx) * 16)), *(const v4i*)(r + (((4 + fq) ^ fx) * 16)));
            const float sc = sc_base[R];
            const v4f z = {0.f, 0.f, 0.f, 0.f};
            const v4f p4 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, z, 0, 0, 0, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[j][e] = __builtin_fmaf(p4[e], sc, acc[j][e]);
        }
    };

    // Chunk barriers: barrier #c has to be passed before the first K block of chunk c is read, i.e. whenever
    // kbl % KC == 0 (the producer passes the same barriers, one per chunk).
    const int rounds = nkb / NPF;
    int kbl = 0;
    for (int r = 0; r + 1 < rounds; ++r) {              // steady state: every slot is refilled after use
        const uint8_t* nbase = wbase + (size_t)(r + 1) * NPF * 128;       // the K blocks one ring ahead
#define DSV3_STEADY(P_) if (P_ < NPF) { if (kbl % KC == 0) wg_barrier(); \
        step(std::integral_constant<int, NPF - 1>{}, P_, wlo[P_ < NPF ? P_ : 0], whi[P_ < NPF ? P_ : 0], kbl); ++kbl; DSV3_FETCH(P_, nbase) }
        DSV3_STEADY(0) DSV3_STEADY(1) DSV3_STEADY(2) DSV3_STEADY(3) DSV3_STEADY(4) DSV3_STEADY(5) DSV3_STEADY(6) DSV3_STEADY(7)
#undef DSV3_STEADY
    }
    {                                                   // last round: the ring drains
#define DSV3_DRAIN(P_) if (P_ < NPF) { if (kbl % KC == 0) wg_barrier(); \
        step(std::integral_constant<int, (NPF - 1 - P_ > 0 ? NPF - 1 - P_ : 0)>{}, P_, wlo[P_ < NPF ? P_ : 0], whi[P_ < NPF ? P_ : 0], kbl); ++kbl; }
        DSV3_DRAIN(0) DSV3_DRAIN(1) DSV3_DRAIN(2) DSV3_DRAIN(3) DSV3_DRAIN(4) DSV3_DRAIN(5) DSV3_DRAIN(6) DSV3_DRAIN(7)
#undef DSV3_DRAIN
#undef DSV3_FETCH
    }

    // ---- store: lane holds c[m = 16j + fr][n0 + 4*fq .. +3]
    const size_t slab = (size_t)blockIdx.y * M * N;
#pragma unroll
    for (int j = 0; j < MT; ++j) {
        const int m = j * 16 + fr, n = n0 + fq * 4;
        if (m >= M) continue;
        const size_t idx = slab + (size_t)m * N + n;
        if (out_dtype == DSV3_F32 && (N & 3) == 0 && n + 3 < N) {        // split-K slabs: one 16-byte store
            *(v4f*)((float*)out + idx) = acc[j];
            continue;
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (n + e >= N) break;
            if (out_dtype == DSV3_F32)       ((float*)out)[idx + e] = acc[j][e];
            else if (out_dtype == DSV3_BF16) ((uint16_t*)out)[idx + e] = cvt_out<DSV3_BF16>(acc[j][e]);
            else                             ((uint16_t*)out)[idx + e] = cvt_out<DSV3_F16>(acc[j][e]);
        }
    }
}

struct Plan { bool ok; int mt, npf, splits, nkb, consumers; };

// Usable when N gives enough groups of 64 (128) rows and the K range splits evenly into ring-sized pieces.
inline Plan make_plan(int64_t m, int64_t n, int64_t k) {
    Plan p{};
    p.ok = false;
    // (M <= 16 and short K ranges are served better by the kernels that split K inside the workgroup)
    if (m <= 16 || m > 64 || k < 1024 || k % 128 || n * k >= (1ll << 32)) return p;
    p.mt = (int)((m + 15) / 16);
    if (p.mt == 3) p.mt = 4;                                    // 3 sub-tiles run as 4 (chunk size stays a power of two)
    // eight consumer wavefronts share an activation chunk where N gives enough groups of 128 rows (half the
    // activation traffic per weight byte: wq_b 1536 -> 24576 at 64 rows 18.0 -> 16.9 us, wq_a 15.1 -> 14.3), four
    // otherwise (wkv_a 7168 -> 576: 11.0 against 12.5 us)
    p.consumers = n >= 1024 ? 8 : 4;
    const int64_t kb = k / 128, groups = (n + 16 * p.consumers - 1) / (16 * p.consumers);
    if (groups < 4) return p;                                   // a handful of rows: not worth a streaming plan
    const int64_t capacity = 256 * (p.consumers == 4 ? 3 : 1);     // resident workgroups (3 per CU with five wavefronts, 1 with nine)
    // K blocks per workgroup: a divisor of kb that is a multiple of the ring depth; take the split count that
    // fills one round best
    int best_nkb = 0, best_npf = 0;
    int64_t best_wgs = 0;
    for (int npf : {8, 4}) {
        if (npf == 8 && p.mt > 1) continue;                     // the deeper ring only fits the register budget with one sub-tile
        for (int64_t nkb = npf; nkb <= kb; nkb += npf) {
            if (kb % nkb) continue;
            const int64_t wgs = groups * (kb / nkb);
            if (wgs > capacity && (kb / nkb) > 1) continue;
            if (wgs > best_wgs) { best_wgs = wgs; best_nkb = (int)nkb; best_npf = npf; }
        }
        if (best_nkb) break;
    }
    if (!best_nkb) return p;
    p.ok = true;
    p.npf = best_npf;
    p.nkb = best_nkb;
    p.splits = (int)(kb / best_nkb);
    return p;
}

template <int MT, int NPF>
void launch_cfg(const Plan& p, const void* a, const float* a_s, const void* b, const float* b_s,
                void* out, int od, int m, int n, int k, hipStream_t st) {
    constexpr int KC = MT == 1 ? (NPF < 8 ? NPF : 8) : (MT == 2 ? 4 : 2);
    const size_t lds = 2 * (size_t)KC * 16 * MT * (128 + 4);
    const int group_rows = 16 * p.consumers;
    const dim3 grid((unsigned)((n + group_rows - 1) / group_rows), (unsigned)p.splits);
    hipLaunchKernelGGL((fp8_gemm_stream_kernel<MT, NPF, KC>), grid, dim3((p.consumers + 1) * kWave), lds, st,
                       (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, out, od, m, n, k, p.nkb);
}

}  // namespace stream

bool stream_supported(int64_t m, int64_t n, int64_t k) { return stream::make_plan(m, n, k).ok; }

size_t stream_workspace_bytes(int64_t m, int64_t n, int64_t k) {
    const stream::Plan p = stream::make_plan(m, n, k);
    return (p.ok && p.splits > 1) ? (size_t)p.splits * (size_t)m * (size_t)n * sizeof(float) : 0;
}

int launch_stream(const void* a, const float* a_s, const void* b, const float* b_s, void* c, int c_dtype,
                  int64_t m, int64_t n, int64_t k, void* ws, int* splits_out, hipStream_t st) {
    using namespace stream;
    const Plan p = make_plan(m, n, k);
    if (!p.ok) return DSV3_ERR_BAD_SHAPE;
    void* out = p.splits > 1 ? ws : c;
    const int od = p.splits > 1 ? (int)DSV3_F32 : c_dtype;
    *splits_out = p.splits;
#define DSV3_CASE(MT_, NPF_) launch_cfg<MT_, NPF_>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st); break
    switch (p.mt * 10 + p.npf) {
        case 24: DSV3_CASE(2, 4);
        case 44: DSV3_CASE(4, 4);
        default: return DSV3_ERR_BAD_SHAPE;
    }
#undef DSV3_CASE
    return launch_status();
}

}  // namespace dsv3
