// fp8_gemm for decode shapes with a wide enough N: producer / consumer weight-streaming kernel
// (reference arithmetic: inference/kernel.py:145-172).
//
// A workgroup is up to nine wavefronts.  Up to eight CONSUMERS each own a 16-row strip of b (a strip lies inside one
// 128-row block of weight scales; a workgroup's strips may lie in two) and walk
// the workgroup's K range; their weights go straight from global memory into the MFMA register layout through a
// ring of NPF K blocks whose loads and waits are written out explicitly (inline asm), so that exactly NPF-1
// blocks stay in flight behind the one being multiplied.  One more wavefront is the PRODUCER: it copies the
// activations the consumers share (chunks of KC K blocks x 16*MT rows, plus their scales and the weight scales of
// those K blocks) into a ring of LDS buffers with global_load_lds, AHEAD chunks ahead of the one the consumers
// read, so that a chunk's trip from L2 is hidden behind the chunks before it (with one chunk in flight at a time
// the chunks' round trips added up to half of the kernel).  Keeping the two streams in different wavefronts matters
// because vector loads retire in issue order per wavefront: an activation load in a consumer's queue would force
// its weight ring to drain at every chunk boundary.  One fence-free workgroup barrier per chunk hands a filled
// buffer to the consumers and tells the producer that the chunk before it has been read.
#include <cstdio>
#include <cstdlib>
#include "common.hpp"
#include <type_traits>

namespace dsv3 {
namespace stream {

typedef const __attribute__((address_space(1))) void* gptr_t;
typedef __attribute__((address_space(3))) void* lptr_t;

constexpr int kMaxConsumers = 8;          // consumer wavefronts per workgroup: 2 .. 8, chosen per launch (blockDim.x / 64 - 1)
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
// KC: K blocks per activation chunk (divides NPF or is a multiple of it -- only has to divide the K range);
// AHEAD: chunks requested ahead of the one being waited for; NBUF >= AHEAD + 2 LDS buffers (when the producer
// requests chunk c + AHEAD it has passed barrier c - 1, so the consumers are done with chunk c - 2 and older).
template <int KC, int ROWS> struct ChunkCfg {
    static constexpr int BYTES = KC * ROWS * 128;
    static constexpr int DMA = BYTES / 1024;               // 1 KiB global_load_lds instructions per chunk
    static constexpr int SC_DMA = (KC * ROWS + 63) / 64;   // 4-byte copies of the activation scales
    static constexpr int PER = DMA + SC_DMA + 1;           // ... plus one for the weight scales
};
constexpr size_t lds_bytes(int kc, int rows, int nbuf) { return (size_t)nbuf * ((size_t)kc * rows * (128 + 4) + 64 * 4); }

template <int N> struct ProducerWait;   // vmcnt(N)
#define DSV3_PWAIT(N_) template <> struct ProducerWait<N_> { static __device__ __forceinline__ void on() { asm volatile("s_waitcnt vmcnt(" #N_ ")" ::: "memory"); } };
DSV3_PWAIT(0) DSV3_PWAIT(10) DSV3_PWAIT(19) DSV3_PWAIT(20) DSV3_PWAIT(30) DSV3_PWAIT(38) DSV3_PWAIT(57)
#undef DSV3_PWAIT

// WPE: wavefronts per SIMD the register budget is sized for (4: three workgroups of five wavefronts per compute unit,
// 128 VGPRs; 3: one workgroup of nine, 168 VGPRs: room to read a K block's activation fragments before the wait for
// its weights)
template <int MT, int NPF, int KC, int AHEAD, int NBUF, int WPE = (NBUF >= 5 ? 3 : 4)>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(WPE, WPE))) void fp8_gemm_stream_kernel(
        const uint8_t* __restrict__ a, const float* __restrict__ a_s,
        const uint8_t* __restrict__ b, const float* __restrict__ b_s,
        void* __restrict__ out, int out_dtype,      // F32 slabs [gridDim.y][M][N] when gridDim.y > 1, else c
        int M, int N, int K, int nkb) {             // nkb: K blocks per workgroup, a multiple of NPF and of KC
    constexpr int ROWS = 16 * MT;
    using CC = ChunkCfg<KC, ROWS>;
    constexpr int CHUNK_BYTES = CC::BYTES, DMA = CC::DMA, SC_DMA = CC::SC_DMA, PER = CC::PER;
    static_assert(NBUF >= AHEAD + 2 && AHEAD <= 3 && (PER == 19 || PER == 10), "ring of chunk buffers; the producer's counted waits");
    static_assert((KC * ROWS) % 64 == 0, "whole wavefront copies of the activation scales");
    extern __shared__ __attribute__((aligned(1024))) uint8_t lds[];
    float* lds_as = (float*)(lds + NBUF * CHUNK_BYTES);    // [NBUF][KC*ROWS]: a_s of the chunk's rows and K blocks
    float* lds_bs = lds_as + NBUF * (KC * ROWS);           // [NBUF][2][32]: b_s of the chunk's K blocks for the first and the
                                                           // second 128-row block the workgroup's strips lie in (KC entries each)

    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int KB = K >> 7;
    const int kb0 = blockIdx.y * nkb;
    const int nchunks = nkb / KC;

    const int consumers = (int)(blockDim.x >> 6) - 1, group_rows = consumers * 16;
    // When the rows of b lie a multiple of 16 KiB apart (16384 -> 7168), workgroups that sit at the same K offset at the
    // same time all ask the same few memory channels: a 117 MB weight took 29 us where neighbouring K took 21-23 us for
    // the same bytes.  There the workgroups do not all walk their K range from its first block: each starts
    // UNIT-sized steps further in, by its index, and wraps around (22 us).  UNIT is a whole number of ring rounds and
    // of activation chunks.  Other K keep the common order: their workgroups then share the activation chunks in L2
    // (7168 -> 1536 at 64 rows: 9.4 against 10.2 us).
    constexpr int UNIT = (NPF % KC == 0) ? NPF : (KC % NPF == 0 ? KC : NPF * KC / 2);
    const int units = nkb / UNIT;
    const int rot = (K & 16383) ? 0 : (int)((blockIdx.x + 3u * blockIdx.y) % (unsigned)units) * UNIT;
    auto k_of = [&](int kbl) { const int t = kbl + rot; return t >= nkb ? t - nkb : t; };    // kbl a multiple of KC or NPF
    if (wave == consumers) {
        // ------------------------------------------------------------------ producer
        // Everything goes global -> LDS without passing through registers: an ordinary load issued behind
        // direct-to-LDS loads would hold the wavefront until those have landed.
        const int nb_lo = min((int)(blockIdx.x * group_rows) >> 7, (N - 1) >> 7);
        const int nb_hi = min((int)(blockIdx.x * group_rows + group_rows - 1) >> 7, (N - 1) >> 7);     // nb_lo or nb_lo + 1
        const float* bs_src = b_s + (size_t)(lane < 32 ? nb_lo : nb_hi) * KB + kb0;
        auto request = [&](int c) {
            const int buf = c % NBUF, kfirst = k_of(c * KC);           // the chunk's first K block
#pragma unroll
            for (int i = 0; i < DMA; ++i) {
                const int R = i * 8 + (lane >> 3);                     // slab row = kbl*ROWS + m
                const int m = min(R % ROWS, M - 1), kb = kfirst + R / ROWS;
                const uint8_t* src = a + (size_t)m * K + (size_t)(kb0 + kb) * 128 + (((lane & 7) ^ swz(R)) * 16);
                __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(lds + buf * CHUNK_BYTES + i * 1024), 16, 0, 0);
            }
#pragma unroll
            for (int i = 0; i < SC_DMA; ++i) {
                const int idx = i * 64 + lane;
                const int m = min(idx % ROWS, M - 1), kb = kfirst + idx / ROWS;
                __builtin_amdgcn_global_load_lds((gptr_t)(a_s + (size_t)m * KB + kb0 + kb),
                                                 (lptr_t)(lds_as + buf * (KC * ROWS) + i * 64), 4, 0, 0);
            }
            __builtin_amdgcn_global_load_lds((gptr_t)(bs_src + kfirst + min(lane & 31, KC - 1)), (lptr_t)(lds_bs + buf * 64), 4, 0, 0);
        };
        for (int c = 0; c < AHEAD && c < nchunks; ++c) request(c);
        for (int c = 0; c < nchunks; ++c) {
            if (c + AHEAD < nchunks) request(c + AHEAD);
            // chunk c has landed when at most the chunks requested after it are outstanding
            const int later = min(AHEAD, nchunks - 1 - c);
            if (AHEAD >= 3 && later == 3) ProducerWait<3 * PER>::on();
            else if (AHEAD >= 2 && later == 2) ProducerWait<2 * PER>::on();
            else if (AHEAD >= 1 && later == 1) ProducerWait<PER>::on();
            else ProducerWait<0>::on();
            wg_barrier();                                              // barrier #c: chunk c is ready, chunk c-1 has been read
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
    // which of the workgroup's two weight-scale rows this strip belongs to (0 or 32: offset into a buffer's b_s)
    const int bs_sel = (min(n0, N - 1) >> 7) != (min((int)(blockIdx.x * group_rows), N - 1) >> 7) ? 32 : 0;

    v4i wlo[NPF], whi[NPF];
#define DSV3_FETCH(P_, BASE_) if (P_ < NPF) { DSV3_GLOAD(wlo[P_ < NPF ? P_ : 0], off_lo, BASE_, P_ * 128); DSV3_GLOAD(whi[P_ < NPF ? P_ : 0], off_hi, BASE_, P_ * 128); }
    const uint8_t* wfirst = wbase + (size_t)k_of(0) * 128;
    DSV3_FETCH(0, wfirst) DSV3_FETCH(1, wfirst) DSV3_FETCH(2, wfirst) DSV3_FETCH(3, wfirst)
    DSV3_FETCH(4, wfirst) DSV3_FETCH(5, wfirst) DSV3_FETCH(6, wfirst) DSV3_FETCH(7, wfirst)

    v4f acc[MT];
#pragma unroll
    for (int j = 0; j < MT; ++j) acc[j] = (v4f){0.f, 0.f, 0.f, 0.f};

    // one K block: wait for ring slot p (LEFT = blocks issued after it that may stay in flight), multiply
    auto step = [&](auto left_tag, int p_, v4i& lo, v4i& hi, int kbl) {
        (void)p_;
        constexpr int LEFT = decltype(left_tag)::value;
        // With registers to spare (WPE == 3) the block's activation fragments and scales are read from LDS before the
        // wait for its weights, so the LDS latency of MT dependent read -> MFMA pairs is not paid behind that wait.
        constexpr bool EARLY = WPE == 3;
        const int c = kbl / KC, t = kbl % KC, buf = c % NBUF;
        const uint8_t* act = lds + buf * CHUNK_BYTES;
        const float* sc_base = lds_as + buf * (KC * ROWS);
        auto fragment = [&](int j) {
            const int R = t * ROWS + j * 16 + fr, fx = swz(R);
            const uint8_t* r = act + R * 128;
            return join(*(const v4i*)(r + ((fq ^ fx) * 16)), *(const v4i*)(r + (((4 + fq) ^ fx) * 16)));
        };
        v8i af[MT];
        float sc[MT];
        const float bs = lds_bs[buf * 64 + bs_sel + t];
        if (EARLY) {
#pragma unroll
            for (int j = 0; j < MT; ++j) { af[j] = fragment(j); sc[j] = sc_base[t * ROWS + j * 16 + fr] * bs; }
        }
        WaitFor<2 * LEFT>::on(lo, hi);
        const v8i wf = untangle(lo, hi);
#pragma unroll
        for (int j = 0; j < MT; ++j) {
            if (!EARLY) { af[j] = fragment(j); sc[j] = sc_base[t * ROWS + j * 16 + fr] * bs; }
            const v4f z = {0.f, 0.f, 0.f, 0.f};
            const v4f p4 = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af[j], z, 0, 0, 0, 0, 0, 0);
#pragma unroll
            for (int e = 0; e < 4; ++e) acc[j][e] = __builtin_fmaf(p4[e], sc[j], acc[j][e]);
        }
    };

    // Chunk barriers: barrier #c has to be passed before the first K block of chunk c is read, i.e. whenever
    // kbl % KC == 0 (the producer passes the same barriers, one per chunk).
    const int rounds = nkb / NPF;
    int kbl = 0;
    for (int r = 0; r + 1 < rounds; ++r) {              // steady state: every slot is refilled after use
        const uint8_t* nbase = wbase + (size_t)k_of((r + 1) * NPF) * 128;  // the K blocks one ring ahead
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
        if ((N & 3) == 0 && n + 3 < N) {                                 // four results per store
            if (out_dtype == DSV3_F32)       *(v4f*)((float*)out + idx) = acc[j];
            else if (out_dtype == DSV3_BF16) *(v2u*)((uint16_t*)out + idx) = v2u{ pack_bf16(acc[j][0], acc[j][1]), pack_bf16(acc[j][2], acc[j][3]) };
            else                             *(v2u*)((uint16_t*)out + idx) = v2u{ pack_f16(acc[j][0], acc[j][1]), pack_f16(acc[j][2], acc[j][3]) };
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

struct Plan { bool ok; int mt, npf, splits, nkb, consumers, per_cu; };

// DSV3_STREAM_PLAN="consumers,nkb,npf,per_cu" pins the plan (tuning aid; the values must fit the problem).
inline bool forced_plan(int& consumers, int& nkb, int& npf, int& per_cu) {
    const char* e = std::getenv("DSV3_STREAM_PLAN");         // (read at every call: a sweep changes it between launches)
    return e && std::sscanf(e, "%d,%d,%d,%d", &consumers, &nkb, &npf, &per_cu) == 4;
}

// Usable when N gives enough strips and the K range splits evenly into ring-sized pieces.
// mt_min: smallest number of 16-row sub-tiles to plan for (a launch of up to 16 rows may run as two sub-tiles when the
// K range does not divide into the one-sub-tile configuration's chunks).
//
// The plan is the number of consumers per workgroup (16 weight rows each), the K blocks per workgroup, the ring depth
// and how many workgroups a compute unit holds at a time (one of up to nine wavefronts at 168 registers, two of up to
// eight at 128, three of up to five).  Candidates are priced with a model fitted to sweeps over the projections of
// the 671B configuration (1 .. 64 rows): a launch takes as long as its busiest compute unit needs for its weight
// bytes, at a rate that grows with the bytes its resident consumers keep in flight, plus its activation chunks from
// L2, plus per-round start-up and chunk barriers, plus, with K slices, a slab of partial sums each and the launch that
// adds them.
inline Plan make_plan_mt(int64_t m, int64_t n, int64_t k, int mt_min) {
    Plan p{};
    p.ok = false;
    int fc = 0, fnkb = 0, fnpf = 0, fpc = 0;
    const bool forced = forced_plan(fc, fnkb, fnpf, fpc);
    if (m < 1 || m > 64 || k < 512 || k % 128 || n * k >= (1ll << 32)) return p;
    p.mt = (int)((m + 15) / 16);
    if (p.mt < mt_min) p.mt = mt_min;
    if (p.mt == 3) p.mt = 4;                                    // 3 sub-tiles run as 4 (chunk size stays a power of two)
    const int64_t kb = k / 128, strips = (n + 15) / 16;
    const bool long_stream = n * k / 256 >= (256 << 10);        // a quarter of a megabyte and more per compute unit
    double best = 1e30;
    for (int c = 8; c >= 2; --c)
    for (int64_t per_cu : {1, 2, 3}) {
        const int64_t groups = (strips + c - 1) / c;
        if ((per_cu == 3) != (c <= 4) || (per_cu == 2 && (c > 7 || p.mt > 2))) continue;
        if (!forced && groups < 4) continue;                    // a handful of weight rows is not worth a streaming plan
        for (int npf : {8, 6, 4}) {
            // what fits the register budgets without spilling: one sub-tile any ring, two sub-tiles six blocks (eight
            // with 168 registers), four sub-tiles four blocks
            if ((p.mt == 4 && npf > 4) || (p.mt == 2 && npf == 8 && per_cu > 1)) continue;
            const int kc = p.mt == 1 ? (npf == 8 ? 8 : 4) : (p.mt == 2 ? 4 : 2);     // K blocks per activation chunk
            for (int64_t nkb = npf; nkb <= kb; nkb += npf) {
                if (kb % nkb || nkb % kc) continue;
                if (forced && (c != fc || nkb != fnkb || npf != fnpf || per_cu != fpc)) continue;
                const int64_t slices = kb / nkb, wgs = groups * slices;
                if (wgs > 256 * per_cu && slices > 1) continue;           // one resident round when partial sums are in play
                if (!forced && (slices > 16 || wgs < 64)) continue;       // (outside what the model below was fitted on)
                // (us; KB / us.  The constants come from a least-regret fit over every valid plan of thirteen weight
                // shapes at 1, 8, 32 and 64 rows, timed on the device: the model's pick is within 3 % of the best
                // measured plan on 45 of the 52 cells and within 9 % on all.)
                const double wg_kb = c * 16.0 * nkb * 0.128;               // KB of weights per workgroup
                const int64_t busiest = (wgs + 255) / 256;                 // workgroups on the busiest compute unit
                const int64_t rounds = (busiest + per_cu - 1) / per_cu;    // ... one after the other
                const double in_flight = (double)(busiest < per_cu ? busiest : per_cu) * c * (npf < nkb ? npf : nkb) * 2.0;
                const double rate = long_stream ? 52.6 * in_flight / (in_flight + 19.8)
                                                : 124.7 * in_flight / (in_flight + 2.5);
                double us = busiest * wg_kb / rate;                        // the weight stream
                us += busiest * (16.0 * p.mt) * nkb * 0.128 / 82.0;        // its activation chunks, from L2
                us += 2.63 * (p.mt - 1) * busiest * nkb / 56.0;            // more sub-tiles per K block and consumer
                if (slices > 1) us += 0.8 + 2.0 * slices * m * n * 4e-6 / 2.66;   // reduce launch, slabs written and read
                us += rounds * (0.15 + 0.186 * (nkb / kc) * c / 8.0);      // start-up, and a barrier of c + 1 wavefronts per chunk
                us += per_cu == 1 ? 0.10 : per_cu == 2 ? 0.40 : 0.0;
                if (us < best) { best = us; p.ok = true; p.consumers = c; p.nkb = (int)nkb; p.npf = npf; p.splits = (int)slices; p.per_cu = (int)per_cu; }
            }
        }
    }
    // One and two rows: the kernel that splits K inside the workgroup is equal or better (and quantises the activations
    // itself for linear()) except where this one needs no K slices or the weight has few strips (7168 -> 576: 36)
    if (p.ok && !forced && m <= 2 && p.splits > 1 && strips >= 64) p.ok = false;
    return p;
}

inline Plan make_plan(int64_t m, int64_t n, int64_t k) {
    Plan p = make_plan_mt(m, n, k, 1);
    // 9 .. 16 rows on a K range without one-sub-tile chunks: two sub-tiles, the second one padding
    if (!p.ok && m >= 9 && m <= 16) p = make_plan_mt(m, n, k, 2);
    return p;
}

template <int MT, int NPF>
int launch_cfg(const Plan& p, const void* a, const float* a_s, const void* b, const float* b_s,
                void* out, int od, int m, int n, int k, hipStream_t st) {
    constexpr int KC = MT == 1 ? (NPF == 8 ? 8 : 4) : (MT == 2 ? 4 : 2);
    const int group_rows = 16 * p.consumers;
    const dim3 grid((unsigned)((n + group_rows - 1) / group_rows), (unsigned)p.splits);
    if (p.per_cu == 2) {
        // two workgroups of up to eight wavefronts per compute unit: four buffers (68 KiB), two chunks ahead
        if constexpr (MT <= 2 && !(MT == 2 && NPF == 8)) {
            auto kern = fp8_gemm_stream_kernel<MT, NPF, KC, 2, 4, 4>;
            constexpr size_t lds = lds_bytes(KC, 16 * MT, 4);
            static LdsGrant grant;
            if (!grant.ensure((const void*)kern, (int)lds)) return DSV3_ERR_LAUNCH;
            hipLaunchKernelGGL(kern, grid, dim3((p.consumers + 1) * kWave), lds, st, (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, out, od, m, n, k, p.nkb);
        } else return DSV3_ERR_BAD_SHAPE;
    } else if (p.per_cu == 1) {
        // one workgroup per compute unit (six to nine wavefronts): five buffers, three chunks ahead
        auto kern = fp8_gemm_stream_kernel<MT, NPF, KC, 3, 5>;
        constexpr size_t lds = lds_bytes(KC, 16 * MT, 5);
        static LdsGrant grant;
        if (!grant.ensure((const void*)kern, (int)lds)) return DSV3_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, dim3((p.consumers + 1) * kWave), lds, st, (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, out, od, m, n, k, p.nkb);
    } else if constexpr (!(MT == 2 && NPF == 8)) {
        // three workgroups of up to five wavefronts per compute unit: three buffers (51 KiB), one chunk ahead
        auto kern = fp8_gemm_stream_kernel<MT, NPF, KC, 1, 3>;
        constexpr size_t lds = lds_bytes(KC, 16 * MT, 3);
        static LdsGrant grant;
        if (!grant.ensure((const void*)kern, (int)lds)) return DSV3_ERR_LAUNCH;
        hipLaunchKernelGGL(kern, grid, dim3((p.consumers + 1) * kWave), lds, st, (const uint8_t*)a, a_s, (const uint8_t*)b, b_s, out, od, m, n, k, p.nkb);
    }
    return launch_status();
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
    switch (p.mt * 10 + p.npf) {
        case 18: return launch_cfg<1, 8>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        case 14: return launch_cfg<1, 4>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        case 16: return launch_cfg<1, 6>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        case 24: return launch_cfg<2, 4>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        case 26: return launch_cfg<2, 6>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        case 28: return launch_cfg<2, 8>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        case 44: return launch_cfg<4, 4>(p, a, a_s, b, b_s, out, od, (int)m, (int)n, (int)k, st);
        default: return DSV3_ERR_BAD_SHAPE;
    }
}

}  // namespace dsv3
