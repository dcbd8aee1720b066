// Expert selection of the router, after its linear layer (reference: inference/model.py:577-598):
//     s      = sigmoid(logits)            (bf16, like the reference's tensor)   | softmax(logits) in binary32
//     sel    = s + bias                   (binary32; bias optional)
//     groups : score of a group = sum of its two largest sel (with bias) or its largest (without);
//              the topk_groups best groups stay, the others are masked to -inf
//     idx    = the topk largest sel, in descending order
//     w      = s[idx];  sigmoid: w = bf16(w / bf16(sum w));  w = bf16(w * route_scale)
// One wavefront per token, four tokens per workgroup.  Expert e sits in lane e % 64, slot e / 64.  The reference
// runs this as about fifteen small tensor operations per call (250 us at 4096 tokens, 70 us at one); here it is
// one launch.  Ties go to the lower index (torch.topk leaves them unspecified).
#include "common.hpp"
#include <math.h>

namespace dsv3 {
namespace {

// Wavefront-wide reductions that leave the result in every lane: four DPP steps inside each row of 16 lanes, then
// the four row results are read into scalar registers and combined -- no LDS traffic (a cross-row shuffle is an LDS
// permute of ~100 cycles, and the selection below is a chain of two dozen such reductions).
template <int CTRL> __device__ __forceinline__ int dpp_mov(int v) {
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, true);
}
template <class Op> __device__ __forceinline__ int wave_reduce(int v, Op op) {
    v = op(v, dpp_mov<0xB1>(v));      // quad_perm [1,0,3,2]
    v = op(v, dpp_mov<0x4E>(v));      // quad_perm [2,3,0,1]
    v = op(v, dpp_mov<0x141>(v));     // row_half_mirror
    v = op(v, dpp_mov<0x140>(v));     // row_mirror: every lane of a row holds the row's result
    const int r0 = __builtin_amdgcn_readlane(v, 0), r1 = __builtin_amdgcn_readlane(v, 16);
    const int r2 = __builtin_amdgcn_readlane(v, 32), r3 = __builtin_amdgcn_readlane(v, 48);
    return op(op(r0, r1), op(r2, r3));
}
__device__ __forceinline__ float wave_max(float x) {
    return __builtin_bit_cast(float, wave_reduce(__builtin_bit_cast(int, x), [](int a, int b) {
        return __builtin_bit_cast(int, fmaxf(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b))); }));
}
__device__ __forceinline__ float wave_sum(float x) {
    return __builtin_bit_cast(float, wave_reduce(__builtin_bit_cast(int, x), [](int a, int b) {
        return __builtin_bit_cast(int, __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b)); }));
}
__device__ __forceinline__ int wave_min(int x) { return wave_reduce(x, [](int a, int b) { return a < b ? a : b; }); }

struct Best { float v; int i; };
// largest value over the wavefront, lowest index among equals; every lane gets the result
__device__ __forceinline__ Best wave_argmax(Best x) {
    Best r;
    r.v = wave_max(x.v);
    r.i = wave_min(x.v == r.v ? x.i : 0x7fffffff);
    return r;
}
__device__ __forceinline__ Best better(Best a, Best b) {
    return (b.v > a.v || (b.v == a.v && b.i < a.i)) ? b : a;
}

constexpr int kTokensPerWg = 4;

template <int EPL>   // expert slots per lane: experts <= 64 * EPL
__global__ __launch_bounds__(64 * kTokensPerWg) void gate_route_kernel(
        const uint16_t* __restrict__ logits, const float* __restrict__ bias, uint16_t* __restrict__ w_out,
        int64_t* __restrict__ idx_out, int tokens, int experts, int topk, int n_groups, int topk_groups,
        int sigmoid, float route_scale) {
    __shared__ float sh[kTokensPerWg][EPL * 64];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int token = blockIdx.x * kTokensPerWg + wave;
    if (token >= tokens) return;                  // no workgroup barrier below
    const float ninf = -INFINITY;

    float orig[EPL], sel[EPL];
#pragma unroll
    for (int s = 0; s < EPL; ++s) {
        const int e = s * 64 + lane;
        orig[s] = e < experts ? bf16lo_to_f32(logits[(int64_t)token * experts + e]) : ninf;
    }
    if (sigmoid) {
#pragma unroll
        for (int s = 0; s < EPL; ++s) orig[s] = round_bf16(1.f / (1.f + expf(-orig[s])));     // padding: sigmoid(-inf) = 0
    } else {
        float m = ninf;
#pragma unroll
        for (int s = 0; s < EPL; ++s) m = fmaxf(m, orig[s]);
        m = wave_max(m);
        float sum = 0.f;
#pragma unroll
        for (int s = 0; s < EPL; ++s) { orig[s] = expf(orig[s] - m); sum += orig[s]; }        // padding: exp(-inf) = 0
        sum = wave_sum(sum);
#pragma unroll
        for (int s = 0; s < EPL; ++s) orig[s] = orig[s] / sum;
    }
#pragma unroll
    for (int s = 0; s < EPL; ++s) {
        const int e = s * 64 + lane;
        sel[s] = e < experts ? (bias ? orig[s] + bias[e] : orig[s]) : ninf;
    }

    if (n_groups > 1) {
        float* mine = sh[wave];
        const int gsz = experts / n_groups;
        Best gs = { ninf, lane };
        if (gsz == 32) {
            // a group is one half of a wavefront in one slot (the 671B router: 256 experts in 8 groups): its two
            // largest values by merging (top1, top2) pairs of disjoint lane sets -- four DPP steps inside each row
            // of 16 lanes, then the two rows of a half through scalar lane reads; every lane stays busy
#pragma unroll
            for (int s = 0; s < EPL; ++s) {
                float t1 = sel[s], t2 = ninf;
                auto merge = [&](float o1, float o2) {
                    const float lo = fminf(t1, o1);
                    t1 = fmaxf(t1, o1);
                    t2 = fmaxf(lo, fmaxf(t2, o2));
                };
                auto f = [](float x) { return __builtin_bit_cast(int, x); };
                auto g = [](int x) { return __builtin_bit_cast(float, x); };
                { const float o1 = g(dpp_mov<0xB1>(f(t1))), o2 = g(dpp_mov<0xB1>(f(t2))); merge(o1, o2); }
                { const float o1 = g(dpp_mov<0x4E>(f(t1))), o2 = g(dpp_mov<0x4E>(f(t2))); merge(o1, o2); }
                { const float o1 = g(dpp_mov<0x141>(f(t1))), o2 = g(dpp_mov<0x141>(f(t2))); merge(o1, o2); }
                { const float o1 = g(dpp_mov<0x140>(f(t1))), o2 = g(dpp_mov<0x140>(f(t2))); merge(o1, o2); }
#pragma unroll
                for (int h = 0; h < 2; ++h) {                      // group 2 s + h: rows 2 h and 2 h + 1
                    const float a1 = g(__builtin_amdgcn_readlane(f(t1), 32 * h)), a2 = g(__builtin_amdgcn_readlane(f(t2), 32 * h));
                    const float b1 = g(__builtin_amdgcn_readlane(f(t1), 32 * h + 16)), b2 = g(__builtin_amdgcn_readlane(f(t2), 32 * h + 16));
                    const float top1 = fmaxf(a1, b1), top2 = fmaxf(fminf(a1, b1), fmaxf(a2, b2));
                    if (lane == 2 * s + h && 2 * s + h < n_groups) gs.v = bias ? top1 + top2 : top1;
                }
            }
        } else {
            // any other group size: through LDS, lane g walks group g
#pragma unroll
            for (int s = 0; s < EPL; ++s) mine[s * 64 + lane] = sel[s];
            // lanes below read what other lanes of the wavefront have just written: order the LDS stores before the
            // loads for the compiler too (the hardware retires a wavefront's LDS operations in order)
            __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
            __builtin_amdgcn_wave_barrier();
            __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
            if (lane < n_groups) {
                float top1 = ninf, top2 = ninf;
                for (int j = 0; j < gsz; ++j) {
                    const float v = mine[lane * gsz + j];
                    if (v > top1) { top2 = top1; top1 = v; }
                    else if (v > top2) top2 = v;
                }
                gs.v = bias ? top1 + top2 : top1;
            }
        }
        uint64_t keep = 0;
        for (int t = 0; t < topk_groups; ++t) {
            const Best b = wave_argmax(gs);
            keep |= 1ull << b.i;
            if (lane == b.i) gs.v = ninf;
            // a group that was already taken can only win again when nothing finite is left; its bit is set
        }
#pragma unroll
        for (int s = 0; s < EPL; ++s) {
            const int e = s * 64 + lane;
            if (e < experts && !((keep >> (e / gsz)) & 1)) sel[s] = ninf;
        }
    }

    float my_w = 0.f;                              // lane t keeps the weight of the t-th selected expert
    for (int t = 0; t < topk; ++t) {
        Best loc = { ninf, 0x7fffffff };
#pragma unroll
        for (int s = 0; s < EPL; ++s) {
            const int e = s * 64 + lane;
            if (e < experts) loc = better(loc, Best{ sel[s], e });
        }
        const Best b = wave_argmax(loc);
        // the winner's unbiased score: slot b.i / 64 of lane b.i % 64, fetched with a lane read (b is uniform)
        const int win = __builtin_amdgcn_readfirstlane(b.i);
        float cand = 0.f;
#pragma unroll
        for (int s = 0; s < EPL; ++s) {
            if (s == (win >> 6)) cand = orig[s];
            if (s * 64 + lane == win) sel[s] = ninf;
        }
        const float w = __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, cand), win & 63));
        if (lane == t) my_w = w;
        if (lane == 0) idx_out[(int64_t)token * topk + t] = b.i;
    }
    if (sigmoid) {
        const float sum = round_bf16(wave_sum(lane < topk ? my_w : 0.f));
        my_w = round_bf16(my_w / sum);
    }
    my_w = my_w * route_scale;                     // binary32 product, rounded once to bf16 on the store
    if (lane < topk) w_out[(int64_t)token * topk + lane] = (uint16_t)(pack_bf16(my_w, 0.f) & 0xffffu);
}

}  // namespace

int launch_gate_route(const void* logits, const float* bias, void* weights, int64_t* indices, int64_t tokens,
                      int experts, int topk, int n_groups, int topk_groups, int score_func, float route_scale,
                      hipStream_t st) {
    const dim3 grid((unsigned)((tokens + kTokensPerWg - 1) / kTokensPerWg)), block(64 * kTokensPerWg);
    const int sig = score_func == DSV3_SCORE_SIGMOID;
#define DSV3_GATE_LAUNCH(EPL)                                                                                     \
    hipLaunchKernelGGL(gate_route_kernel<EPL>, grid, block, 0, st, (const uint16_t*)logits, bias, (uint16_t*)weights, \
                       indices, (int)tokens, experts, topk, n_groups, topk_groups, sig, route_scale)
    if (experts <= 64) DSV3_GATE_LAUNCH(1);
    else if (experts <= 128) DSV3_GATE_LAUNCH(2);
    else if (experts <= 256) DSV3_GATE_LAUNCH(4);
    else DSV3_GATE_LAUNCH(8);
#undef DSV3_GATE_LAUNCH
    return launch_status();
}

}  // namespace dsv3
