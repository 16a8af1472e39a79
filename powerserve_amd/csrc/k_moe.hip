// Mixture-of-experts routing for the layer-list models (PS_FF_MOE_SWIGLU).  The experts' matrix products are grouped launches of the dense kernels
// (k_dense.hip); here is what decides who goes where, all fp32:
//   moe_route_kernel    a block per token: router logits, sigmoid scores, the `top` largest, the shared expert's gate
//   moe_plan_kernel     the token-expert slots sorted by expert (counts, offsets, list) for the tiled products
//   moe_combine_kernel  a token's `top` per-slot results summed into the residual stream
#include "ps_seq.h"

#include <cmath>

static __device__ __forceinline__ float moe_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
static __device__ __forceinline__ float moe_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

typedef float moe_f4 __attribute__((ext_vector_type(4)));
// One block of four waves per token; dynamic LDS: experts + 1 floats (the token's scores, the shared gate's logit).  The rows of the router (and the
// shared gate's row as one more) are dealt to the waves; a row's K numbers are read as 16-byte pieces, four in flight per lane.
__global__ __launch_bounds__(256) void moe_route_kernel(const float *h, long long ldh, const float *router, const float *shared_gate, int experts, int top, int norm_top,
                                                        long long K, int32_t *sel, float *wgt, float *sgate) {
    extern __shared__ float sc[];
    const int t = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const float *x = h + (long long)t * ldh;
    const bool vec = K % 4 == 0 && ldh % 4 == 0;
    for (int e = wave; e < experts + (shared_gate ? 1 : 0); e += 4) {
        const float *w = e < experts ? router + (long long)e * K : shared_gate;
        float a = 0.f;
        if (vec) {
            float a4[4] = {0.f, 0.f, 0.f, 0.f};
            for (long long k0 = 0; k0 < K; k0 += 1024) {
                moe_f4 wv[4], xv[4];
#pragma unroll
                for (int u = 0; u < 4; u++) {
                    const long long k = k0 + 256 * u + 4 * lane;
                    const bool in = k < K;
                    wv[u] = in ? *(const moe_f4 *)(w + k) : moe_f4{0.f, 0.f, 0.f, 0.f};
                    xv[u] = in ? *(const moe_f4 *)(x + k) : moe_f4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int u = 0; u < 4; u++)
#pragma unroll
                    for (int i = 0; i < 4; i++) a4[i] = fmaf(wv[u][i], xv[u][i], a4[i]);
            }
            a = (a4[0] + a4[1]) + (a4[2] + a4[3]);
        } else {
            for (long long k = lane; k < K; k += 64) a = fmaf(w[k], x[k], a);
        }
        a = moe_wave_sum(a);
        if (lane == 0) sc[e] = moe_sigmoid(a);
    }
    __syncthreads();
    if (wave) return;
    if (shared_gate && lane == 0) sgate[t] = sc[experts];
    // the top: lane l proposes the best of experts l, l + 64, ..., the wave agrees on (largest score, lowest index), the winner is struck out
    float total = 0.f;
    for (int i = 0; i < top; i++) {
        float best = -1.f;
        int at = 0x7fffffff;
        for (int e = lane; e < experts; e += 64)
            if (sc[e] > best) { best = sc[e]; at = e; }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
        if (lane == 0) { sel[(long long)t * top + i] = at; wgt[(long long)t * top + i] = best; sc[at] = -2.f; }
        total += best;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (norm_top && lane < top) wgt[(long long)t * top + lane] /= total;
}
void psk_moe_route(hipStream_t st, const float *h, int64_t ldh, const float *router, const float *shared_gate, int experts, int top, int norm_top, int64_t K, int T,
                   int32_t *sel, float *wgt, float *sgate) {
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(256), (size_t)(experts + 1) * 4, st, h, (long long)ldh, router, shared_gate, experts, top, norm_top, (long long)K, sel,
                       wgt, sgate);
}

// one block; dynamic LDS: 2 x experts ints.  Counts, offsets, then every slot takes the next free place of its expert.  Which place a slot gets is up to the
// atomics, and it does not matter: a row of a tiled product is summed over k in the same order wherever in a tile it sits.
__global__ __launch_bounds__(1024) void moe_plan_kernel(const int32_t *sel, int S, int experts, int32_t *seg, int32_t *list) {
    extern __shared__ int pl[];
    int *cnt = pl, *cur = pl + experts;
    const int tid = threadIdx.x, nt = blockDim.x;
    for (int e = tid; e < experts; e += nt) cnt[e] = 0;
    __syncthreads();
    for (int s = tid; s < S; s += nt) atomicAdd(&cnt[sel[s]], 1);
    __syncthreads();
    if (tid == 0) {
        int at = 0;
        for (int e = 0; e < experts; e++) { seg[e] = at; cur[e] = at; at += cnt[e]; }
        seg[experts] = at;
    }
    __syncthreads();
    for (int s = tid; s < S; s += nt) list[atomicAdd(&cur[sel[s]], 1)] = s;
}
void psk_moe_plan(hipStream_t st, const int32_t *sel, int S, int experts, int32_t *seg, int32_t *list) {
    hipLaunchKernelGGL(moe_plan_kernel, dim3(1), dim3(S >= 1024 ? 1024 : 256), (size_t)experts * 8, st, sel, S, experts, seg, list);
}

__global__ void moe_combine_kernel(float *x, const float *y, int top, float alpha, long long n) {
    const long long t = blockIdx.x;
    for (long long i = threadIdx.x; i < n; i += blockDim.x) {
        float a = 0.f;
        for (int k = 0; k < top; k++) a += y[(t * top + k) * n + i];
        x[t * n + i] += alpha * a;
    }
}
void psk_moe_combine(hipStream_t st, float *x, const float *y, int top, float alpha, int64_t n, int T) {
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, x, y, top, alpha, (long long)n);
}
