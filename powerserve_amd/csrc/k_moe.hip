// Mixture-of-experts routing for the layer-list models (PS_FF_MOE_SWIGLU, PS_FF_MOE_RELU2).  The experts' matrix products are grouped launches of the dense kernels
// (k_dense.hip); here is what decides who goes where, all fp32:
//   moe_route_kernel    a block per token: router logits, sigmoid or soft-max scores, a correction and a group limit on the choice, the `top` largest,
//                       the shared expert's gate
//   moe_plan_kernel     the token-expert slots sorted by expert (counts, offsets, list) for the tiled products
//   moe_combine_kernel  a token's `top` per-slot results summed into the residual stream; an identity expert's share is its weight times the input
#include "ps_seq.h"

#include <cmath>

static __device__ __forceinline__ float moe_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
static __device__ __forceinline__ float moe_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

typedef float moe_f4 __attribute__((ext_vector_type(4)));
// One block of four waves per token.  The rows of the router (and the shared gate's row as one more) are dealt to the waves; a row's K numbers are read as
// 16-byte pieces, four in flight per lane.  Then wave 0 alone: scores (sigmoid, or soft-max over all rows), the choice scores (score + correction), the
// groups that stay in the race, and `top` rounds of (largest choice score, lowest index); the weights are the SCORES of the chosen.
// dynamic LDS: [rows + 1] scores, [rows] choice scores, [groups] group scores.
__global__ __launch_bounds__(256) void moe_route_kernel(const float *h, long long ldh, const float *router, const float *shared_gate, int experts, int top, int norm_top,
                                                        long long K, int softmax, const float *correction, int n_groups, int keep, int32_t *sel, float *wgt,
                                                        float *sgate) {
    extern __shared__ float sc[];
    float *ch = sc + experts + 1, *gs = ch + experts;
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
        if (lane == 0) sc[e] = softmax && e < experts ? a : moe_sigmoid(a);
    }
    __syncthreads();
    if (wave) return;
    if (shared_gate && lane == 0) sgate[t] = sc[experts];
    if (softmax) {
        float mx = -INFINITY, sum = 0.f;
        for (int e = lane; e < experts; e += 64) mx = fmaxf(mx, sc[e]);
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 64));
        for (int e = lane; e < experts; e += 64) sum += expf(sc[e] - mx);
        sum = moe_wave_sum(sum);
        for (int e = lane; e < experts; e += 64) sc[e] = expf(sc[e] - mx) / sum;
    }
    for (int e = lane; e < experts; e += 64) ch[e] = sc[e] + (correction ? correction[e] : 0.f);
    __builtin_amdgcn_wave_barrier();
    __threadfence_block();
    // (largest value, lowest index) over the wave's proposals
    auto agree = [&](float &best, int &at) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            const float ob = __shfl_xor(best, o, 64);
            const int oa = __shfl_xor(at, o, 64);
            if (ob > best || (ob == best && oa < at)) { best = ob; at = oa; }
        }
    };
    if (n_groups > 0) { // a group's score is its best choice score; the rows of every group outside the `keep` best leave the race
        const int size = experts / n_groups;
        for (int g = lane; g < n_groups; g += 64) {
            float b = -INFINITY;
            for (int e = g * size; e < (g + 1) * size; e++) b = fmaxf(b, ch[e]);
            gs[g] = b;
        }
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
        for (int i = 0; i < keep; i++) {
            float best = -INFINITY;
            int at = 0x7fffffff;
            for (int g = lane; g < n_groups; g += 64)
                if (gs[g] > best) { best = gs[g]; at = g; }
            agree(best, at);
            if (lane == 0 && at != 0x7fffffff) gs[at] = -INFINITY; // (struck out = kept)
            __builtin_amdgcn_wave_barrier();
            __threadfence_block();
        }
        for (int e = lane; e < experts; e += 64)
            if (gs[e / size] != -INFINITY) ch[e] = -INFINITY;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    float total = 0.f;
    for (int i = 0; i < top; i++) {
        float best = -INFINITY;
        int at = 0x7fffffff;
        for (int e = lane; e < experts; e += 64)
            if (ch[e] > best) { best = ch[e]; at = e; }
        agree(best, at);
        const bool any = at != 0x7fffffff; // (nothing left in the race: the slot goes to row 0 with weight 0)
        const float w = any ? sc[at] : 0.f;
        if (lane == 0) { sel[(long long)t * top + i] = any ? at : 0; wgt[(long long)t * top + i] = w; if (any) ch[at] = -INFINITY; }
        total += w;
        __builtin_amdgcn_wave_barrier();
        __threadfence_block();
    }
    if (norm_top && lane < top) wgt[(long long)t * top + lane] /= total;
}
void psk_moe_route(hipStream_t st, const float *h, int64_t ldh, const float *router, const float *shared_gate, int experts, int top, int norm_top, int64_t K, int T,
                   int32_t *sel, float *wgt, float *sgate, int softmax, const float *correction, int n_groups, int keep) {
    hipLaunchKernelGGL(moe_route_kernel, dim3(T), dim3(256), (size_t)(2 * experts + 1 + (n_groups > 0 ? n_groups : 0)) * 4, st, h, (long long)ldh, router, shared_gate,
                       experts, top, norm_top, (long long)K, softmax, correction, n_groups, keep, sel, wgt, sgate);
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

// x[t] += alpha * sum_k (slot t top + k: its product's result y[slot], or -- a slot whose choice is an identity expert, sel >= n_real -- wgt[slot] * h[t]);
// y NULL: the products have been added already and only the identity slots are left.
__global__ void moe_combine_kernel(float *x, const float *y, int top, float alpha, long long n, const int32_t *sel, const float *wgt, int n_real, const float *h,
                                   long long ldh) {
    const long long t = blockIdx.x;
    for (long long i = threadIdx.x; i < n; i += blockDim.x) {
        float a = 0.f;
        for (int k = 0; k < top; k++) {
            const long long s = t * top + k;
            if (sel && sel[s] >= n_real) a = fmaf(wgt[s], h[t * ldh + i], a);
            else if (y) a += y[s * n + i];
        }
        x[t * n + i] += alpha * a;
    }
}
void psk_moe_combine(hipStream_t st, float *x, const float *y, int top, float alpha, int64_t n, int T, const int32_t *sel, const float *wgt, int n_real, const float *h,
                     int64_t ldh) {
    hipLaunchKernelGGL(moe_combine_kernel, dim3(T), dim3(256), 0, st, x, y, top, alpha, (long long)n, sel, wgt, n_real, h, (long long)ldh);
}
