// Mechanisms of the layer-list models that are not matrix products: RMS norms (with the residual add), causal convolutions over time
// with a per-sequence tail, and the two recurrent scans (wkv, gated delta rule).  Everything here is fp32.
//
// The scans: a head's state S [d][dv] is split by COLUMN over threads -- every column j evolves on its own in both recurrences
// (S_ij <- decay S_ij + k_i x_j needs only column j) -- and each column over R lanes of 16 rows each, so a step is 16 fused
// multiply-adds per lane and one R-lane butterfly; the per-token vectors of a head (r, k, decays; unit q and k) are staged eight tokens
// at a time through LDS, where their per-token scalars are reduced once for all columns.
#include "ps_seq.h"

#include <cmath>

static __device__ __forceinline__ float sq_block_sum(float v, float *red) { // 256 threads
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return red[0] + red[1] + red[2] + red[3];
}
static __device__ __forceinline__ float sq_silu(float x) { return x / (1.f + expf(-x)); }
static __device__ __forceinline__ float sq_softplus(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// (a row in `groups` equal consecutive parts, each with its own mean square: block (row, part) works on n = the part's length)
__global__ __launch_bounds__(256) void sq_rmsnorm_kernel(const float *x, long long ldx, const int32_t *idx, const float *w, float offset, float eps, long long n,
                                                         float *y, long long ldy) {
    __shared__ float red[4];
    const long long r = idx ? idx[blockIdx.x] : blockIdx.x, part = (long long)blockIdx.y * n;
    const float *xr = x + r * ldx + part;
    w += part;
    float s = 0.f;
    for (long long i = threadIdx.x; i < n; i += 256) s += xr[i] * xr[i];
    s = sq_block_sum(s, red);
    const float inv = 1.f / sqrtf(s / (float)n + eps);
    float *yr = y + (long long)blockIdx.x * ldy + part;
    for (long long i = threadIdx.x; i < n; i += 256) yr[i] = xr[i] * inv * (offset + w[i]);
}
void psk_rmsnorm(hipStream_t st, const float *x, int64_t ldx, const int32_t *idx, const float *w, float offset, float eps, int64_t n, int rows, float *y, int64_t ldy,
                 int groups) {
    if (rows <= 0) return;
    hipLaunchKernelGGL(sq_rmsnorm_kernel, dim3(rows, groups), dim3(256), 0, st, x, (long long)ldx, idx, w, offset, eps, (long long)(n / groups), y, (long long)ldy);
}

// The front of a parallel layer without an input filter, one block per row:  x = sum_j mix[j] X_j  over the nmix streams X_j = src + j stride (mix NULL: the last
// of them as it is), kept in xout (NULL: not kept; it may be the last stream itself); then, over `groups` equal parts of the row each with its own mean square,
// h = x / rms * (offset + w1) and h2 = x / rms * (offset + w2): two norms of the same vector share their statistics (w1 / w2 NULL: not wanted).
// center: a layer norm instead -- the part's mean is taken off and the variance is the mean of the squared deviations (two passes over the row in LDS).
// dynamic LDS: n + 2 groups floats.
__global__ __launch_bounds__(1024) void sq_front_kernel(const float *src, long long stride, int nmix, const float *mix, const int32_t *idx, float *xout, const float *w1,
                                                       float *h, const float *w2, float *h2, int groups, float offset, float eps, long long n, int center) {
    extern __shared__ float fr[];
    float *xs = fr, *inv = fr + n, *mean = inv + groups;
    const long long r = idx ? idx[blockIdx.x] : blockIdx.x, o = (long long)blockIdx.x * n;
    const int tid = threadIdx.x, nt = blockDim.x;
    for (long long i = tid; i < n; i += nt) {
        float v;
        if (mix) {
            v = 0.f;
            for (int j = 0; j < nmix; j++) v = fmaf(mix[j], src[j * stride + r * n + i], v);
        } else {
            v = src[(nmix - 1) * stride + r * n + i];
        }
        xs[i] = v;
        if (xout) xout[o + i] = v;
    }
    if (!w1 && !w2) return;
    __syncthreads();
    const long long gs = n / groups;
    for (int g = tid >> 6; g < groups; g += nt >> 6) {
        float mu = 0.f;
        if (center) {
            for (long long i = tid & 63; i < gs; i += 64) mu += xs[g * gs + i];
#pragma unroll
            for (int o2 = 32; o2 > 0; o2 >>= 1) mu += __shfl_xor(mu, o2, 64);
            mu /= (float)gs;
        }
        float s = 0.f;
        for (long long i = tid & 63; i < gs; i += 64) { const float dv = xs[g * gs + i] - mu; s += dv * dv; }
#pragma unroll
        for (int o2 = 32; o2 > 0; o2 >>= 1) s += __shfl_xor(s, o2, 64);
        if ((tid & 63) == 0) { inv[g] = 1.f / sqrtf(s / (float)gs + eps); mean[g] = mu; }
    }
    __syncthreads();
    for (long long i = tid; i < n; i += nt) {
        const float v = (xs[i] - mean[i / gs]) * inv[i / gs];
        if (w1) h[o + i] = v * (offset + w1[i]);
        if (w2) h2[o + i] = v * (offset + w2[i]);
    }
}
void psk_front(hipStream_t st, const float *src, int64_t stride, int nmix, const float *mix, const int32_t *idx, float *xout, const float *w1, float *h, const float *w2,
               float *h2, int groups, float offset, float eps, int64_t n, int rows, int center) {
    if (rows <= 0) return;
    static unsigned long long mask = 0;
    if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)sq_front_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipLaunchKernelGGL(sq_front_kernel, dim3(rows), dim3(rows <= 8 && n >= 2048 ? 1024 : 256), (size_t)(n + 2 * groups) * 4, st, src, (long long)stride, nmix, mix, idx, xout, w1, h, w2, h2, groups, offset, eps,
                       (long long)n, center);
}

__global__ __launch_bounds__(256) void sq_norm_residual_kernel(float *x, const float *y, const float *w, float offset, float eps, long long n) {
    __shared__ float red[4];
    const long long at = ((long long)blockIdx.x * gridDim.y + blockIdx.y) * n; // (block (row, part) of a row of gridDim.y parts)
    const float *yr = y + at;
    float *xr = x + at;
    w += (long long)blockIdx.y * n;
    float s = 0.f;
    for (long long i = threadIdx.x; i < n; i += 256) s += yr[i] * yr[i];
    s = sq_block_sum(s, red);
    const float inv = 1.f / sqrtf(s / (float)n + eps);
    for (long long i = threadIdx.x; i < n; i += 256) xr[i] += yr[i] * inv * (offset + w[i]);
}
void psk_norm_residual(hipStream_t st, float *x, const float *y, const float *w, float offset, float eps, int64_t n, int rows, int groups) {
    if (rows <= 0) return;
    hipLaunchKernelGGL(sq_norm_residual_kernel, dim3(rows, groups), dim3(256), 0, st, x, y, w, offset, eps, (long long)(n / groups));
}

// ---------------------------------------------------------------------------------------------------- causal convolution with a tail
#define SQ_CONV_CHUNK 8 // tokens per thread: a portion spreads over T / 8 times as many threads as channels
static __device__ __forceinline__ void sq_conv_tail(float *tail, const float *in, long long ldi, int taps, long long C, int T, long long c) {
    // new tail row i = input of token T - (taps-1) + i; before this step's first token: the old tail's row T + i (ascending i never reads a row already written)
    for (int i = 0; i < taps - 1; i++) {
        const int r = T + i - (taps - 1);
        tail[(long long)i * C + c] = r >= 0 ? in[(long long)r * ldi + c] : tail[(long long)(T + i) * C + c];
    }
}
__global__ __launch_bounds__(256) void sq_conv_kernel(const ps_seq_step *step, long long tail_off, const float *in, long long ldi, const float *w, int taps, int mode,
                                                      long long C, int T, float *out, long long ldo) {
    const long long c = (long long)blockIdx.x * 256 + threadIdx.x;
    if (c >= C) return;
    float *tail = step->state + tail_off;
    const int tb = blockIdx.y * SQ_CONV_CHUNK, te = min(T, tb + SQ_CONV_CHUNK);
    for (int t = tb; t < te; t++) {
        float s = 0.f;
        for (int j = 0; j < taps; j++) {
            const int r = t - taps + 1 + j;
            const float v = r >= 0 ? in[(long long)r * ldi + c] : tail[(long long)(taps - 1 + r) * C + c];
            s = fmaf(w[c * taps + j], v, s);
        }
        out[(long long)t * ldo + c] = mode == 0 ? in[(long long)t * ldi + c] + s : sq_silu(s);
    }
    if (gridDim.y == 1) sq_conv_tail(tail, in, ldi, taps, C, T, c); // one thread owns the channel: it has read what it overwrites
}
__global__ __launch_bounds__(256) void sq_conv_tail_kernel(const ps_seq_step *step, long long tail_off, const float *in, long long ldi, int taps, long long C, int T) {
    const long long c = (long long)blockIdx.x * 256 + threadIdx.x;
    if (c < C) sq_conv_tail(step->state + tail_off, in, ldi, taps, C, T, c);
}
void psk_causal_conv(hipStream_t st, const ps_seq_step *step, int64_t tail_off, const float *in, int64_t ldi, const float *w, int taps, int mode, int64_t C, int T,
                     float *out, int64_t ldo) {
    const unsigned gx = (unsigned)((C + 255) / 256), gy = (unsigned)((T + SQ_CONV_CHUNK - 1) / SQ_CONV_CHUNK);
    hipLaunchKernelGGL(sq_conv_kernel, dim3(gx, gy), dim3(256), 0, st, step, (long long)tail_off, in, (long long)ldi, w, taps, mode, (long long)C, T, out, (long long)ldo);
    if (gy > 1 && taps > 1) hipLaunchKernelGGL(sq_conv_tail_kernel, dim3(gx), dim3(256), 0, st, step, (long long)tail_off, in, (long long)ldi, taps, (long long)C, T);
}

__global__ void sq_state_store_kernel(const ps_seq_step *step, long long off, const float *src, long long n) {
    float *dst = step->state + off;
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) dst[i] = src[i];
}
void psk_state_store(hipStream_t st, const ps_seq_step *step, int64_t off, const float *src, int64_t n) {
    hipLaunchKernelGGL(sq_state_store_kernel, dim3((unsigned)min((long long)((n + 255) / 256), 1024ll)), dim3(256), 0, st, step, (long long)off, src, (long long)n);
}
__global__ void sq_fill_kernel(float *p, float v, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) p[i] = v;
}
void psk_fill(hipStream_t st, float *p, float v, int64_t n) {
    if (n <= 0) return;
    hipLaunchKernelGGL(sq_fill_kernel, dim3((unsigned)min((long long)((n + 255) / 256), 4096ll)), dim3(256), 0, st, p, v, (long long)n);
}
__global__ void sq_copy_kernel(const float *s, float *d, long long n) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) d[i] = s[i];
}
void psk_copy(hipStream_t st, const float *src, float *dst, int64_t n) {
    if (n <= 0) return;
    hipLaunchKernelGGL(sq_copy_kernel, dim3((unsigned)min((long long)((n + 255) / 256), 4096ll)), dim3(256), 0, st, src, dst, (long long)n);
}


// A single token's sublayer boundary in one launch (one block):  x += y / rms(y) * (offset + wb)   (where y is given), then, where wn is given,
// h = conv(x / rms(x) * (offset + wn)) with the convolution's residual form and its tail brought up to date -- three launches of the kernels above.
__global__ __launch_bounds__(1024) void sq_boundary1_kernel(const ps_seq_step *step, float *x, const float *y, const float *wb, const float *wn, const float *cw,
                                                            int taps, long long tail_off, float offset, float eps, long long n, float *h, float *hn) {
    __shared__ float red[16];
    const int tid = threadIdx.x, nw = blockDim.x >> 6;
    auto block_sum = [&](float v) {
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
        __syncthreads();
        if ((tid & 63) == 0) red[tid >> 6] = v;
        __syncthreads();
        float s = 0.f;
        for (int w = 0; w < nw; w++) s += red[w];
        return s;
    };
    float s2 = 0.f;
    if (y) {
        float s1 = 0.f;
        for (long long i = tid; i < n; i += blockDim.x) s1 += y[i] * y[i];
        const float inv = 1.f / sqrtf(block_sum(s1) / (float)n + eps);
        for (long long i = tid; i < n; i += blockDim.x) {
            const float v = x[i] + y[i] * inv * (offset + wb[i]);
            x[i] = v;
            s2 += v * v;
        }
    } else {
        for (long long i = tid; i < n; i += blockDim.x) s2 += x[i] * x[i];
    }
    if (!wn) return;
    const float inv = 1.f / sqrtf(block_sum(s2) / (float)n + eps);
    float *tail = step->state + tail_off;
    for (long long c = tid; c < n; c += blockDim.x) { // (a thread re-reads only what it wrote itself)
        const float v = x[c] * inv * (offset + wn[c]);
        if (hn) hn[c] = v;
        float s = cw[c * taps + taps - 1] * v;
        for (int j = 0; j < taps - 1; j++) s = fmaf(cw[c * taps + j], tail[(long long)j * n + c], s);
        h[c] = v + s;
        for (int j = 0; j + 1 < taps - 1; j++) tail[(long long)j * n + c] = tail[(long long)(j + 1) * n + c];
        if (taps > 1) tail[(long long)(taps - 2) * n + c] = v;
    }
}
void psk_boundary1(hipStream_t st, const ps_seq_step *step, float *x, const float *y, const float *wb, const float *wn, const float *cw, int taps, int64_t tail_off,
                   float offset, float eps, int64_t n, float *h, float *hn) {
    hipLaunchKernelGGL(sq_boundary1_kernel, dim3(1), dim3(n >= 2048 ? 1024 : 256), 0, st, step, x, y, wb, wn, cw, taps, (long long)tail_off, offset, eps, (long long)n, h, hn);
}

// ---------------------------------------------------------------------------------------------------- recurrent scans
typedef float sq_f4 __attribute__((ext_vector_type(4)));
#define SQ_NR 16 // state rows per lane (lane s of a column holds rows 16 s .. 16 s + 15: its per-token vectors are four 16-byte LDS reads each)
#define SQ_TC 8  // tokens staged per round
#define SQ_PF 8  // staged numbers per thread and vector: SQ_TC * 16 R / 256 <= 8 for R <= 16
static inline int sq_lanes_per_col(int d) { int R = 1; while (R * SQ_NR < d) R *= 2; return R; }


// sum over the R (1, 2, 4, 8 or 16) adjacent lanes of a column, every lane gets the total: data-parallel-primitive moves inside a row of 16
// lanes (neighbour, other pair, mirrored half, mirrored row) instead of trips through the LDS crossbar
static __device__ __forceinline__ float sq_dpp(float v, int ctrl_sel) {
    const int x = __float_as_int(v);
    int y;
    if (ctrl_sel == 0) y = __builtin_amdgcn_update_dpp(0, x, 0xB1, 0xF, 0xF, false);       // quad_perm [1, 0, 3, 2]
    else if (ctrl_sel == 1) y = __builtin_amdgcn_update_dpp(0, x, 0x4E, 0xF, 0xF, false);  // quad_perm [2, 3, 0, 1]
    else if (ctrl_sel == 2) y = __builtin_amdgcn_update_dpp(0, x, 0x141, 0xF, 0xF, false); // row_half_mirror
    else y = __builtin_amdgcn_update_dpp(0, x, 0x140, 0xF, 0xF, false);                    // row_mirror
    return __int_as_float(y);
}
static __device__ __forceinline__ float sq_col_sum(float v, int R) {
    if (R > 1) v += sq_dpp(v, 0);
    if (R > 2) v += sq_dpp(v, 1);
    if (R > 4) v += sq_dpp(v, 2);
    if (R > 8) v += sq_dpp(v, 3);
    return v;
}

// The scan of a state with a decay per key channel, S [d][dv] per head, in its two forms:
//   GLA = 0 (wkv)  o_j = sum_i r_i (S_ij + bonus_i k_i v_j), then S_ij <- w_i S_ij + k_i v_j,  w = exp(-exp(z))
//   GLA = 1        S_ij <- w_i S_ij + k_i v_j, then o_j = sum_i (qscale r_i) S_ij,              w = sigmoid(z)^inv_tau = exp(-softplus(-z) inv_tau)
// LDS: rs, ks, ws [TC][dp] (dp = NR * R, rows >= d zero), sc [TC] (sum_i r_i bonus_i k_i)
template <int GLA>
__global__ __launch_bounds__(256) void sq_decay_scan_kernel(const ps_seq_step *step, long long state_off, const float *r, const float *k, const float *v, const float *z,
                                                            long long ld, long long ldz, const float *bonus, int d, int dv, float qscale, float inv_tau, int R, int T,
                                                            float *o, long long ldo) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int dp = SQ_NR * R, cpb = 256 / R;
    float *rs = lds, *ks = rs + SQ_TC * dp, *ws = ks + SQ_TC * dp, *sc = ws + SQ_TC * dp;
    const int h = blockIdx.y, tid = threadIdx.x, s = tid % R, j = blockIdx.x * cpb + tid / R;
    const bool col = j < dv;
    float *S0 = step->state + state_off + (long long)h * d * dv;
    float S[SQ_NR];
#pragma unroll
    for (int m = 0; m < SQ_NR; m++) {
        const int i = s * SQ_NR + m;
        S[m] = (col && i < d) ? S0[(long long)i * dv + j] : 0.f;
    }
    const long long hb = (long long)h * d, vb = (long long)h * dv;
    // the next round's inputs are requested before the current round's steps run, and land in LDS after them
    float pa[SQ_PF], pb[SQ_PF], pc[SQ_PF], pv[SQ_TC];
    auto fetch = [&](int t0) {
        const int nt = min(SQ_TC, T - t0);
#pragma unroll
        for (int e = 0; e < SQ_PF; e++) {
            const int x = tid + 256 * e, t = x / dp, i = x % dp;
            const bool in = x < SQ_TC * dp && t < nt && i < d;
            const long long at = (long long)(t0 + (in ? t : 0)) * ld + hb + (in ? i : 0);
            pa[e] = in ? r[at] : 0.f;
            pb[e] = in ? k[at] : 0.f;
            pc[e] = in ? z[(long long)(t0 + t) * ldz + hb + i] : (GLA ? INFINITY : -INFINITY); // w = 1: with k = 0 a token that is not there leaves the state alone
        }
#pragma unroll
        for (int t = 0; t < SQ_TC; t++) pv[t] = (col && t < nt) ? v[(long long)(t0 + t) * ld + vb + j] : 0.f;
    };
    fetch(0);
    for (int t0 = 0; t0 < T; t0 += SQ_TC) {
        const int nt = min(SQ_TC, T - t0);
        __syncthreads();
#pragma unroll
        for (int e = 0; e < SQ_PF; e++) {
            const int x = tid + 256 * e;
            if (x < SQ_TC * dp) {
                rs[x] = GLA ? pa[e] * qscale : pa[e];
                ks[x] = pb[e];
                ws[x] = GLA ? expf(-sq_softplus(-pc[e]) * inv_tau) : expf(-expf(pc[e]));
            }
        }
        float vj[SQ_TC];
#pragma unroll
        for (int t = 0; t < SQ_TC; t++) vj[t] = pv[t];
        __syncthreads();
        if (t0 + SQ_TC < T) fetch(t0 + SQ_TC);
        for (int t = tid >> 6; !GLA && t < SQ_TC; t += 4) { // one wave per token
            float a = 0.f;
            for (int i = tid & 63; i < d; i += 64) a += rs[t * dp + i] * bonus[hb + i] * ks[t * dp + i];
#pragma unroll
            for (int x = 32; x > 0; x >>= 1) a += __shfl_xor(a, x, 64);
            if ((tid & 63) == 0) sc[t] = a;
        }
        __syncthreads();
        // (no branch per token: the steps of a round are one block of straight-line code the compiler can interleave; padded tokens are neutral)
#pragma unroll
        for (int t = 0; t < SQ_TC; t++) {
            {
                const sq_f4 *rt = (const sq_f4 *)(rs + t * dp + s * SQ_NR), *kt = (const sq_f4 *)(ks + t * dp + s * SQ_NR), *wt = (const sq_f4 *)(ws + t * dp + s * SQ_NR);
                float pp[4] = {0.f, 0.f, 0.f, 0.f}; // four short chains instead of one of sixteen
#pragma unroll
                for (int m4 = 0; m4 < SQ_NR / 4; m4++) {
                    const sq_f4 r4 = rt[m4], k4 = kt[m4], w4 = wt[m4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        if constexpr (GLA) {
                            S[4 * m4 + e] = fmaf(w4[e], S[4 * m4 + e], k4[e] * vj[t]);
                            pp[e] = fmaf(r4[e], S[4 * m4 + e], pp[e]);
                        } else {
                            pp[e] = fmaf(r4[e], S[4 * m4 + e], pp[e]);
                            S[4 * m4 + e] = fmaf(w4[e], S[4 * m4 + e], k4[e] * vj[t]);
                        }
                    }
                }
                const float p = sq_col_sum((pp[0] + pp[1]) + (pp[2] + pp[3]), R);
                if (col && s == 0 && t < nt) o[(long long)(t0 + t) * ldo + vb + j] = GLA ? p : fmaf(vj[t], sc[t], p);
            }
        }
    }
#pragma unroll
    for (int m = 0; m < SQ_NR; m++) {
        const int i = s * SQ_NR + m;
        if (col && i < d) S0[(long long)i * dv + j] = S[m];
    }
}
void psk_wkv_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *r, const float *k, const float *v, const float *z, int64_t ld,
                  const float *bonus, int H, int d, int T, float *o, int64_t ldo) {
    const int R = sq_lanes_per_col(d), cpb = 256 / R;
    const size_t lds = (size_t)(3 * SQ_TC * SQ_NR * R + SQ_TC) * 4;
    hipLaunchKernelGGL(sq_decay_scan_kernel<0>, dim3((d + cpb - 1) / cpb, H), dim3(256), lds, st, step, (long long)state_off, r, k, v, z, (long long)ld, (long long)ld, bonus, d, d, 1.f, 1.f,
                       R, T, o, (long long)ldo);
}
void psk_gla_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *q, const float *k, const float *v, int64_t ld, const float *z, int64_t ldz,
                  float tau, int H, int d, int dv, int T, float *o, int64_t ldo) {
    const int R = sq_lanes_per_col(d), cpb = 256 / R;
    const size_t lds = (size_t)(3 * SQ_TC * SQ_NR * R + SQ_TC) * 4;
    hipLaunchKernelGGL(sq_decay_scan_kernel<1>, dim3((dv + cpb - 1) / cpb, H), dim3(256), lds, st, step, (long long)state_off, q, k, v, z, (long long)ld, (long long)ldz, nullptr, d, dv,
                       1.f / sqrtf((float)d), 1.f / tau, R, T, o, (long long)ldo);
}

// LDS: qs, ks [TC][dp]; per token: g, beta, kq
__global__ __launch_bounds__(256) void sq_delta_scan_kernel(const ps_seq_step *step, long long state_off, const float *q, const float *k, const float *v,
                                                            const float *braw, const float *araw, long long ld, long long ldb, const float *a_log, const float *dt_bias, int H,
                                                            int KH, int d, int dv, int R, int T, float *o, long long ldo) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int dp = SQ_NR * R, cpb = 256 / R;
    float *qs = lds, *ks = qs + SQ_TC * dp, *gs = ks + SQ_TC * dp, *bs = gs + SQ_TC, *kq = bs + SQ_TC;
    const int h = blockIdx.y, tid = threadIdx.x, s = tid % R, j = blockIdx.x * cpb + tid / R;
    const bool col = j < dv;
    float *S0 = step->state + state_off + (long long)h * d * dv;
    float S[SQ_NR];
#pragma unroll
    for (int m = 0; m < SQ_NR; m++) {
        const int i = s * SQ_NR + m;
        S[m] = (col && i < d) ? S0[(long long)i * dv + j] : 0.f;
    }
    const long long qb = (long long)(h / (H / KH)) * d, vb = (long long)h * dv;
    const float qscale = 1.f / sqrtf((float)d), na = -expf(a_log[h]), db = dt_bias[h];
    float pa[SQ_PF], pb[SQ_PF], pv[SQ_TC], pg = 0.f, pbeta = 0.f;
    auto fetch = [&](int t0) {
        const int nt = min(SQ_TC, T - t0);
#pragma unroll
        for (int e = 0; e < SQ_PF; e++) {
            const int x = tid + 256 * e, t = x / dp, i = x % dp;
            const bool in = x < SQ_TC * dp && t < nt && i < d;
            const long long at = (long long)(t0 + (in ? t : 0)) * ld + qb + (in ? i : 0);
            pa[e] = in ? q[at] : 0.f;
            pb[e] = in ? k[at] : 0.f;
        }
        if (tid < SQ_TC) {
            const bool in = tid < nt;
            pg = in ? araw[(long long)(t0 + tid) * ldb + h] : 0.f;
            pbeta = in ? braw[(long long)(t0 + tid) * ldb + h] : -INFINITY; // sigmoid(-inf) = 0
        }
#pragma unroll
        for (int t = 0; t < SQ_TC; t++) pv[t] = (col && t < nt) ? v[(long long)(t0 + t) * ld + vb + j] : 0.f;
    };
    fetch(0);
    for (int t0 = 0; t0 < T; t0 += SQ_TC) {
        const int nt = min(SQ_TC, T - t0);
        __syncthreads();
#pragma unroll
        for (int e = 0; e < SQ_PF; e++) {
            const int x = tid + 256 * e;
            if (x < SQ_TC * dp) {
                qs[x] = pa[e];
                ks[x] = pb[e];
            }
        }
        if (tid < SQ_TC) {
            gs[tid] = tid < nt ? expf(na * sq_softplus(pg + db)) : 1.f;
            bs[tid] = 1.f / (1.f + expf(-pbeta));
        }
        float vj[SQ_TC];
#pragma unroll
        for (int t = 0; t < SQ_TC; t++) vj[t] = pv[t];
        __syncthreads();
        if (t0 + SQ_TC < T) fetch(t0 + SQ_TC);
        for (int t = tid >> 6; t < SQ_TC; t += 4) { // one wave per token: unit vectors, then k . q
            float a = 0.f, b = 0.f;
            for (int i = tid & 63; i < d; i += 64) {
                a += qs[t * dp + i] * qs[t * dp + i];
                b += ks[t * dp + i] * ks[t * dp + i];
            }
#pragma unroll
            for (int x = 32; x > 0; x >>= 1) {
                a += __shfl_xor(a, x, 64);
                b += __shfl_xor(b, x, 64);
            }
            const float iq = qscale / sqrtf(a + 1e-6f), ik = 1.f / sqrtf(b + 1e-6f);
            float c = 0.f;
            for (int i = tid & 63; i < d; i += 64) {
                const float qn = qs[t * dp + i] * iq, kn = ks[t * dp + i] * ik;
                qs[t * dp + i] = qn;
                ks[t * dp + i] = kn;
                c += qn * kn;
            }
#pragma unroll
            for (int x = 32; x > 0; x >>= 1) c += __shfl_xor(c, x, 64);
            if ((tid & 63) == 0) kq[t] = c;
        }
        __syncthreads();
#pragma unroll
        for (int t = 0; t < SQ_TC; t++) {
            { // (padded tokens: g = 1, beta = 0, k = 0 -- the state stays)
                const sq_f4 *qt = (const sq_f4 *)(qs + t * dp + s * SQ_NR), *kt = (const sq_f4 *)(ks + t * dp + s * SQ_NR);
                const float g = gs[t];
                sq_f4 k4[SQ_NR / 4];
                float a1[4] = {0.f, 0.f, 0.f, 0.f}, a2[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int m4 = 0; m4 < SQ_NR / 4; m4++) {
                    const sq_f4 q4 = qt[m4];
                    k4[m4] = kt[m4];
#pragma unroll
                    for (int e = 0; e < 4; e++) {
                        S[4 * m4 + e] *= g;
                        a1[e] = fmaf(k4[m4][e], S[4 * m4 + e], a1[e]);
                        a2[e] = fmaf(q4[e], S[4 * m4 + e], a2[e]);
                    }
                }
                const float p1 = sq_col_sum((a1[0] + a1[1]) + (a1[2] + a1[3]), R), p2 = sq_col_sum((a2[0] + a2[1]) + (a2[2] + a2[3]), R);
                const float u = bs[t] * (vj[t] - p1);
#pragma unroll
                for (int m4 = 0; m4 < SQ_NR / 4; m4++)
#pragma unroll
                    for (int e = 0; e < 4; e++) S[4 * m4 + e] = fmaf(k4[m4][e], u, S[4 * m4 + e]);
                if (col && s == 0 && t < nt) o[(long long)(t0 + t) * ldo + vb + j] = fmaf(u, kq[t], p2); // S_new^T q = (g S)^T q + u (k . q)
            }
        }
    }
#pragma unroll
    for (int m = 0; m < SQ_NR; m++) {
        const int i = s * SQ_NR + m;
        if (col && i < d) S0[(long long)i * dv + j] = S[m];
    }
}
void psk_delta_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *q, const float *k, const float *v, const float *braw,
                    const float *araw, int64_t ld, int64_t ldb, const float *a_log, const float *dt_bias, int H, int KH, int d, int dv, int T, float *o, int64_t ldo) {
    const int R = sq_lanes_per_col(d), cpb = 256 / R;
    const size_t lds = (size_t)(2 * SQ_TC * SQ_NR * R + 3 * SQ_TC) * 4;
    hipLaunchKernelGGL(sq_delta_scan_kernel, dim3((dv + cpb - 1) / cpb, H), dim3(256), lds, st, step, (long long)state_off, q, k, v, braw, araw, (long long)ld, (long long)ldb, a_log,
                       dt_bias, H, KH, d, dv, R, T, o, (long long)ldo);
}

__global__ __launch_bounds__(64) void sq_headnorm_gate_kernel(float *o, long long ldo, const float *g, long long ldg, const float *w, int w_stride, float eps, int dv) {
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    float *oh = o + (long long)t * ldo + (long long)h * dv;
    const float *gh = g + (long long)t * ldg + (long long)h * dv, *wh = w + (long long)h * w_stride;
    float s = 0.f;
    for (int j = lane; j < dv; j += 64) s += oh[j] * oh[j];
#pragma unroll
    for (int x = 32; x > 0; x >>= 1) s += __shfl_xor(s, x, 64);
    const float inv = 1.f / sqrtf(s / (float)dv + eps);
    for (int j = lane; j < dv; j += 64) oh[j] = oh[j] * inv * wh[j] * sq_silu(gh[j]);
}
void psk_headnorm_gate(hipStream_t st, float *o, int64_t ldo, const float *g, int64_t ldg, const float *w, int w_stride, float eps, int H, int dv, int T) {
    hipLaunchKernelGGL(sq_headnorm_gate_kernel, dim3(T, H), dim3(64), 0, st, o, (long long)ldo, g, (long long)ldg, w, w_stride, eps, dv);
}


// ---------------------------------------------------------------------------------------------------- element-wise gated recurrence (minGRU)
// y[t] = [ z | u | g ] pre-activations (C each, row stride ldy).  Per channel  a_t = 1 - sigmoid(z_t),  b_t = sigmoid(z_t) cand(u_t)  with
// cand(u) = u + 1/2 (u >= 0), sigmoid(u) (u < 0);  S_t = a_t S_(t-1) + b_t;  o[t] = S_t silu(g_t).  The state [C] is fp32 at step->state + state_off.
// A block is 64 channels x NCH time chunks: every chunk first folds its own tokens from zero (A = prod a, B), the chunks' (A, B) meet in LDS, each chunk
// takes the state in front of it and walks its tokens again, now storing.  One chunk (a short step): a single walk.
static __device__ __forceinline__ float sq_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }
__global__ __launch_bounds__(1024) void sq_mingru_kernel(const ps_seq_step *step, long long state_off, const float *y, long long ldy, long long C, int T, float *o,
                                                         long long ldo) {
    __shared__ float As[16][64], Bs[16][64];
    const int lane = threadIdx.x, ch = threadIdx.y, nch = blockDim.y;
    const long long c = (long long)blockIdx.x * 64 + lane;
    const bool in = c < C;
    const int per = (T + nch - 1) / nch, tb = ch * per, te = min(T, tb + per);
    const float *yz = y + c, *yu = y + C + c, *yg = y + 2 * C + c;
    float *state = step->state + state_off;
    float S = in ? state[c] : 0.f; // (read before the barrier below: the chunk with the last token overwrites it when it is done)
    if (nch > 1) {
        float A = 1.f, B = 0.f;
        if (in)
            for (int t = tb; t < te; t++) {
                const float z = sq_sigmoid(yz[(long long)t * ldy]), u = yu[(long long)t * ldy];
                const float cand = u >= 0.f ? u + 0.5f : sq_sigmoid(u), a = 1.f - z;
                A *= a;
                B = fmaf(a, B, z * cand);
            }
        As[ch][lane] = A;
        Bs[ch][lane] = B;
        __syncthreads();
        if (in)
            for (int j = 0; j < ch; j++) S = fmaf(As[j][lane], S, Bs[j][lane]);
    }
    if (!in) return;
    for (int t = tb; t < te; t++) {
        const float z = sq_sigmoid(yz[(long long)t * ldy]), u = yu[(long long)t * ldy], gg = yg[(long long)t * ldy];
        const float cand = u >= 0.f ? u + 0.5f : sq_sigmoid(u);
        S = fmaf(1.f - z, S, z * cand);
        o[(long long)t * ldo + c] = S * sq_silu(gg);
    }
    if (te == T && tb < T) state[c] = S; // (the chunk that holds the last token)
}
void psk_mingru_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *y, int64_t ldy, int64_t C, int T, float *o, int64_t ldo) {
    const int nch = T >= 256 ? 16 : T >= 64 ? 8 : T >= 16 ? 4 : 1;
    hipLaunchKernelGGL(sq_mingru_kernel, dim3((unsigned)((C + 63) / 64)), dim3(64, nch), 0, st, step, (long long)state_off, y, (long long)ldy, (long long)C, T, o,
                       (long long)ldo);
}
