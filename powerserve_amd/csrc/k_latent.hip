// Latent attention of the layer-list models: what a token leaves behind is its normalised key-value latent c (kv_rank numbers) and one rotated
// key part shared by all heads (rot_dim numbers), kept in a per-sequence RING of `cap` rows (row = position mod cap; cap >= window - 1 + the
// widest step, so a step never overwrites a row one of its own tokens still sees).  Scores, soft-max and the weighted sum are fp32.  cos and sin of the
// rotation may carry a common factor (rot_mag: frequency scaling by wavelength stretches both), and a head's output a sigmoid gate.
//   latent_prep_kernel   norms of the two latents, rotation of the shared key part, ring append
//   latent_attn_kernel   one wave per (token, head) over per-head keys / values expanded from the ring rows of the window (the plain form)
//   latent_attn_mfma_kernel / latent_absorbed_kernel (+ fold, combine, unfold): the matrix-core forms for a portion and for a single token, below
#include "ps_attn_dev.h"
#include "ps_seq.h"

#include <cmath>

static __device__ __forceinline__ float la_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
static __device__ __forceinline__ float la_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}

__global__ __launch_bounds__(256) void latent_prep_kernel(const ps_seq_step *step, long long ring_off, int cap, const float *y, long long ldy, const float *qnorm,
                                                          const float *kvnorm, float eps, int q_rank, int kv_rank, int rot_dim, int rot_dims, const float *freq, float *cq,
                                                          long long ldcq, float rot_mag) {
    __shared__ float red[8];
    const int t = blockIdx.x, tid = threadIdx.x;
    const long long pos = step->pos0 + t;
    const float *yt = y + (long long)t * ldy, *ckv = yt + q_rank, *kr = ckv + kv_rank;
    float *ring = step->state + ring_off + (pos % cap) * (long long)(kv_rank + rot_dim);
    float a = 0.f, b = 0.f;
    for (int i = tid; i < q_rank; i += 256) a += yt[i] * yt[i];
    for (int i = tid; i < kv_rank; i += 256) b += ckv[i] * ckv[i];
    a = la_wave_sum(a);
    b = la_wave_sum(b);
    if ((tid & 63) == 0) { red[tid >> 6] = a; red[4 + (tid >> 6)] = b; }
    __syncthreads();
    const float ia = q_rank > 0 ? 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)q_rank + eps) : 0.f; // (q_rank 0: the queries do not pass a latent)
    const float ib = 1.f / sqrtf((red[4] + red[5] + red[6] + red[7]) / (float)kv_rank + eps);
    for (int i = tid; i < q_rank; i += 256) cq[(long long)t * ldcq + i] = yt[i] * ia * qnorm[i];
    for (int i = tid; i < kv_rank; i += 256) ring[i] = ckv[i] * ib * kvnorm[i];
    const int half = rot_dims / 2; // the first rot_dims of the part are rotated, pairs (i, i + rot_dims / 2); the rest passes unchanged
    for (int i = tid; i < half; i += 256) {
        const float ang = (float)pos * freq[i], c = cosf(ang) * rot_mag, s = sinf(ang) * rot_mag;
        const float u = kr[i], v = kr[i + half];
        ring[kv_rank + i] = u * c - v * s;
        ring[kv_rank + half + i] = v * c + u * s;
    }
    for (int i = 2 * half + tid; i < rot_dim; i += 256) ring[kv_rank + i] = kr[i];
}
void psk_latent_prep(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *y, int64_t ldy, const float *qnorm, const float *kvnorm,
                     float eps, int q_rank, int kv_rank, int rot_dim, int rot_dims, const float *freq, int T, float *cq, int64_t ldcq, float rot_mag) {
    hipLaunchKernelGGL(latent_prep_kernel, dim3(T), dim3(256), 0, st, step, (long long)ring_off, cap, y, (long long)ldy, qnorm, kvnorm, eps, q_rank, kv_rank, rot_dim,
                       rot_dims, freq, cq, (long long)ldcq, rot_mag);
}

// dynamic LDS: qs [d + dr], ps [64]
#define LA_NV 4 // value columns per lane: dv <= 256
__global__ __launch_bounds__(64) void latent_attn_kernel(const ps_seq_step *step, long long ring_off, int cap, const float *q, long long ldq, const float *kv,
                                                         long long ldkv, const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window,
                                                         float scale, float *o, long long ldo, float rot_mag, const float *gate, long long ldg) {
    extern __shared__ float lds[];
    float *qs = lds, *ps = lds + d + dr;
    const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
    const long long pos0 = step->pos0, p = pos0 + t;
    const long long first = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0; // position of kv row 0
    const long long lo = p - window + 1 > 0 ? p - window + 1 : 0;
    const float *qt = q + (long long)t * ldq + (long long)h * (d + dr);
    const int half = rot_dims / 2;
    for (int i = lane; i < d; i += 64) qs[i] = qt[i];
    for (int i = 2 * half + lane; i < dr; i += 64) qs[d + i] = qt[d + i];
    for (int i = lane; i < half; i += 64) {
        const float ang = (float)p * freq[i], c = cosf(ang) * rot_mag, s = sinf(ang) * rot_mag;
        const float u = qt[d + i], v = qt[d + half + i];
        qs[d + i] = u * c - v * s;
        qs[d + half + i] = v * c + u * s;
    }
    __syncthreads();
    const float *ring = step->state + ring_off;
    const long long rs = kv_rank + dr;
    float m = -INFINITY, l = 0.f, acc[LA_NV];
#pragma unroll
    for (int x = 0; x < LA_NV; x++) acc[x] = 0.f;
    for (long long j0 = lo; j0 <= p; j0 += 64) {
        const long long j = j0 + lane;
        float s = -INFINITY;
        if (j <= p) {
            const float *kn = kv + (j - first) * ldkv + (long long)h * d;
            const float *kr = ring + (j % cap) * rs + kv_rank;
            float a = 0.f;
            for (int i = 0; i < d; i++) a = fmaf(qs[i], kn[i], a);
            for (int i = 0; i < dr; i++) a = fmaf(qs[d + i], kr[i], a);
            s = a * scale;
        }
        const float mn = fmaxf(m, la_wave_max(s));
        const float corr = expf(m - mn), pj = j <= p ? expf(s - mn) : 0.f; // (m = -inf in the first round: corr = 0, acc and l are 0)
        l = l * corr + la_wave_sum(pj);
        m = mn;
        __syncthreads();
        ps[lane] = pj;
        __syncthreads();
        const int nk = (int)min((long long)64, p - j0 + 1);
#pragma unroll
        for (int x = 0; x < LA_NV; x++) acc[x] *= corr;
        for (int kk = 0; kk < nk; kk++) {
            const float *vr = kv + (j0 + kk - first) * ldkv + (long long)H * d + (long long)h * dv;
            const float pk = ps[kk];
#pragma unroll
            for (int x = 0; x < LA_NV; x++)
                if (lane + 64 * x < dv) acc[x] = fmaf(pk, vr[lane + 64 * x], acc[x]);
        }
    }
    const float il = (gate ? 1.f / (1.f + expf(-gate[(long long)t * ldg + h])) : 1.f) / l;
#pragma unroll
    for (int x = 0; x < LA_NV; x++)
        if (lane + 64 * x < dv) o[(long long)t * ldo + (long long)h * dv + lane + 64 * x] = acc[x] * il;
}
void psk_latent_attn(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int64_t ldq, const float *kv, int64_t ldkv,
                     const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window, float scale, int T, float *o, int64_t ldo, float rot_mag,
                     const float *gate, int64_t ldg) {
    hipLaunchKernelGGL(latent_attn_kernel, dim3(T, H), dim3(64), (size_t)(d + dr + 64) * 4, st, step, (long long)ring_off, cap, q, (long long)ldq, kv, (long long)ldkv,
                       freq, H, d, dr, rot_dims, dv, kv_rank, window, scale, o, (long long)ldo, rot_mag, gate, (long long)ldg);
}

// ---------------------------------------------------------------------------------------------------- matrix-core form
// One wave attends 16 rows to tiles of 16 keys, fp32 throughout on v_mfma_f32_16x16x4_f32:
//   scores   S[16 x 16] = Q[16 x DK] K^T: the keys come straight from memory as 16-byte pieces (lane (key l % 16, quarter l / 16) holds 4
//            consecutive dimensions; the row operand is read from LDS in the same order, so the sum runs over a permutation of the dimensions)
//   soft-max online, in the accumulator layout (lane holds rows 4 (l / 16) + i of key column l % 16; a row's 16 lanes reduce by butterfly)
//   output   O[16 x DV] += P V: P goes through a 16 x 17 LDS patch into the row-operand layout; V comes as 16-byte pieces of 4 consecutive
//            columns, so accumulator tile jj of a 64-column group holds columns 4 (l % 16) + jj -- undone at the final store.
// A "row" is a (token, head) pair.  Two drivers use it: a prompt's portion over per-head keys / values expanded from the ring (rows = 16
// consecutive tokens of one head), and the single-token step in the ABSORBED form -- rows = heads, every head's query folded through its key
// expansion into latent space (q~_h = W_uk,h^T q_h), keys AND values the ring's latents themselves, the value expansion applied afterwards to
// the attended latent -- where the ring is read once for all heads and nothing is expanded per key.
// a prompt's portion: block = 64 consecutive tokens of one head (a wave per 16), keys / values expanded per head in kv (position first + row)
// dynamic LDS: 4 x (16 x qld + 16 x 17)
template <int NJ>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(const ps_seq_step *step, long long ring_off, int cap, const float *q, long long ldq, const float *kv,
                                                               long long ldkv, const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window,
                                                               float scale, int T, float *o, long long ldo, float rot_mag, const float *gate, long long ldg) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lq = lane >> 4, h = blockIdx.y;
    const int qld = d + dr + 4;
    float *qs = lds + wave * (16 * qld + 16 * 17), *pt = qs + 16 * qld;
    const long long pos0 = step->pos0;
    const int t0 = blockIdx.x * 64 + wave * 16;
    if (t0 >= T) return; // (no block-wide barrier below: waves are on their own)
    const long long first = pos0 - window + 1 > 0 ? pos0 - window + 1 : 0;
    const int half = rot_dims / 2;
    // this wave's 16 query rows into LDS (no index division, one sincos per rotated pair and row)
    for (int r = 0; r < 16; r++) {
        const int t = t0 + r;
        const bool in = t < T;
        const float *qt = q + (long long)(in ? t : 0) * ldq + (long long)h * (d + dr);
        float *qr = qs + r * qld;
        for (int c = lane; c < d; c += 64) qr[c] = in ? qt[c] : 0.f;
        for (int c = 2 * half + lane; c < dr; c += 64) qr[d + c] = in ? qt[d + c] : 0.f;
        for (int i = lane; i < half; i += 64) {
            const float ang = (float)(pos0 + t) * freq[i], cs = cosf(ang) * rot_mag, sn = sinf(ang) * rot_mag;
            const float u = in ? qt[d + i] : 0.f, v = in ? qt[d + half + i] : 0.f;
            qr[d + i] = u * cs - v * sn;
            qr[d + half + i] = v * cs + u * sn;
        }
    }
    __builtin_amdgcn_wave_barrier();
    const la_src k1 = {kv + (long long)h * d, ldkv, first, 0};
    const la_src k2 = {step->state + ring_off + kv_rank, (long long)(kv_rank + dr), 0, cap};
    const la_src vs = {kv + (long long)H * d + (long long)h * dv, ldkv, first, 0};
    long long rowlo[4], rowhi[4];
    float m[4], l[4];
    la_f4 acc[NJ];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const long long rp = pos0 + t0 + 4 * lq + i;
        const bool in = t0 + 4 * lq + i < T;
        rowlo[i] = in && rp - window + 1 > 0 ? rp - window + 1 : 0;
        rowhi[i] = in ? rp + 1 : 0;
        m[i] = -INFINITY; l[i] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[j] = la_f4{0.f, 0.f, 0.f, 0.f};
    const long long plast = pos0 + (t0 + 15 < T ? t0 + 15 : T - 1), pfirst = pos0 + t0;
    const long long lo = pfirst - window + 1 > 0 ? pfirst - window + 1 : 0;
    for (long long j0 = lo; j0 <= plast; j0 += 16) la_tile<NJ>(qs, qld, pt, k1, k2, vs, d, dr, dv, j0, plast + 1, rowlo, rowhi, scale, m, l, acc);
#pragma unroll
    for (int J = 0; J < NJ / 4; J++)
#pragma unroll
        for (int i = 0; i < 4; i++) { // a lane's four tiles of a 64-column group are four consecutive columns: one 16-byte store
            const int t = t0 + 4 * lq + i, c = 64 * J + 4 * lr;
            if (t < T && c < dv) {
                const float il = (gate ? 1.f / (1.f + expf(-gate[(long long)t * ldg + h])) : 1.f) / l[i];
                *(la_f4 *)(o + (long long)t * ldo + (long long)h * dv + c) = la_f4{acc[4 * J][i] * il, acc[4 * J + 1][i] * il, acc[4 * J + 2][i] * il, acc[4 * J + 3][i] * il};
            }
        }
}

bool psk_latent_attn_mfma_ok(int d, int dr, int dv) { return d % 16 == 0 && dr % 16 == 0 && dv % 4 == 0 && dv <= 128 && (size_t)4 * (16 * (d + dr + 4) + 16 * 17) * 4 <= 160 * 1024; }
void psk_latent_attn_mfma(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int64_t ldq, const float *kv, int64_t ldkv,
                          const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window, float scale, int T, float *o, int64_t ldo, float rot_mag,
                          const float *gate, int64_t ldg) {
    const size_t lds = (size_t)4 * (16 * (d + dr + 4) + 16 * 17) * 4;
    static unsigned long long mask = 0;
    if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)latent_attn_mfma_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipLaunchKernelGGL(latent_attn_mfma_kernel<8>, dim3((T + 63) / 64, H), dim3(256), lds, st, step, (long long)ring_off, cap, q, (long long)ldq, kv, (long long)ldkv, freq,
                       H, d, dr, rot_dims, dv, kv_rank, window, scale, T, o, (long long)ldo, rot_mag, gate, (long long)ldg);
}

// ---------------------------------------------------------------------------------------------------- single token, absorbed
// qa[h][r] = sum_i q[h][i] Wuk[h * d + i][r]: a head's query folded into latent space.  One block per head, a thread per latent index.
template <typename WT>
__global__ __launch_bounds__(256) void latent_fold_q_kernel(const float *q, int qstride, const WT *wuk, int d, int R, float *qa) {
    __shared__ float part[4][64];
    const int h = blockIdx.x, r = blockIdx.y * 64 + (threadIdx.x & 63), grp = threadIdx.x >> 6; // block: 64 latent indices x 4 slices of the head's rows
    const float *qh = q + (long long)h * qstride;
    float a = 0.f;
    if (r < R) {
#pragma unroll 8
        for (int i = grp; i < d; i += 4) {
            float w;
            if constexpr (sizeof(WT) == 2) w = __uint_as_float((unsigned)wuk[((long long)h * d + i) * R + r] << 16);
            else w = wuk[((long long)h * d + i) * R + r];
            a = fmaf(qh[i], w, a);
        }
    }
    part[grp][threadIdx.x & 63] = a;
    __syncthreads();
    if (grp == 0 && r < R) qa[(long long)h * R + r] = part[0][threadIdx.x] + part[1][threadIdx.x] + part[2][threadIdx.x] + part[3][threadIdx.x];
}
// o[h][x] = sum_r Wuv[h * dv + x][r] ol[h][r]: the value expansion of the attended latent.  A wave per output row.
template <typename WT>
__global__ __launch_bounds__(256) void latent_unfold_v_kernel(const float *ol, const WT *wuv, int dv, int R, int rows, float *o, const float *gate) {
    const int row = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (row >= rows) return;
    const float *x = ol + (long long)(row / dv) * R;
    float a = 0.f;
    for (int r = lane; r < R; r += 64) {
        float w;
        if constexpr (sizeof(WT) == 2) w = __uint_as_float((unsigned)wuv[(long long)row * R + r] << 16);
        else w = wuv[(long long)row * R + r];
        a = fmaf(w, x[r], a);
    }
    a = la_wave_sum(a);
    if (lane == 0) o[row] = gate ? a / (1.f + expf(-gate[row / dv])) : a; // (the head's output gate)
}

// rows = heads (16 per block), keys = ring rows; wave w of block (split s, head tile) takes key tile 4 s + w of the window.  Partials:
// per (key tile, head) R unnormalised outputs, then m and l.  dynamic LDS: 16 x qld + 4 x 16 x 17
template <int NJ>
__global__ __launch_bounds__(256) void latent_absorbed_kernel(const ps_seq_step *step, long long ring_off, int cap, const float *qa, const float *q, int qstride, int d,
                                                              int dr, int rot_dims, const float *freq, int H, int R, int window, float scale, float *part, float rot_mag) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lq = lane >> 4, h0 = blockIdx.y * 16;
    const int qld = R + dr + 4;
    float *qs = lds, *pt = lds + 16 * qld + wave * 16 * 17;
    const long long p = step->pos0;
    const long long lo = p - window + 1 > 0 ? p - window + 1 : 0;
    const int half = rot_dims / 2;
    // the 16 heads' folded queries and rotated parts into LDS: wave w takes rows w, w + 4, ...; every head turns by the same angles
    for (int r = wave; r < 16; r += 4) {
        const int h = h0 + r;
        float *qr = qs + r * qld;
        for (int c = lane; c < R; c += 64) qr[c] = h < H ? qa[(long long)h * R + c] : 0.f;
        for (int c = 2 * half + lane; c < dr; c += 64) qr[R + c] = h < H ? q[(long long)h * qstride + d + c] : 0.f;
    }
    for (int i = lane; i < half; i += 64) {
        const float ang = (float)p * freq[i], cs = cosf(ang) * rot_mag, sn = sinf(ang) * rot_mag;
        for (int r = wave; r < 16; r += 4) {
            const int h = h0 + r;
            const float *qt = q + (long long)(h < H ? h : 0) * qstride + d;
            const float u = h < H ? qt[i] : 0.f, v = h < H ? qt[half + i] : 0.f;
            qs[r * qld + R + i] = u * cs - v * sn;
            qs[r * qld + R + half + i] = v * cs + u * sn;
        }
    }
    __syncthreads();
    const long long tile = (long long)blockIdx.x * 4 + wave, j0 = lo + tile * 16;
    const float *ring = step->state + ring_off;
    const la_src k1 = {ring, (long long)(R + dr), 0, cap}, k2 = {ring + R, (long long)(R + dr), 0, cap};
    long long rowlo[4], rowhi[4];
    float m[4], l[4];
    la_f4 acc[NJ];
#pragma unroll
    for (int i = 0; i < 4; i++) { rowlo[i] = h0 + 4 * lq + i < H ? lo : 0; rowhi[i] = h0 + 4 * lq + i < H ? p + 1 : 0; m[i] = -INFINITY; l[i] = 0.f; }
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[j] = la_f4{0.f, 0.f, 0.f, 0.f};
    if (j0 <= p) la_tile<NJ>(qs, qld, pt, k1, k2, k1, R, dr, R, j0, p + 1, rowlo, rowhi, scale, m, l, acc);
    // partial of (tile, head): [o[R], m, l, -, -] (rows of R + 4 floats: 16-byte stores)
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int h = h0 + 4 * lq + i;
        if (h >= H) continue;
        float *pp = part + ((long long)tile * H + h) * (R + 4);
        if (lr == 0) { pp[R] = m[i]; pp[R + 1] = l[i]; }
#pragma unroll
        for (int J = 0; J < NJ / 4; J++) {
            const int c = 64 * J + 4 * lr;
            if (c < R) *(la_f4 *)(pp + c) = la_f4{acc[4 * J][i], acc[4 * J + 1][i], acc[4 * J + 2][i], acc[4 * J + 3][i]};
        }
    }
}
// ol[h][c] = sum_tiles exp(m_t - M) o_t[c] / sum_tiles exp(m_t - M) l_t
__global__ __launch_bounds__(256) void latent_combine_kernel(const ps_seq_step *step, const float *part, int H, int R, int window, int max_tiles, float *ol) {
    extern __shared__ float wts[]; // [max_tiles] weights exp(m_t - M), then their l-weighted sum in red
    __shared__ float red[4];
    const int h = blockIdx.x, tid = threadIdx.x;
    const long long p = step->pos0, lo = p - window + 1 > 0 ? p - window + 1 : 0;
    int nt = (int)((p - lo) / 16 + 1);
    if (nt > max_tiles) nt = max_tiles;
    float mx = -INFINITY;
    for (int t = tid; t < nt; t += 256) mx = fmaxf(mx, part[((long long)t * H + h) * (R + 4) + R]);
    mx = la_wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float ls = 0.f;
    for (int t = tid; t < nt; t += 256) {
        const float *pp = part + ((long long)t * H + h) * (R + 4) + R;
        const float w = pp[0] == -INFINITY ? 0.f : expf(pp[0] - M);
        wts[t] = w;
        ls = fmaf(w, pp[1], ls);
    }
    ls = la_wave_sum(ls);
    if ((tid & 63) == 0) red[tid >> 6] = ls;
    __syncthreads();
    const float L = red[0] + red[1] + red[2] + red[3];
    for (int c = tid; c < R; c += 256) {
        float a = 0.f;
#pragma unroll 8
        for (int t = 0; t < nt; t++) a = fmaf(wts[t], part[((long long)t * H + h) * (R + 4) + c], a);
        ol[(long long)h * R + c] = a / L;
    }
}

bool psk_latent_absorbed_ok(int d, int dr, int dv, int R) { return R % 16 == 0 && dr % 16 == 0 && R <= 512 && (size_t)(16 * (R + dr + 4) + 4 * 16 * 17) * 4 <= 160 * 1024; }
size_t psk_latent_absorbed_scratch(int H, int R, int window) { return ((size_t)((window + 15) / 16 + 4) * H * (R + 4) + (size_t)2 * H * R) * 4; }
// q [H][d + dr] (row stride qstride) -> o [H * dv]; ukv: rows uk | uv of the expansion matrix [H d + H dv][R]; scratch from psk_latent_absorbed_scratch
void psk_latent_absorbed(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int qstride, const ps_dense *ukv, const float *freq,
                         int H, int d, int dr, int rot_dims, int dv, int R, int window, float scale, float *scratch, float *o, float rot_mag, const float *gate) {
    const int max_tiles = (window + 15) / 16 + 1; // (a window that does not start on a tile's edge touches one tile more)
    float *qa = scratch, *ol = qa + (size_t)H * R, *part = ol + (size_t)H * R;
    const bool bf = ukv->dtype == PS_BF16;
    if (bf) hipLaunchKernelGGL(latent_fold_q_kernel<unsigned short>, dim3(H, (R + 63) / 64), dim3(256), 0, st, q, qstride, (const unsigned short *)ukv->data, d, R, qa);
    else hipLaunchKernelGGL(latent_fold_q_kernel<float>, dim3(H, (R + 63) / 64), dim3(256), 0, st, q, qstride, (const float *)ukv->data, d, R, qa);
    const size_t lds = (size_t)(16 * (R + dr + 4) + 4 * 16 * 17) * 4;
    const dim3 grid((max_tiles + 3) / 4, (H + 15) / 16);
    if (R <= 128) {
        static unsigned long long mask = 0;
        if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)latent_absorbed_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        hipLaunchKernelGGL(latent_absorbed_kernel<8>, grid, dim3(256), lds, st, step, (long long)ring_off, cap, qa, q, qstride, d, dr, rot_dims, freq, H, R, window, scale, part, rot_mag);
    } else {
        static unsigned long long mask = 0;
        if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)latent_absorbed_kernel<32>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
        hipLaunchKernelGGL(latent_absorbed_kernel<32>, grid, dim3(256), lds, st, step, (long long)ring_off, cap, qa, q, qstride, d, dr, rot_dims, freq, H, R, window, scale, part, rot_mag);
    }
    hipLaunchKernelGGL(latent_combine_kernel, dim3(H), dim3(256), (size_t)grid.x * 4 * 4, st, step, part, H, R, window, (int)grid.x * 4, ol);
    const int rows = H * dv;
    if (bf) hipLaunchKernelGGL(latent_unfold_v_kernel<unsigned short>, dim3((rows + 3) / 4), dim3(256), 0, st, ol, (const unsigned short *)ukv->data + (size_t)H * d * R, dv, R, rows, o, gate);
    else hipLaunchKernelGGL(latent_unfold_v_kernel<float>, dim3((rows + 3) / 4), dim3(256), 0, st, ol, (const float *)ukv->data + (size_t)H * d * R, dv, R, rows, o, gate);
}
