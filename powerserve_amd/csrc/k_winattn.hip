// Windowed attention with pooled blocks of the layer-list models (PS_MIX_WINATTN): grouped-query soft-max attention in which a token at
// position p sees the `window` positions up to itself and, beside them, ONE key and value for every block of `pool` consecutive positions that
// lies wholly before that window (the means of the block's keys / values as the ring holds them); a per-head sink adds exp(sink) to the
// denominator, a per-head temperature multiplies the scores, a sigmoid gate (per head, or element by element) the output; the q / k norms are taken over
// the whole projection or per head, and a head's value may be made a unit-rms vector as it is cached.  What a sequence keeps: a RING of the last
// `cap` tokens' keys and values (row = position mod cap; cap >= window - 1 + the widest step) and the block means, one row per block, which
// grow with the sequence.  Scores, soft-max and the weighted sums are fp32.
//   winattn_prep_kernel    norms over the whole q / k projections, rotation, ring append            (one or a few blocks per token)
//   winattn_pool_kernel    block sums in position order, turned into means when a block is complete  (a thread per channel and block)
//   winattn_kernel         one wave per (token, head) over [visible blocks | window]: the plain form, any size
//   winattn_mfma_kernel    a portion on the fp32 matrix cores, 16 tokens of a head per wave (ps_attn_dev.h)
//   winattn_step_kernel + winattn_merge_kernel   a single token: rows = the heads that share a key / value group, a key tile per wave
#include "ps_attn_dev.h"
#include "ps_seq.h"

#include <algorithm>
#include <cmath>

static __device__ __forceinline__ float wa_wave_sum(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
    return v;
}
static __device__ __forceinline__ float wa_wave_max(float v) {
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
    return v;
}
// blocks of `pool` positions wholly before the window of a query at p: block b is seen when b pool + pool - 1 <= p - window
static __device__ __forceinline__ long long wa_blocks(long long p, int window, int pool) {
    const long long n = p - window + 1;
    return (pool > 0 && n > 0) ? n / pool : 0;
}

// y[t] = [ q (H d) | k (G d) | v (G dv) | ... ].  q -> qo[t] normed and rotated; k (normed, rotated) and v -> ring row pos mod cap: [G d | G dv].
// A step of ONE token also brings its block's sum up to date here (the thread that wrote a channel adds it: the same sum, in the same order, as
// winattn_pool_kernel makes for a portion).  dynamic LDS: rot_dims floats (cos | sin of the token's angles, shared by all heads).
__global__ __launch_bounds__(256) void winattn_prep_kernel(const ps_seq_step *step, long long ring_off, int cap, long long pool_off, int pool, const float *y,
                                                           long long ldy, const float *qnorm, const float *knorm, float eps, int H, int G, int d, int dv, int rot_dims,
                                                           int pairing, const float *freq, float *qo, long long ldq, float qt_coef, int qt_every, int head_norm,
                                                           int v_unit) {
    extern __shared__ float cs[];
    __shared__ float red[8];
    const int t = blockIdx.x, tid = threadIdx.x;
    const long long pos = step->pos0 + t;
    const int nq = H * d, nk = G * d, nv = G * dv, half = rot_dims / 2;
    const float *qt = y + (long long)t * ldy, *kt = qt + nq, *vt = kt + nk;
    float *ring = step->state + ring_off + (pos % cap) * (long long)(nk + nv);
    // a query temperature that grows with the position in steps of qt_every tokens: 1 + coef ln(floor((pos + 1) / every) + 1)
    const float qtemp = qt_every > 0 ? 1.f + qt_coef * logf((float)((pos + 1) / qt_every) + 1.f) : 1.f;
    for (int i = tid; i < half; i += 256) {
        const float ang = (float)pos * freq[i];
        cs[i] = cosf(ang);
        cs[half + i] = sinf(ang);
    }
    float a = 0.f, b = 0.f;
    if (qnorm && !head_norm) for (int i = tid; i < nq; i += 256) a += qt[i] * qt[i];
    if (knorm && !head_norm) for (int i = tid; i < nk; i += 256) b += kt[i] * kt[i];
    a = wa_wave_sum(a);
    b = wa_wave_sum(b);
    if ((tid & 63) == 0) { red[tid >> 6] = a; red[4 + (tid >> 6)] = b; }
    __syncthreads();
    const float ia = qnorm && !head_norm ? 1.f / sqrtf((red[0] + red[1] + red[2] + red[3]) / (float)nq + eps) : 1.f;
    const float ib = knorm && !head_norm ? 1.f / sqrtf((red[4] + red[5] + red[6] + red[7]) / (float)nk + eps) : 1.f;
    // element i of a projection (c = its index in its head): normed, and where c < rot_dims turned together with its partner; wc: 1 = one weight vector of d
    // numbers for every head (indexed by c), 0 = a weight per element of the projection
    auto turned = [&](const float *src, const float *w, float inv, int i, int wc) {
        const int c = i % d;
        if (w && wc) w += c - i;
        const float self = src[i] * inv * (w ? w[i] : 1.f);
        if (c >= 2 * half) return self;
        int partner, pair;
        bool first;
        if (pairing == PS_ROT_NEIGHBOURS) { partner = i - c + (c ^ 1); pair = c >> 1; first = !(c & 1); }
        else { first = c < half; partner = first ? i + half : i - half; pair = first ? c : c - half; }
        const float other = src[partner] * inv * (w ? w[partner] : 1.f);
        return first ? self * cs[pair] - other * cs[half + pair] : self * cs[pair] + other * cs[half + pair];
    };
    // the block of a single token: its sum so far (nothing before the block's first position), the mean once the block is complete
    const bool own_pool = pool > 0 && gridDim.x == 1;
    const long long pb = own_pool ? pos / pool : 0;
    float *mean = step->state + pool_off + pb * (long long)(nk + nv);
    auto pooled = [&](int c, float v) {
        if (!own_pool) return;
        const float sum = (pos == pb * pool ? 0.f : mean[c]) + v;
        mean[c] = pos == pb * pool + pool - 1 ? sum / (float)pool : sum;
    };
    if (head_norm || v_unit) {
        // statistics per head: a WAVE per head (the heads of q, then k, then v, dealt over the token's blocks and their waves) sums, norms, turns and stores it
        const int lane = tid & 63;
        for (int hd = blockIdx.y * 4 + (tid >> 6); hd < H + 2 * G; hd += 4 * gridDim.y) {
            const bool isq = hd < H, isk = !isq && hd < H + G;
            const int n = isq || isk ? d : dv, e0 = isq ? hd * d : isk ? (hd - H) * d : (hd - H - G) * dv; // (e0: the head's first element in its projection)
            const float *src = isq ? qt : isk ? kt : vt, *w = isq ? qnorm : isk ? knorm : nullptr;
            const bool own = isq || isk ? head_norm && w : v_unit != 0;
            float ss = 0.f;
            if (own) for (int c = lane; c < n; c += 64) ss += src[e0 + c] * src[e0 + c];
            ss = wa_wave_sum(ss);
            const float inv = own ? 1.f / sqrtf(ss / (float)n + eps) : isq ? ia : isk ? ib : 1.f;
            for (int c = lane; c < n; c += 64) {
                if (isq) { qo[(long long)t * ldq + e0 + c] = turned(qt, qnorm, inv, e0 + c, head_norm) * qtemp; continue; }
                const float v = isk ? turned(kt, knorm, inv, e0 + c, head_norm) : vt[e0 + c] * inv;
                const int i = isk ? e0 + c : nk + e0 + c;
                ring[i] = v;
                pooled(i, v);
            }
        }
        return;
    }
    // the elements of q | k | v are spread over the blocks of a token (gridDim.y; every block has made the sums above for itself)
    for (int e = blockIdx.y * 256 + tid; e < nq + nk + nv; e += 256 * gridDim.y) {
        if (e < nq) {
            qo[(long long)t * ldq + e] = turned(qt, qnorm, ia, e, 0) * qtemp;
        } else {
            const int i = e - nq;
            const float v = i < nk ? turned(kt, knorm, ib, i, 0) : vt[i - nk];
            ring[i] = v;
            pooled(i, v);
        }
    }
}

// Block sums of the ring rows this step appended, in position order (so the result does not depend on how the tokens were cut into steps); a
// block that the step completes is stored as its mean.  A block whose first position the step brings starts from zero: nothing is cleared.
__global__ __launch_bounds__(256) void winattn_pool_kernel(const ps_seq_step *step, long long ring_off, int cap, long long pool_off, int pool, int rs) {
    const int c = blockIdx.x * 256 + threadIdx.x;
    if (c >= rs) return;
    const long long pos0 = step->pos0, end = pos0 + step->n, b = pos0 / pool + blockIdx.y, pb = b * pool;
    const long long from = pb > pos0 ? pb : pos0, to = pb + pool < end ? pb + pool : end;
    if (from >= to) return;
    const float *ring = step->state + ring_off;
    float *mean = step->state + pool_off + b * rs;
    float s = from == pb ? 0.f : mean[c];
    for (long long p = from; p < to; p++) s += ring[(p % cap) * rs + c];
    mean[c] = to == pb + pool ? s / (float)pool : s;
}

void psk_winattn_prep(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *y, int64_t ldy, const float *qnorm,
                      const float *knorm, float eps, int H, int G, int d, int dv, int rot_dims, int pairing, const float *freq, int T, float *q, int64_t ldq, float qt_coef,
                      int qt_every, int head_norm, int v_unit) {
    const int total = H * d + G * (d + dv);
    // few tokens: a token's elements over several blocks; with statistics per head, its heads (four per block)
    const int split = head_norm || v_unit ? (T >= 64 ? std::min(2, (H + 2 * G + 3) / 4) : std::min(32, (H + 2 * G + 3) / 4)) : T >= 64 ? 1 : std::min(16, (total + 511) / 512);
    hipLaunchKernelGGL(winattn_prep_kernel, dim3(T, split), dim3(256), (size_t)(rot_dims + 2) * 4, st, step, (long long)ring_off, cap, (long long)pool_off, pool, y,
                       (long long)ldy, qnorm, knorm, eps, H, G, d, dv, rot_dims, pairing, freq, q, (long long)ldq, qt_coef, qt_every, head_norm, v_unit);
    if (pool > 0 && T > 1) {
        const int rs = G * (d + dv);
        hipLaunchKernelGGL(winattn_pool_kernel, dim3((rs + 255) / 256, (T - 1) / pool + 2), dim3(256), 0, st, step, (long long)ring_off, cap, (long long)pool_off, pool, rs);
    }
}

// the sink joins a finished online soft-max (m running maximum, l denominator): returns the factor for the accumulated values
static __device__ __forceinline__ float wa_finish(float m, float l, const float *sink, int h) {
    if (!sink) return 1.f / l;
    const float sk = sink[h], M = fmaxf(m, sk), c = expf(m - M); // (m = -inf cannot happen: a token sees itself)
    return c / (l * c + expf(sk - M));
}
static __device__ __forceinline__ float wa_sigmoid(float x) { return 1.f / (1.f + expf(-x)); }

// dynamic LDS: qs [d], ps [64].  Keys in one index space: [visible blocks | window tokens].
#define WA_NV 4 // value columns per lane: dv <= 256
__global__ __launch_bounds__(64) void winattn_kernel(const ps_seq_step *step, long long ring_off, int cap, long long pool_off, int pool, const float *q, long long ldq,
                                                     const float *gate, long long ldg, const float *temp, const float *sink, int H, int G, int d, int dv, int window,
                                                     float scale, float *o, long long ldo, float softcap, int gate_elem) {
    extern __shared__ float lds[];
    float *qs = lds, *ps = lds + d;
    const int t = blockIdx.x, h = blockIdx.y, g = h / (H / G), lane = threadIdx.x;
    const long long p = step->pos0 + t, lo = p - window + 1 > 0 ? p - window + 1 : 0, nb = wa_blocks(p, window, pool), nkeys = nb + (p - lo + 1);
    const float *qt = q + (long long)t * ldq + (long long)h * d;
    for (int i = lane; i < d; i += 64) qs[i] = qt[i];
    __syncthreads();
    const long long rs = (long long)G * (d + dv);
    const float *ring = step->state + ring_off, *means = step->state + pool_off;
    auto row = [&](long long n) { return n < nb ? means + n * rs : ring + ((lo + n - nb) % cap) * rs; };
    const float sc = scale * (temp ? temp[h] : 1.f);
    float m = -INFINITY, l = 0.f, acc[WA_NV];
#pragma unroll
    for (int x = 0; x < WA_NV; x++) acc[x] = 0.f;
    for (long long n0 = 0; n0 < nkeys; n0 += 64) {
        const long long n = n0 + lane;
        float s = -INFINITY;
        if (n < nkeys) {
            const float *kn = row(n) + (long long)g * d;
            float a = 0.f;
            for (int i = 0; i < d; i++) a = fmaf(qs[i], kn[i], a);
            s = a * sc;
            if (softcap > 0.f) s = softcap * tanhf(s / softcap);
        }
        const float mn = fmaxf(m, wa_wave_max(s));
        const float corr = expf(m - mn), pj = n < nkeys ? expf(s - mn) : 0.f;
        l = l * corr + wa_wave_sum(pj);
        m = mn;
        __syncthreads();
        ps[lane] = pj;
        __syncthreads();
        const int nk = (int)min((long long)64, nkeys - n0);
#pragma unroll
        for (int x = 0; x < WA_NV; x++) acc[x] *= corr;
        for (int kk = 0; kk < nk; kk++) {
            const float *vr = row(n0 + kk) + (long long)G * d + (long long)g * dv;
            const float pk = ps[kk];
#pragma unroll
            for (int x = 0; x < WA_NV; x++)
                if (lane + 64 * x < dv) acc[x] = fmaf(pk, vr[lane + 64 * x], acc[x]);
        }
    }
    const float f = wa_finish(m, l, sink, h) * (gate && !gate_elem ? wa_sigmoid(gate[(long long)t * ldg + h]) : 1.f);
#pragma unroll
    for (int x = 0; x < WA_NV; x++)
        if (lane + 64 * x < dv) {
            const long long c = (long long)h * dv + lane + 64 * x;
            o[(long long)t * ldo + c] = acc[x] * f * (gate && gate_elem ? wa_sigmoid(gate[(long long)t * ldg + c]) : 1.f);
        }
}
void psk_winattn(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *q, int64_t ldq, const float *gate,
                 int64_t ldg, const float *temp, const float *sink, int H, int G, int d, int dv, int window, float scale, int T, float *o, int64_t ldo, float softcap,
                 int gate_elem) {
    hipLaunchKernelGGL(winattn_kernel, dim3(T, H), dim3(64), (size_t)(d + 64) * 4, st, step, (long long)ring_off, cap, (long long)pool_off, pool, q, (long long)ldq, gate,
                       (long long)ldg, temp, sink, H, G, d, dv, window, scale, o, (long long)ldo, softcap, gate_elem);
}

// ---------------------------------------------------------------------------------------------------- matrix-core forms (ps_attn_dev.h)
// A portion: block = 64 consecutive tokens of one head (a wave per 16).  The visible block means first (key index = block), then the window's ring rows
// (key index = position), one online soft-max over both.  dynamic LDS: 4 x (16 x (d + 4) + 16 x 17)
template <int NJ>
__global__ __launch_bounds__(256) void winattn_mfma_kernel(const ps_seq_step *step, long long ring_off, int cap, long long pool_off, int pool, const float *q, long long ldq,
                                                           const float *gate, long long ldg, const float *temp, const float *sink, int H, int G, int d, int dv, int window,
                                                           float scale, int T, float *o, long long ldo, float softcap, int gate_elem) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lq = lane >> 4, h = blockIdx.y, g = h / (H / G);
    const int qld = d + 4;
    float *qs = lds + wave * (16 * qld + 16 * 17), *pt = qs + 16 * qld;
    const long long pos0 = step->pos0;
    const int t0 = blockIdx.x * 64 + wave * 16;
    if (t0 >= T) return; // (no block-wide barrier below: waves are on their own)
    for (int r = 0; r < 16; r++) {
        const int t = t0 + r;
        const float *qt = q + (long long)(t < T ? t : 0) * ldq + (long long)h * d;
        for (int c = lane; c < d; c += 64) qs[r * qld + c] = t < T ? qt[c] : 0.f;
    }
    __builtin_amdgcn_wave_barrier();
    const long long rs = (long long)G * (d + dv);
    const float *ring = step->state + ring_off, *means = step->state + pool_off;
    const float sc = scale * (temp ? temp[h] : 1.f);
    long long rowlo[4], rowhi[4], blo[4], bhi[4];
    float m[4], l[4];
    la_f4 acc[NJ];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const long long rp = pos0 + t0 + 4 * lq + i;
        const bool in = t0 + 4 * lq + i < T;
        rowlo[i] = in && rp - window + 1 > 0 ? rp - window + 1 : 0;
        rowhi[i] = in ? rp + 1 : 0;
        blo[i] = 0;
        bhi[i] = in ? wa_blocks(rp, window, pool) : 0;
        m[i] = -INFINITY; l[i] = 0.f;
    }
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[j] = la_f4{0.f, 0.f, 0.f, 0.f};
    const long long plast = pos0 + (t0 + 15 < T ? t0 + 15 : T - 1), pfirst = pos0 + t0;
    const long long nbmax = wa_blocks(plast, window, pool);
    {
        const la_src k1 = {means + (long long)g * d, rs, 0, 0}, vs = {means + (long long)G * d + (long long)g * dv, rs, 0, 0};
        for (long long j0 = 0; j0 < nbmax; j0 += 16) la_tile<NJ>(qs, qld, pt, k1, k1, vs, d, 0, dv, j0, nbmax, blo, bhi, sc, m, l, acc, softcap);
    }
    {
        const la_src k1 = {ring + (long long)g * d, rs, 0, cap}, vs = {ring + (long long)G * d + (long long)g * dv, rs, 0, cap};
        const long long lo = pfirst - window + 1 > 0 ? pfirst - window + 1 : 0;
        for (long long j0 = lo; j0 <= plast; j0 += 16) la_tile<NJ>(qs, qld, pt, k1, k1, vs, d, 0, dv, j0, plast + 1, rowlo, rowhi, sc, m, l, acc, softcap);
    }
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int t = t0 + 4 * lq + i;
        if (t >= T) continue;
        const float f = wa_finish(m[i], l[i], sink, h) * (gate && !gate_elem ? wa_sigmoid(gate[(long long)t * ldg + h]) : 1.f);
#pragma unroll
        for (int J = 0; J < NJ / 4; J++) { // a lane's four tiles of a 64-column group are four consecutive columns: one 16-byte store
            const int c = 64 * J + 4 * lr;
            if (c >= dv) continue;
            la_f4 r = la_f4{acc[4 * J][i] * f, acc[4 * J + 1][i] * f, acc[4 * J + 2][i] * f, acc[4 * J + 3][i] * f};
            if (gate && gate_elem) {
                const float *gp = gate + (long long)t * ldg + (long long)h * dv + c;
#pragma unroll
                for (int e = 0; e < 4; e++) r[e] *= wa_sigmoid(gp[e]);
            }
            *(la_f4 *)(o + (long long)t * ldo + (long long)h * dv + c) = r;
        }
    }
}

static size_t wa_mfma_lds(int d) { return (size_t)4 * (16 * (d + 4) + 16 * 17) * 4; }
// the sizes the matrix-core forms take: 16-byte pieces of keys (d a multiple of 16) and values (dv of 4, at most 128 columns per head)
bool psk_winattn_mfma_ok(int d, int dv) { return d % 16 == 0 && dv % 4 == 0 && dv <= 128 && wa_mfma_lds(d) <= 160 * 1024; }
void psk_winattn_mfma(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *q, int64_t ldq, const float *gate,
                      int64_t ldg, const float *temp, const float *sink, int H, int G, int d, int dv, int window, float scale, int T, float *o, int64_t ldo, float softcap,
                      int gate_elem) {
    static unsigned long long mask = 0;
    if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)winattn_mfma_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    hipLaunchKernelGGL(winattn_mfma_kernel<8>, dim3((T + 63) / 64, H), dim3(256), wa_mfma_lds(d), st, step, (long long)ring_off, cap, (long long)pool_off, pool, q,
                       (long long)ldq, gate, (long long)ldg, temp, sink, H, G, d, dv, window, scale, T, o, (long long)ldo, softcap, gate_elem);
}

// A single token.  Rows = the heads that share key / value group g (16 per block); the keys are cut into tiles of 16 in one index space -- tiles
// 0 .. nbt - 1 the visible block means, then the window from its first position -- and wave w of block (x, head tile, g) takes tile 4 x + w.
// Partials per (tile, head): [o[dv] unnormalised, m, l, -, -], merged by winattn_merge_kernel, where the sink and the gate come in.
// dynamic LDS: 16 x (d + 4) + 4 x 16 x 17
template <int NJ>
__global__ __launch_bounds__(256) void winattn_step_kernel(const ps_seq_step *step, long long ring_off, int cap, long long pool_off, int pool, const float *q,
                                                           const float *temp, int H, int G, int d, int dv, int window, float scale, float *part, float softcap) {
    extern __shared__ __attribute__((aligned(16))) float lds[];
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63, lr = lane & 15, lq = lane >> 4, g = blockIdx.z, hpg = H / G, r0 = blockIdx.y * 16;
    const int qld = d + 4;
    float *qs = lds, *pt = lds + 16 * qld + wave * 16 * 17;
    const long long p = step->pos0, lo = p - window + 1 > 0 ? p - window + 1 : 0, nb = wa_blocks(p, window, pool), nbt = (nb + 15) / 16;
    const long long tile = (long long)blockIdx.x * 4 + wave, ntiles = nbt + (p - lo) / 16 + 1;
    // the group's 16 queries into LDS, each already times its head's temperature (the scores of a tile then share one scale)
    for (int r = wave; r < 16; r += 4) {
        const int hh = r0 + r, h = g * hpg + hh;
        const float tp = hh < hpg && temp ? temp[h] : 1.f;
        for (int c = lane; c < d; c += 64) qs[r * qld + c] = hh < hpg ? q[(long long)h * d + c] * tp : 0.f;
    }
    __syncthreads();
    if (tile >= ntiles) return;
    const long long rs = (long long)G * (d + dv);
    const float *base = tile < nbt ? step->state + pool_off : step->state + ring_off;
    const la_src k1 = {base + (long long)g * d, rs, 0, tile < nbt ? 0 : (long long)cap}, vs = {base + (long long)G * d + (long long)g * dv, rs, 0, tile < nbt ? 0 : (long long)cap};
    const long long j0 = tile < nbt ? tile * 16 : lo + (tile - nbt) * 16, jend = tile < nbt ? nb : p + 1;
    long long rowlo[4], rowhi[4];
    float m[4], l[4];
    la_f4 acc[NJ];
#pragma unroll
    for (int i = 0; i < 4; i++) { const bool in = r0 + 4 * lq + i < hpg; rowlo[i] = 0; rowhi[i] = in ? jend : 0; m[i] = -INFINITY; l[i] = 0.f; }
#pragma unroll
    for (int j = 0; j < NJ; j++) acc[j] = la_f4{0.f, 0.f, 0.f, 0.f};
    la_tile<NJ>(qs, qld, pt, k1, k1, vs, d, 0, dv, j0, jend, rowlo, rowhi, scale, m, l, acc, softcap);
    const int dvp = dv + 4;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int hh = r0 + 4 * lq + i;
        if (hh >= hpg) continue;
        float *pp = part + (tile * H + g * hpg + hh) * dvp;
        if (lr == 0) { pp[dv] = m[i]; pp[dv + 1] = l[i]; }
#pragma unroll
        for (int J = 0; J < NJ / 4; J++) {
            const int c = 64 * J + 4 * lr;
            if (c < dv) *(la_f4 *)(pp + c) = la_f4{acc[4 * J][i], acc[4 * J + 1][i], acc[4 * J + 2][i], acc[4 * J + 3][i]};
        }
    }
}
// o[h][c] = gate_h * sum_tiles exp(m_t - M) o_t[c] / (sum_tiles exp(m_t - M) l_t + exp(sink_h - M)),  M = max(max_t m_t, sink_h)
__global__ __launch_bounds__(256) void winattn_merge_kernel(const ps_seq_step *step, const float *part, const float *gate, const float *sink, int pool, int H, int dv,
                                                            int window, int max_tiles, float *o, int gate_elem) {
    extern __shared__ float wts[]; // [max_tiles] weights exp(m_t - M)
    __shared__ float red[4];
    const int h = blockIdx.x, tid = threadIdx.x, dvp = dv + 4;
    const long long p = step->pos0, lo = p - window + 1 > 0 ? p - window + 1 : 0, nb = wa_blocks(p, window, pool);
    long long ntl = (nb + 15) / 16 + (p - lo) / 16 + 1;
    const int nt = (int)(ntl < max_tiles ? ntl : max_tiles);
    float mx = sink ? sink[h] : -INFINITY;
    for (int t = tid; t < nt; t += 256) mx = fmaxf(mx, part[((long long)t * H + h) * dvp + dv]);
    mx = wa_wave_max(mx);
    if ((tid & 63) == 0) red[tid >> 6] = mx;
    __syncthreads();
    const float M = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    __syncthreads();
    float ls = 0.f;
    for (int t = tid; t < nt; t += 256) {
        const float *pp = part + ((long long)t * H + h) * dvp + dv;
        const float w = pp[0] == -INFINITY ? 0.f : expf(pp[0] - M);
        wts[t] = w;
        ls = fmaf(w, pp[1], ls);
    }
    ls = wa_wave_sum(ls);
    if ((tid & 63) == 0) red[tid >> 6] = ls;
    __syncthreads();
    const float L = red[0] + red[1] + red[2] + red[3] + (sink ? expf(sink[h] - M) : 0.f);
    const float f = (gate && !gate_elem ? wa_sigmoid(gate[h]) : 1.f) / L;
    for (int c = tid; c < dv; c += 256) {
        float a = 0.f;
#pragma unroll 8
        for (int t = 0; t < nt; t++) a = fmaf(wts[t], part[((long long)t * H + h) * dvp + c], a);
        o[(long long)h * dv + c] = a * f * (gate && gate_elem ? wa_sigmoid(gate[(long long)h * dv + c]) : 1.f);
    }
}

static int wa_max_tiles(int window, int pool, int64_t max_context) {
    const int64_t nb = pool > 0 ? max_context / pool + 1 : 0;
    return (int)((nb + 15) / 16 + (window + 15) / 16 + 1); // (a window that does not start on a tile's edge touches one tile more)
}
size_t psk_winattn_step_scratch(int H, int dv, int window, int pool, int64_t max_context) {
    return (size_t)(wa_max_tiles(window, pool, max_context) + 4) * H * (dv + 4) * 4;
}
// q [H * d] -> o [H * dv]; gate [H] raw or NULL; scratch from psk_winattn_step_scratch
void psk_winattn_step(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *q, const float *gate, const float *temp,
                      const float *sink, int H, int G, int d, int dv, int window, float scale, int64_t max_context, float *scratch, float *o, float softcap, int gate_elem) {
    const int max_tiles = wa_max_tiles(window, pool, max_context);
    const size_t lds = (size_t)(16 * (d + 4) + 4 * 16 * 17) * 4;
    static unsigned long long mask = 0;
    if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)winattn_step_kernel<8>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    const dim3 grid((max_tiles + 3) / 4, (H / G + 15) / 16, G);
    hipLaunchKernelGGL(winattn_step_kernel<8>, grid, dim3(256), lds, st, step, (long long)ring_off, cap, (long long)pool_off, pool, q, temp, H, G, d, dv, window, scale, scratch, softcap);
    hipLaunchKernelGGL(winattn_merge_kernel, dim3(H), dim3(256), (size_t)grid.x * 4 * 4, st, step, scratch, gate, sink, pool, H, dv, window, (int)grid.x * 4, o, gate_elem);
}
