// Internal launchers of the layer-list models (include/ps_hip.h, "layer-list models"): dense mat-mul / mat-vec (k_dense.hip),
// norms, causal convolutions, token-shift, recurrent scans (k_seqmix.hip), latent attention (k_latent.hip).  All enqueue on `st`;
// none waits.  Activations are fp32 row-major [tokens][features] with an explicit row stride.
#pragma once
#include "ps_internal.h"

struct ps_dense {
    int dtype = PS_BF16; // PS_BF16 or PS_F32
    int64_t N = 0, K = 0;
    void *data = nullptr;
};

// What every kernel of a step reads from DEVICE memory, so that one captured launch sequence replays for any position and slot:
//   pos0 = position of the step's first token, n = tokens in the step, state = the slot's state block
struct ps_seq_step {
    int64_t pos0;
    int32_t n, slot;
    float *state;
    int32_t token0; // single-token steps: the token to embed (greedy decoding feeds its own arg-max back here)
    int32_t _pad;
};

enum { PSD_ACT_NONE = 0, PSD_ACT_XIELU = 1, PSD_ACT_TANH = 2,
       PSD_ACT_SILU_PAIR = 3,   // rows 2i / 2i + 1 of W are a gate and its partner: out[t][i] = silu(row 2i) * (row 2i + 1), N / 2 outputs (bias: one per row, added first)
       PSD_ACT_RELU_PAIR = 4,   // the same with relu on the gate
       PSD_ACT_RELU2 = 5 };     // max(z, 0)^2

// out[t][n] = alpha * act(sum_k A(t, k) W[n][k] + bias[n]),  t < T
//   A(t, k) = a[row(t)][k], row(t) = t, or (a_row0 + t) mod a_mod when a_mod > 0 (rows of a ring), or, where a_step is given, rows of the
//   ring starting at the device-side a_step->pos0 + a_row0 (clamped at 0) -- see k_latent.hip;
//   with mu: the token-shift mix a[t][k] + (prev(t)[k] - a[t][k]) * mu[k], prev(t) = t ? a[t-1] : shift0.
// In the bf16 mode A is rounded to bfloat16 (nearest even) before the product; accumulation is fp32 in both modes.
struct psk_dense_args {
    const ps_dense *w = nullptr;
    const float *a = nullptr;
    int64_t lda = 0, a_row0 = 0, a_mod = 0;
    const ps_seq_step *a_step = nullptr; // ring rows relative to the step's position (a_row0 = offset, usually negative)
    int T = 0;
    float *out = nullptr;
    int64_t ldo = 0;
    const float *bias = nullptr;
    int act = PSD_ACT_NONE;
    float act_p = 0.f, act_q = 0.f, alpha = 1.f; // xIELU: act_p = softplus(p), act_q = 1/2 + softplus(q)
    int accum = 0; // 1: out += the result (the residual stream takes a sublayer's output projection directly)
    const float *mu = nullptr, *shift0 = nullptr;
    int force_tiled = 0; // 1: the plain tiled mat-mul whatever the shape (A/B against the mat-vec and the wide mat-mul)
    void *pack = nullptr; // scratch for the wide mat-mul's bfloat16 copy of A (T rounded up to 128 rows of K); without it the plain tiled kernel runs
    size_t pack_bytes = 0;
    const float *out_scale = nullptr; // [T] device: row t of the result is multiplied by out_scale[t] (beside alpha)
    // ---- grouped products: w holds `groups` matrices of N / groups rows one after the other, and every row of the product belongs to one of them.
    // T counts SLOTS; slot s reads A row s / g_adiv times g_scale[s] (NULL: 1), uses matrix g_sel[s] and lands in output row s / g_odiv.
    // More than 8 slots: the slots sorted by matrix come as g_list with g_seg [groups + 1] (moe plan), a tile never mixes matrices; g_odiv > 1 is then not
    // taken (two slots of a row would meet: the caller sums per-slot results).  At most 8 slots x g_inner: a mat-vec per output row, which adds the g_inner
    // slots r g_inner .. r g_inner + g_inner - 1 of row r (T counts rows there, g_odiv is ignored).
    int groups = 0, g_adiv = 1, g_odiv = 1, g_inner = 1;
    const int32_t *g_sel = nullptr, *g_seg = nullptr, *g_list = nullptr;
    const float *g_scale = nullptr;
    // the grouped mat-vec only (an output per row, no activation): a slot whose g_sel is not below `groups` has no matrix -- an identity expert -- and adds
    // g_ident_w[slot] * g_ident[row][n] to output n of its row instead of a product (g_ident NULL: nothing)
    const float *g_ident = nullptr, *g_ident_w = nullptr;
    int64_t g_ident_ld = 0;
};
int psk_dense(hipStream_t st, const psk_dense_args &a);
void psk_dense_widen(hipStream_t st, const uint16_t *bf16, int64_t n, float *out);
// out[t][:] = table[token(t)][:] * scale; tokens device int32 (step != NULL and T == 1: the token is step->token0)
void psk_embed(hipStream_t st, const ps_dense *table, const int32_t *tokens, const ps_seq_step *step, int T, float scale, float *out, int64_t ldo);
// out[r] = index of the first maximum of x[r][0..n)
void psk_argmax_rows(hipStream_t st, const float *x, int64_t n, int rows, int32_t *out);

// ---- k_seqmix.hip
// y[r] = x[row(r)] / sqrt(mean(x^2) + eps) * (offset + w),  row(r) = idx ? idx[r] : r
//   (groups > 1: the row in that many equal consecutive parts, each divided by its own root mean square)
void psk_rmsnorm(hipStream_t st, const float *x, int64_t ldx, const int32_t *idx, const float *w, float offset, float eps, int64_t n, int rows, float *y, int64_t ldy,
                 int groups = 1);
// x[r] += y[r] / sqrt(mean(y^2) + eps) * (offset + w)
void psk_norm_residual(hipStream_t st, float *x, const float *y, const float *w, float offset, float eps, int64_t n, int rows, int groups = 1);
// The front of a parallel layer that has no input filter, in one launch: x[r] = sum_j mix[j] X_j[row(r)] over the nmix streams X_j = src + j stride (mix NULL:
// the last stream alone), row(r) = idx ? idx[r] : r, stored to xout[r] (NULL: not kept); then h[r] = norm(x) (offset + w1) and h2[r] = norm(x) (offset + w2) with
// the norm taken over `groups` parts -- two norms of one vector share their statistics.  w1 / w2 NULL: that output is not made.
void psk_front(hipStream_t st, const float *src, int64_t stride, int nmix, const float *mix, const int32_t *idx, float *xout, const float *w1, float *h, const float *w2,
               float *h2, int groups, float offset, float eps, int64_t n, int rows,
               int center = 0); // 1: layer norms -- (x - mean) / sqrt(mean((x - mean)^2) + eps) over each part
// Element-wise gated recurrence.  y[t] = [ z | u | g ] (C each): S <- (1 - sigmoid(z)) S + sigmoid(z) c(u), c(u) = sigmoid(u) for negative u, else u + 0.5;
// o[t] = S silu(g).  State [C] fp32 at step->state + state_off.
void psk_mingru_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *y, int64_t ldy, int64_t C, int T, float *o, int64_t ldo);
// Causal convolution over time on each channel, taps taken from the step's rows and, before them, from the sequence's tail (the last taps - 1
// inputs of earlier steps, [taps - 1][C] at step->state + tail_off): out[t][c] = f(sum_j w[c][j] in(t - taps + 1 + j)[c]); mode 0: f = in(t) + sum
// (a residual around the convolution), mode 1: f = silu(sum).  The tail is brought up to date behind it.
void psk_causal_conv(hipStream_t st, const ps_seq_step *step, int64_t tail_off, const float *in, int64_t ldi, const float *w, int taps, int mode,
                     int64_t C, int T, float *out, int64_t ldo);
// One token's sublayer boundary fused: x += norm_b(y) (y may be NULL), then h = conv(norm(x)) in the residual form with the tail update (wn may be NULL: stop after x);
// hn (may be NULL) also receives norm(x) itself, for a sublayer that reads the unfiltered input
void psk_boundary1(hipStream_t st, const ps_seq_step *step, float *x, const float *y, const float *wb, const float *wn, const float *cw, int taps, int64_t tail_off,
                   float offset, float eps, int64_t n, float *h, float *hn);
// state row copy: (step->state + off)[0..n) = src[0..n)
void psk_state_store(hipStream_t st, const ps_seq_step *step, int64_t off, const float *src, int64_t n);
void psk_fill(hipStream_t st, float *p, float v, int64_t n);
void psk_copy(hipStream_t st, const float *src, float *dst, int64_t n);

// wkv scan.  r, k, v, z: [T][H*d] (row stride ld), z = the decay's pre-activation (w = exp(-exp(z))); bonus [H*d]; state [H][d][d] fp32 at
// step->state + state_off.  o[t][h][j] = sum_i r_i (S_ij + bonus_i k_i v_j), then S_ij = w_i S_ij + k_i v_j.
void psk_wkv_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *r, const float *k, const float *v, const float *z, int64_t ld,
                  const float *bonus, int H, int d, int T, float *o, int64_t ldo);
// gated linear attention scan.  q, k [T][H*d], v [T][H*dv] (row stride ld), z [T][H*d] (row stride ldz) the decay's pre-activation; state [H][d][dv] fp32.
// Per head: S <- diag(sigmoid(z)^(1/tau)) S + k v^T, then o = S^T (q d^-1/2).
void psk_gla_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *q, const float *k, const float *v, int64_t ld, const float *z, int64_t ldz,
                  float tau, int H, int d, int dv, int T, float *o, int64_t ldo);
// gated delta rule scan.  q, k: [T][KH*d] after convolution + silu (unit-normalised here, q also times d^-1/2), v [T][H*dv] (row stride ld), braw / araw [T][H] (row stride ldb);
// per head: g = exp(-exp(a_log) softplus(araw + dt_bias)), beta = sigmoid(braw); S = g S; u = beta (v - S^T k); S += k u^T; o = S^T q.
void psk_delta_scan(hipStream_t st, const ps_seq_step *step, int64_t state_off, const float *q, const float *k, const float *v, const float *braw,
                    const float *araw, int64_t ld, int64_t ldb, const float *a_log, const float *dt_bias, int H, int KH, int d, int dv, int T, float *o, int64_t ldo);
// o[t][h][:] = o / sqrt(mean_j o^2 + eps) * w(h, :) * silu(g[t][h][:]);  w_stride = dv (a weight per head) or 0 (one shared by the heads)
void psk_headnorm_gate(hipStream_t st, float *o, int64_t ldo, const float *g, int64_t ldg, const float *w, int w_stride, float eps, int H, int dv, int T);

// ---- k_moe.hip
// Router of a mixture of experts, fp32: scores = sigmoid(router h[t]), or (softmax) the soft-max over all `experts` rows; choice scores = scores + correction (NULL: none);
// with n_groups > 0 only rows of the `keep` groups (equal runs of neighbours) with the largest best choice score stay in the race; the `top` largest choice scores
// (ties: the lower index) -> sel[t top + i], wgt[t top + i] (their SCORES, divided by their sum where norm_top); sgate[t] = sigmoid(shared_gate . h[t]) where given.
void psk_moe_route(hipStream_t st, const float *h, int64_t ldh, const float *router, const float *shared_gate, int experts, int top, int norm_top, int64_t K, int T,
                   int32_t *sel, float *wgt, float *sgate, int softmax = 0, const float *correction = nullptr, int n_groups = 0, int keep = 0);
// The S slots sorted by expert: seg [experts + 1] (slots of expert e are list[seg[e] .. seg[e + 1])), list [S]
void psk_moe_plan(hipStream_t st, const int32_t *sel, int S, int experts, int32_t *seg, int32_t *list);
// x[t] += alpha * sum_i (y[t top + i], or, for a slot whose sel >= n_real (an identity expert), wgt[slot] * h[t]);  y NULL: only the identity slots; sel NULL: only y
void psk_moe_combine(hipStream_t st, float *x, const float *y, int top, float alpha, int64_t n, int T, const int32_t *sel = nullptr, const float *wgt = nullptr,
                     int n_real = 0, const float *h = nullptr, int64_t ldh = 0);

// ---- k_latent.hip
// One token per block.  y[t] = [ dq (q_rank) | ckv (kv_rank) | kr (rot_dim) ]:  cq[t] = rmsnorm(dq) * qnorm;  ring row (pos mod cap):
// c = rmsnorm(ckv) * kvnorm, kr with its first rot_dims numbers rotated at pos (pairs (i, i + rot_dims/2), angle pos * freq[i]).  Ring at step->state + ring_off: [cap][kv_rank + rot_dim].
void psk_latent_prep(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *y, int64_t ldy, const float *qnorm, const float *kvnorm,
                     float eps, int q_rank, int kv_rank, int rot_dim, int rot_dims, const float *freq, int T, float *cq, int64_t ldcq,
                     float rot_mag = 1.f); // cos and sin of every rotation of this mixer are multiplied by rot_mag (the same value in all its launches); q_rank 0: no query latent
// Windowed soft-max attention over expanded keys / values.  q [T][H*(d+dr)] (rotated part not yet rotated), kv [Nw][H*d + H*dv] for the positions
// first .. first + Nw - 1 where first = max(0, pos0 - window + 1) (the caller expands exactly these ring rows), rotated key parts from the ring.
void psk_latent_attn(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int64_t ldq, const float *kv, int64_t ldkv,
                     const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window, float scale, int T, float *o, int64_t ldo,
                     float rot_mag = 1.f, const float *gate = nullptr, int64_t ldg = 0); // gate [T][H] raw: head h of token t times sigmoid(gate[t][h]) (all forms)
// The same attention on the matrix cores (fp32 MFMA), 16 tokens of a head per wave; _ok: the sizes it takes (d, dr multiples of 16, dv of 4, dv <= 128).
bool psk_latent_attn_mfma_ok(int d, int dr, int dv);
void psk_latent_attn_mfma(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int64_t ldq, const float *kv, int64_t ldkv,
                          const float *freq, int H, int d, int dr, int rot_dims, int dv, int kv_rank, int window, float scale, int T, float *o, int64_t ldo,
                          float rot_mag = 1.f, const float *gate = nullptr, int64_t ldg = 0);
// Single-token step in the absorbed form: nothing is expanded per key, the ring's latents are keys and values for all heads at once.
// q [H][d + dr] (row stride qstride, rotated part not yet rotated) -> o [H * dv].  ukv: rows uk | uv.  _ok: kv_rank, dr multiples of 16, kv_rank <= 512.
bool psk_latent_absorbed_ok(int d, int dr, int dv, int R);
size_t psk_latent_absorbed_scratch(int H, int R, int window);
void psk_latent_absorbed(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, const float *q, int qstride, const ps_dense *ukv, const float *freq,
                         int H, int d, int dr, int rot_dims, int dv, int R, int window, float scale, float *scratch, float *o, float rot_mag = 1.f,
                         const float *gate = nullptr);

// ---- k_winattn.hip
// y[t] = [ q (H d) | k (G d) | v (G dv) | ... ]: RMS norms over the whole q / k projections (qnorm / knorm, NULL: none), rotation of the first rot_dims numbers of
// every head at the token's position (pairing: ps_rot_pairing; angle of pair i: pos * freq[i]); q -> q[t], k and v -> the ring row pos mod cap ([G d | G dv], ring at
// step->state + ring_off); then the block means ([block][G d | G dv] at step->state + pool_off, pool > 0) are brought up to date.
void psk_winattn_prep(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *y, int64_t ldy, const float *qnorm,
                      const float *knorm, float eps, int H, int G, int d, int dv, int rot_dims, int pairing, const float *freq, int T, float *q, int64_t ldq,
                      float qt_coef = 0.f, int qt_every = 0, // qt_every > 0: q[t] times 1 + qt_coef ln(floor((pos + 1) / qt_every) + 1)
                      int head_norm = 0, // 1: qnorm / knorm are [d] and the norms are taken per head
                      int v_unit = 0);   // 1: every head's value divided by its own root mean square
// o[t][h] = gate(t, h) * soft-max attention of q[t][h] over the visible block means and the window's ring rows, scores times scale * temp[h], exp(sink[h]) in the
// denominator; gate [T][..] raw (sigmoid here; column h, row stride ldg), temp / sink / gate may be NULL.
void psk_winattn(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *q, int64_t ldq, const float *gate,
                 int64_t ldg, const float *temp, const float *sink, int H, int G, int d, int dv, int window, float scale, int T, float *o, int64_t ldo,
                 float softcap = 0.f, // softcap > 0 (all three forms): score <- softcap tanh(score / softcap) behind scale and temperature
                 int gate_elem = 0);  // 1 (all three forms): gate [T][H dv], one sigmoid per output element instead of one per head
// The same attention on the fp32 matrix cores for a portion, 16 tokens of a head per wave; _ok: the sizes it takes (d a multiple of 16, dv of 4, dv <= 128).
bool psk_winattn_mfma_ok(int d, int dv);
void psk_winattn_mfma(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *q, int64_t ldq, const float *gate,
                      int64_t ldg, const float *temp, const float *sink, int H, int G, int d, int dv, int window, float scale, int T, float *o, int64_t ldo,
                      float softcap = 0.f, int gate_elem = 0);
// A single token on the matrix cores: rows = the heads of a key / value group, the keys spread over waves, partials merged in a second launch (same sizes).
size_t psk_winattn_step_scratch(int H, int dv, int window, int pool, int64_t max_context);
void psk_winattn_step(hipStream_t st, const ps_seq_step *step, int64_t ring_off, int cap, int64_t pool_off, int pool, const float *q, const float *gate, const float *temp,
                      const float *sink, int H, int G, int d, int dv, int window, float scale, int64_t max_context, float *scratch, float *o, float softcap = 0.f,
                      int gate_elem = 0);
