// Dense (unquantized) matrices of the layer-list models: bfloat16 operands with fp32 accumulation on v_mfma_f32_16x16x32_bf16, or
// fp32 throughout on v_mfma_f32_16x16x4_f32 (one rounding per product, fp32 adds: a true fp32 product, no reduced-precision mode).
//   dense_mm_kernel<WT>   tiled mat-mul, 64 tokens x 64 outputs per work-group of four waves, any T / N / K (edges zero-filled)
//   dense_mm_fast_kernel  bf16, K % 64 == 0, more than 8 tokens: 128 x 128 tiles over an operand packed to bf16 by dense_pack_kernel
//   dense_mv_kernel<WT,C> a few tokens (C <= 8 columns): the activation rows live in LDS, a wave streams four weight rows at a time
// All take the same operand description (ps_seq.h psk_dense_args): ring rows, the token-shift mix and the epilogue
// (bias, xIELU / tanh, scale) are part of the launch, so no mixer needs a kernel of its own around its projections.
#include "ps_seq.h"

#include <cmath>

typedef float dn_f4 __attribute__((ext_vector_type(4)));
typedef __bf16 dn_bf8 __attribute__((ext_vector_type(8)));
typedef unsigned short dn_us8 __attribute__((ext_vector_type(8)));

static __device__ __forceinline__ unsigned short dn_f2bf(float f) { // round to nearest even
    unsigned u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (unsigned short)((u >> 16) | 0x40);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (unsigned short)(u >> 16);
}
static __device__ __forceinline__ float dn_bf2f(unsigned short b) { return __uint_as_float((unsigned)b << 16); }

struct dn_args {
    const void *w;
    const float *a;
    long long lda, a_row0, a_mod;
    const ps_seq_step *a_step;
    int T;
    long long N, K;
    float *out;
    long long ldo;
    const float *bias;
    int act;
    float act_p, act_q, alpha;
    const float *mu, *shift0;
    int accum;
    const float *out_scale;
    // grouped products (ps_seq.h): N is one matrix's rows, wstride the elements between matrices
    int groups, g_adiv, g_odiv, g_inner;
    const int32_t *g_sel, *g_seg, *g_list;
    const float *g_scale;
    long long wstride;
    const float *g_ident, *g_ident_w; // grouped mat-vec: a slot without a matrix adds g_ident_w[slot] * g_ident[row][n] to output n
    long long g_ident_ld;
};

// rows of A that exist and where they start (ring rows relative to the step's position)
static __device__ __forceinline__ void dn_rows(const dn_args &g, long long &row0, int &T) {
    row0 = g.a_row0;
    T = g.T;
    if (g.g_seg) { // the slots of matrix blockIdx.z: entries row0 .. row0 + T - 1 of the sorted list
        row0 = g.g_seg[blockIdx.z];
        T = g.g_seg[blockIdx.z + 1] - (int)row0;
        return;
    }
    if (g.a_step) {
        const long long p = g.a_step->pos0 + g.a_row0;
        row0 = p > 0 ? p : 0;
        const long long have = g.a_step->pos0 + g.a_step->n - row0;
        if (have < T) T = (int)have;
    }
}
static __device__ __forceinline__ const float *dn_arow(const dn_args &g, long long row0, int t) {
    long long r = row0 + t;
    if (g.g_list) r = g.g_list[r] / g.g_adiv;
    if (g.a_mod > 0) r %= g.a_mod;
    return g.a + r * g.lda;
}
static __device__ __forceinline__ float dn_aval(const dn_args &g, long long row0, int t, long long k) {
    if (g.g_list) return dn_arow(g, row0, t)[k] * (g.g_scale ? g.g_scale[g.g_list[row0 + t]] : 1.f);
    const float x = dn_arow(g, row0, t)[k];
    if (!g.mu) return x;
    const float p = t ? dn_arow(g, row0, t - 1)[k] : g.shift0[k];
    return x + (p - x) * g.mu[k];
}
static __device__ __forceinline__ float dn_epi(const dn_args &g, float acc, long long n) {
    if (g.bias) acc += g.bias[n];
    if (g.act == PSD_ACT_XIELU) {
        if (acc > 0.f) acc = g.act_p * acc * acc + 0.5f * acc;
        else acc = g.act_q * (expm1f(acc) - acc) + 0.5f * acc;
    } else if (g.act == PSD_ACT_TANH) {
        acc = tanhf(acc);
    } else if (g.act == PSD_ACT_RELU2) {
        acc = acc > 0.f ? acc * acc : 0.f;
    }
    return acc * g.alpha;
}
static __device__ __forceinline__ float dn_silu(float x) { return x / (1.f + expf(-x)); }
// Result acc of (token t, weight row n) goes to its place.  other: the result of row n ^ 1 (the paired activation needs both; every lane of the wave calls
// this with both values, only the even row stores).
static __device__ __forceinline__ void dn_put(const dn_args &g, long long t, long long n, float acc, float other, bool in) {
    const float rs = in && g.out_scale ? g.out_scale[t] : 1.f;
    if (g.act == PSD_ACT_SILU_PAIR || g.act == PSD_ACT_RELU_PAIR) {
        if (in && !(n & 1)) {
            float *p = g.out + t * g.ldo + (n >> 1);
            if (g.bias) { acc += g.bias[n]; other += g.bias[n + 1]; }
            const float v = (g.act == PSD_ACT_SILU_PAIR ? dn_silu(acc) : fmaxf(acc, 0.f)) * other * g.alpha * rs;
            *p = g.accum ? *p + v : v;
        }
        return;
    }
    if (!in) return;
    float *p = g.out + t * g.ldo + n;
    const float v = dn_epi(g, acc, n) * rs;
    *p = g.accum ? *p + v : v;
}
// the output row of local row t (t < T): itself, or where the sorted list sends its slot
static __device__ __forceinline__ long long dn_orow(const dn_args &g, long long row0, int t, int T) {
    if (!g.g_list) return t;
    return t < T ? g.g_list[row0 + t] / g.g_odiv : 0;
}

// ---------------------------------------------------------------------------------------------------- tiled mat-mul
template <typename WT> struct dn_tile;
template <> struct dn_tile<unsigned short> { static constexpr int BK = 32, LD = 40; typedef unsigned short S; }; // LDS rows padded to 80 B
template <> struct dn_tile<float> { static constexpr int BK = 16, LD = 20; typedef float S; };

template <typename WT>
__global__ __launch_bounds__(256) void dense_mm_kernel(dn_args g) {
    constexpr int BK = dn_tile<WT>::BK, LD = dn_tile<WT>::LD;
    typedef typename dn_tile<WT>::S S;
    __shared__ __attribute__((aligned(16))) S As[64 * LD];
    __shared__ __attribute__((aligned(16))) S Bs[64 * LD];
    long long row0;
    int T;
    dn_rows(g, row0, T);
    const int t0 = blockIdx.y * 64;
    if (t0 >= T) return; // (uniform per work-group: no barrier is skipped by part of it)
    const long long n0 = (long long)blockIdx.x * 64;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1;
    const int lr = lane & 15, lq = lane >> 4;
    const WT *W = (const WT *)g.w + (g.g_seg ? (long long)blockIdx.z * g.wstride : 0);
    dn_f4 acc[2][2];
    for (int i = 0; i < 2; i++)
        for (int j = 0; j < 2; j++) acc[i][j] = dn_f4{0.f, 0.f, 0.f, 0.f};
    constexpr int PER = 64 * BK / 256; // elements of each tile a thread stages: 8 (bf16) or 4 (fp32)
    const int srow = tid / (BK / PER), sk = (tid % (BK / PER)) * PER;
    for (long long k0 = 0; k0 < g.K; k0 += BK) {
        { // A: tokens t0 .. t0+63
            const int t = t0 + srow;
            S tmp[PER];
#pragma unroll
            for (int e = 0; e < PER; e++) {
                const long long k = k0 + sk + e;
                const float v = (t < T && k < g.K) ? dn_aval(g, row0, t, k) : 0.f;
                if constexpr (sizeof(WT) == 2) tmp[e] = dn_f2bf(v);
                else tmp[e] = v;
            }
#pragma unroll
            for (int e = 0; e < PER; e++) As[srow * LD + sk + e] = tmp[e];
        }
        { // B: weight rows n0 .. n0+63
            const long long n = n0 + srow;
            const long long k = k0 + sk;
            S tmp[PER];
            if (n < g.N && k + PER <= g.K && ((g.K * (long long)sizeof(WT)) % 16 == 0)) {
                const dn_f4 raw = *(const dn_f4 *)(W + n * g.K + k); // 16 bytes: 8 bf16 or 4 floats
                __builtin_memcpy(tmp, &raw, 16);
            } else {
#pragma unroll
                for (int e = 0; e < PER; e++) tmp[e] = (n < g.N && k + e < g.K) ? W[n * g.K + k + e] : (S)0;
            }
#pragma unroll
            for (int e = 0; e < PER; e++) Bs[srow * LD + sk + e] = tmp[e];
        }
        __syncthreads();
        if constexpr (sizeof(WT) == 2) {
            dn_bf8 fa[2], fb[2];
#pragma unroll
            for (int i = 0; i < 2; i++) {
                dn_us8 ra = *(const dn_us8 *)&As[(wm * 32 + i * 16 + lr) * LD + lq * 8];
                dn_us8 rb = *(const dn_us8 *)&Bs[(wn * 32 + i * 16 + lr) * LD + lq * 8];
                __builtin_memcpy(&fa[i], &ra, 16);
                __builtin_memcpy(&fb[i], &rb, 16);
            }
#pragma unroll
            for (int i = 0; i < 2; i++)
#pragma unroll
                for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        } else {
#pragma unroll
            for (int kk = 0; kk < BK; kk += 4) {
                float fa[2], fb[2];
#pragma unroll
                for (int i = 0; i < 2; i++) {
                    fa[i] = As[(wm * 32 + i * 16 + lr) * LD + kk + lq];
                    fb[i] = Bs[(wn * 32 + i * 16 + lr) * LD + kk + lq];
                }
#pragma unroll
                for (int i = 0; i < 2; i++)
#pragma unroll
                    for (int j = 0; j < 2; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x4f32(fa[i], fb[j], acc[i][j], 0, 0, 0);
            }
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
        for (int j = 0; j < 2; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int t = t0 + wm * 32 + i * 16 + lq * 4 + e;
                const long long n = n0 + wn * 32 + j * 16 + lr;
                dn_put(g, dn_orow(g, row0, t, T), n, acc[i][j][e], __shfl_xor(acc[i][j][e], 1, 64), t < T && n < g.N); // (row n ^ 1 is the neighbouring lane's)
            }
}

// ---------------------------------------------------------------------------------------------------- a few tokens: mat-vec
// Dynamic LDS: C rows of K activations, as bf16-rounded fp32 values (bf16 mode: the same operand rounding as the tiled kernel) or fp32.
template <typename WT, int C>
__global__ __launch_bounds__(256) void dense_mv_kernel(dn_args g) {
    extern __shared__ __attribute__((aligned(16))) float xs[]; // [C][Kp]
    long long row0;
    int T;
    dn_rows(g, row0, T);
    const long long K = g.K, Kp = (K + 7) / 8 * 8;
    for (long long i = threadIdx.x; i < (long long)C * Kp; i += 256) {
        const int c = (int)(i / Kp);
        const long long k = i % Kp;
        float v = (c < T && k < K) ? dn_aval(g, row0, c, k) : 0.f;
        if constexpr (sizeof(WT) == 2) v = dn_bf2f(dn_f2bf(v));
        xs[i] = v;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const WT *W = (const WT *)g.w;
    constexpr int RW = 4, VE = 16 / (int)sizeof(WT); // rows per wave at a time; elements per 16-byte load
    const bool vec = (K * (long long)sizeof(WT)) % 16 == 0;
    for (long long nb = ((long long)blockIdx.x * 4 + wave) * RW; nb < g.N; nb += (long long)gridDim.x * 4 * RW) {
        float acc[RW][C];
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int c = 0; c < C; c++) acc[r][c] = 0.f;
        if (vec) {
            // two 16-byte pieces of each of the four rows in flight per lane (8 KiB per wave and round)
            for (long long k = (long long)lane * VE; k < K; k += 128 * VE) {
                const long long k2 = k + 64 * VE;
                const bool two = k2 < K;
                dn_f4 raw[2][RW];
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    const long long n = nb + r < g.N ? nb + r : g.N - 1;
                    raw[0][r] = __builtin_nontemporal_load((const dn_f4 *)(W + n * K + k));
                    raw[1][r] = two ? __builtin_nontemporal_load((const dn_f4 *)(W + n * K + k2)) : dn_f4{0.f, 0.f, 0.f, 0.f};
                }
#pragma unroll
                for (int u = 0; u < 2; u++) {
                    const long long ku = u ? (two ? k2 : k) : k; // (the second piece is zero where there is none: any valid x offset will do)
#pragma unroll
                    for (int r = 0; r < RW; r++) {
                        float wv[VE];
                        if constexpr (sizeof(WT) == 2) {
                            unsigned short h[8];
                            __builtin_memcpy(h, &raw[u][r], 16);
#pragma unroll
                            for (int e = 0; e < 8; e++) wv[e] = dn_bf2f(h[e]);
                        } else {
                            __builtin_memcpy(wv, &raw[u][r], 16);
                        }
#pragma unroll
                        for (int c = 0; c < C; c++) {
                            const float *x = xs + (long long)c * Kp + ku;
#pragma unroll
                            for (int e = 0; e < VE; e++) acc[r][c] = fmaf(wv[e], x[e], acc[r][c]);
                        }
                    }
                }
            }
        } else {
            for (long long k = lane; k < K; k += 64)
#pragma unroll
                for (int r = 0; r < RW; r++) {
                    const long long n = nb + r < g.N ? nb + r : g.N - 1;
                    float wv;
                    if constexpr (sizeof(WT) == 2) wv = dn_bf2f(((const unsigned short *)W)[n * K + k]);
                    else wv = ((const float *)W)[n * K + k];
#pragma unroll
                    for (int c = 0; c < C; c++) acc[r][c] = fmaf(wv, xs[(long long)c * Kp + k], acc[r][c]);
                }
        }
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int c = 0; c < C; c++) {
#pragma unroll
                for (int o = 32; o > 0; o >>= 1) acc[r][c] += __shfl_xor(acc[r][c], o, 64);
            }
#pragma unroll
        for (int r = 0; r < RW; r++)
#pragma unroll
            for (int c = 0; c < C; c++) dn_put(g, c, nb + r, acc[r][c], acc[r ^ 1][c], lane == 0 && nb + r < g.N && c < T); // (nb is a multiple of four)
    }
}


// Grouped mat-vec (ps_seq.h, grouped products): block row r = one output row, which adds its g_inner slots; slot s = r g_inner + i reads A row s / g_adiv
// times g_scale[s] and the matrix g_sel[s].  Dynamic LDS: [g_inner][Kp] activations, rounded as in dense_mv_kernel.  A wave streams RW weight rows at a
// time, two 16-byte pieces of each in flight; small matrices take fewer rows per wave so that the launch still has waves for every CU.
template <typename WT, int RW>
__global__ __launch_bounds__(256) void dense_mv_grouped_kernel(dn_args g) {
    extern __shared__ __attribute__((aligned(16))) float xs[]; // [inner][Kp]
    const long long K = g.K, Kp = (K + 7) / 8 * 8;
    const int r = blockIdx.y, inner = g.g_inner;
    for (long long i = threadIdx.x; i < (long long)inner * Kp; i += 256) {
        const int c = (int)(i / Kp);
        const long long k = i % Kp, s = (long long)r * inner + c;
        float v = k < K ? g.a[(s / g.g_adiv) * g.lda + k] * (g.g_scale ? g.g_scale[s] : 1.f) : 0.f;
        if constexpr (sizeof(WT) == 2) v = dn_bf2f(dn_f2bf(v));
        xs[i] = v;
    }
    __syncthreads();
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    constexpr int VE = 16 / (int)sizeof(WT);
    const bool vec = (K * (long long)sizeof(WT)) % 16 == 0;
    for (long long nb = ((long long)blockIdx.x * 4 + wave) * RW; nb < g.N; nb += (long long)gridDim.x * 4 * RW) {
        float acc[RW];
        float ident = 0.f; // the summed weights of the row's slots that have no matrix (identity experts)
#pragma unroll
        for (int q = 0; q < RW; q++) acc[q] = 0.f;
        for (int c = 0; c < inner; c++) {
            const int sel = g.g_sel[(long long)r * inner + c];
            if (sel >= g.groups) { // (no product for this slot; the same for every lane of the block)
                if (g.g_ident) ident += g.g_ident_w[(long long)r * inner + c];
                continue;
            }
            const WT *W = (const WT *)g.w + (long long)sel * g.wstride;
            const float *x = xs + (long long)c * Kp;
            if (vec) {
                for (long long k = (long long)lane * VE; k < K; k += 128 * VE) {
                    const long long k2 = k + 64 * VE;
                    const bool two = k2 < K;
                    dn_f4 raw[2][RW];
#pragma unroll
                    for (int q = 0; q < RW; q++) {
                        const long long n = nb + q < g.N ? nb + q : g.N - 1;
                        raw[0][q] = __builtin_nontemporal_load((const dn_f4 *)(W + n * K + k));
                        raw[1][q] = two ? __builtin_nontemporal_load((const dn_f4 *)(W + n * K + k2)) : dn_f4{0.f, 0.f, 0.f, 0.f};
                    }
#pragma unroll
                    for (int u = 0; u < 2; u++) {
                        const long long ku = u ? (two ? k2 : k) : k; // (the second piece is zero where there is none: any valid x offset will do)
#pragma unroll
                        for (int q = 0; q < RW; q++) {
                            float wv[VE];
                            if constexpr (sizeof(WT) == 2) {
                                unsigned short h[8];
                                __builtin_memcpy(h, &raw[u][q], 16);
#pragma unroll
                                for (int e = 0; e < 8; e++) wv[e] = dn_bf2f(h[e]);
                            } else {
                                __builtin_memcpy(wv, &raw[u][q], 16);
                            }
#pragma unroll
                            for (int e = 0; e < VE; e++) acc[q] = fmaf(wv[e], x[ku + e], acc[q]);
                        }
                    }
                }
            } else {
                for (long long k = lane; k < K; k += 64)
#pragma unroll
                    for (int q = 0; q < RW; q++) {
                        const long long n = nb + q < g.N ? nb + q : g.N - 1;
                        float wv;
                        if constexpr (sizeof(WT) == 2) wv = dn_bf2f(((const unsigned short *)W)[n * K + k]);
                        else wv = ((const float *)W)[n * K + k];
                        acc[q] = fmaf(wv, x[k], acc[q]);
                    }
            }
        }
#pragma unroll
        for (int q = 0; q < RW; q++) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) acc[q] += __shfl_xor(acc[q], o, 64);
        }
        if (ident != 0.f && lane == 0) {
#pragma unroll
            for (int q = 0; q < RW; q++)
                if (nb + q < g.N) acc[q] = fmaf(ident, g.g_ident[(long long)r * g.g_ident_ld + nb + q], acc[q]);
        }
#pragma unroll
        for (int q = 0; q < RW; q++) dn_put(g, r, nb + q, acc[q], acc[RW > 1 ? (q ^ 1) : q], lane == 0 && nb + q < g.N);
    }
}
template <typename WT, int RW>
static void dn_launch_mv_grouped(hipStream_t st, const dn_args &g, int rows, size_t lds) {
    static unsigned long long mask = 0;
    if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)dense_mv_grouped_kernel<WT, RW>, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    long long blocks = (g.N + 4 * RW - 1) / (4 * RW);
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL((dense_mv_grouped_kernel<WT, RW>), dim3((unsigned)blocks, (unsigned)rows), dim3(256), lds, st, g);
}

// ---------------------------------------------------------------------------------------------------- wide mat-mul (bf16, K % 64 == 0)
// The A operand is first packed to bfloat16 [Tp][K] (Tp = T rounded up to 128, rows beyond T zero; the ring rows and the token-shift mix
// are resolved there), then 128 tokens x 128 outputs per work-group: four waves of 64 x 64 (4 x 4 tiles of v_mfma_f32_16x16x32_bf16), K in
// steps of 64 through LDS (rows padded to 144 B), the next step's 16-byte global loads in flight while the matrix cores run the current one.
__global__ __launch_bounds__(256) void dense_pack_kernel(dn_args g, unsigned short *out, int Tp) {
    long long row0 = g.a_row0;
    int T = g.T;
    if (!g.g_list) dn_rows(g, row0, T); // (grouped: all T slots in the order of the sorted list, whatever their matrix)
    else row0 = 0;
    const long long per_row = g.K / 8, total = (long long)Tp * per_row;
    for (long long i = (long long)blockIdx.x * 256 + threadIdx.x; i < total; i += (long long)gridDim.x * 256) {
        const int t = (int)(i / per_row);
        const long long k = (i % per_row) * 8;
        dn_us8 v;
#pragma unroll
        for (int e = 0; e < 8; e++) v[e] = t < T ? dn_f2bf(dn_aval(g, row0, t, k + e)) : (unsigned short)0;
        *(dn_us8 *)(out + (long long)t * g.K + k) = v;
    }
}

#define DN_FLD 72 // LDS row stride in bf16: 64 + 8
__global__ __launch_bounds__(256) void dense_mm_fast_kernel(dn_args g, const unsigned short *A) {
    __shared__ __attribute__((aligned(16))) unsigned short As[128 * DN_FLD];
    __shared__ __attribute__((aligned(16))) unsigned short Bs[128 * DN_FLD];
    long long row0;
    int T;
    dn_rows(g, row0, T);
    const int t0 = blockIdx.y * 128;
    if (t0 >= T) return;
    const long long n0 = (long long)blockIdx.x * 128;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wm = wave >> 1, wn = wave & 1, lr = lane & 15, lq = lane >> 4;
    const unsigned short *W = (const unsigned short *)g.w + (g.g_seg ? (long long)blockIdx.z * g.wstride : 0);
    if (g.g_seg) A += row0 * g.K; // (the packed operand is in list order: this matrix's slots start at row0; a tile's rows beyond them are another matrix's or zero, and are not stored)
    const long long K = g.K;
    // staging: 128 rows x 64 k = 1024 pieces of 16 bytes per operand, four per thread: row = (tid >> 3) + 32 i, k piece = tid & 7
    const int sr = tid >> 3, sk = (tid & 7) * 8;
    const unsigned short *ap[4], *bp[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        ap[i] = A + (long long)(t0 + sr + 32 * i) * K + sk; // (the packed operand has Tp rows: always there)
        long long n = n0 + sr + 32 * i;
        if (n >= g.N) n = g.N - 1;
        bp[i] = W + n * K + sk;
    }
    dn_f4 ra[4], rb[4];
#pragma unroll
    for (int i = 0; i < 4; i++) { ra[i] = *(const dn_f4 *)ap[i]; rb[i] = *(const dn_f4 *)bp[i]; }
    dn_f4 acc[4][4];
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++) acc[i][j] = dn_f4{0.f, 0.f, 0.f, 0.f};
    for (long long k0 = 0; k0 < K; k0 += 64) {
#pragma unroll
        for (int i = 0; i < 4; i++) {
            *(dn_f4 *)&As[(sr + 32 * i) * DN_FLD + sk] = ra[i];
            *(dn_f4 *)&Bs[(sr + 32 * i) * DN_FLD + sk] = rb[i];
        }
        __syncthreads();
        if (k0 + 64 < K) {
#pragma unroll
            for (int i = 0; i < 4; i++) { ra[i] = *(const dn_f4 *)(ap[i] + k0 + 64); rb[i] = *(const dn_f4 *)(bp[i] + k0 + 64); }
        }
#pragma unroll
        for (int kk = 0; kk < 64; kk += 32) {
            dn_bf8 fa[4], fb[4];
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const dn_f4 xa = *(const dn_f4 *)&As[(wm * 64 + i * 16 + lr) * DN_FLD + kk + lq * 8];
                const dn_f4 xb = *(const dn_f4 *)&Bs[(wn * 64 + i * 16 + lr) * DN_FLD + kk + lq * 8];
                __builtin_memcpy(&fa[i], &xa, 16);
                __builtin_memcpy(&fb[i], &xb, 16);
            }
#pragma unroll
            for (int i = 0; i < 4; i++)
#pragma unroll
                for (int j = 0; j < 4; j++) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fa[i], fb[j], acc[i][j], 0, 0, 0);
        }
        __syncthreads();
    }
#pragma unroll
    for (int i = 0; i < 4; i++)
#pragma unroll
        for (int j = 0; j < 4; j++)
#pragma unroll
            for (int e = 0; e < 4; e++) {
                const int t = t0 + wm * 64 + i * 16 + lq * 4 + e;
                const long long n = n0 + wn * 64 + j * 16 + lr;
                dn_put(g, dn_orow(g, row0, t, T), n, acc[i][j][e], __shfl_xor(acc[i][j][e], 1, 64), t < T && n < g.N);
            }
}

template <typename WT, int C>
static void dn_launch_mv(hipStream_t st, const dn_args &g) {
    const size_t lds = (size_t)C * ((g.K + 7) / 8 * 8) * 4;
    static unsigned long long mask = 0;
    if (ps_first_on_device(&mask)) (void)hipFuncSetAttribute((const void *)dense_mv_kernel<WT, C>, hipFuncAttributeMaxDynamicSharedMemorySize, 64 * 1024);
    long long blocks = (g.N + 15) / 16;
    if (blocks > 2048) blocks = 2048;
    hipLaunchKernelGGL((dense_mv_kernel<WT, C>), dim3((unsigned)blocks), dim3(256), lds, st, g);
}

int psk_dense(hipStream_t st, const psk_dense_args &a) {
    if (!a.w || a.T <= 0) return 0;
    dn_args g;
    g.w = a.w->data; g.a = a.a; g.lda = a.lda; g.a_row0 = a.a_row0; g.a_mod = a.a_mod; g.a_step = a.a_step; g.T = a.T;
    g.N = a.w->N; g.K = a.w->K; g.out = a.out; g.ldo = a.ldo; g.bias = a.bias; g.act = a.act; g.act_p = a.act_p; g.act_q = a.act_q;
    g.alpha = a.alpha; g.mu = a.mu; g.shift0 = a.shift0; g.accum = a.accum; g.out_scale = a.out_scale;
    g.groups = 0; g.g_adiv = 1; g.g_odiv = 1; g.g_inner = 1; g.g_sel = nullptr; g.g_seg = nullptr; g.g_list = nullptr; g.g_scale = nullptr; g.wstride = 0;
    g.g_ident = a.g_ident; g.g_ident_w = a.g_ident_w; g.g_ident_ld = a.g_ident_ld;
    const bool bf = a.w->dtype == PS_BF16;
    const size_t kp4 = (size_t)((g.K + 7) / 8 * 8) * 4;
    if (a.groups > 0) {
        g.groups = a.groups; g.N = a.w->N / a.groups; g.wstride = g.N * g.K;
        g.g_adiv = a.g_adiv; g.g_odiv = a.g_odiv; g.g_inner = a.g_inner; g.g_sel = a.g_sel; g.g_scale = a.g_scale;
        if (!a.g_list) { // a mat-vec per output row (T rows of g_inner slots each); four rows per wave only where that still leaves about 1024 waves
            const long long waves4 = (g.N + 3) / 4 * a.T;
            const int RW = waves4 >= 1024 ? 4 : (waves4 >= 512 || g.act == PSD_ACT_SILU_PAIR || g.act == PSD_ACT_RELU_PAIR) ? 2 : 1; // (a gate / up pair sits in one wave)
            const size_t lds = kp4 * a.g_inner;
            if (bf) {
                if (RW == 4) dn_launch_mv_grouped<unsigned short, 4>(st, g, a.T, lds);
                else if (RW == 2) dn_launch_mv_grouped<unsigned short, 2>(st, g, a.T, lds);
                else dn_launch_mv_grouped<unsigned short, 1>(st, g, a.T, lds);
            } else {
                if (RW == 4) dn_launch_mv_grouped<float, 4>(st, g, a.T, lds);
                else if (RW == 2) dn_launch_mv_grouped<float, 2>(st, g, a.T, lds);
                else dn_launch_mv_grouped<float, 1>(st, g, a.T, lds);
            }
            return 0;
        }
        g.g_seg = a.g_seg; g.g_list = a.g_list;
        const int Tp = (a.T + 127) / 128 * 128 + 128; // (a tile may start anywhere in the list and runs 127 rows on)
        if (bf && !a.force_tiled && g.K % 64 == 0 && a.pack && (size_t)Tp * g.K * 2 <= a.pack_bytes) {
            long long pb = ((long long)Tp * (g.K / 8) + 255) / 256;
            if (pb > 8192) pb = 8192;
            hipLaunchKernelGGL(dense_pack_kernel, dim3((unsigned)pb), dim3(256), 0, st, g, (unsigned short *)a.pack, Tp);
            hipLaunchKernelGGL(dense_mm_fast_kernel, dim3((unsigned)((g.N + 127) / 128), (unsigned)((a.T + 127) / 128), (unsigned)a.groups), dim3(256), 0, st, g,
                               (const unsigned short *)a.pack);
            return 0;
        }
        const dim3 grid((unsigned)((g.N + 63) / 64), (unsigned)((a.T + 63) / 64), (unsigned)a.groups);
        if (bf) hipLaunchKernelGGL(dense_mm_kernel<unsigned short>, grid, dim3(256), 0, st, g);
        else hipLaunchKernelGGL(dense_mm_kernel<float>, grid, dim3(256), 0, st, g);
        return 0;
    }
    if (!a.force_tiled && a.T <= 8) {
        const int C = a.T <= 1 ? 1 : a.T <= 2 ? 2 : a.T <= 4 ? 4 : 8;
        if (kp4 * C <= 64 * 1024) {
            if (bf) {
                if (C == 1) dn_launch_mv<unsigned short, 1>(st, g);
                else if (C == 2) dn_launch_mv<unsigned short, 2>(st, g);
                else if (C == 4) dn_launch_mv<unsigned short, 4>(st, g);
                else dn_launch_mv<unsigned short, 8>(st, g);
            } else {
                if (C == 1) dn_launch_mv<float, 1>(st, g);
                else if (C == 2) dn_launch_mv<float, 2>(st, g);
                else if (C == 4) dn_launch_mv<float, 4>(st, g);
                else dn_launch_mv<float, 8>(st, g);
            }
            return 0;
        }
    }
    const int Tp = (a.T + 127) / 128 * 128;
    if (bf && !a.force_tiled && a.T > 8 && g.K % 64 == 0 && a.pack && (size_t)Tp * g.K * 2 <= a.pack_bytes) {
        long long pb = ((long long)Tp * (g.K / 8) + 255) / 256;
        if (pb > 8192) pb = 8192;
        hipLaunchKernelGGL(dense_pack_kernel, dim3((unsigned)pb), dim3(256), 0, st, g, (unsigned short *)a.pack, Tp);
        hipLaunchKernelGGL(dense_mm_fast_kernel, dim3((unsigned)((g.N + 127) / 128), (unsigned)(Tp / 128)), dim3(256), 0, st, g, (const unsigned short *)a.pack);
        return 0;
    }
    dim3 grid((unsigned)((g.N + 63) / 64), (unsigned)((a.T + 63) / 64));
    if (bf) hipLaunchKernelGGL(dense_mm_kernel<unsigned short>, grid, dim3(256), 0, st, g);
    else hipLaunchKernelGGL(dense_mm_kernel<float>, grid, dim3(256), 0, st, g);
    return 0;
}

// ---------------------------------------------------------------------------------------------------- upload, embedding, arg-max
__global__ void dense_widen_kernel(const unsigned short *in, long long n, float *out) {
    for (long long i = (long long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long long)gridDim.x * blockDim.x) out[i] = dn_bf2f(in[i]);
}
void psk_dense_widen(hipStream_t st, const uint16_t *bf16, int64_t n, float *out) {
    long long blocks = (n + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(dense_widen_kernel, dim3((unsigned)blocks), dim3(256), 0, st, bf16, (long long)n, out);
}

__global__ void dense_embed_kernel(const void *table, int is_bf16, long long K, const int32_t *tokens, const ps_seq_step *step, float scale, float *out,
                                   long long ldo) {
    const int t = blockIdx.x;
    const long long tok = (tokens ? tokens[t] : step->token0);
    for (long long k = threadIdx.x; k < K; k += blockDim.x)
        out[t * ldo + k] = (is_bf16 ? dn_bf2f(((const unsigned short *)table)[tok * K + k]) : ((const float *)table)[tok * K + k]) * scale;
}
void psk_embed(hipStream_t st, const ps_dense *table, const int32_t *tokens, const ps_seq_step *step, int T, float scale, float *out, int64_t ldo) {
    hipLaunchKernelGGL(dense_embed_kernel, dim3(T), dim3(256), 0, st, table->data, table->dtype == PS_BF16 ? 1 : 0, (long long)table->K, tokens, step, scale, out,
                       (long long)ldo);
}

__global__ __launch_bounds__(256) void dense_argmax_kernel(const float *x, long long n, int32_t *out) {
    __shared__ float bv[256];
    __shared__ long long bi[256];
    const float *row = x + (long long)blockIdx.x * n;
    float best = -INFINITY;
    long long at = n;
    for (long long i = threadIdx.x; i < n; i += 256) {
        const float v = row[i];
        if (v > best || (v == best && i < at)) { best = v; at = i; }
    }
    bv[threadIdx.x] = best;
    bi[threadIdx.x] = at;
    __syncthreads();
    for (int s = 128; s > 0; s >>= 1) {
        if ((int)threadIdx.x < s) {
            const float v = bv[threadIdx.x + s];
            const long long i = bi[threadIdx.x + s];
            if (v > bv[threadIdx.x] || (v == bv[threadIdx.x] && i < bi[threadIdx.x])) { bv[threadIdx.x] = v; bi[threadIdx.x] = i; }
        }
        __syncthreads();
    }
    if (threadIdx.x == 0) out[blockIdx.x] = (int32_t)(bi[0] < n ? bi[0] : 0);
}
void psk_argmax_rows(hipStream_t st, const float *x, int64_t n, int rows, int32_t *out) {
    hipLaunchKernelGGL(dense_argmax_kernel, dim3(rows), dim3(256), 0, st, x, (long long)n, out);
}

extern "C" {
int ps_hip_dense_upload(ps_hip_ctx *c, const uint16_t *host, int64_t N, int64_t K, int as_f32, ps_dense **out) {
    *out = nullptr;
    if (N <= 0 || K <= 0) PS_FAIL(c, "dense_upload: empty matrix");
    PS_CHECK(c, hipSetDevice(c->device));
    auto w = new ps_dense();
    w->N = N; w->K = K; w->dtype = as_f32 ? PS_F32 : PS_BF16;
    const size_t n = (size_t)N * K;
    uint16_t *raw = nullptr;
    if (ps_dev_malloc((void **)&raw, n * 2 + 64) != hipSuccess) { delete w; PS_FAIL(c, "dense_upload: out of device memory"); }
    if (hipMemcpyAsync(raw, host, n * 2, hipMemcpyHostToDevice, c->stream) != hipSuccess) { (void)ps_dev_free(raw); delete w; PS_FAIL(c, "dense_upload: copy"); }
    if (as_f32) {
        float *f = nullptr;
        if (ps_dev_malloc((void **)&f, n * 4 + 64) != hipSuccess) { (void)ps_dev_free(raw); delete w; PS_FAIL(c, "dense_upload: out of device memory"); }
        psk_dense_widen(c->stream, raw, (int64_t)n, f);
        w->data = f;
    } else {
        w->data = raw;
    }
    hipError_t e = hipStreamSynchronize(c->stream);
    if (as_f32) (void)ps_dev_free(raw);
    if (e != hipSuccess) { (void)ps_dev_free(w->data); delete w; PS_FAIL(c, std::string("dense_upload: ") + hipGetErrorString(e)); }
    *out = w;
    return 0;
}
void ps_hip_dense_free(ps_hip_ctx *c, ps_dense *w) {
    if (!w) return;
    if (c) (void)hipStreamSynchronize(c->stream);
    (void)ps_dev_free(w->data);
    delete w;
}
int ps_hip_dense_matmul(ps_hip_ctx *c, const ps_dense *w, const float *x, int T, float *out, float alpha) {
    if (!w || T <= 0) PS_FAIL(c, "dense_matmul: bad argument");
    psk_dense_args a;
    a.w = w; a.a = x; a.lda = w->K; a.T = T; a.out = out; a.ldo = w->N; a.alpha = alpha;
    psk_dense(c->stream, a);
    PS_CHECK(c, hipGetLastError());
    return 0;
}
}
