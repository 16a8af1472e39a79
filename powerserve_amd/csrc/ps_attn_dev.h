// One 16-row x 16-key step of soft-max attention on the fp32 matrix cores (v_mfma_f32_16x16x4_f32), shared by the attention kernels of the
// layer-list models (k_latent.hip, k_winattn.hip):
//   scores   S[16 x 16] = Q[16 x DK] K^T: the keys come straight from memory as 16-byte pieces (lane (key l % 16, quarter l / 16) holds 4
//            consecutive dimensions; the row operand is read from LDS in the same order, so the sum runs over a permutation of the dimensions)
//   soft-max online, in the accumulator layout (lane holds rows 4 (l / 16) + i of key column l % 16; a row's 16 lanes reduce by butterfly)
//   output   O[16 x DV] += P V: P goes through a 16 x 17 LDS patch into the row-operand layout; V comes as 16-byte pieces of 4 consecutive
//            columns, so accumulator tile jj of a 64-column group holds columns 4 (l % 16) + jj -- undone at the final store.
// A "row" is a (token, head) pair.
#pragma once
#include <hip/hip_runtime.h>

#include <cmath>

typedef float la_f4 __attribute__((ext_vector_type(4)));

struct la_src { // where key j's row lives: base + ((j - sub) mod `mod`) * ld   (mod 0: no wrap)
    const float *base;
    long long ld, sub, mod;
};
static __device__ __forceinline__ const float *la_row(const la_src &s, long long j) {
    long long r = j - s.sub;
    if (s.mod > 0) r %= s.mod;
    return s.base + r * s.ld;
}

// qs: this wave's 16 rows in LDS, row stride qld floats, [DK1 | DK2]; pt: its 16 x 17 patch.  Accumulator row i of this lane (rows 4 (l / 16) + i)
// sees key j when rowlo[i] <= j < rowhi[i] (a row that does not exist: rowhi = rowlo) and j < jend; j indexes whatever the sources hold (positions
// of a window, blocks of a pooled store).  NJ: accumulator tiles (DV <= 16 NJ).
template <int NJ>
static __device__ __forceinline__ void la_tile(const float *qs, int qld, float *pt, const la_src &k1, const la_src &k2, const la_src &vs, int DK1, int DK2, int DV,
                                               long long j0, long long jend, const long long (&rowlo)[4], const long long (&rowhi)[4], float scale, float (&m)[4], float (&l)[4],
                                               la_f4 (&acc)[NJ], float softcap = 0.f) { // softcap > 0: score <- softcap tanh(score / softcap) behind the scale
    const int lane = threadIdx.x & 63, lr = lane & 15, lq = lane >> 4;
    const long long jk = j0 + lr < jend ? j0 + lr : jend - 1; // (a key row that exists; masked below)
    la_f4 s4 = {0.f, 0.f, 0.f, 0.f};
    const float *kr1 = la_row(k1, jk) + 4 * lq, *kr2 = la_row(k2, jk) + 4 * lq, *qr = qs + lr * qld + 4 * lq;
    // eight 16-byte key pieces in flight per lane ahead of their 32 matrix instructions
    for (int g0 = 0; g0 < DK1 + DK2; g0 += 128) {
        la_f4 b[8], a[8];
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int g = g0 + 16 * u;
            b[u] = g < DK1 ? *(const la_f4 *)(kr1 + g) : (g < DK1 + DK2 ? *(const la_f4 *)(kr2 + (g - DK1)) : la_f4{0.f, 0.f, 0.f, 0.f});
        }
#pragma unroll
        for (int u = 0; u < 8; u++) {
            const int g = g0 + 16 * u;
            a[u] = g < DK1 + DK2 ? *(const la_f4 *)(qr + g) : la_f4{0.f, 0.f, 0.f, 0.f};
        }
#pragma unroll
        for (int u = 0; u < 8; u++)
            if (g0 + 16 * u < DK1 + DK2) {
#pragma unroll
                for (int e = 0; e < 4; e++) s4 = __builtin_amdgcn_mfma_f32_16x16x4f32(a[u][e], b[u][e], s4, 0, 0, 0);
            }
    }
    const long long j = j0 + lr;
    float p[4], corr[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const bool vis = j < jend && j >= rowlo[i] && j < rowhi[i];
        float sv = s4[i] * scale;
        if (softcap > 0.f) sv = softcap * tanhf(sv / softcap);
        const float s = vis ? sv : -INFINITY;
        float tm = s;
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) tm = fmaxf(tm, __shfl_xor(tm, o, 64));
        const float mn = fmaxf(m[i], tm);
        corr[i] = mn == -INFINITY ? 1.f : expf(m[i] - mn);
        p[i] = mn == -INFINITY ? 0.f : expf(s - mn);
        float ts = p[i];
#pragma unroll
        for (int o = 1; o < 16; o <<= 1) ts += __shfl_xor(ts, o, 64);
        l[i] = l[i] * corr[i] + ts;
        m[i] = mn;
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int i = 0; i < 4; i++) pt[(4 * lq + i) * 17 + lr] = p[i];
    __builtin_amdgcn_wave_barrier();
    float pa[4];
#pragma unroll
    for (int s = 0; s < 4; s++) pa[s] = pt[lr * 17 + 4 * s + lq];
    __builtin_amdgcn_wave_barrier();
    const float *vr[4];
#pragma unroll
    for (int s = 0; s < 4; s++) {
        const long long jv = j0 + 4 * s + lq < jend ? j0 + 4 * s + lq : jend - 1; // (weight 0 beyond the end)
        vr[s] = la_row(vs, jv) + 4 * lr;
    }
    la_f4 bn[4];
#pragma unroll
    for (int s = 0; s < 4; s++) bn[s] = 4 * lr < DV ? *(const la_f4 *)(vr[s]) : la_f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int J = 0; J < NJ / 4; J++) {
        if (64 * J < DV) { // (uniform)
            la_f4 b[4];
#pragma unroll
            for (int s = 0; s < 4; s++) b[s] = bn[s];
            if (J + 1 < NJ / 4 && 64 * (J + 1) < DV) { // the next 64 columns' pieces are requested before this group's matrix instructions
                const bool in = 64 * (J + 1) + 4 * lr < DV;
#pragma unroll
                for (int s = 0; s < 4; s++) bn[s] = in ? *(const la_f4 *)(vr[s] + 64 * (J + 1)) : la_f4{0.f, 0.f, 0.f, 0.f};
            }
#pragma unroll
            for (int jj = 0; jj < 4; jj++) {
                la_f4 a = acc[4 * J + jj];
#pragma unroll
                for (int i = 0; i < 4; i++) a[i] *= corr[i];
#pragma unroll
                for (int s = 0; s < 4; s++) a = __builtin_amdgcn_mfma_f32_16x16x4f32(pa[s], b[s][jj], a, 0, 0, 0);
                acc[4 * J + jj] = a;
            }
        }
    }
}
