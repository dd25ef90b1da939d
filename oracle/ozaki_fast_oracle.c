/*
 * Oracle: Ozaki-II reduced-precision ("fast") CRT tier.
 * TEST INFRASTRUCTURE ONLY - see eshkol_oracle.h.
 *
 * Restates ozaki_ii_fast_dispatch (lib/backend/gpu/gpu_memory.mm:2802-3012) and
 * its three kernels (lib/backend/gpu/metal_softfloat.h:4126-4246):
 *   moduli   the n largest prime powers <= cap, cap the largest p with
 *            K floor(p/2)^2 < 2^24 (and <= 255)        gpu_memory.mm:2802-2842
 *   E        floor((log2 P - log2 K - 2) / 2), in [1, 52]   gpu_memory.mm:2853-2855
 *   e_i,f_j  frexp exponents of the row / column maxima     gpu_memory.mm:2886-2905
 *   split    round-half-up(|x| 2^(E - e)) with x's sign, modulo p, centred with
 *            +p/2 kept positive; subnormal x count as 0     metal_softfloat.h:4148-4178
 *   product  G_l = A_l B_l, exact
 *   accum    S += ((G mod p) q mod p) / p in float-float, reduced modulo 1
 *                                                          metal_softfloat.h:4183-4207
 *   final    C = centred frac(S) * P * 2^(e_i + f_j - 2E) in float-float,
 *            widened hi + lo                               metal_softfloat.h:4210-4246
 * The float-float steps are restated operation for operation (compile with
 * -ffp-contract=off; fma only where the shader says fma). Besides that
 * restatement, oracle_ozaki_fast_exact_value gives the tier's integer product
 * sum_k a_int b_int scaled back, in long double: what every reconstruction of
 * the same residues approximates.
 */
#include "eshkol_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* gpu_memory.mm:2831-2835 */
int oracle_ozaki_fast_cap(uint64_t K) {
    int cap = (int)floor(2.0 * sqrt(16777216.0 / (double)K));
    if (cap > 255) cap = 255;
    while (cap > 2 && (double)K * floor(cap / 2.0) * floor(cap / 2.0) >= 16777216.0) cap--;
    return cap;
}

/* gpu_memory.mm:2802-2814; returns the count actually produced */
int oracle_ozaki_fast_moduli(int cap, int n_mod, int* out) {
    int pp[64], npp = 0;
    for (int p = 2; p <= cap; p++) {
        int pr = 1;
        for (int d = 2; d * d <= p; d++) if (p % d == 0) { pr = 0; break; }
        if (!pr) continue;
        long v = p, best = p;
        while (v * p <= cap) { v *= p; best = v; }
        pp[npp++] = (int)best;
    }
    for (int i = 0; i < npp; i++)                 /* descending */
        for (int j = i + 1; j < npp; j++)
            if (pp[j] > pp[i]) { int t = pp[i]; pp[i] = pp[j]; pp[j] = t; }
    if (npp > n_mod) npp = n_mod;
    for (int i = 0; i < npp; i++) out[i] = pp[i];
    return npp;
}

static long modinv(long a, long m) {
    long t = 0, nt = 1, r = m, nr = ((a % m) + m) % m;
    while (nr != 0) { long q = r / nr, x = t - q * nt; t = nt; nt = x; x = r - q * nr; r = nr; nr = x; }
    return (t % m + m) % m;
}

/* gpu_memory.mm:2844-2857 */
int oracle_ozaki_fast_constants(uint64_t K, int n_mod_req, OracleFastConstants* c) {
    memset(c, 0, sizeof *c);
    c->cap = oracle_ozaki_fast_cap(K);
    if (c->cap < 2) return -4;
    if (n_mod_req > 16) n_mod_req = 16;
    if (n_mod_req < 2) n_mod_req = 2;
    c->num_moduli = oracle_ozaki_fast_moduli(c->cap, n_mod_req, c->moduli);
    if (c->num_moduli < 2) return -4;
    unsigned __int128 P = 1;
    for (int l = 0; l < c->num_moduli; l++) P *= (unsigned)c->moduli[l];
    double logP = 0;
    for (int l = 0; l < c->num_moduli; l++) {
        unsigned __int128 Pp = P / (unsigned)c->moduli[l];
        c->q[l] = (int)modinv((long)(Pp % (unsigned)c->moduli[l]), c->moduli[l]);
        logP += log2((double)c->moduli[l]);
    }
    c->log2P = logP;
    int E = (int)floor((logP - log2((double)K) - 2.0) / 2.0);
    if (E > 52) E = 52;
    if (E < 1) E = 1;
    c->E = E;
    c->P = (double)P;
    c->P_hi = (float)c->P;
    c->P_lo = (float)(c->P - (double)c->P_hi);
    return 0;
}

/* gpu_memory.mm:2886-2905 */
void oracle_ozaki_fast_exponents(const double* A, const double* B, uint64_t M, uint64_t K, uint64_t N,
                                 int32_t* ei, int32_t* fj) {
    for (uint64_t i = 0; i < M; i++) {
        double mu = 0.0;
        for (uint64_t k = 0; k < K; k++) { double v = fabs(A[i * K + k]); if (v > mu) mu = v; }
        int e = 0;
        if (mu != 0.0) frexp(mu, &e);
        ei[i] = e;
    }
    for (uint64_t j = 0; j < N; j++) {
        double mx = 0.0;
        for (uint64_t k = 0; k < K; k++) { double v = fabs(B[k * N + j]); if (v > mx) mx = v; }
        int e = 0;
        if (mx != 0.0) frexp(mx, &e);
        fj[j] = e;
    }
}

/* metal_softfloat.h:4148-4178: the scaled integer (signed) of one element */
static int64_t fast_scaled(double x, int es, int E) {
    uint64_t bits;
    memcpy(&bits, &x, 8);
    const int sign = (int)(bits >> 63), exp = (int)((bits >> 52) & 0x7ff);
    if (exp == 0) return 0;
    uint64_t m = (bits & 0xfffffffffffffull) | (1ull << 52);
    const int sh = (exp - 1075) + E - es;
    int s = -sh;
    if (s > 53) return 0;
    if (s < 0) s = 0;
    if (s >= 1) m += 1ull << (s - 1);
    m >>= s;
    return sign ? -(int64_t)m : (int64_t)m;
}
static int8_t fast_residue(int64_t v, int p) {
    int64_t r = v % p;
    if (r < 0) r += p;                    /* the shader: r = |v| mod p, then p - r for negatives: same class */
    return (int8_t)((r > (p >> 1)) ? r - p : r);
}

/* planes [n][rows][K], rows of A or columns of B */
void oracle_ozaki_fast_split_a(const double* A, uint64_t M, uint64_t K, const int32_t* ei,
                               const OracleFastConstants* c, int8_t* planes, int64_t* scaled) {
    for (uint64_t i = 0; i < M; i++)
        for (uint64_t k = 0; k < K; k++) {
            const int64_t v = fast_scaled(A[i * K + k], ei[i], c->E);
            if (scaled) scaled[i * K + k] = v;
            for (int l = 0; l < c->num_moduli; l++)
                planes[((uint64_t)l * M + i) * K + k] = fast_residue(v, c->moduli[l]);
        }
}
void oracle_ozaki_fast_split_b(const double* B, uint64_t K, uint64_t N, const int32_t* fj,
                               const OracleFastConstants* c, int8_t* planes, int64_t* scaled) {
    for (uint64_t k = 0; k < K; k++)
        for (uint64_t j = 0; j < N; j++) {
            const int64_t v = fast_scaled(B[k * N + j], fj[j], c->E);
            if (scaled) scaled[j * K + k] = v;
            for (int l = 0; l < c->num_moduli; l++)
                planes[((uint64_t)l * N + j) * K + k] = fast_residue(v, c->moduli[l]);
        }
}

/* G_l = A_l B_l^T exactly; out[n][M][N] int32 (|G| <= K (cap/2)^2 < 2^24) */
void oracle_ozaki_fast_products(const int8_t* a_planes, const int8_t* b_planes, uint64_t M, uint64_t K, uint64_t N,
                                int n, int32_t* G) {
    for (int l = 0; l < n; l++)
        for (uint64_t i = 0; i < M; i++)
            for (uint64_t j = 0; j < N; j++) {
                const int8_t* a = a_planes + ((uint64_t)l * M + i) * K;
                const int8_t* b = b_planes + ((uint64_t)l * N + j) * K;
                int64_t s = 0;
                for (uint64_t k = 0; k < K; k++) s += (int64_t)a[k] * (int64_t)b[k];
                G[((uint64_t)l * M + i) * N + j] = (int32_t)s;
            }
}

/* metal_softfloat.h:4126-4144 */
static void df_add(float ahi, float alo, float bhi, float blo, float* rhi, float* rlo) {
    float s = ahi + bhi;
    float bb = s - ahi;
    float err = (ahi - (s - bb)) + (bhi - bb);
    float lo = alo + blo + err;
    float t = s + lo;
    *rlo = lo - (t - s);
    *rhi = t;
}
static void df_mul(float ahi, float alo, float bhi, float blo, float* rhi, float* rlo) {
    float p = ahi * bhi;
    float e = fmaf(ahi, bhi, -p);
    e += ahi * blo + alo * bhi;
    float t = p + e;
    *rlo = e - (t - p);
    *rhi = t;
}

/* accum for every modulus, then finalize: the reference's float-float result */
void oracle_ozaki_fast_reconstruct(const int32_t* G, uint64_t M, uint64_t N, const OracleFastConstants* c,
                                   const int32_t* ei, const int32_t* fj, double* C) {
    const uint64_t mn = M * N;
    for (uint64_t i = 0; i < M; i++)
        for (uint64_t j = 0; j < N; j++) {
            const uint64_t idx = i * N + j;
            float shi = 0.0f, slo = 0.0f;
            for (int l = 0; l < c->num_moduli; l++) {                 /* metal_softfloat.h:4183-4207 */
                const int p = c->moduli[l], q = c->q[l];
                const int Gi = G[(uint64_t)l * mn + idx];
                const int gg = ((Gi % p) + p) % p;
                const int u = (gg * q) % p;
                const float pf = (float)p;
                const float thi = (float)u / pf;
                const float tlo = fmaf(-thi, pf, (float)u) / pf;
                float rhi, rlo;
                df_add(shi, slo, thi, tlo, &rhi, &rlo);
                const float fl = floorf(rhi);
                if (fl != 0.0f) df_add(rhi, rlo, -fl, 0.0f, &rhi, &rlo);
                shi = rhi; slo = rlo;
            }
            float fl = floorf(shi), fhi, flo;                         /* metal_softfloat.h:4226-4245 */
            df_add(shi, slo, -fl, 0.0f, &fhi, &flo);
            const float fl2 = floorf(fhi);
            if (fl2 != 0.0f) df_add(fhi, flo, -fl2, 0.0f, &fhi, &flo);
            if (fhi >= 0.5f) df_add(fhi, flo, -1.0f, 0.0f, &fhi, &flo);
            const int scale = ei[i] + fj[j] - 2 * c->E;
            const float w = ldexpf(1.0f, scale);
            const float Whi = c->P_hi * w, Wlo = c->P_lo * w;
            float chi, clo;
            df_mul(fhi, flo, Whi, Wlo, &chi, &clo);
            C[idx] = (double)chi + (double)clo;                       /* gpu_memory.mm:2990 */
        }
}

/* The integer the residues encode, scaled back: sum_k a_int b_int * 2^(e_i + f_j - 2E). */
void oracle_ozaki_fast_exact_value(const int64_t* a_scaled, const int64_t* b_scaled, uint64_t M, uint64_t K, uint64_t N,
                                   const OracleFastConstants* c, const int32_t* ei, const int32_t* fj, double* C) {
    for (uint64_t i = 0; i < M; i++)
        for (uint64_t j = 0; j < N; j++) {
            __int128 s = 0;
            for (uint64_t k = 0; k < K; k++) s += (__int128)a_scaled[i * K + k] * (__int128)b_scaled[j * K + k];
            C[i * N + j] = (double)ldexpl((long double)s, ei[i] + fj[j] - 2 * c->E);
        }
}

int oracle_matmul_ozaki_fast_f64(const double* A, const double* B, double* C,
                                 uint64_t M, uint64_t K, uint64_t N, int n_mod) {
    OracleFastConstants c;
    int rc = oracle_ozaki_fast_constants(K, n_mod, &c);
    if (rc != 0) return rc;
    int32_t* ei = malloc(M * sizeof *ei);
    int32_t* fj = malloc(N * sizeof *fj);
    int8_t* ap = malloc((size_t)c.num_moduli * M * K);
    int8_t* bp = malloc((size_t)c.num_moduli * N * K);
    int32_t* G = malloc((size_t)c.num_moduli * M * N * sizeof *G);
    if (!ei || !fj || !ap || !bp || !G) { free(ei); free(fj); free(ap); free(bp); free(G); return -2; }
    oracle_ozaki_fast_exponents(A, B, M, K, N, ei, fj);
    oracle_ozaki_fast_split_a(A, M, K, ei, &c, ap, NULL);
    oracle_ozaki_fast_split_b(B, K, N, fj, &c, bp, NULL);
    oracle_ozaki_fast_products(ap, bp, M, K, N, c.num_moduli, G);
    oracle_ozaki_fast_reconstruct(G, M, N, &c, ei, fj, C);
    free(ei); free(fj); free(ap); free(bp); free(G);
    return 0;
}
