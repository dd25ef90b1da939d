/*
 * Oracle: Ozaki-II CRT exact tier, and the MLP layer built on it.
 * TEST INFRASTRUCTURE ONLY - see eshkol_oracle.h.
 *
 * Restates the host side of ozaki_ii_dispatch (lib/backend/gpu/gpu_memory.mm:
 * 227-453, 2474-2665) and the arithmetic of its modular GEMM kernel
 * (lib/backend/gpu/metal_softfloat.h:3907-4100). Two deliberate differences,
 * both invisible modulo p_l:
 *   - residues are taken with exact integer arithmetic instead of the float
 *     formula x - p*rint(x*(1/p)), whose product p*rint(..) can exceed 2^53
 *     at the top of the range (gpu_memory.mm:2580);
 *   - the representative at the tie of the even modulus 256 is -128, so every
 *     residue fits int8.
 * The accumulations S1 += sl1*w, S2 += sl2*w (gpu_memory.mm:2637-2638) are
 * stated as fma(): that is what the reference's compiler (clang, contraction
 * on within a statement) emits on the machines the Metal path runs on.
 * Compile with -ffp-contract=off.
 *
 * One addition that is not the reference: oracle_ozaki_crt_constants_aligned
 * gives the same constants with the CRT weights split at a common bit position
 * (the split the library offers as an option, where the reference's own split
 * makes the accumulation inexact). It is pinned by exact integer arithmetic in
 * tests/test_oracle_ozaki.py, not by the reference.
 */
#include "eshkol_oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* gpu_memory.mm:227-233 */
const int ORACLE_OZAKI_MODULI[49] = {
    256, 255, 253, 251, 247, 241, 239, 233, 229, 227,
    223, 217, 211, 199, 197, 193, 191, 181, 179, 173,
    167, 163, 157, 151, 149, 139, 137, 131, 127, 113,
    109, 107, 103, 101,  97,  89,  83,  79,  73,  71,
     67,  61,  59,  53,  47,  43,  41,  37,  29
};

/* gpu_memory.mm:282-296 */
static int64_t ext_gcd(int64_t a, int64_t b, int64_t* x, int64_t* y) {
    if (a == 0) { *x = 0; *y = 1; return b; }
    int64_t x1, y1;
    int64_t g = ext_gcd(b % a, a, &x1, &y1);
    *x = y1 - (b / a) * x1;
    *y = x1;
    return g;
}
static int mod_inverse(int64_t a, int64_t m) {
    int64_t x, y;
    ext_gcd(a % m, m, &x, &y);
    return (int)((x % m + m) % m);
}

/* gpu_memory.mm:301-341, clamp of 344-353. With aligned != 0 the weights
 * s_l = (P / p_l) q_l are split at one common bit position instead (not in the
 * reference): the reference takes the upper 40 bits of each weight by a
 * Veltkamp split relative to that weight's own exponent, so the lowest bit of
 * sl1 sits anywhere from 2^81 to 2^88 for sixteen moduli, and the sum of
 * sl1_l w_l (up to 2^137) is then not always representable: on operands drawn
 * from N(0,1) about one element in 150 comes back wrong by a multiple of 2^81 in
 * the scaled integer, 2^-25 of a typical element. Aligned, every sl1 is a
 * multiple of 2^e with e = bits(P) + 7 + ceil(log2 n) - 53, the partial sums
 * are exact, and what is left are roundings of the low parts, about 2^-60 of
 * a row's scale. */
static void crt_constants(int n, int aligned, OracleCRTConstants* crt) {
    if (n < 2) n = 2;
    if (n > ORACLE_OZAKI_MAX_MODULI) n = ORACLE_OZAKI_MAX_MODULI;
    memset(crt, 0, sizeof *crt);
    crt->num_moduli = n;
    __int128 P = 1;
    for (int l = 0; l < n; l++) P *= ORACLE_OZAKI_MODULI[l];
    crt->P1 = (double)P;
    __int128 P1_int = (__int128)crt->P1;
    crt->P2 = (double)(P - P1_int);
    crt->Pinv = 1.0 / (double)P;
    crt->log2P = log2((double)P);
    int bits_P = 0;
    for (__int128 t = P; t > 0; t >>= 1) bits_P++;
    for (int l = 0; l < n; l++) {
        int p = ORACLE_OZAKI_MODULI[l];
        __int128 Pp = P / p;
        crt->q[l] = mod_inverse((int64_t)(Pp % p), p);
        __int128 s = Pp * (__int128)crt->q[l];
        int bits_to_remove = 8 + (int)ceil(log2((double)n));
        if (aligned) {
            const int e = bits_P + (bits_to_remove - 1) - 53;
            __int128 hi = s;
            if (e > 0) hi = ((s + ((__int128)1 << (e - 1))) >> e) << e;
            crt->sl1[l] = (double)hi;                 /* at most bits_P - e <= 53 significant bits: exact */
            crt->sl2[l] = (double)(s - hi);
            continue;
        }
        double s_d = (double)s;
        double factor = (double)(1LL << (bits_to_remove + 1)) + 1.0;
        double t = factor * s_d;
        double hi = t - s_d;
        crt->sl1[l] = t - hi;
        __int128 sl1_int = (__int128)crt->sl1[l];
        crt->sl2[l] = (double)(s - sl1_int);
    }
}

void oracle_ozaki_crt_constants(int n, OracleCRTConstants* crt) { crt_constants(n, 0, crt); }
void oracle_ozaki_crt_constants_aligned(int n, OracleCRTConstants* crt) { crt_constants(n, 1, crt); }

/* oracle_matmul_ozaki_crt_f64 and oracle_mlp_layer_f64 use the aligned weights while this is set */
static int g_aligned_weights = 0;
void oracle_ozaki_crt_use_aligned_weights(int on) { g_aligned_weights = on != 0; }

static void row_col_max(const double* A, const double* B, uint64_t M, uint64_t K, uint64_t N,
                        double* rmax, double* cmax) {
    for (uint64_t i = 0; i < M; i++) {
        double mx = 0.0;
        for (uint64_t k = 0; k < K; k++) { double v = fabs(A[i * K + k]); if (v > mx) mx = v; }
        rmax[i] = mx;
    }
    for (uint64_t j = 0; j < N; j++) cmax[j] = 0.0;
    for (uint64_t k = 0; k < K; k++)
        for (uint64_t j = 0; j < N; j++) { double v = fabs(B[k * N + j]); if (v > cmax[j]) cmax[j] = v; }
}

static void frac_from_max(const double* rmax, const double* cmax, uint64_t M, uint64_t N,
                          double* frac_A, double* frac_B) {
    double fa = 0.0, fb = 0.0;
    for (uint64_t i = 0; i < M; i++)
        if (rmax[i] > 0.0) { double lg = log2(rmax[i]); double f = lg - floor(lg); if (f > fa) fa = f; }
    for (uint64_t j = 0; j < N; j++)
        if (cmax[j] > 0.0) { double lg = log2(cmax[j]); double f = lg - floor(lg); if (f > fb) fb = f; }
    *frac_A = fa; *frac_B = fb;
}

/* gpu_memory.mm:376-420 */
void oracle_ozaki_frac_bounds(const double* A, const double* B,
                              uint64_t M, uint64_t K, uint64_t N,
                              double* frac_A, double* frac_B) {
    double* r = (double*)malloc((size_t)M * sizeof(double));
    double* c = (double*)malloc((size_t)N * sizeof(double));
    row_col_max(A, B, M, K, N, r, c);
    frac_from_max(r, c, M, N, frac_A, frac_B);
    free(r); free(c);
}

/* gpu_memory.mm:362-367, 433-453 */
int oracle_ozaki_adaptive_n(const double* A, const double* B,
                            uint64_t M, uint64_t K, uint64_t N, int max_moduli) {
    if (max_moduli > ORACLE_OZAKI_MAX_MODULI) max_moduli = ORACLE_OZAKI_MAX_MODULI;
    if (max_moduli < 2) max_moduli = 2;
    double fa, fb;
    oracle_ozaki_frac_bounds(A, B, M, K, N, &fa, &fb);
    double cumul[50];
    cumul[0] = 0.0;
    for (int i = 0; i < 49; i++) cumul[i + 1] = cumul[i] + log2((double)ORACLE_OZAKI_MODULI[i]);
    const double log2K = log2((double)K);
    for (int n = 2; n <= max_moduli; n++) {
        double emax = floor((cumul[n] - 1.0 - log2K - fa - fb) / 2.0);
        if (emax >= 52.0) return n;
    }
    return max_moduli;
}

/* gpu_memory.mm:2510-2532 */
int oracle_ozaki_crt_scaling(const double* A, const double* B,
                             uint64_t M, uint64_t K, uint64_t N,
                             const OracleCRTConstants* crt, int* mu, int* nu) {
    double* r = (double*)malloc((size_t)M * sizeof(double));
    double* c = (double*)malloc((size_t)N * sizeof(double));
    row_col_max(A, B, M, K, N, r, c);
    double fa, fb;
    frac_from_max(r, c, M, N, &fa, &fb);
    int E = (int)floor((crt->log2P - 1.0 - log2((double)K) - fa - fb) / 2.0);
    if (E > 52) E = 52;
    if (E < 0) E = 0;
    for (uint64_t i = 0; i < M; i++) mu[i] = (r[i] == 0.0) ? 0 : E - (int)floor(log2(r[i]));
    for (uint64_t j = 0; j < N; j++) nu[j] = (c[j] == 0.0) ? 0 : E - (int)floor(log2(c[j]));
    free(r); free(c);
    return E;
}

/* Residue of trunc(v * 2^sh) for each modulus, representative in [-p/2, p/2). */
static inline void residues_of(double v, int sh, int num_moduli, int8_t* out, uint64_t stride) {
    double scale = ldexp(1.0, sh);               /* gpu_memory.mm:2539 */
    double x = trunc(v * scale);                 /* gpu_memory.mm:2541 */
    int64_t t = (int64_t)x;                      /* |x| < 2^53: exact */
    for (int l = 0; l < num_moduli; l++) {
        int p = ORACLE_OZAKI_MODULI[l];
        int r = (int)(t % p);                    /* C remainder: sign of t */
        if (r < 0) r += p;                       /* [0, p) */
        if (2 * r >= p) r -= p;                  /* [-p/2, p/2) */
        out[(uint64_t)l * stride] = (int8_t)r;
    }
}

/* gpu_memory.mm:2538-2542, 2573-2580 */
void oracle_ozaki_crt_split_a(const double* A, uint64_t M, uint64_t K,
                              const int* mu, int num_moduli, int8_t* a_planes) {
    const uint64_t tot = M * K;
    for (uint64_t i = 0; i < M; i++)
        for (uint64_t k = 0; k < K; k++)
            residues_of(A[i * K + k], mu[i], num_moduli, a_planes + i * K + k, tot);
}

/* gpu_memory.mm:2543-2547, 2581-2582; planes stored transposed (K contiguous). */
void oracle_ozaki_crt_split_b(const double* B, uint64_t K, uint64_t N,
                              const int* nu, int num_moduli, int8_t* b_planes) {
    const uint64_t tot = K * N;
    for (uint64_t k = 0; k < K; k++)
        for (uint64_t j = 0; j < N; j++)
            residues_of(B[k * N + j], nu[j], num_moduli, b_planes + j * K + k, tot);
}

/* metal_softfloat.h:3907-4100: the kernel keeps its float accumulator exact by
 * partial reductions; the value it returns is the symmetric residue of the
 * exact integer sum, which is what is computed here. */
void oracle_ozaki_crt_products(const int8_t* a_planes, const int8_t* b_planes,
                               uint64_t M, uint64_t K, uint64_t N, int num_moduli,
                               int8_t* w_planes, int32_t* acc32) {
    for (int l = 0; l < num_moduli; l++) {
        const int p = ORACLE_OZAKI_MODULI[l];
        const int8_t* Al = a_planes + (uint64_t)l * M * K;
        const int8_t* Bl = b_planes + (uint64_t)l * N * K;
        #pragma omp parallel for schedule(static)
        for (uint64_t i = 0; i < M; i++)
            for (uint64_t j = 0; j < N; j++) {
                const int8_t* a = Al + i * K;
                const int8_t* b = Bl + j * K;
                int64_t acc = 0;
                for (uint64_t k0 = 0; k0 < K; k0 += 65536) {
                    uint64_t k1 = (k0 + 65536 < K) ? k0 + 65536 : K;
                    int32_t part = 0;
                    for (uint64_t k = k0; k < k1; k++) part += (int32_t)a[k] * (int32_t)b[k];
                    acc += part;
                }
                if (acc32) acc32[(uint64_t)l * M * N + i * N + j] = (int32_t)acc;
                int r = (int)(acc % p);
                if (r < 0) r += p;
                if (2 * r >= p) r -= p;
                w_planes[(uint64_t)l * M * N + i * N + j] = (int8_t)r;
            }
    }
}

/* gpu_memory.mm:2626-2655 */
void oracle_ozaki_crt_reconstruct(const int8_t* w_planes, uint64_t M, uint64_t N,
                                  const OracleCRTConstants* crt,
                                  const int* mu, const int* nu, double* C) {
    const uint64_t tot = M * N;
    const double P1 = crt->P1, P2 = crt->P2, Pinv = crt->Pinv;
    for (uint64_t i = 0; i < M; i++) {
        double mu_inv = ldexp(1.0, -mu[i]);
        for (uint64_t j = 0; j < N; j++) {
            uint64_t idx = i * N + j;
            double S1 = 0.0, S2 = 0.0;
            for (int l = 0; l < crt->num_moduli; l++) {
                double w = (double)w_planes[(uint64_t)l * tot + idx];
                S1 = fma(crt->sl1[l], w, S1);
                S2 = fma(crt->sl2[l], w, S2);
            }
            double s = S1 + S2;
            double Q = round(s * Pinv);
            double h1 = fma(-P1, Q, S1);
            double h2 = fma(-P2, Q, S2);
            double c_prime = h1 + h2;
            double t = c_prime * mu_inv;
            C[idx] = t * ldexp(1.0, -nu[j]);
        }
    }
}

static int all_finite(const double* x, uint64_t n) {
    for (uint64_t i = 0; i < n; i++) if (!isfinite(x[i])) return 0;
    return 1;
}

/* gpu_memory.mm:2474-2665 */
int oracle_matmul_ozaki_crt_f64(const double* A, const double* B, double* C,
                                uint64_t M, uint64_t K, uint64_t N,
                                int num_moduli, int adaptive) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0) return -1;
    if (!all_finite(A, M * K) || !all_finite(B, K * N)) return -1;
    if (num_moduli < 2) num_moduli = 2;
    if (num_moduli > ORACLE_OZAKI_MAX_MODULI) num_moduli = ORACLE_OZAKI_MAX_MODULI;
    if (adaptive) num_moduli = oracle_ozaki_adaptive_n(A, B, M, K, N, num_moduli);
    OracleCRTConstants crt;
    crt_constants(num_moduli, g_aligned_weights, &crt);
    int* mu = (int*)malloc((size_t)M * sizeof(int));
    int* nu = (int*)malloc((size_t)N * sizeof(int));
    int8_t* ap = (int8_t*)malloc((size_t)num_moduli * M * K);
    int8_t* bp = (int8_t*)malloc((size_t)num_moduli * K * N);
    int8_t* wp = (int8_t*)malloc((size_t)num_moduli * M * N);
    int rc = -1;
    if (mu && nu && ap && bp && wp) {
        oracle_ozaki_crt_scaling(A, B, M, K, N, &crt, mu, nu);
        int ok = 1;
        for (uint64_t i = 0; i < M && ok; i++) if (mu[i] > 1023 || mu[i] < -1022) ok = 0;
        for (uint64_t j = 0; j < N && ok; j++) if (nu[j] > 1023 || nu[j] < -1022) ok = 0;
        if (ok) {
            oracle_ozaki_crt_split_a(A, M, K, mu, num_moduli, ap);
            oracle_ozaki_crt_split_b(B, K, N, nu, num_moduli, bp);
            oracle_ozaki_crt_products(ap, bp, M, K, N, num_moduli, wp, NULL);
            oracle_ozaki_crt_reconstruct(wp, M, N, &crt, mu, nu, C);
            rc = 0;
        }
    }
    free(mu); free(nu); free(ap); free(bp); free(wp);
    return rc;
}

/* ---- the reference's own representatives ------------------------------------------
 * The functions above take every residue by integer arithmetic in [-p/2, p/2), so
 * the class 128 of the modulus 256 is always -128. The reference computes its
 * residues in floating point, where the half-way case of the one even modulus
 * comes out as +128 or -128 by the parity of the rounded quotient:
 *   inputs  (gpu_memory.mm:2573-2583)       a_l = (float)(A' - p rint(A' (1/p))), in double
 *   products (metal_softfloat.h:3907-4100)  float sums of 63 k-blocks of 16 (1008 k),
 *            each reduced as v - p rint(v (1/p)) in float and added up, the total
 *            reduced the same way once more.
 * Modulo p nothing changes, so the exact product is the same; but the
 * reference's weighted sum S1 is not exact (its weights end at different bits),
 * and +128 instead of -128 moves that sum by 256 s_0 = P q_0, so its rounding
 * errors fall differently. This restates the reference's choice operation for
 * operation, to count on how many elements that matters.
 *   mode 1: the input formula applied to the exact sum (what a host statement of
 *           the modular product by the reference's own residue formula gives);
 *   mode 2: the Metal kernel's order: reference representatives of the inputs,
 *           partial reductions every 1008 k in float, final reduction in float.
 * w16[l*M*N + i*N + j] in [-128, 128]. */
static inline double ref_residue_f64(double x, int p) {
    const double pd = (double)p, inv = 1.0 / pd;                  /* gpu_memory.mm:2576-2580 */
    return x - pd * rint(x * inv);
}
static inline float ref_residue_f32(float v, float pf, float pinv) {
    return v - pf * rintf(v * pinv);                              /* metal_softfloat.h:4063-4064 */
}

void oracle_ozaki_crt_products_refrep(const double* A, const double* B,
                                      uint64_t M, uint64_t K, uint64_t N,
                                      const int* mu, const int* nu, int num_moduli, int mode,
                                      int16_t* w16) {
    float* ar = (float*)malloc((size_t)M * K * sizeof(float));
    float* br = (float*)malloc((size_t)N * K * sizeof(float));
    for (int l = 0; l < num_moduli; l++) {
        const int p = ORACLE_OZAKI_MODULI[l];
        const float pf = (float)p, pinv = 1.0f / pf;
        for (uint64_t i = 0; i < M; i++)
            for (uint64_t k = 0; k < K; k++)
                ar[i * K + k] = (float)ref_residue_f64(trunc(A[i * K + k] * ldexp(1.0, mu[i])), p);
        for (uint64_t k = 0; k < K; k++)
            for (uint64_t j = 0; j < N; j++)
                br[j * K + k] = (float)ref_residue_f64(trunc(B[k * N + j] * ldexp(1.0, nu[j])), p);
        #pragma omp parallel for schedule(static)
        for (uint64_t i = 0; i < M; i++)
            for (uint64_t j = 0; j < N; j++) {
                const float* a = ar + i * K;
                const float* b = br + j * K;
                float w;
                if (mode == 2) {
                    float partial = 0.0f;
                    for (uint64_t k0 = 0; k0 < K; k0 += 1008) {
                        const uint64_t k1 = (k0 + 1008 < K) ? k0 + 1008 : K;
                        int32_t v = 0;                            /* |v| <= 1008 * 128^2 < 2^24: exact in float too */
                        for (uint64_t k = k0; k < k1; k++) v += (int32_t)a[k] * (int32_t)b[k];
                        partial += ref_residue_f32((float)v, pf, pinv);
                    }
                    w = ref_residue_f32(partial, pf, pinv);
                } else {
                    int64_t v = 0;
                    for (uint64_t k = 0; k < K; k++) v += (int64_t)a[k] * (int64_t)b[k];
                    w = (float)ref_residue_f64((double)v, p);
                }
                w16[(uint64_t)l * M * N + i * N + j] = (int16_t)w;
            }
    }
    free(ar); free(br);
}

/* The exact tier with the reference's representatives (mode as above); the
 * accumulation is oracle_ozaki_crt_reconstruct's, operation for operation, on
 * residues that may be +128. Also counts the elements whose residue modulo 256
 * is the half-way class (n_half) and those among them that came out as +128
 * (n_plus): only these can differ from oracle_matmul_ozaki_crt_f64. */
int oracle_matmul_ozaki_crt_refrep_f64(const double* A, const double* B, double* C,
                                       uint64_t M, uint64_t K, uint64_t N,
                                       int num_moduli, int mode,
                                       uint64_t* n_half, uint64_t* n_plus) {
    if (!A || !B || !C || M == 0 || K == 0 || N == 0 || (mode != 1 && mode != 2)) return -1;
    if (!all_finite(A, M * K) || !all_finite(B, K * N)) return -1;
    if (num_moduli < 2) num_moduli = 2;
    if (num_moduli > ORACLE_OZAKI_MAX_MODULI) num_moduli = ORACLE_OZAKI_MAX_MODULI;
    OracleCRTConstants crt;
    crt_constants(num_moduli, g_aligned_weights, &crt);
    int* mu = (int*)malloc((size_t)M * sizeof(int));
    int* nu = (int*)malloc((size_t)N * sizeof(int));
    int16_t* w16 = (int16_t*)malloc((size_t)num_moduli * M * N * sizeof(int16_t));
    oracle_ozaki_crt_scaling(A, B, M, K, N, &crt, mu, nu);
    oracle_ozaki_crt_products_refrep(A, B, M, K, N, mu, nu, num_moduli, mode, w16);
    const uint64_t tot = M * N;
    uint64_t half = 0, plus = 0;
    for (uint64_t i = 0; i < M; i++) {
        const double mu_inv = ldexp(1.0, -mu[i]);
        for (uint64_t j = 0; j < N; j++) {
            const uint64_t idx = i * N + j;
            if (w16[idx] == 128 || w16[idx] == -128) { half++; plus += w16[idx] == 128; }
            double S1 = 0.0, S2 = 0.0;
            for (int l = 0; l < crt.num_moduli; l++) {
                const double w = (double)w16[(uint64_t)l * tot + idx];
                S1 = fma(crt.sl1[l], w, S1);
                S2 = fma(crt.sl2[l], w, S2);
            }
            const double s = S1 + S2;
            const double Q = round(s * crt.Pinv);
            const double c_prime = fma(-crt.P1, Q, S1) + fma(-crt.P2, Q, S2);
            C[idx] = (c_prime * mu_inv) * ldexp(1.0, -nu[j]);
        }
    }
    if (n_half) *n_half = half;
    if (n_plus) *n_plus = plus;
    free(mu); free(nu); free(w16);
    return 0;
}

/* BASELINE config 5: one dense layer through the exact tier. The add is the
 * broadcast of b over rows (runtime_tensor_math.cpp:672-740), the activation is
 * std::tanh applied elementwise (lib/core/model_io.cpp:709). */
int oracle_mlp_layer_f64(const double* X, const double* W, const double* b, double* Y,
                         uint64_t batch, uint64_t in_f, uint64_t out_f, int num_moduli) {
    int rc = oracle_matmul_ozaki_crt_f64(X, W, Y, batch, in_f, out_f, num_moduli, 0);
    if (rc != 0) return rc;
    for (uint64_t i = 0; i < batch; i++)
        for (uint64_t j = 0; j < out_f; j++) {
            double v = Y[i * out_f + j];
            if (b) v = v + b[j];
            Y[i * out_f + j] = tanh(v);
        }
    return 0;
}
