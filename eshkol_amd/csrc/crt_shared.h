/*
 * Pieces the two CRT tiers (exact: ozaki_crt.hip, fast: ozaki_fast.hip) share:
 * the byte form of a scaled operand element, the byte weights of a modulus, and
 * the host-side hand-off of the row and column maxima's exponents.
 */
#ifndef ESHKOL_HIP_CRT_SHARED_H
#define ESHKOL_HIP_CRT_SHARED_H

#include <hip/hip_runtime.h>
#include <stdint.h>

/* An integer s of magnitude below 2^53 as eight bytes: the low seven of its
 * 64-bit two's complement, and 1 or 0 in the eighth for negative or not. Its
 * value is sum_{i<7} b_i 256^i - b_7 256^7. */
struct Scaled { uint32_t lo, hi; };

/* x * 2^sh as such an integer, read straight off the bit pattern of x (sh is
 * chosen by the callers so that the magnitude stays below 2^53).
 * HALF_UP false: truncated towards zero (the exact tier, gpu_memory.mm:2560-2590);
 * subnormal x are scaled like any other value.
 * HALF_UP true: magnitude rounded half up, subnormal x count as zero (the fast
 * tier's split, metal_softfloat.h:4148-4178). */
template <bool HALF_UP>
__device__ __forceinline__ Scaled scaled_integer(double x, int sh) {
    const uint64_t bits = __double_as_longlong(x);
    const int e = (int)((bits >> 52) & 0x7ff);
    uint64_t mant = bits & 0xfffffffffffffull;
    int e_eff = 1;
    if (e != 0) { mant |= 1ull << 52; e_eff = e; }
    else if (HALF_UP) mant = 0;
    const int rs = 1075 - e_eff - sh;          /* value = mant * 2^-rs; rs <= 0 is excluded by the callers */
    uint64_t t = mant;
    if (HALF_UP) {
        if (rs > 53) t = 0;
        else if (rs > 0) t = (mant + (1ull << (rs - 1))) >> rs;
    } else {
        if (rs >= 64) t = 0;
        else if (rs > 0) t = mant >> rs;
    }
    const uint64_t m = (uint64_t)((int64_t)bits >> 63);
    const uint64_t v = (t ^ m) - m;
    return { (uint32_t)v, (uint32_t)(v >> 32) & 0x01ffffffu };
}

/* Byte weights of a modulus p <= 256: 256^i mod p for the seven magnitude bytes
 * and -(256^7) mod p for the sign byte, four to a word, so that two
 * v_dot4_u32_u8 give x = sum b_i w_i < 2^19 congruent to the integer. */
struct ByteWeights { uint32_t lo, hi; };
constexpr ByteWeights byte_weights(int modulus) {
    const uint32_t p = (uint32_t)modulus;
    uint32_t c[8] = {}, pw = 1u % p;
    for (int i = 0; i < 8; i++) { c[i] = pw; pw = pw * 256u % p; }
    c[7] = (p - c[7]) % p;
    return { c[0] | c[1] << 8 | c[2] << 16 | c[3] << 24, c[4] | c[5] << 8 | c[6] << 16 | c[7] << 24 };
}

/* One step of a maximum of magnitudes. A NaN or an infinity anywhere makes the result
 * +inf, which the tiers read as "not representable, use the native GEMM". */
__device__ __forceinline__ void eshkol_absmax_step(double v, double* m) {
    const double a = fabs(v);
    if (!(a <= 1.7976931348623157e308)) *m = __builtin_inf();
    else if (a > *m) *m = a;
}

/* E - floor(log2 m) for a maximum m > 0 (exponent field; subnormals by their
 * leading bit), 0 for m = 0: the per-row shift of the CRT tiers when E does not
 * depend on the operands (gpu_memory.mm:2524-2532). */
__device__ __forceinline__ int32_t eshkol_shift_of_maximum(double m, int E) {
    if (!(m > 0.0)) return 0;
    const unsigned long long bits = (unsigned long long)__double_as_longlong(m);
    const int ef = (int)(bits >> 52);
    const int e = ef ? ef - 1023 : (63 - __clzll((long long)(bits & 0xfffffffffffffull))) - 1074;
    return E - e;
}

/* ---- maxima with the shifts beside them (implemented in elementwise.hip) ------------
 * hip_rowabsmax_f64 / hip_colabsmax_f64 that also write, when shift is not null,
 * shift[i] = E - floor(log2 max_i) (0 for a maximum of zero): what the split of a
 * CRT tier needs when its exponent E is known before the operands are looked at. */
int eshkol_rowabsmax_shift_f64(const double* A, uint64_t M, uint64_t K, double zero_value,
                               double* rmax, int32_t* shift, int E, hipStream_t stream, hipEvent_t done = nullptr);
int eshkol_colabsmax_shift_f64(const double* X, uint64_t K, uint64_t R, double zero_value,
                               double* cmax, int32_t* shift, int E, hipStream_t stream, hipEvent_t done = nullptr);
/* done, when given, becomes the completion event of the launch's last kernel
 * (the kernel's own completion signal: no marker is queued behind it, which
 * would hold the next kernel of the stream back by 6-7 us). */

/* ---- exponents of the maxima (implemented in ozaki_crt.hip) ---------------------- */

/* What the host learns about one operand's row (or column) maxima. */
struct CrtMaxima {
    int nonfinite;              /* a NaN or an infinity among them */
    int nonzero;                /* at least one maximum > 0 */
    int e_min, e_max;           /* range of floor(log2 max) over the maxima > 0 */
};
constexpr int32_t CRT_FL_ZERO = INT32_MIN;      /* exponent entry of a maximum of zero */

/* Queues the scan of the two vectors of maxima for its summary (a NaN or an
 * infinity among them? the range of their exponents), on a stream of the
 * library's own behind everything queued on st so far: what follows on st does
 * not wait for it. The summary is written to host memory by the device; ask for
 * it after queueing the rest of the pipeline. Returns the summary's ticket, 0 on
 * failure. For callers whose shifts came with the maxima (above). For a small
 * product (operand_elems = M K + K N) the scan is queued on st itself: there the
 * device waits for the host, and three calls cost more than ten microseconds in line. */
uint32_t eshkol_crt_scan_launch_aside(const double* amax, uint64_t M, const double* bmax, uint64_t N, hipStream_t st,
                                      uint64_t operand_elems, bool event_attached = false);
/* The event the side stream waits for before that scan, or null when a product of
 * this size has its scan queued in line. A caller that hands it to the launcher
 * of the last maxima kernel (`done` above) passes event_attached = true and
 * spares the stream a marker; otherwise the event is recorded behind st. */
hipEvent_t eshkol_crt_scan_event(uint64_t operand_elems);
/* The two CRT tiers print one marker line per call, as the reference does per
 * dispatch (gpu_memory.mm:2503; its gates count those lines). A dispatcher that
 * runs one product as several calls (row panels) lets the first call print and
 * silences the rest with this switch. */
void eshkol_crt_set_quiet(int quiet);
int eshkol_crt_quiet(void);

/* Waits for that summary and fills out[0] (A) and out[1] (B). 0 on success. */
int eshkol_crt_scan_result(uint32_t ticket, CrtMaxima out[2], hipStream_t st);

#endif
