"""Pins of the oracle's restatement of the reduced-precision CRT tier
(gpu_memory.mm:2802-3012, metal_softfloat.h:4126-4246). The reference's own
path needs Metal, so the restatement is pinned by what the mathematics fixes:
the moduli by their definition, the split by exact rational arithmetic in
Python, the products and the CRT identity by Python integers, and the
float-float reconstruction by its distance from the exact integer result."""
from fractions import Fraction
import math

import numpy as np
import pytest

import oracle
from eshkol_amd import synth


def prime_powers_upto(cap):
    out = []
    for p in range(2, cap + 1):
        if all(p % d for d in range(2, int(p ** 0.5) + 1)):
            v = p
            while v * p <= cap:
                v *= p
            out.append(v)
    return sorted(out, reverse=True)


@pytest.mark.parametrize("K", [1, 64, 512, 1000, 4096, 8192, 65536, 131071, 2 ** 22])
def test_cap_and_moduli(K):
    cap = oracle.lib().oracle_ozaki_fast_cap(oracle.u64(K))
    # the largest admissible p/2: one f32 GEMM of residues in [-p/2, p/2] stays exact
    assert cap <= 255 and K * (cap // 2) ** 2 < 2 ** 24
    assert cap >= 254 or K * ((cap + 2) // 2) ** 2 >= 2 ** 24
    assert cap == min(255, math.floor(2.0 * math.sqrt(2 ** 24 / K))) or K * ((cap + 1) // 2) ** 2 >= 2 ** 24
    for n in (2, 5, 11, 16):
        rc, c = oracle.fast_constants(K, n)
        if len(prime_powers_upto(cap)) < 2:
            assert rc == -4
            continue
        assert rc == 0
        mods = list(c.moduli[:c.num_moduli])
        assert mods == prime_powers_upto(cap)[:n]
        assert all(math.gcd(a, b) == 1 for i, a in enumerate(mods) for b in mods[i + 1:])
        P = math.prod(mods)
        assert c.P == float(P) and abs(c.log2P - math.log2(P)) < 1e-9
        assert c.E == min(52, max(1, math.floor((math.log2(P) - math.log2(K) - 2.0) / 2.0)))
        for p, q in zip(mods, c.q):
            assert (P // p) * q % p == 1
        assert float(c.P_hi) + float(c.P_lo) == pytest.approx(float(P), rel=2 ** -45)


def test_known_moduli_at_8192():
    rc, c = oracle.fast_constants(8192, 11)
    assert rc == 0 and c.cap == 90
    assert list(c.moduli[:11]) == [89, 83, 81, 79, 73, 71, 67, 64, 61, 59, 53]
    assert c.E == 26


def exact_scaled(x, e, E):
    """round-half-up(|x| 2^(E-e)) with the sign of x, in exact rational arithmetic."""
    if x == 0.0 or abs(x) < 2.0 ** -1022:
        return 0
    f = Fraction(abs(x)) * Fraction(2) ** (E - e)
    n = math.floor(f + Fraction(1, 2))
    return -n if x < 0 else n


@pytest.mark.parametrize("seed,shape", [(1, (5, 7, 4)), (2, (9, 33, 6)), (3, (16, 130, 12))])
def test_split_products_and_crt_identity(seed, shape):
    M, K, N = shape
    A, B = synth.wide_range(seed, (M, K), -12, 12), synth.wide_range(seed + 50, (K, N), -12, 12)
    A[0, :] = 0.0; A[1, 2] = 5e-324; A[2, 0] = -A[2, 0]; B[:, 1] = 0.0
    st = oracle.ozaki_fast_stages(A, B, 11)
    E, mods = st["E"], st["moduli"]
    for i in range(M):
        mx = np.abs(A[i]).max()
        assert st["ei"][i] == (0 if mx == 0 else math.frexp(mx)[1])
        for k in range(K):
            v = exact_scaled(A[i, k], int(st["ei"][i]), E)
            assert int(st["a_int"][i, k]) == v
            for l, p in enumerate(mods):
                r = int(st["a_planes"][l, i, k])
                assert (r - v) % p == 0 and -(p // 2) <= r <= p // 2 and (r != -(p // 2) or p % 2 == 1)
    for j in range(N):
        for k in range(K):
            assert int(st["b_int"][j, k]) == exact_scaled(B[k, j], int(st["fj"][j]), E)
    # exact products, and the CRT identity: the integer dot product is the unique class in (-P/2, P/2]
    P = math.prod(mods)
    for i in range(M):
        for j in range(N):
            V = sum(int(a) * int(b) for a, b in zip(st["a_int"][i], st["b_int"][j]))
            assert abs(V) < P // 2
            acc = 0
            for l, p in enumerate(mods):
                g = int(st["G"][l, i, j])
                assert g == sum(int(a) * int(b) for a, b in zip(st["a_planes"][l, i], st["b_planes"][l, j]))
                acc += (g % p) * st["q"][l] % p * (P // p)
            acc %= P
            if acc > P // 2:
                acc -= P
            assert acc == V
            want = float(Fraction(V) * Fraction(2) ** (int(st["ei"][i]) + int(st["fj"][j]) - 2 * E))
            assert st["C_exact"][i, j] == want
            # the float-float reconstruction: within 2^-40 of P at the element's scale
            tol = P * 2.0 ** (int(st["ei"][i]) + int(st["fj"][j]) - 2 * E - 40)
            assert abs(st["C"][i, j] - want) <= tol


def test_accuracy_of_the_tier_default_moduli():
    """The reference calls the default (11 moduli) its ~1e-8 tier."""
    A, B = synth.normal(7, (48, 600)), synth.normal(8, (600, 40))
    rc, Cf = oracle.matmul_ozaki_fast(A, B, 11)
    assert rc == 0
    ref = A @ B
    assert np.abs(Cf - ref).max() / np.abs(ref).max() < 5e-8
    # more moduli keep more bits of the operands, but the float-float reconstruction resolves
    # about 2^-45 of P whatever P is: past the point where P outgrows the products it stops helping
    rc, C16 = oracle.matmul_ozaki_fast(A, B, 16)
    assert rc == 0 and np.abs(C16 - ref).max() / np.abs(ref).max() < 5e-8
