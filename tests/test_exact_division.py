"""The kernels divide by a chunk constant b as float(double(a) * y) with y ~= 1/b in double
(csrc/dq_tile16.cuh: div_by, div_exact).  Checked here on the host, in numpy's IEEE arithmetic, against the
binary32 division the reference's kernels perform (csrc/cuda_hierarchical_mee.cu:88-96): the product form is the
correctly rounded quotient whenever the quotient is a normal number, it is NOT for quotients that lie half-way
between two subnormal numbers, and the rule the kernels apply (a subnormal, non-zero product takes the division)
closes that gap.  The device's reciprocal is accurate to about one unit in the last place of a double, on either
side: every property is checked for the correctly rounded reciprocal and for its two neighbours."""
import numpy as np

F32_MIN_NORMAL = np.float32(2.0 ** -126)


def reciprocals(b):
    y = 1.0 / b.astype(np.float64)
    return [y, np.nextafter(y, np.inf), np.nextafter(y, -np.inf)]


def product_form(a, y):
    return (a.astype(np.float64) * y).astype(np.float32)


def corrected_form(a, b, y):
    """div_exact: the product, and the division itself where the product is a subnormal number other than zero"""
    q = product_form(a, y)
    sub = (np.abs(q) < F32_MIN_NORMAL) & (q != 0)
    with np.errstate(under="ignore"):
        return np.where(sub, a / b, q)


def same_bits(x, y):
    return x.view(np.uint32) == y.view(np.uint32)


def test_product_form_is_the_quotient_when_the_quotient_is_normal():
    rng = np.random.default_rng(1)
    n = 2_000_000
    # random significands and exponents, and quotients steered next to rounding boundaries: a = (k + 1/2) ulp * b
    a = rng.integers(1 << 23, 1 << 24, n).astype(np.float32) * np.float32(2.0) ** rng.integers(-60, 60, n).astype(np.float32)
    b = rng.integers(1 << 23, 1 << 24, n).astype(np.float32) * np.float32(2.0) ** rng.integers(-60, 60, n).astype(np.float32)
    near = ((rng.integers(1 << 23, 1 << 24, n) + 0.5) * b.astype(np.float64)).astype(np.float32)
    for num in (a, near, -a):
        want = num / b
        normal = np.abs(want) >= F32_MIN_NORMAL
        assert normal.all()
        for y in reciprocals(b):
            assert same_bits(product_form(num, y), want).all()


def tie_operands():
    """a / b = m 2^-150 with m odd: exactly half-way between two subnormal numbers"""
    a, b = [], []
    for e in range(1, 40):
        for D in (3, 5, 7, 9, 11, 13, 15, 255, 1785, 65535, 0x7fffff, 0xffffff):
            for m in (1, 3, 5, 7, 9, 255, 4097, (1 << 22) + 1, (1 << 23) - 1):
                bb = float(D) * 2.0 ** e
                aa = float(m) * float(D) * 2.0 ** (e - 150)
                if np.float32(aa) == aa and np.float32(bb) == bb and aa < 2.0 ** 100:
                    a.append(aa)
                    b.append(bb)
    return np.array(a, np.float32), np.array(b, np.float32)


def test_product_form_misses_ties_between_subnormal_numbers_and_the_corrected_form_does_not():
    a, b = tie_operands()
    assert a.size > 1000
    with np.errstate(under="ignore"):
        want = a / b
    assert (np.abs(want) < F32_MIN_NORMAL).all()
    missed = 0
    for y in reciprocals(b):
        missed += int((~same_bits(product_form(a, y), want)).sum())
        assert same_bits(corrected_form(a, b, y), want).all()
        assert same_bits(corrected_form(-a, b, y), -want).all()
    assert missed > 0  # the hazard is real: the error of the reciprocal decides a tie


def test_corrected_form_on_random_subnormal_quotients():
    rng = np.random.default_rng(2)
    n = 1_000_000
    b = rng.integers(1 << 23, 1 << 24, n).astype(np.float32) * np.float32(2.0) ** rng.integers(-20, 60, n).astype(np.float32)
    target = rng.integers(0, 1 << 24, n).astype(np.float64) * 2.0 ** -149 * rng.choice([1.0, 0.5, 0.25, 2.0 ** -10], n)
    a = (target * b.astype(np.float64)).astype(np.float32)
    with np.errstate(under="ignore"):
        want = a / b
    for y in reciprocals(b):
        assert same_bits(corrected_form(a, b, y), want).all()
        # a product that rounds to zero needs no division: the quotient rounds to zero as well
        q = product_form(a, y)
        assert (want[q == 0] == 0).all()


def test_sixteen_bit_elements_meet_no_tie_below_a_world_size_of_3_times_2_to_17():
    """bfloat16 elements are multiples of 2^-133: v / world = m 2^-150 with m odd needs world = D 2^e, e >= 17.  Checked by
    brute force over every positive bfloat16 pattern whose quotient is subnormal, for world sizes that are not powers of two."""
    pat = np.arange(1, 0x7f80, dtype=np.uint32)
    v = (pat << 16).view(np.float32)
    for world in (3, 5, 6, 7, 12, 24, 48, 96, 1000, 65535, 3 << 16, (1 << 17) + 2):
        w = np.float32(world)
        with np.errstate(under="ignore"):
            want = v / w
        for y in reciprocals(np.full(v.shape, w, np.float32)):
            assert same_bits(product_form(v, y), want).all(), world
    # ... and from 3 * 2^17 on there is one
    w = np.float32(3 << 17)
    v = np.array([3 * 2.0 ** -133], np.float32)
    assert (v.view(np.uint32) & 0xffff) == 0
    assert float(v[0]) / float(w) == 2.0 ** -150


# ---- binary16 operands: the corrected single-precision quotient of the binary16 encoders ------------------------------

def corrected_quotient(a, b, y):
    """div_half_operands (csrc/dq_scaling_tile16.hip): q0 = RN32(a y); rem = fma(-q0, b, a); RN32(fma(rem, y, q0)).  The two
    fused operations are evaluated in double: q0 b (24 x 11 bits) and a - q0 b are exact there, rem y (24 x 24 bits) too, and
    the last sum is rounded to double before it is rounded to binary32 -- where that could differ from the single rounding of
    the fused operation (the double lands on a binary32 tie) the caller's comparison falls back to exact fractions."""
    q0 = (a * y).astype(np.float32)
    rem = (a.astype(np.float64) - q0.astype(np.float64) * b.astype(np.float64))
    assert np.array_equal(rem.astype(np.float32).astype(np.float64), rem)          # the remainder fits binary32
    return (q0.astype(np.float64) + rem * y.astype(np.float64)).astype(np.float32)


def test_corrected_quotient_of_binary16_operands_is_the_binary32_quotient_for_every_pair_of_significands():
    """Every binary16 number is an 11-bit integer times a power of two, and scaling either operand by a power of two scales
    quotient, reciprocal and remainder exactly (no operand of the encoders brings them near the ends of the binary32
    range): all 1024 x 1024 pairs of normalised significands cover every pair of binary16 operands.  Checked for the
    reciprocal the kernels use, the double reciprocal rounded to binary32, which is RN32(1 / b) itself."""
    from fractions import Fraction
    sig = np.arange(1024, 2048, dtype=np.float32)
    a, b = (m.reshape(-1) for m in np.meshgrid(sig, sig, indexing="ij"))
    y64 = 1.0 / b.astype(np.float64)
    y = y64.astype(np.float32)
    for yd in reciprocals(b):                                   # the device's double reciprocal may be an ulp off
        assert np.array_equal(yd.astype(np.float32), y)
    got = corrected_quotient(a, b, y)
    want = a / b                                                # numpy's binary32 division is IEEE
    bad = np.flatnonzero(got != want)
    for i in bad:                                               # (the emulation's double rounding: settle exactly)
        q0 = Fraction(float(np.float32(a[i] * y[i])))
        exact = q0 + (Fraction(float(a[i])) - q0 * Fraction(float(b[i]))) * Fraction(float(y[i]))
        assert abs(exact - Fraction(float(want[i]))) <= abs(exact - Fraction(float(got[i]))), (a[i], b[i])
    assert bad.size < 8
    # and with a few scalings of the operands, subnormal binary16 numerators included
    for ea, eb in ((-24, 0), (-24, 15), (15, -24), (-10, 5), (0, -14)):
        a2, b2 = np.ldexp(a, ea).astype(np.float32), np.ldexp(b, eb).astype(np.float32)
        y2 = (1.0 / b2.astype(np.float64)).astype(np.float32)
        assert np.array_equal(corrected_quotient(a2, b2, y2) == a2 / b2, got == want)


def test_binary16_rounding_of_a_quotient_of_binary16_operands_sees_no_double_rounding():
    """RN16(RN32(a / b)) == RN16(a / b): a quotient of two 11-bit significands that is not itself a binary16 tie stays two
    binary32 ulps clear of every such tie, so the binary32 rounding in between never moves it onto or across one."""
    sig = np.arange(1024, 2048, dtype=np.float64)
    a, b = (m.reshape(-1) for m in np.meshgrid(sig, sig, indexing="ij"))
    q = a / b                                                   # double: 2^-53, far below the distances at stake
    once = q.astype(np.float16)
    twice = q.astype(np.float32).astype(np.float16)
    assert np.array_equal(once.view(np.uint16), twice.view(np.uint16))
