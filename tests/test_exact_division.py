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
