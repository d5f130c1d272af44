"""java.util.Random restated in the library (omega_jrandom_*, host code): known answers of the Java class library,
an independent Python restatement of the specified algorithm, and the RandomUtils.normal_ composition.  CPU only."""
import importlib
import math

import numpy as np

JR = importlib.import_module("omega-ai_amd.java_random")

MASK = (1 << 48) - 1


class PyRandom:
    """The algorithm as the Java SE specification of java.util.Random states it, in plain Python integers."""

    def __init__(self, seed):
        self.s = (seed ^ 0x5DEECE66D) & MASK
        self.nxt = None

    def next(self, bits):
        self.s = (self.s * 0x5DEECE66D + 0xB) & MASK
        v = self.s >> (48 - bits)
        return v - (1 << bits) if v >= 1 << (bits - 1) and bits == 32 else v

    def nextDouble(self):
        return ((self.next(26) << 27) + self.next(27)) * 2.0 ** -53

    def polar_pair(self):
        while True:
            v1, v2 = 2 * self.nextDouble() - 1, 2 * self.nextDouble() - 1
            s = v1 * v1 + v2 * v2
            if 0 < s < 1:
                return v1, v2, s


def test_known_answers_of_the_java_class_library():
    # new Random(0) / new Random(42): first nextInt(), nextDouble(), nextGaussian() as every JDK prints them
    for seed, ni, nd, g in ((0, -1155484576, 0.730967787376657, [0.8025330637390305, -0.9015460884175122, 2.080920790428163]),
                            (42, -1170105035, 0.7275636800328681, [1.1419053154730547])):
        assert JR.JavaRandom(seed).nextInt() == ni
        assert JR.JavaRandom(seed).nextDouble() == nd
        r = JR.JavaRandom(seed)
        assert [r.nextGaussian() for _ in g] == g
    # (the last one separates StrictMath.log = fdlibm from glibc's log, which gives one unit in the last place more)


def test_matches_the_specified_algorithm():
    for seed in (1, -7, 2**40 + 3, 123456789):
        a, b = JR.JavaRandom(seed), PyRandom(seed)
        assert [a.nextInt() for _ in range(50)] == [b.next(32) for _ in range(50)]
        assert [a.nextDouble() for _ in range(50)] == [b.nextDouble() for _ in range(50)]
        # nextGaussian: same uniform draws and rejections; the value within one ulp of libm's (fdlibm's log is not
        # correctly rounded, neither is it wrong by more than one unit)
        a, b = JR.JavaRandom(seed), PyRandom(seed)
        for _ in range(200):
            v1, v2, s = b.polar_pair()
            m = math.sqrt(-2 * math.log(s) / s)
            g1, g2 = a.nextGaussian(), a.nextGaussian()            # the second comes from the kept value
            assert abs(g1 - v1 * m) <= 2 * math.ulp(g1) and abs(g2 - v2 * m) <= 2 * math.ulp(g2)
    # setSeed drops the kept second value
    a = JR.JavaRandom(5)
    a.nextGaussian()
    a.setSeed(5)
    assert a.nextGaussian() == JR.JavaRandom(5).nextGaussian()


def test_normal_is_randomutils_normal():
    r = JR.JavaRandom(42)
    got = r.normal_(1001, 0.01, 0.02)
    r2 = JR.JavaRandom(42)
    want = np.array([np.float32(float(np.float32(0.02)) * r2.nextGaussian() + float(np.float32(0.01))) for _ in range(1001)],
                    np.float32)
    assert np.array_equal(got, want)
    assert got[0] == np.float32(float(np.float32(0.02)) * 1.1419053154730547 + float(np.float32(0.01)))
    big = JR.JavaRandom(7).normal_(400000, 0.01, 0.02).astype(np.float64)
    assert abs(big.mean() - 0.01) < 5 * 0.02 / math.sqrt(big.size) and abs(big.std() - 0.02) < 5 * 0.02 / math.sqrt(2 * big.size)


def test_house_style_init_order():
    class Rec:
        embedDim, hidden, nExperts, nShared, hasBias = 6, 4, 3, 1, False

        def __init__(self):
            self.calls = []

        def set_gate(self, Wg, bg=None):
            self.calls.append(("gate", Wg.copy()))

        def set_expert(self, g, W1, W3, W2):
            self.calls.append((g, W1.copy(), W3.copy(), W2.copy()))

    rec = Rec()
    arrays = JR.init_layer(rec, JR.JavaRandom(99))
    flat = JR.JavaRandom(99).normal_(3 * 6 + 4 * 3 * 4 * 6, 0.01, 0.02)
    assert np.array_equal(rec.calls[0][1].ravel(), flat[:18])
    o = 18
    for g in range(4):                                             # linear1, linear2, linear3 = W1, W2, W3
        _, W1, W3, W2 = rec.calls[1 + g]
        assert np.array_equal(W1.ravel(), flat[o:o + 24]) and W1.shape == (4, 6)
        assert np.array_equal(W2.ravel(), flat[o + 24:o + 48]) and W2.shape == (6, 4)
        assert np.array_equal(W3.ravel(), flat[o + 48:o + 72])
        o += 72
    assert arrays["W2"].shape == (4, 6, 4)
