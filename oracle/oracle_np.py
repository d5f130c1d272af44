"""Independent NumPy restatements used to pin the C oracle (test infrastructure only).

Nothing here calls the C oracle: each function is written from the definition (or from the
reference kernel text it cites) so that a mistake in either implementation shows up as a
mismatch in tests/test_oracle_*.py.
"""
import numpy as np

GAMMA = np.uint64(0x9E3779B97F4A7C15)
GAMMA2 = np.uint64(0xD1342543DE82EF95)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)

INV_ODD = [float.fromhex(h) for h in (
    "0x1.0000000000000p+0", "0x1.5555555555555p-2", "0x1.999999999999ap-3", "0x1.2492492492492p-3",
    "0x1.c71c71c71c71cp-4", "0x1.745d1745d1746p-4", "0x1.3b13b13b13b14p-4", "0x1.1111111111111p-4",
    "0x1.e1e1e1e1e1e1ep-5", "0x1.af286bca1af28p-5", "0x1.8618618618618p-5")]
INV_FACT = [float.fromhex(h) for h in (
    "0x1.0000000000000p+0", "0x1.0000000000000p+0", "0x1.0000000000000p-1", "0x1.5555555555555p-3",
    "0x1.5555555555555p-5", "0x1.1111111111111p-7", "0x1.6c16c16c16c17p-10", "0x1.a01a01a01a01ap-13",
    "0x1.a01a01a01a01ap-16", "0x1.71de3a556c734p-19", "0x1.27e4fb7789f5cp-22", "0x1.ae64567f544e4p-26",
    "0x1.1eed8eff8d898p-29", "0x1.6124613a86d09p-33", "0x1.93974a8c07c9dp-37", "0x1.ae7f3e733b81fp-41",
    "0x1.ae7f3e733b81fp-45", "0x1.952c77030ad4ap-49", "0x1.6827863b97d97p-53", "0x1.2f49b46814157p-57",
    "0x1.e542ba4020225p-62")]
LN2 = float.fromhex("0x1.62e42fefa39efp-1")
PI_4 = float.fromhex("0x1.921fb54442d18p-1")
SQRT_HALF = float.fromhex("0x1.6a09e667f3bcdp-1")


def _mix64(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def stream_key(seed, stream):
    with np.errstate(over="ignore"):
        s = np.array([stream], np.uint64) * GAMMA2 + np.uint64(1)
        return _mix64(np.array([seed], np.uint64) ^ _mix64(s))[0]


def fill_normal(n, seed, stream, std, first=0):
    """Counter-based N(0,std): SplitMix64 + Box-Muller in double with +,-,*,/,sqrt only."""
    with np.errstate(over="ignore"):
        key = stream_key(seed, stream)
        i = np.arange(first, first + n, dtype=np.uint64)
        h1 = _mix64(key + GAMMA * (np.uint64(2) * i + np.uint64(1)))
        h2 = _mix64(key + GAMMA * (np.uint64(2) * i + np.uint64(2)))
    u = ((h1 >> np.uint64(11)) + np.uint64(1)).astype(np.float64) * 2.0 ** -53
    m, e = np.frexp(u)
    low = m < SQRT_HALF
    m = np.where(low, m * 2.0, m)
    e = np.where(low, e - 1, e)
    s = (m - 1.0) / (m + 1.0)
    s2 = s * s
    p = np.full_like(s, INV_ODD[10])
    for k in range(9, -1, -1):
        p = p * s2 + INV_ODD[k]
    ln = e.astype(np.float64) * LN2 + 2.0 * s * p
    r = np.sqrt(-2.0 * ln)
    th = ((h2 >> np.uint64(8)) & np.uint64((1 << 53) - 1)).astype(np.float64) * 2.0 ** -53 * PI_4
    t2 = th * th
    c = np.full_like(th, INV_FACT[18])
    sn = np.full_like(th, INV_FACT[19])
    for k in range(8, -1, -1):
        c = INV_FACT[2 * k] - t2 * c
        sn = INV_FACT[2 * k + 1] - t2 * sn
    sn = th * sn
    z = r * np.where(((h2 >> np.uint64(62)) & np.uint64(1)) == 1, sn, c)
    z = np.where((h2 >> np.uint64(63)) == 1, -z, z)
    return (z * float(std)).astype(np.float32)


def round_bf16(a):
    """fp32 -> bf16 (round to nearest even) -> fp32."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = (u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))) & np.uint64(0xFFFF0000)
    return u.astype(np.uint32).view(np.float32).reshape(np.shape(a))


def to_bf16_bits(a):
    """fp32 array (already bf16-representable or not) -> uint16 bf16 bit patterns (RNE)."""
    return (round_bf16(a).view(np.uint32) >> 16).astype(np.uint16)


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, np.uint16).astype(np.uint32) << 16).view(np.float32)


def softmax_3pass(logits):
    """Row softmax exactly as the reference's thread-per-row kernel / safeSoftmax_3pass:
    max, e=(float)exp(x-max) with a running fp32 sum in index order, divide."""
    logits = np.asarray(logits, np.float32)
    mx = logits.max(axis=1, keepdims=True)
    e = np.exp((logits - mx).astype(np.float64)).astype(np.float32)
    s = np.zeros(logits.shape[0], np.float32)
    for i in range(logits.shape[1]):
        s = (s + e[:, i]).astype(np.float32)
    return (e / s[:, None]).astype(np.float32)


def topk_stable(p, K, renorm):
    """Top-k by stable descending sort: equal values keep ascending expert order."""
    ids = np.argsort(-p.astype(np.float64), axis=1, kind="stable")[:, :K].astype(np.int32)
    w = np.take_along_axis(p, ids, axis=1).astype(np.float32)
    if renorm:
        s = np.zeros(p.shape[0], np.float32)
        for j in range(K):
            s = (s + w[:, j]).astype(np.float32)
        w = (w / s[:, None]).astype(np.float32)
    return ids, w


def dispatch_argsort(ids, E):
    """counts / offsets / dst / src_row from a stable sort of the pair list by expert id."""
    T, K = ids.shape
    flat = ids.reshape(-1)
    counts = np.bincount(flat, minlength=E).astype(np.int32)
    offsets = np.concatenate([[0], np.cumsum(counts)]).astype(np.int32)
    order = np.argsort(flat, kind="stable")          # order[r] = pair placed at row r
    dst = np.empty(T * K, np.int32)
    dst[order] = np.arange(T * K, dtype=np.int32)
    src_row = (order // K).astype(np.int32)
    return counts, offsets, dst, src_row


def silu64(v):
    return v / (1.0 + np.exp(-v))


def dense_moe_fp64(x, ids, w, W1, W3, W2, E, Es=0):
    """Dense-MoE identity in fp64, no permutation anywhere:
    out[t] = sum_e [sum_j w[t,j]*(ids[t,j]==e)] * SwiGLU_e(x[t]) + sum_s SwiGLU_{E+s}(x[t])."""
    x = x.astype(np.float64)
    T, d = x.shape
    out = np.zeros((T, d))
    for e in range(E + Es):
        if e < E:
            coef = ((ids == e) * w.astype(np.float64)).sum(axis=1)
            sel = np.nonzero(coef != 0)[0] if True else None
            sel = np.nonzero((ids == e).any(axis=1))[0]
        else:
            coef = np.ones(T)
            sel = np.arange(T)
        if len(sel) == 0:
            continue
        xs = x[sel]
        h = silu64(xs @ W1[e].astype(np.float64).T) * (xs @ W3[e].astype(np.float64).T)
        out[sel] += coef[sel, None] * (h @ W2[e].astype(np.float64).T)
    return out


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-300))


def rmsnorm_lanes(x, gamma, bf16=False):
    """rmsnorm_forward_kernel2 (RMSKernel.cu:185-223) written from the kernel text: 32 lanes per row, lane l adds
    x[i]^2 for i = l, l+32, ... with one fused multiply-add per step, xor butterfly 16..1 over the lanes,
    rms = sqrt(sum/C + 1e-6), out = (x/rms)*weight - every operation rounded to float32 as the kernel does.
    (The fused multiply-add is emulated in float64: the product of two float32 is exact there.)"""
    x = np.asarray(x, np.float32)
    T, d = x.shape
    pad = (-d) % 32
    xp = np.concatenate([x, np.zeros((T, pad), np.float32)], axis=1).reshape(T, -1, 32)
    s = np.zeros((T, 32), np.float32)
    for j in range(xp.shape[1]):
        v = xp[:, j, :].astype(np.float64)
        s = (v * v + s.astype(np.float64)).astype(np.float32)
    lanes = np.arange(32)
    for m in (16, 8, 4, 2, 1):
        s = (s + s[:, lanes ^ m]).astype(np.float32)
    rms = np.sqrt((s[:, 0] / np.float32(d)).astype(np.float32) + np.float32(1e-6)).astype(np.float32)
    h = ((x / rms[:, None]).astype(np.float32) * np.asarray(gamma, np.float32)[None, :]).astype(np.float32)
    if bf16:
        h = round_bf16(h)
    return h, rms
