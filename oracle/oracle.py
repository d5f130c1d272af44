"""ctypes front end of the C oracle (oracle/libomega_oracle.so).

Test infrastructure only: imported by tests/, by the smoke check and by the benchmark's
cpu_baseline leg; never by the shipped package.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libomega_oracle.so")


def build(force=False):
    """Compile the oracle with gcc (seconds)."""
    if force or not os.path.exists(_SO):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"], stdout=subprocess.DEVNULL)
    return _SO


_lib = None

_f = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")


def lib():
    global _lib
    if _lib is None:
        build()
        L = C.CDLL(_SO)
        L.orc_stream_key.restype = C.c_uint64
        L.orc_stream_key.argtypes = [C.c_uint64, C.c_uint64]
        L.orc_fill_normal.argtypes = [_f, C.c_uint64, C.c_uint64, C.c_uint64, C.c_double, C.c_uint64]
        L.orc_round_bf16.argtypes = [_f, C.c_uint64]
        L.orc_gate.argtypes = [_f, _f, C.c_void_p, C.c_int, C.c_int, C.c_int, _f]
        L.orc_softmax.argtypes = [_f, C.c_int, C.c_int, _f]
        L.orc_topk.argtypes = [_f, C.c_int, C.c_int, C.c_int, C.c_int, _i, _f]
        L.orc_dispatch.argtypes = [_i, C.c_int, C.c_int, C.c_int, _i, _i, _i, _i]
        L.orc_gather.argtypes = [_f, _i, C.c_int, C.c_int, _f]
        L.orc_swiglu_rows.argtypes = [_f, C.c_int, _f, _f, _f, C.c_int, C.c_int, C.c_int, _f, _f]
        L.orc_combine.argtypes = [_f, _i, _f, C.c_void_p, C.c_int, C.c_int, C.c_int, C.c_int, C.c_int, _f]
        L.orc_moe_tokens.argtypes = [_f, _i, _f, _f, _f, _f] + [C.c_int] * 6 + [_i, C.c_int, _f]
        L.orc_moe_forward.argtypes = [_f, _f, C.c_void_p, _f, _f, _f] + [C.c_int] * 8 + [_f, _f, _i, _f, _i, _i, _i, _i, _f]
        L.orc_rmsnorm.argtypes = [_f, _f, C.c_int, C.c_int, C.c_int, _f, _f]
        L.orc_block_tokens.argtypes = [_f, _f, _i, _f, _f, _f, _f] + [C.c_int] * 6 + [_i, C.c_int, _f]
        L.orc_block_forward.argtypes = ([_f, _f, _f, C.c_void_p, _f, _f, _f] + [C.c_int] * 8
                                        + [_f, _f, _f, _f, _i, _f, _i, _i, _i, _i, _f])
        L.orc_moe_backward.argtypes = ([_f, _f, _f, C.c_void_p, _f, _f, _f] + [C.c_int] * 8
                                       + [_f, _f, C.c_void_p, _f, _f, _f, _f, _f])
        L.orc_moe_backward_routed.argtypes = ([_f, _f, _f, _f, _i, _i, _f, _f, _f, _f] + [C.c_int] * 9 + [_f, _f, _f])
        L.orc_rmsnorm_backward.argtypes = [_f, _f, _f, _f, C.c_void_p, C.c_int, C.c_int, C.c_int, _f, _f]
        L.orc_block_backward.argtypes = ([_f, _f, _f, _f, C.c_void_p, _f, _f, _f] + [C.c_int] * 8
                                         + [_f, _f, _f, C.c_void_p, _f, _f, _f, _f])
        L.orc_adamw_correction.restype = C.c_float
        L.orc_adamw_correction.argtypes = [C.c_float, C.c_int]
        L.orc_adamw.argtypes = [_f, _f, _f, _f, C.c_long] + [C.c_float] * 7
        L.orc_cpu_baseline_forward.restype = C.c_double
        L.orc_cpu_baseline_forward.argtypes = [_f, _f, C.c_void_p, _f, _f, _f] + [C.c_int] * 8 + [_f]
        L.orc_cpu_sgemm_tn.argtypes = [C.c_int, C.c_int, C.c_int, _f, C.c_int, _f, C.c_int, _f, C.c_int, C.c_int]
        _lib = L
    return _lib


def _opt(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def fill_normal(n, seed, stream, std, first=0):
    out = np.empty(int(n), np.float32)
    lib().orc_fill_normal(out, int(n), int(seed), int(stream), float(std), int(first))
    return out


def round_bf16(a):
    out = np.ascontiguousarray(a, np.float32).copy()
    lib().orc_round_bf16(out.reshape(-1), out.size)
    return out


def gate(x, Wg, bg=None):
    T, d = x.shape
    E = Wg.shape[0]
    out = np.empty((T, E), np.float32)
    lib().orc_gate(x, Wg, _opt(bg), T, d, E, out)
    return out


def softmax(logits):
    T, E = logits.shape
    out = np.empty((T, E), np.float32)
    lib().orc_softmax(np.ascontiguousarray(logits), T, E, out)
    return out


def topk(p, K, renorm):
    T, E = p.shape
    ids = np.empty((T, K), np.int32)
    w = np.empty((T, K), np.float32)
    lib().orc_topk(np.ascontiguousarray(p), T, E, K, int(renorm), ids, w)
    return ids, w


def dispatch(ids, E):
    T, K = ids.shape
    counts = np.empty(E, np.int32)
    offsets = np.empty(E + 1, np.int32)
    dst = np.empty(T * K, np.int32)
    src_row = np.empty(T * K, np.int32)
    lib().orc_dispatch(np.ascontiguousarray(ids), T, K, E, counts, offsets, dst, src_row)
    return counts, offsets, dst, src_row


def swiglu_rows(xg, W1, W3, W2, bf16=False):
    rows, d = xg.shape
    H = W1.shape[0]
    y = np.empty((rows, d), np.float32)
    lib().orc_swiglu_rows(np.ascontiguousarray(xg), rows, W1, W3, W2, d, H, int(bf16), y, np.empty(H, np.float32))
    return y


def moe_tokens(x, ids, w, W1, W3, W2, E, Es, tokens, bf16=False):
    """Layer output for the listed tokens only (routing given)."""
    T, d = x.shape
    K = ids.shape[1]
    H = W1.shape[1]
    tok = np.ascontiguousarray(tokens, np.int32)
    out = np.empty((len(tok), d), np.float32)
    lib().orc_moe_tokens(x, np.ascontiguousarray(ids), np.ascontiguousarray(w), W1, W3, W2, d, H, E, K, Es,
                         int(bf16), tok, len(tok), out)
    return out


def moe_forward(x, Wg, bg, W1, W3, W2, K, renorm, Es=0, bf16=False):
    """Whole layer; W1,W3: [E+Es,H,d], W2: [E+Es,d,H]. Returns a dict of every intermediate."""
    T, d = x.shape
    E = Wg.shape[0]
    H = W1.shape[1]
    P = T * K
    r = dict(logits=np.empty((T, E), np.float32), p=np.empty((T, E), np.float32), ids=np.empty((T, K), np.int32),
             w=np.empty((T, K), np.float32), counts=np.empty(E, np.int32), offsets=np.empty(E + 1, np.int32),
             dst=np.empty(P, np.int32), src_row=np.empty(P, np.int32), out=np.empty((T, d), np.float32))
    lib().orc_moe_forward(x, Wg, _opt(bg), W1, W3, W2, T, d, E, K, H, Es, int(renorm), int(bf16), r["logits"],
                          r["p"], r["ids"], r["w"], r["counts"], r["offsets"], r["dst"], r["src_row"], r["out"])
    return r


def rmsnorm(x, gamma, bf16=False):
    """Pre-norm of the block: returns (h [T,d], rms [T])."""
    T, d = x.shape
    h, rms = np.empty((T, d), np.float32), np.empty(T, np.float32)
    lib().orc_rmsnorm(np.ascontiguousarray(x), np.ascontiguousarray(gamma, np.float32), T, d, int(bf16), h, rms)
    return h, rms


def block_tokens(x, h, ids, w, W1, W3, W2, E, Es, tokens, bf16=False):
    """x + layer(h) for the listed tokens only (h = rmsnorm(x) for all tokens, routing given)."""
    T, d = x.shape
    K = ids.shape[1]
    H = W1.shape[1]
    tok = np.ascontiguousarray(tokens, np.int32)
    out = np.empty((len(tok), d), np.float32)
    lib().orc_block_tokens(x, np.ascontiguousarray(h), np.ascontiguousarray(ids), np.ascontiguousarray(w), W1, W3, W2,
                           d, H, E, K, Es, int(bf16), tok, len(tok), out)
    return out


def block_forward(x, gamma, Wg, bg, W1, W3, W2, K, renorm, Es=0, bf16=False):
    """out = x + layer(rmsnorm(x)); returns every intermediate, including h and rms."""
    T, d = x.shape
    E = Wg.shape[0]
    H = W1.shape[1]
    P = T * K
    r = dict(h=np.empty((T, d), np.float32), rms=np.empty(T, np.float32), logits=np.empty((T, E), np.float32),
             p=np.empty((T, E), np.float32), ids=np.empty((T, K), np.int32), w=np.empty((T, K), np.float32),
             counts=np.empty(E, np.int32), offsets=np.empty(E + 1, np.int32), dst=np.empty(P, np.int32),
             src_row=np.empty(P, np.int32), out=np.empty((T, d), np.float32))
    lib().orc_block_forward(x, np.ascontiguousarray(gamma, np.float32), Wg, _opt(bg), W1, W3, W2, T, d, E, K, H, Es,
                            int(renorm), int(bf16), r["h"], r["rms"], r["logits"], r["p"], r["ids"], r["w"],
                            r["counts"], r["offsets"], r["dst"], r["src_row"], r["out"])
    return r


def moe_backward(x, dout, Wg, bg, W1, W3, W2, K, renorm, Es=0, bf16=False):
    """Backward of the whole layer for the output gradient dout [T,d]; the forward quantities are recomputed.
    Returns dict(dx, dWg, dbg (None without bias), dW1, dW3, dW2, dw [T,K], dlogits [T,E])."""
    T, d = x.shape
    E = Wg.shape[0]
    G, H = W1.shape[0], W1.shape[1]
    r = dict(dx=np.empty((T, d), np.float32), dWg=np.empty((E, d), np.float32),
             dbg=None if bg is None else np.empty(E, np.float32), dW1=np.empty((G, H, d), np.float32),
             dW3=np.empty((G, H, d), np.float32), dW2=np.empty((G, d, H), np.float32),
             dw=np.empty((T, K), np.float32), dlogits=np.empty((T, E), np.float32))
    lib().orc_moe_backward(x, np.ascontiguousarray(dout, np.float32), Wg, _opt(bg), W1, W3, W2, T, d, E, K, H, Es,
                           int(renorm), int(bf16), r["dx"], r["dWg"], _opt(r["dbg"]), r["dW1"], r["dW3"], r["dW2"],
                           r["dw"], r["dlogits"])
    return r


def moe_backward_routed(x, dout, Wg, p, ids, wid, w, W1, W3, W2, Es, renorm, bf16=False):
    """Backward for a few tokens of a larger batch with their routing given: p [n,E] gate probabilities, ids [n,K]
    experts as the gate numbers them, wid [n,K] the same experts as indices into W1/W3/W2 (Ew routed experts, then Es
    shared), w [n,K].  Returns dict(dx, dw, dlogits)."""
    n, d = x.shape
    E, K, H, Ew = p.shape[1], ids.shape[1], W1.shape[1], W1.shape[0] - Es
    r = dict(dx=np.empty((n, d), np.float32), dw=np.empty((n, K), np.float32), dlogits=np.empty((n, E), np.float32))
    c = np.ascontiguousarray
    lib().orc_moe_backward_routed(c(x, np.float32), c(dout, np.float32), c(Wg, np.float32), c(p, np.float32),
                                  c(ids, np.int32), c(wid, np.int32), c(w, np.float32), c(W1), c(W3), c(W2), n, d, E, Ew, K,
                                  H, Es, int(renorm), int(bf16), r["dx"], r["dw"], r["dlogits"])
    return r


def rmsnorm_backward(x, dh, gamma, rms, resid=None, bf16=False):
    """Backward of the pre-norm: returns (dx [T,d], dgamma [d]); resid (the gradient that bypasses the norm) is added to dx."""
    T, d = x.shape
    dx, dg = np.empty((T, d), np.float32), np.empty(d, np.float32)
    c = np.ascontiguousarray
    lib().orc_rmsnorm_backward(c(x, np.float32), c(dh, np.float32), c(gamma, np.float32), c(rms, np.float32),
                               _opt(None if resid is None else c(resid, np.float32)), T, d, int(bf16), dx, dg)
    return dx, dg


def block_backward(x, gamma, dout, Wg, bg, W1, W3, W2, K, renorm, Es=0, bf16=False):
    """Backward of out = x + layer(rmsnorm(x)).  Returns dict(dx, dgamma, dWg, dbg, dW1, dW3, dW2, dh)."""
    T, d = x.shape
    E = Wg.shape[0]
    G, H = W1.shape[0], W1.shape[1]
    r = dict(dx=np.empty((T, d), np.float32), dgamma=np.empty(d, np.float32), dWg=np.empty((E, d), np.float32),
             dbg=None if bg is None else np.empty(E, np.float32), dW1=np.empty((G, H, d), np.float32),
             dW3=np.empty((G, H, d), np.float32), dW2=np.empty((G, d, H), np.float32), dh=np.empty((T, d), np.float32))
    c = np.ascontiguousarray
    lib().orc_block_backward(c(x, np.float32), c(gamma, np.float32), c(dout, np.float32), Wg, _opt(bg), W1, W3, W2, T, d, E,
                             K, H, Es, int(renorm), int(bf16), r["dx"], r["dgamma"], r["dWg"], _opt(r["dbg"]), r["dW1"],
                             r["dW3"], r["dW2"], r["dh"])
    return r


def adamw(w, grad, mw, vw, lr, beta1, beta2, wd, train_time, eps=1e-8):
    """One AdamW step of the reference's adamw_kernel on flat copies; returns (w, mw, vw) as new arrays."""
    w, mw, vw = (np.ascontiguousarray(a, np.float32).copy().reshape(-1) for a in (w, mw, vw))
    g = np.ascontiguousarray(grad, np.float32).reshape(-1)
    L = lib()
    L.orc_adamw(w, g, mw, vw, w.size, lr, beta1, beta2, L.orc_adamw_correction(beta1, train_time),
                L.orc_adamw_correction(beta2, train_time), eps, wd)
    shape = np.shape(grad)
    return w.reshape(shape), mw.reshape(shape), vw.reshape(shape)


def cpu_baseline_forward(x, Wg, bg, W1, W3, W2, K, renorm, Es, n_threads):
    """Reference-CPU-style forward (column-major j8->p->i sgemm, one task per expert). Returns (seconds, out)."""
    T, d = x.shape
    E = Wg.shape[0]
    H = W1.shape[1]
    out = np.empty((T, d), np.float32)
    s = lib().orc_cpu_baseline_forward(x, Wg, _opt(bg), W1, W3, W2, T, d, E, K, H, Es, int(renorm), int(n_threads), out)
    return s, out


def cpu_sgemm_tn(A, B, n_threads=1):
    """Column-major C[m,n] = A^T B with A stored [k,m] col-major == row-major [m,k]; B row-major [n,k].
    Returns row-major [n,m]."""
    m, k = A.shape
    n = B.shape[0]
    Cm = np.zeros((n, m), np.float32)
    lib().orc_cpu_sgemm_tn(m, n, k, np.ascontiguousarray(A), k, np.ascontiguousarray(B), k, Cm, m, n_threads)
    return Cm
