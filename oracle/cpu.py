"""numpy front end of oracle/kernels.cpp (ctypes). Test infrastructure only.

Every wrapper takes and returns C-contiguous numpy arrays; float arrays are
float32, token ids / targets uint32. The reference citations live next to the
C++ functions.
"""
import ctypes as C
import os

import numpy as np

from . import build as _build

_lib = None

_f = np.float32
_FP = C.POINTER(C.c_float)
_U32P = C.POINTER(C.c_uint32)
_U16P = C.POINTER(C.c_uint16)
_SZ = C.c_size_t


def lib():
    global _lib
    if _lib is None:
        path = _build.LIB
        if not os.path.exists(path):
            path = _build.build()
        _lib = C.CDLL(path)
        _lib.orc_sum_squares_partial.restype = _SZ
        _lib.orc_num_threads.restype = C.c_int
    return _lib


def _p(a):
    return a.ctypes.data_as(_FP)


def _c(a, dtype=_f):
    return np.ascontiguousarray(a, dtype=dtype)


def num_threads():
    return int(lib().orc_num_threads())


def set_num_threads(n):
    lib().orc_set_num_threads(C.c_int(int(n)))


def pack_f16(x):
    """f32 -> f16 bit patterns (uint16), round to nearest even."""
    x = _c(x)
    out = np.empty(x.shape, dtype=np.uint16)
    lib().orc_pack_f16(_p(x), out.ctypes.data_as(_U16P), _SZ(x.size))
    return out


def unpack_f16(bits):
    bits = _c(bits, np.uint16)
    out = np.empty(bits.shape, dtype=_f)
    lib().orc_unpack_f16(bits.ctypes.data_as(_U16P), _p(out), _SZ(bits.size))
    return out


def round_f16(x):
    """The f32 values an f16-stored weight holds."""
    return unpack_f16(pack_f16(x))


def transpose(x):
    x = _c(x)
    rows, cols = x.shape
    out = np.empty((cols, rows), dtype=_f)
    lib().orc_transpose(_p(x), _p(out), _SZ(rows), _SZ(cols))
    return out


def matmul(a, b):
    """a[M,K] @ b[K,N]."""
    a, b = _c(a), _c(b)
    M, K = a.shape
    K2, N = b.shape
    assert K == K2, (a.shape, b.shape)
    out = np.empty((M, N), dtype=_f)
    lib().orc_matmul(_p(a), _p(b), _p(out), _SZ(M), _SZ(K), _SZ(N), C.c_int(0))
    return out


def matmul_bt(a, b):
    """a[M,K] @ b[N,K]^T."""
    a, b = _c(a), _c(b)
    M, K = a.shape
    N, K2 = b.shape
    assert K == K2, (a.shape, b.shape)
    out = np.empty((M, N), dtype=_f)
    lib().orc_matmul(_p(a), _p(b), _p(out), _SZ(M), _SZ(K), _SZ(N), C.c_int(1))
    return out


def matmul_at(a, b):
    """a[K,M]^T @ b[K,N]."""
    a, b = _c(a), _c(b)
    K, M = a.shape
    K2, N = b.shape
    assert K == K2, (a.shape, b.shape)
    out = np.empty((M, N), dtype=_f)
    lib().orc_matmul(_p(a), _p(b), _p(out), _SZ(M), _SZ(K), _SZ(N), C.c_int(2))
    return out


def rms_norm(x, w, eps):
    x, w = _c(x), _c(w)
    size = x.shape[-1]
    rows = x.size // size
    out = np.empty_like(x)
    lib().orc_rms_norm(_p(x), _p(w), _p(out), _SZ(rows), _SZ(size), C.c_float(eps))
    return out


def rms_norm_backward(x, w, g, eps):
    x, w, g = _c(x), _c(w), _c(g)
    size = x.shape[-1]
    rows = x.size // size
    gx = np.empty_like(x)
    gw = np.empty_like(w)
    lib().orc_rms_norm_backward(_p(x), _p(w), _p(g), _p(gx), _p(gw), _SZ(rows), _SZ(size),
                                C.c_float(eps))
    return gx, gw


def rope(x, head_dim, pos, theta, inverse=False):
    """Out of place; x is [batch, seq, hidden] or [seq, hidden]."""
    x = _c(x).copy()
    if x.ndim == 2:
        batch, (seq, hidden) = 1, x.shape
    else:
        batch, seq, hidden = x.shape
    lib().orc_rope(_p(x), _SZ(batch), _SZ(seq), _SZ(hidden), _SZ(head_dim), _SZ(pos),
                   C.c_float(theta), C.c_int(1 if inverse else 0))
    return x


def attention(q, k, v, causal=True, causal_offset=0):
    """q [B,Sq,H,D], k/v [B,Sk,Hkv,D] -> (out [B,Sq,H,D], lse [B,H,Sq])."""
    q, k, v = _c(q), _c(k), _c(v)
    B, Sq, H, D = q.shape
    _, Sk, Hkv, _ = k.shape
    out = np.empty_like(q)
    lse = np.empty((B, H, Sq), dtype=_f)
    lib().orc_attention(_p(q), _p(k), _p(v), _p(out), _p(lse), _SZ(B), _SZ(Sq), _SZ(Sk), _SZ(H),
                        _SZ(Hkv), _SZ(D), C.c_int(1 if causal else 0), _SZ(causal_offset))
    return out, lse


def attention_backward(q, k, v, out, d_out, causal=True, causal_offset=0):
    q, k, v, out, d_out = _c(q), _c(k), _c(v), _c(out), _c(d_out)
    B, Sq, H, D = q.shape
    _, Sk, Hkv, _ = k.shape
    dq = np.empty_like(q)
    dk = np.empty_like(k)
    dv = np.empty_like(v)
    lib().orc_attention_backward(_p(q), _p(k), _p(v), _p(out), _p(d_out), _p(dq), _p(dk), _p(dv),
                                 _SZ(B), _SZ(Sq), _SZ(Sk), _SZ(H), _SZ(Hkv), _SZ(D),
                                 C.c_int(1 if causal else 0), _SZ(causal_offset))
    return dq, dk, dv


def add(a, b):
    a, b = _c(a), _c(b)
    out = np.empty_like(a)
    lib().orc_add(_p(a), _p(b), _p(out), _SZ(a.size))
    return out


def scale(x, s):
    x = _c(x).copy()
    lib().orc_scale(_p(x), _SZ(x.size), C.c_float(s))
    return x


def silu_gate(a, b):
    """silu(a) * b."""
    a, b = _c(a), _c(b)
    out = np.empty_like(a)
    lib().orc_silu_gate(_p(a), _p(b), _p(out), _SZ(a.size))
    return out


def silu_gate_backward(a, b, g):
    a, b, g = _c(a), _c(b), _c(g)
    ga = np.empty_like(a)
    gb = np.empty_like(a)
    lib().orc_silu_gate_backward(_p(a), _p(b), _p(g), _p(ga), _p(gb), _SZ(a.size))
    return ga, gb


def embedding(table, ids):
    table = _c(table)
    ids = _c(ids, np.uint32)
    vocab, hidden = table.shape
    out = np.empty(ids.shape + (hidden,), dtype=_f)
    lib().orc_embedding(_p(table), _SZ(vocab), _SZ(hidden), ids.ctypes.data_as(_U32P),
                        _SZ(ids.size), _p(out))
    return out


def masked_cross_entropy(logits, targets, weights):
    """-> (grad [rows, vocab], row_loss [rows])."""
    logits = _c(logits)
    vocab = logits.shape[-1]
    rows = logits.size // vocab
    targets = _c(targets, np.uint32)
    weights = _c(weights)
    assert targets.size == rows and weights.size == rows
    grad = np.empty_like(logits)
    row_loss = np.empty(rows, dtype=_f)
    lib().orc_masked_cross_entropy(_p(logits), targets.ctypes.data_as(_U32P), _p(weights),
                                   _p(grad), _p(row_loss), _SZ(rows), _SZ(vocab))
    return grad, row_loss


def sum_squares_partial(x, out, offset):
    x = _c(x)
    return int(lib().orc_sum_squares_partial(_p(x), _SZ(x.size), _p(out), _SZ(offset)))


def adamw_update(w, g, m, v, lr, beta1=0.9, beta2=0.999, eps=1e-8, weight_decay=0.01, t=1.0):
    """In place on w, m, v (float32, C-contiguous)."""
    for a in (w, m, v):
        assert a.dtype == _f and a.flags.c_contiguous
    g = _c(g)
    lib().orc_adamw_update(_p(w), _p(g), _p(m), _p(v), _SZ(w.size), C.c_float(lr), C.c_float(beta1),
                           C.c_float(beta2), C.c_float(eps), C.c_float(weight_decay), C.c_float(t))
