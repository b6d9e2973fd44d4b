"""ctypes bindings of the CPU oracle (liboracle.so) and, where it was built,
of the reference's own CPU path (_ref/libref.so).  TEST INFRASTRUCTURE: only
tests, the smoke check and the benchmark's CPU-baseline leg import this."""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
ROUND_ACT_BF16 = 1
PAR_TOKENS = 2

_f = np.ctypeslib.ndpointer(dtype=np.float32, flags="C_CONTIGUOUS")
_i = np.ctypeslib.ndpointer(dtype=np.int32, flags="C_CONTIGUOUS")
_u8 = np.ctypeslib.ndpointer(dtype=np.uint8, flags="C_CONTIGUOUS")


def build(force: bool = False) -> None:
    so = os.path.join(_HERE, "liboracle.so")
    if force or not os.path.exists(so):
        subprocess.check_call(["make", "-C", _HERE, "liboracle.so"] + (["-B"] if force else []))


def _opt(a, dtype):
    if a is None:
        return None
    assert a.dtype == dtype and a.flags["C_CONTIGUOUS"]
    return a.ctypes.data_as(C.c_void_p)


_lib = None


def _load(path):
    L = C.CDLL(path)
    L.oracle_f32_to_bf16.restype = C.c_uint16
    L.oracle_f32_to_bf16.argtypes = [C.c_float]
    L.oracle_bf16_to_f32.restype = C.c_float
    L.oracle_bf16_to_f32.argtypes = [C.c_uint16]
    L.oracle_round_to_bf16.argtypes = [_f, C.c_size_t]
    L.oracle_matmul.argtypes = [_f, _f, _f, C.c_int, C.c_int]
    L.oracle_topk.argtypes = [_f, _i, _f, C.c_int, C.c_int]
    L.oracle_softmax.argtypes = [_f, C.c_int]
    L.oracle_router.argtypes = [_f, C.c_void_p, _f, _f] + [C.c_int] * 4 + [_f, _i, _f]
    L.oracle_dispatch.argtypes = [_i, C.c_void_p] + [C.c_int] * 3 + [_i, _i, C.c_void_p]
    L.oracle_expert_token.argtypes = [_f] * 5 + [C.c_int, C.c_int, C.c_float, C.c_int, _f, _f]
    L.oracle_moe_layer.argtypes = ([_f, C.c_void_p] + [_f] * 6 + [C.c_int] * 5 +
                                       [C.c_float, C.c_int, _f, C.c_void_p, C.c_void_p, C.c_void_p])
    L.oracle_mxfp4_dequant.argtypes = [_u8, _u8, C.c_size_t, _f]
    L.oracle_rmsnorm.argtypes = [_f, _f, _f, C.c_int]
    L.oracle_num_threads.restype = C.c_int
    return L


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = _load(os.path.join(_HERE, "liboracle.so"))
    return _lib


def lib_native():
    """The restatement compiled on this host with -O3 -march=native -fopenmp (the
    flags of the reference's OpenMP build); built on first use.  Used by the
    benchmark's CPU-baseline leg only: the checker of the tests stays the
    portable build."""
    so = os.path.join(_HERE, "_native", "liboracle_native.so")
    subprocess.check_call(["make", "-s", "-B", "-C", _HERE, "native"])
    return _load(so)


def f32_to_bf16(x: float) -> int:
    return int(lib().oracle_f32_to_bf16(x))


def round_to_bf16(a: np.ndarray) -> np.ndarray:
    out = np.ascontiguousarray(a, dtype=np.float32).copy()
    lib().oracle_round_to_bf16(out.reshape(-1), out.size)
    return out


def matmul(x, w):
    d, n = w.shape
    out = np.empty(d, dtype=np.float32)
    lib().oracle_matmul(out, np.ascontiguousarray(x, np.float32), np.ascontiguousarray(w, np.float32), n, d)
    return out


def topk(score, K):
    score = np.ascontiguousarray(score, np.float32)
    v = np.zeros(K, np.float32)
    i = np.zeros(K, np.int32)
    lib().oracle_topk(v, i, score, score.shape[0], K)
    return v, i


def softmax(x):
    x = np.ascontiguousarray(x, np.float32).copy()
    lib().oracle_softmax(x, x.shape[0])
    return x


def router(x, pos, wr, br, K):
    T, H = x.shape
    E = wr.shape[0]
    score = np.zeros((T, E), np.float32)
    ti = np.zeros((T, K), np.int32)
    tv = np.zeros((T, K), np.float32)
    lib().oracle_router(x, _opt(pos, np.int32), wr, br, T, H, E, K, score, ti, tv)
    return score, ti, tv


def dispatch(topk_i, pos, E):
    T, K = topk_i.shape
    offsets = np.zeros(E + 1, np.int32)
    perm = np.full(T * K, -1, np.int32)
    inv = np.full(T * K, -1, np.int32)
    lib().oracle_dispatch(np.ascontiguousarray(topk_i, np.int32), _opt(pos, np.int32), T, E, K,
                          offsets, perm, inv.ctypes.data_as(C.c_void_p))
    return offsets, perm[:offsets[E]].copy(), inv.reshape(T, K)


def expert_token(t, w1, b1, w2, b2, limit, mode=0):
    H = t.shape[0]
    IM = w2.shape[1]
    scratch = np.zeros(3 * IM, np.float32)
    y = np.zeros(H, np.float32)
    lib().oracle_expert_token(t, w1, b1, w2, b2, H, IM, limit, mode, scratch, y)
    return y


def moe_layer(x, pos, wr, br, w1, b1, w2, b2, K, limit, mode=0, want_routing=False, use_lib=None):
    T, H = x.shape
    E = wr.shape[0]
    IM = w2.shape[2]
    out = np.zeros((T, H), np.float32)
    score = np.zeros((T, E), np.float32) if want_routing else None
    ti = np.zeros((T, K), np.int32) if want_routing else None
    tv = np.zeros((T, K), np.float32) if want_routing else None
    (use_lib or lib()).oracle_moe_layer(x, _opt(pos, np.int32), wr, br, w1, b1, w2, b2, T, H, IM, E, K,
                           limit, mode, out, _opt(score, np.float32), _opt(ti, np.int32),
                           _opt(tv, np.float32))
    return (out, score, ti, tv) if want_routing else out


def rmsnorm(x, weight):
    """Row-wise oracle_rmsnorm of x [T, H] (or [H])."""
    x2 = np.ascontiguousarray(np.atleast_2d(x), np.float32)
    w = np.ascontiguousarray(weight, np.float32)
    out = np.empty_like(x2)
    for t in range(x2.shape[0]):
        lib().oracle_rmsnorm(out[t], x2[t], w, x2.shape[1])
    return out.reshape(np.shape(x))


def ffn_block(x, pos, rms_w, wr, br, w1, b1, w2, b2, K, limit, mode=0):
    """The FFN block on a bf16 residual stream: t = bf16(rmsnorm(x) * w)
    (run.cpp:660; the layer's input is bf16 on the GPU path, defines.h:107),
    out = moe_layer(t) (run.cpp:662-745), x' = bf16(x + out) (run.cpp:748-750;
    utility.cpp:158-173 rounds the sum to bf16).  Rows with pos < 0 keep x.
    Returns (x', t)."""
    x = np.ascontiguousarray(x, np.float32)
    t = round_to_bf16(rmsnorm(x, rms_w))
    out = moe_layer(t, pos, wr, br, w1, b1, w2, b2, K, limit, mode=mode)
    xn = round_to_bf16(x + out)
    if pos is not None:
        inactive = np.asarray(pos) < 0
        xn[inactive] = x[inactive]
    return xn, t


def mxfp4_dequant(blocks, scales):
    blocks = np.ascontiguousarray(blocks, np.uint8)
    scales = np.ascontiguousarray(scales, np.uint8)
    n = scales.size
    assert blocks.size == n * 16
    out = np.zeros(n * 32, np.float32)
    lib().oracle_mxfp4_dequant(blocks.reshape(-1), scales.reshape(-1), n, out)
    return out.reshape(scales.shape[:-1] + (scales.shape[-1] * 32,))


def num_threads() -> int:
    return int(lib().oracle_num_threads())


# ---- the reference's own CPU path, compiled from its sources (optional) ----

_ref = None


def ref_available() -> bool:
    return os.path.exists(os.path.join(_HERE, "_ref", "libref.so"))


def ref():
    global _ref
    if _ref is None:
        L = C.CDLL(os.path.join(_HERE, "_ref", "libref.so"))
        L.ref_matmul.argtypes = [_f, _f, _f, C.c_int, C.c_int]
        L.ref_topk.argtypes = [_f, _i, _f, C.c_int, C.c_int]
        L.ref_softmax.argtypes = [_f, C.c_int]
        L.ref_rmsnorm.argtypes = [_f, _f, _f, C.c_int]
        L.ref_moe_forward.argtypes = ([C.c_int] * 5 + [C.c_float] + [_f] * 7 + [_f, _f, _i, _f, _f])
        L.ref_moe_forward.restype = C.c_int
        _ref = L
    return _ref


def ref_moe_forward(emb, wr, br, w1, b1, w2, b2, K, limit):
    T, H = emb.shape
    E = wr.shape[0]
    IM = w2.shape[2]
    t_out = np.zeros((T, H), np.float32)
    score = np.zeros((T, E), np.float32)
    ti = np.zeros((T, K), np.int32)
    tv = np.zeros((T, K), np.float32)
    agg = np.zeros((T, H), np.float32)
    ref().ref_moe_forward(T, H, IM, E, K, limit, emb, wr, br, w1, b1, w2, b2, t_out, score, ti, tv, agg)
    return dict(t=t_out, score=score, topk_i=ti, topk_v=tv, e_agg=agg)
