"""ctypes binding of the C-ABI in include/moe_abi.h (libmi355_moe.so).

Plumbing for tests and the benchmark: device buffers are plain integers
(device addresses) obtained from the library's own allocation helpers, host
data are numpy arrays.  The library is required: if it is missing or fails to
load, importing callers get an error, never a fallback.
"""
from __future__ import annotations

import ctypes as C
import os

import numpy as np

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "libmi355_moe.so")

STAGES = ["router", "dispatch", "gate_up", "down", "combine"]

# every symbol include/moe_abi.h declares
SYMBOLS = [
    "moe_create", "moe_destroy", "moe_upload_layer", "moe_upload_layer_mxfp4", "moe_upload_norm",
    "moe_forward", "moe_block_forward",
    "moe_router",
    "moe_dispatch", "moe_get_dispatch", "moe_experts", "moe_expert_gemms", "moe_combine",
    "moe_dispatch_static", "moe_set_distinct_ids", "moe_profile_enable",
    "moe_profile_read", "moe_weight_bytes", "moe_workspace_bytes", "moe_last_error",
    "moe_version", "moe_dev_alloc", "moe_dev_free", "moe_dev_upload", "moe_dev_download",
    "moe_dev_memset", "moe_dev_sync", "moe_dev_count", "moe_time_forward", "moe_time_forward_each",
    "moe_yardstick_mfma", "moe_yardstick_hbm",
]


class MoeConfig(C.Structure):
    _fields_ = [("hidden", C.c_int), ("inter", C.c_int), ("experts", C.c_int),
                ("topk", C.c_int), ("layers", C.c_int), ("max_tokens", C.c_int),
                ("swiglu_limit", C.c_float)]


class MoeError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"moe status {code}: {msg}")
        self.code = code


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                f"{LIB_PATH} is not built; run `python -c 'import __graft_entry__ as g; g.build()'`")
        L = C.CDLL(LIB_PATH)
        vp, ci, cf = C.c_void_p, C.c_int, C.c_float
        L.moe_create.argtypes = [C.POINTER(MoeConfig), C.POINTER(vp)]
        L.moe_destroy.argtypes = [vp]
        L.moe_upload_layer.argtypes = [vp, ci] + [vp] * 6
        L.moe_upload_layer_mxfp4.argtypes = [vp, ci] + [vp] * 8
        L.moe_forward.argtypes = [vp, ci, vp, vp, ci, vp, ci, vp]
        L.moe_upload_norm.argtypes = [vp, ci, vp]
        L.moe_block_forward.argtypes = [vp, ci, vp, vp, ci, vp]
        L.moe_router.argtypes = [vp, ci, vp, vp, ci, vp, vp, vp, vp]
        L.moe_dispatch.argtypes = [vp, vp, vp, ci, vp]
        L.moe_get_dispatch.argtypes = [vp, vp, vp, ci, vp]
        L.moe_experts.argtypes = [vp, ci, vp, vp, vp, vp, ci, vp, ci, vp]
        L.moe_expert_gemms.argtypes = [vp, ci, vp, ci, vp]
        L.moe_combine.argtypes = [vp, vp, vp, ci, vp, ci, vp]
        L.moe_dispatch_static.argtypes = [vp, vp, ci, ci, vp, vp, vp]
        L.moe_set_distinct_ids.argtypes = [vp, ci]
        L.moe_profile_enable.argtypes = [vp, ci]
        L.moe_profile_read.argtypes = [vp, C.POINTER(cf), C.POINTER(ci)]
        L.moe_weight_bytes.argtypes = [vp]
        L.moe_weight_bytes.restype = C.c_size_t
        L.moe_workspace_bytes.argtypes = [vp]
        L.moe_workspace_bytes.restype = C.c_size_t
        L.moe_last_error.restype = C.c_char_p
        L.moe_version.restype = C.c_char_p
        L.moe_dev_alloc.argtypes = [C.POINTER(vp), C.c_size_t]
        L.moe_dev_free.argtypes = [vp]
        L.moe_dev_upload.argtypes = [vp, vp, C.c_size_t]
        L.moe_dev_download.argtypes = [vp, vp, C.c_size_t]
        L.moe_dev_memset.argtypes = [vp, ci, C.c_size_t]
        L.moe_time_forward.argtypes = [vp, ci, vp, vp, ci, vp, ci, ci, C.POINTER(cf)]
        L.moe_time_forward_each.argtypes = [vp, ci, vp, vp, ci, vp, ci, C.POINTER(cf)]
        L.moe_yardstick_mfma.argtypes = [ci, ci, ci, C.POINTER(C.c_double), C.POINTER(C.c_double)]
        L.moe_yardstick_hbm.argtypes = [C.c_size_t, ci, C.POINTER(C.c_double), C.POINTER(C.c_double)]
        _lib = L
    return _lib


def check(rc: int) -> None:
    if rc != 0:
        raise MoeError(rc, lib().moe_last_error().decode())


def device_count() -> int:
    return int(lib().moe_dev_count())


class DevBuf:
    """A device allocation; freed on close() or garbage collection."""

    def __init__(self, nbytes: int):
        p = C.c_void_p()
        check(lib().moe_dev_alloc(C.byref(p), nbytes))
        self.ptr = p.value
        self.nbytes = nbytes

    @classmethod
    def from_numpy(cls, a: np.ndarray) -> "DevBuf":
        a = np.ascontiguousarray(a)
        b = cls(a.nbytes)
        check(lib().moe_dev_upload(b.ptr, a.ctypes.data, a.nbytes))
        return b

    def upload(self, a: np.ndarray) -> None:
        a = np.ascontiguousarray(a)
        assert a.nbytes <= self.nbytes
        check(lib().moe_dev_upload(self.ptr, a.ctypes.data, a.nbytes))

    def download(self, shape, dtype) -> np.ndarray:
        out = np.empty(shape, dtype=dtype)
        assert out.nbytes <= self.nbytes
        check(lib().moe_dev_download(out.ctypes.data, self.ptr, out.nbytes))
        return out

    def memset(self, value: int = 0) -> None:
        check(lib().moe_dev_memset(self.ptr, value, self.nbytes))

    def close(self) -> None:
        if getattr(self, "ptr", None):
            lib().moe_dev_free(self.ptr)
            self.ptr = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass


def dispatch_static(topk_i, pos, n_tokens, n_experts, offsets, perm, stream=None) -> None:
    """moe_dispatch_static: no handle, no allocation; device buffers in and out."""
    check(lib().moe_dispatch_static(_p(topk_i), _p(pos), n_tokens, n_experts, _p(offsets), _p(perm),
                                    stream))


def yardstick_mfma(n_workgroups: int = 256, iters: int = 20000, data: int = 1):
    """(TFLOP/s, shader GHz) of a register-resident v_mfma_f32_32x32x16_bf16 loop.
    data: 0 zeros, 1 operands of unit scale, 2 unit scale against scale 0.02."""
    tf, ghz = C.c_double(), C.c_double()
    check(lib().moe_yardstick_mfma(n_workgroups, iters, int(data), C.byref(tf), C.byref(ghz)))
    return float(tf.value), float(ghz.value)


def yardstick_hbm(nbytes: int = 1 << 30, iters: int = 10):
    """(copy GB/s counting reads + writes, read-only GB/s) of plain streams over nbytes."""
    c, r = C.c_double(), C.c_double()
    check(lib().moe_yardstick_hbm(nbytes, iters, C.byref(c), C.byref(r)))
    return float(c.value), float(r.value)


def sync() -> None:
    check(lib().moe_dev_sync())


def _p(b):
    if b is None:
        return None
    return b.ptr if isinstance(b, DevBuf) else b


class Moe:
    """Owner of one moe_handle."""

    def __init__(self, hidden, inter, experts, max_tokens, layers=1, topk=4, swiglu_limit=7.0):
        self.cfg = MoeConfig(hidden, inter, experts, topk, layers, max_tokens, swiglu_limit)
        h = C.c_void_p()
        check(lib().moe_create(C.byref(self.cfg), C.byref(h)))
        self.h = h

    def close(self):
        if getattr(self, "h", None):
            lib().moe_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def upload_layer(self, layer, w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2):
        arrs = [np.ascontiguousarray(a, dtype=np.float32)
                for a in (w_router, b_router, w_mlp1, b_mlp1, w_mlp2, b_mlp2)]
        check(lib().moe_upload_layer(self.h, layer, *[a.ctypes.data for a in arrs]))

    def upload_layer_mxfp4(self, layer, w_router, b_router, w1_blocks, w1_scales, b_mlp1,
                           w2_blocks, w2_scales, b_mlp2):
        """Expert matrices as MXFP4: blocks u8 [E, rows, cols/32, 16], scales u8 [E, rows, cols/32]."""
        f = lambda a: np.ascontiguousarray(a, dtype=np.float32)
        u = lambda a: np.ascontiguousarray(a, dtype=np.uint8)
        arrs = [f(w_router), f(b_router), u(w1_blocks), u(w1_scales), f(b_mlp1), u(w2_blocks),
                u(w2_scales), f(b_mlp2)]
        check(lib().moe_upload_layer_mxfp4(self.h, layer, *[a.ctypes.data for a in arrs]))

    def upload_norm(self, layer, rms_w):
        a = np.ascontiguousarray(rms_w, dtype=np.float32)
        check(lib().moe_upload_norm(self.h, layer, a.ctypes.data))

    def block_forward(self, layer, x, pos, n_tokens, stream=None):
        """x: DevBuf of bf16 [n_tokens, H], updated in place."""
        check(lib().moe_block_forward(self.h, layer, _p(x), _p(pos), n_tokens, stream))

    def forward(self, layer, x, pos, n_tokens, out, accumulate=False, stream=None):
        check(lib().moe_forward(self.h, layer, _p(x), _p(pos), n_tokens, _p(out),
                                1 if accumulate else 0, stream))

    def router(self, layer, x, pos, n_tokens, score, topk_i, topk_v, stream=None):
        check(lib().moe_router(self.h, layer, _p(x), _p(pos), n_tokens, _p(score), _p(topk_i),
                               _p(topk_v), stream))

    def dispatch(self, topk_i, pos, n_tokens, stream=None):
        check(lib().moe_dispatch(self.h, _p(topk_i), _p(pos), n_tokens, stream))

    def get_dispatch(self, offsets, perm, n_tokens, stream=None):
        check(lib().moe_get_dispatch(self.h, _p(offsets), _p(perm), n_tokens, stream))

    def experts(self, layer, x, pos, topk_i, topk_v, n_tokens, out, accumulate=False, stream=None):
        check(lib().moe_experts(self.h, layer, _p(x), _p(pos), _p(topk_i), _p(topk_v), n_tokens,
                                _p(out), 1 if accumulate else 0, stream))

    def expert_gemms(self, layer, x, n_tokens, stream=None):
        check(lib().moe_expert_gemms(self.h, layer, _p(x), n_tokens, stream))

    def combine(self, topk_v, pos, n_tokens, out, accumulate=False, stream=None):
        check(lib().moe_combine(self.h, _p(topk_v), _p(pos), n_tokens, _p(out),
                                1 if accumulate else 0, stream))

    def set_distinct_ids(self, distinct=True):
        check(lib().moe_set_distinct_ids(self.h, 1 if distinct else 0))

    def profile_enable(self, n_calls):
        check(lib().moe_profile_enable(self.h, n_calls))

    def profile_read(self):
        ms = (C.c_float * len(STAGES))()
        n = C.c_int()
        check(lib().moe_profile_read(self.h, ms, C.byref(n)))
        return {s: float(ms[i]) for i, s in enumerate(STAGES)}, n.value

    def time_forward(self, layer, x, pos, n_tokens, out, warmup, iters) -> float:
        ms = C.c_float()
        check(lib().moe_time_forward(self.h, layer, _p(x), _p(pos), n_tokens, _p(out), warmup,
                                     iters, C.byref(ms)))
        return float(ms.value)

    def time_forward_each(self, layer, x, pos, n_tokens, out, iters) -> np.ndarray:
        """Durations in ms of `iters` consecutive forward calls (HIP events on one stream)."""
        ms = (C.c_float * iters)()
        check(lib().moe_time_forward_each(self.h, layer, _p(x), _p(pos), n_tokens, _p(out), iters, ms))
        return np.array(ms[:], dtype=np.float64)

    @property
    def weight_bytes(self):
        return int(lib().moe_weight_bytes(self.h))

    @property
    def workspace_bytes(self):
        return int(lib().moe_workspace_bytes(self.h))


def run_layer(moe: Moe, layer: int, x_f32: np.ndarray, pos: np.ndarray | None):
    """Convenience for tests: uploads x (float32 holding bf16 values) as bf16,
    runs the whole layer and the stage-level entry points, and returns host copies."""
    from . import synth
    T, H = x_f32.shape
    E, K = moe.cfg.experts, moe.cfg.topk
    dx = DevBuf.from_numpy(synth.to_bf16_bits(x_f32))
    dpos = DevBuf.from_numpy(pos.astype(np.int32)) if pos is not None else None
    dout = DevBuf(T * H * 4)
    dscore = DevBuf(T * E * 4)
    dscore.memset(0)
    dti = DevBuf(T * K * 4)
    dtv = DevBuf(T * K * 4)
    doff = DevBuf((E + 1) * 4)
    dperm = DevBuf(T * K * 4)
    moe.router(layer, dx, dpos, T, dscore, dti, dtv)
    moe.dispatch(dti, dpos, T)
    moe.get_dispatch(doff, dperm, T)
    moe.forward(layer, dx, dpos, T, dout, accumulate=False)
    sync()
    return dict(out=dout.download((T, H), np.float32), score=dscore.download((T, E), np.float32),
                topk_i=dti.download((T, K), np.int32), topk_v=dtv.download((T, K), np.float32),
                offsets=doff.download((E + 1,), np.int32), perm=dperm.download((T * K,), np.int32))
