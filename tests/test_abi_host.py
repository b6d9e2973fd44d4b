"""The C-ABI library loads, exports every symbol include/moe_abi.h declares, and
its argument validation works -- all without a GPU (no kernel is launched)."""
import ctypes as C
import os
import re

import numpy as np
import pytest

from gpt_oss_amd import abi, synth

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "moe_abi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(moe_[a-z_0-9]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    names = declared_symbols()
    assert len(names) >= 20
    L = abi.lib()
    missing = [n for n in names if not hasattr(L, n)]
    assert not missing, missing
    assert sorted(abi.SYMBOLS) == names
    assert b"gfx950" in L.moe_version()


def _create(**kw):
    cfg = dict(hidden=256, inter=256, experts=8, topk=4, layers=1, max_tokens=64, swiglu_limit=7.0)
    cfg.update(kw)
    c = abi.MoeConfig(*[cfg[k] for k in ("hidden", "inter", "experts", "topk", "layers", "max_tokens",
                                         "swiglu_limit")])
    h = C.c_void_p()
    rc = abi.lib().moe_create(C.byref(c), C.byref(h))
    return rc, h, abi.lib().moe_last_error().decode()


@pytest.mark.parametrize("kw,code,word", [
    (dict(topk=2), -2, "topk"),
    (dict(hidden=100), -2, "multiples of 32"),
    (dict(inter=2880 + 16), -2, "multiples of 32"),
    (dict(experts=2), -2, "experts"),
    (dict(experts=300), -2, "experts"),
    (dict(layers=0), -1, "layers"),
    (dict(max_tokens=0), -1, "max_tokens"),
    (dict(swiglu_limit=0.0), -1, "swiglu_limit"),
])
def test_create_rejects_bad_config(kw, code, word):
    rc, h, msg = _create(**kw)
    assert rc == code and h.value is None
    assert word in msg


def test_null_arguments_are_errors_not_crashes():
    L = abi.lib()
    assert L.moe_create(None, None) == -1
    assert L.moe_forward(None, 0, None, None, 1, None, 0, None) == -1
    assert L.moe_router(None, 0, None, None, 1, None, None, None, None) == -1
    assert L.moe_dispatch(None, None, None, 1, None) == -1
    assert L.moe_experts(None, 0, None, None, None, None, 1, None, 0, None) == -1
    assert L.moe_upload_layer(None, 0, None, None, None, None, None, None) == -1
    assert L.moe_profile_enable(None, 1) == -1
    assert L.moe_destroy(None) == 0
    assert L.moe_weight_bytes(None) == 0


@pytest.mark.skipif(abi.device_count() > 0, reason="only meaningful without a GPU")
def test_fails_loudly_without_gpu():
    rc, h, msg = _create()
    assert rc == -4 and "hip" in msg.lower()
    with pytest.raises(abi.MoeError):
        abi.Moe(256, 256, 8, 64)


def test_synth_bf16_helpers_roundtrip():
    rng = np.random.default_rng(0)
    a = rng.standard_normal(10000).astype(np.float32)
    r = synth.round_bf16(a)
    assert np.array_equal(synth.from_bf16_bits(synth.to_bf16_bits(a)), r)
    assert np.all(np.abs(r - a) <= np.abs(a) * 2.0 ** -8)
    assert np.array_equal(synth.round_bf16(r), r)


def test_synth_is_deterministic_and_thread_count_independent():
    a = synth._normal(3, 4, (3, 1 << 22), 0.02, True)
    b = synth._normal(3, 4, (3 << 22,), 0.02, True)
    assert np.array_equal(a.reshape(-1), b)
    assert abs(float(a.std()) - 0.02) < 2e-4
    x = synth.make_activations(synth.CONFIGS["c2"], tokens=8)
    np.testing.assert_allclose(np.sqrt((x.astype(np.float64) ** 2).mean(axis=1)), 1.0, atol=3e-3)


def test_bench_refuses_more_than_one_gpu_and_needs_a_gpu():
    """bench.py measures one GPU: --gpus 2 exits with a message saying so; with
    no GPU visible it exits rather than falling back to anything."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"],
                       capture_output=True, text=True, timeout=120)
    assert r.returncode == 2 and "one GPU" in r.stderr
    if abi.device_count() == 0:
        r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--steps", "1", "--warmup", "0"],
                           capture_output=True, text=True, timeout=120)
        assert r.returncode == 3 and "no CPU fallback" in r.stderr and r.stdout.strip() == ""
