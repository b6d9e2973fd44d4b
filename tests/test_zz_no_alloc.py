"""moe_dispatch_static, the entry point for callers that cannot allocate:
no handle, no allocation, its working buffers in a device array that is part of
the library image.  Checked through the C-ABI against moe_dispatch +
moe_get_dispatch (bit-exact, as for all integer work) and against the oracle,
on two calls in a row, the second with a smaller input (the array keeps the
first call's contents), and at its limits."""
import numpy as np
import pytest

from gpt_oss_amd import abi
from oracle import binding as ob

pytestmark = pytest.mark.gpu

MAX_TOKENS, MAX_EXPERTS = 8192, 256


def _routing(rng, T, E):
    ti = np.stack([rng.permutation(E)[:4] for _ in range(T)]).astype(np.int32)
    pos = np.where(rng.random(T) < 0.2, -1, 3).astype(np.int32)
    return ti, pos


def _both(m, ti, pos, E):
    T = ti.shape[0]
    dti = abi.DevBuf.from_numpy(ti)
    dpos = abi.DevBuf.from_numpy(pos) if pos is not None else None
    off_a, perm_a = abi.DevBuf((E + 1) * 4), abi.DevBuf(T * 16)
    off_b, perm_b = abi.DevBuf((E + 1) * 4), abi.DevBuf(T * 16)
    for b in (off_b, perm_b):
        b.memset(0x5A)
    m.dispatch(dti, dpos, T)
    m.get_dispatch(off_a, perm_a, T)
    abi.dispatch_static(dti, dpos, T, E, off_b, perm_b)
    abi.sync()
    want_off, want_perm = off_a.download((E + 1,), np.int32), perm_a.download((T * 4,), np.int32)
    got_off, got_perm = off_b.download((E + 1,), np.int32), perm_b.download((T * 4,), np.int32)
    assert np.array_equal(got_off, want_off), "offsets differ from moe_dispatch"
    assert np.array_equal(got_perm, want_perm), "permutation differs from moe_dispatch"
    o_off, o_perm, _ = ob.dispatch(ti, pos, E)
    assert np.array_equal(got_off, o_off) and np.array_equal(got_perm[:o_off[-1]], o_perm)
    assert np.all(got_perm[o_off[-1]:] == -1)


@pytest.mark.parametrize("E", [32, 128])
def test_static_dispatch_matches_handle_dispatch(E):
    rng = np.random.default_rng(E)
    m = abi.Moe(64, 64, E, max_tokens=MAX_TOKENS)
    # two calls in a row, the second smaller: nothing of the first may show
    for T in (5000, 700, MAX_TOKENS, 200, 1):
        ti, pos = _routing(rng, T, E)
        _both(m, ti, pos, E)
    ti, _ = _routing(rng, 300, E)
    _both(m, ti, None, E)


def test_static_dispatch_limits():
    E = 8
    dti = abi.DevBuf(16 * (MAX_TOKENS + 1))
    dti.memset(0)
    off, perm = abi.DevBuf((MAX_EXPERTS + 2) * 4), abi.DevBuf(16 * (MAX_TOKENS + 1))
    with pytest.raises(abi.MoeError) as e:
        abi.dispatch_static(dti, None, MAX_TOKENS + 1, E, off, perm)
    assert e.value.code == -3 and "maximum" in str(e.value)
    with pytest.raises(abi.MoeError) as e:
        abi.dispatch_static(dti, None, 16, MAX_EXPERTS + 1, off, perm)
    assert e.value.code == -3
    with pytest.raises(abi.MoeError) as e:
        abi.dispatch_static(None, None, 16, E, off, perm)
    assert e.value.code == -1
    abi.dispatch_static(dti, None, 0, E, off, perm)  # an empty batch: offsets all zero
    abi.sync()
    assert np.all(off.download((E + 1,), np.int32) == 0)
