"""Stage-level parity of the HIP path through the C-ABI: the stage entry points
compose to the whole layer, the SwiGLU's clamp points, adversarial router
inputs (near ties, exact ties, NaN rows), the error bound of the router's first
pass, and repeatability of the large-batch kernels.

Bars as in test_gpu_parity.py: ids, offsets and permutations bit-exact; outputs
within max-abs 2e-2 and rel-L2 1e-3 of the oracle on the same bf16 inputs."""
import numpy as np
import pytest

from gpt_oss_amd import abi, synth
from oracle import binding as ob

pytestmark = pytest.mark.gpu

W = ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")
BF16_ULP = 2.0 ** -7  # spacing of bf16 values relative to the value, at most


def bf16_layer(shape, tokens=None, seed=0):
    L = synth.make_layer(shape, seed=seed, tokens=tokens)
    return {k: (synth.round_bf16(v) if v.dtype == np.float32 else v) for k, v in L.items()}


def make_moe(shape, L, max_tokens):
    m = abi.Moe(shape.hidden, shape.inter, shape.experts, max_tokens=max_tokens, swiglu_limit=shape.limit)
    m.upload_layer(0, *[L[k] for k in W])
    return m


def next_bf16(a, steps=1):
    """The bf16 value `steps` ulps further from zero."""
    bits = synth.to_bf16_bits(a).astype(np.int32) + steps
    return synth.from_bf16_bits(bits.astype(np.uint16))


# ---------------- stage entry points ----------------

@pytest.mark.parametrize("T", [40, 700, 3000])
def test_stage_entry_points_compose(T):
    """moe_router -> moe_dispatch -> moe_expert_gemms -> moe_combine gives the
    bits of moe_forward, with and without accumulation, and the combine stage is
    the weighted sum of the per-assignment rows in slot order."""
    sh = synth.LayerShape("s", T, 320, 128, 13)
    L = bf16_layer(sh, seed=5)
    m = make_moe(sh, L, T)
    # the router's ids are four different experts per token: with that said, the staged
    # calls run the configuration moe_forward runs (same bits also at 40 tokens, where
    # with so few column tiles the small-batch down GEMM sums its reduction in two parts)
    m.set_distinct_ids(True)
    pos = np.zeros(T, np.int32)
    pos[3::7] = -1
    base = abi.run_layer(m, 0, L["x"], pos)
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(L["x"]))
    dpos = abi.DevBuf.from_numpy(pos)
    dti, dtv = abi.DevBuf(T * 16), abi.DevBuf(T * 16)
    prior = np.random.default_rng(T).standard_normal((T, sh.hidden)).astype(np.float32)
    dout, dacc = abi.DevBuf(T * sh.hidden * 4), abi.DevBuf.from_numpy(prior)
    m.router(0, dx, dpos, T, None, dti, dtv)
    with pytest.raises(abi.MoeError) as e:  # no dispatch of this batch yet
        m.expert_gemms(0, dx, T)
    assert e.value.code == -5
    m.dispatch(dti, dpos, T)
    with pytest.raises(abi.MoeError) as e:  # the GEMMs have not run on this dispatch: y is stale
        m.combine(dtv, dpos, T, dout, accumulate=False)
    assert e.value.code == -5
    m.expert_gemms(0, dx, T)
    m.combine(dtv, dpos, T, dout, accumulate=False)
    m.combine(dtv, dpos, T, dacc, accumulate=True)
    abi.sync()
    assert np.array_equal(dout.download((T, sh.hidden), np.float32), base["out"])
    acc = dacc.download((T, sh.hidden), np.float32)
    assert np.array_equal(acc[pos < 0], prior[pos < 0])
    np.testing.assert_allclose(acc[pos >= 0], prior[pos >= 0] + base["out"][pos >= 0], rtol=0, atol=1e-6)
    # a whole-layer call takes the plan over: the stage calls need a new dispatch
    m.forward(0, dx, dpos, T, dout)
    with pytest.raises(abi.MoeError):
        m.combine(dtv, dpos, T, dout)


@pytest.mark.parametrize("T", [17, 40, 64, 65])
def test_caller_routing_with_distinct_ids(T):
    """moe_set_distinct_ids: with the promise that a token's ids are four
    different experts, moe_experts bounds the rows per expert by T as
    moe_forward does and takes the small-batch kernels up to 64 tokens: the bits
    of moe_forward.  Without it the bound is 4 T and the full-height kernels
    run: the same bits, too."""
    sh = synth.LayerShape("d", T, 2880, 320, 32)
    L = bf16_layer(sh, seed=8)
    m = make_moe(sh, L, 128)
    pos = np.zeros(T, np.int32)
    pos[2::5] = -1
    base = abi.run_layer(m, 0, L["x"], pos)
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(L["x"]))
    dpos = abi.DevBuf.from_numpy(pos)
    dti, dtv = abi.DevBuf.from_numpy(base["topk_i"]), abi.DevBuf.from_numpy(base["topk_v"])
    dout = abi.DevBuf(T * sh.hidden * 4)
    def same(got, distinct):
        # at this shape only batches of up to 5 tokens split the down GEMM's reduction, and
        # those run the small-batch configuration with or without the promise
        assert np.array_equal(got, base["out"]), f"distinct={distinct}"

    for distinct in (False, True, False):
        m.set_distinct_ids(distinct)
        dout.memset(0xFF)
        m.experts(0, dx, dpos, dti, dtv, T, dout)
        abi.sync()
        same(dout.download((T, sh.hidden), np.float32), distinct)
        m.dispatch(dti, dpos, T)
        m.expert_gemms(0, dx, T)
        dout.memset(0xFF)
        m.combine(dtv, dpos, T, dout)
        abi.sync()
        same(dout.download((T, sh.hidden), np.float32), distinct)
    # ids that break the promise must not fault: one expert in all four slots of every token
    m.set_distinct_ids(True)
    bad = np.full((T, 4), 3, np.int32)
    m.experts(0, dx, None, abi.DevBuf.from_numpy(bad), dtv, T, dout)
    abi.sync()


def test_reference_7m_model_shape():
    """The reference's smallest model (export_model_bin/gpt-oss-7m/config.json:
    hidden 32, intermediate 64, 32 experts): sizes that are multiples of 32 but
    not of 64 are padded inside the library.  Whole layer, FFN block and MXFP4
    upload against the oracle; batches on both sides of the small-batch limit."""
    for H, IM, E in ((32, 64, 32), (96, 96, 32), (32, 32, 8)):
        for T in (1, 50, 64, 300, 1100):
            sh = synth.LayerShape("7m", T, H, IM, E)
            L = bf16_layer(sh, seed=H + T)
            m = make_moe(sh, L, T)
            pos = np.zeros(T, np.int32)
            pos[1::6] = -1
            for p in (None, pos):
                R = abi.run_layer(m, 0, L["x"], p)
                _, ti, _ = ob.router(L["x"], p, L["w_router"], L["b_router"], 4)
                off, perm, _ = ob.dispatch(ti, p, E)
                case = f"H={H} IM={IM} E={E} T={T} masked={p is not None}"
                assert np.array_equal(R["topk_i"], ti), case
                assert np.array_equal(R["offsets"], off) and np.array_equal(R["perm"][:off[-1]], perm), case
                rows = np.arange(min(T, 48))
                want = ob.moe_layer(np.ascontiguousarray(L["x"][rows]), None if p is None else np.ascontiguousarray(p[rows]),
                                    *[L[k] for k in W], 4, sh.limit, mode=ob.ROUND_ACT_BF16 | ob.PAR_TOKENS)
                assert np.abs(R["out"][rows] - want).max() <= 2e-2, case
                assert np.linalg.norm(R["out"][rows] - want) <= 1e-3 * np.linalg.norm(want), case
            # the FFN block in place on the bf16 stream
            rng = np.random.default_rng(T)
            rw = synth.round_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
            m.upload_norm(0, rw)
            dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(L["x"]))
            m.block_forward(0, dx, abi.DevBuf.from_numpy(pos), T)
            abi.sync()
            got = synth.from_bf16_bits(dx.download((T, H), np.uint16))
            rows = np.arange(min(T, 32))
            want, _ = ob.ffn_block(np.ascontiguousarray(L["x"][rows]), np.ascontiguousarray(pos[rows]), rw,
                                   *[L[k] for k in W], 4, sh.limit, mode=ob.ROUND_ACT_BF16 | ob.PAR_TOKENS)
            assert np.all(np.abs(got[rows] - want) <= 2e-2 + 2.0 ** -7 * np.abs(want)), f"block H={H} T={T}"
            assert np.array_equal(got[pos < 0], L["x"][pos < 0])
            m.close()
    # MXFP4 upload at sizes that need padding: bit-identical to uploading the decoded matrices
    sh = synth.LayerShape("7q", 200, 96, 96, 8)
    x = synth.round_bf16(synth.make_activations(sh))
    wr, br = (synth.round_bf16(a) for a in synth.make_router(sh))
    b1k, s1, b1, b2k, s2, b2 = synth.make_experts_mxfp4(sh)
    b1, b2 = synth.round_bf16(b1), synth.round_bf16(b2)
    w1, w2 = ob.mxfp4_dequant(b1k, s1), ob.mxfp4_dequant(b2k, s2)
    m4 = abi.Moe(sh.hidden, sh.inter, sh.experts, max_tokens=sh.tokens)
    m4.upload_layer_mxfp4(0, wr, br, b1k, s1, b1, b2k, s2, b2)
    m32 = abi.Moe(sh.hidden, sh.inter, sh.experts, max_tokens=sh.tokens)
    m32.upload_layer(0, wr, br, w1, b1, w2, b2)
    for T in (200, 40):
        a, b = abi.run_layer(m4, 0, x[:T], None), abi.run_layer(m32, 0, x[:T], None)
        assert np.array_equal(a["out"], b["out"]) and np.isfinite(a["out"]).all()
    with pytest.raises(abi.MoeError) as e:
        abi.Moe(48, 64, 8, max_tokens=16)  # not a multiple of 32
    assert e.value.code == -2


def test_yardsticks_run():
    """The measured denominators the benchmark reports: a register-resident MFMA
    loop and plain streams through HBM.  Sanity only: positive, below the
    published peaks, zeros no slower than random operands."""
    tf, ghz = abi.yardstick_mfma(256, 2000, data=1)
    tf2, _ = abi.yardstick_mfma(256, 2000, data=2)
    tf0, _ = abi.yardstick_mfma(256, 2000, data=0)
    assert 200 < tf < 2600 and 200 < tf2 < 2600 and 0.5 < ghz < 3.0 and tf0 > 0.9 * tf
    c, r = abi.yardstick_hbm(1 << 28, 3)
    assert 500 < c < 8200 and 500 < r < 8200


def test_swiglu_clamp_points():
    """The clamp points of run.cpp:709-726 through moe_experts: W1 = 0 so the
    biases are the gate and up values, W2 = I so the activation is the output.
    The gate is clamped from above only, the up value on both sides; a very
    negative gate gives ~0 rather than being clamped to -limit."""
    H = IM = 64
    E, T = 4, 40
    w1 = np.zeros((E, 2 * IM, H), np.float32)
    w2 = np.tile(np.eye(H, IM, dtype=np.float32), (E, 1, 1))
    b2 = np.zeros((E, H), np.float32)
    b1 = np.zeros((E, 2 * IM), np.float32)
    b1[0, 0:2] = (9.0, 0.5)     # gate above the limit -> 7
    b1[0, 2:4] = (1.0, 9.0)     # up above the limit -> 7
    b1[0, 4:6] = (1.0, -9.0)    # up below -limit -> -7
    b1[0, 6:8] = (-30.0, 2.0)   # very negative gate: not clamped from below, ~0
    b1[0, 8:10] = (-9.0, 1.0)   # gate below -limit stays -9
    b1[0, 10:12] = (7.0, 7.0)   # exactly at the limit
    b1[0, 12:14] = (6.96875, -7.0)
    m = abi.Moe(H, IM, E, max_tokens=T, swiglu_limit=7.0)
    m.upload_layer(0, np.zeros((E, H), np.float32), np.zeros(E, np.float32), w1, b1, w2, b2)
    x = synth.round_bf16(np.random.default_rng(0).standard_normal((T, H)).astype(np.float32))
    ti = np.tile(np.arange(4, dtype=np.int32), (T, 1))
    tv = np.tile(np.array([1, 0, 0, 0], np.float32), (T, 1))
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(x))
    dout = abi.DevBuf(T * H * 4)
    m.experts(0, dx, None, abi.DevBuf.from_numpy(ti), abi.DevBuf.from_numpy(tv), T, dout)
    abi.sync()
    y = dout.download((T, H), np.float32)
    assert np.array_equal(y, np.tile(y[0], (T, 1)))  # W1 = 0: every token sees the same values
    sig = lambda g: 1.0 / (1.0 + np.exp(-1.702 * g))
    want = [7 * sig(7) * 1.5, 1 * sig(1) * 8.0, 1 * sig(1) * -6.0, None, -9 * sig(-9) * 2.0,
            7 * sig(7) * 8.0, 6.96875 * sig(6.96875) * -6.0]
    for j, wv in enumerate(want):
        if wv is None:
            assert abs(y[0, j]) < 1e-18
        else:  # the activation is rounded to bf16 (matmul.cpp:1427)
            np.testing.assert_allclose(y[0, j], wv, rtol=BF16_ULP)
    assert np.all(y[0, len(want):] == 0)
    # and against the oracle's own expert with the same rounding point
    yo = ob.expert_token(x[0], w1[0], b1[0], w2[0], b2[0], 7.0, mode=ob.ROUND_ACT_BF16)
    np.testing.assert_allclose(y[0], yo, rtol=BF16_ULP, atol=1e-30)


# ---------------- router: adversarial inputs ----------------

def _check_ids(m, L, x, pos, E):
    R = abi.run_layer(m, 0, x, pos)
    score, ti, tv = ob.router(x, pos, L["w_router"], L["b_router"], 4)
    assert np.array_equal(R["topk_i"], ti), "expert ids differ from the oracle"
    np.testing.assert_allclose(R["topk_v"], tv, rtol=0, atol=1e-6)
    act = np.ones(x.shape[0], bool) if pos is None else pos >= 0
    # logits of experts the router did not have to recompute exactly are its
    # first-pass values: 2e-6, or two float steps of the value where that is more
    np.testing.assert_allclose(R["score"][act], score[act], rtol=2.0 ** -22, atol=2e-6)
    return R, score, ti


@pytest.mark.parametrize("E,T", [(32, 2048), (128, 1000), (256, 300)])
def test_router_near_ties(E, T):
    """Logits one bf16 step of one weight apart, and exactly
    equal ones, at the top of every token's ranking: the first pass of the
    router cannot separate them, the ids must still be the oracle's."""
    H = 2880
    sh = synth.LayerShape("nt", T, H, 64, E)
    L = bf16_layer(sh, seed=11)
    rng = np.random.default_rng(E)
    wr, br = L["w_router"].copy(), L["b_router"].copy()
    base = wr[5].copy()
    group = [1, 5, 6, 9, 17, 20, E - 1, E - 2]
    for n, e in enumerate(group):
        wr[e] = base
        br[e] = 8.0  # lifts the whole group to the top of every token
        if n >= 2:   # experts 1 and 5 stay exactly equal; the others move one weight by one step
            k = int(rng.integers(H))
            wr[e, k] = next_bf16(wr[e, k:k + 1], steps=1 if n % 2 else -1)[0]
    L["w_router"], L["b_router"] = wr, br
    m = make_moe(sh, L, T)
    pos = np.zeros(T, np.int32)
    pos[4::13] = -1
    R, score, ti = _check_ids(m, L, L["x"], pos, E)
    act = pos >= 0
    assert np.isin(ti[act], group).all()  # the test is about the group
    top = np.sort(score[act][:, group], axis=1)[:, ::-1]
    assert np.median(top[:, 0] - top[:, 4]) < 2e-2  # and its members really are that close
    both = np.array([(1 in r) and (5 in r) for r in ti])
    assert both.any()
    for r in ti[both]:
        assert list(r).index(1) < list(r).index(5)  # exact tie: the lower id first


def test_router_first_pass_error_bound():
    """The first pass decides a token only when its logits are further apart
    than twice kGamma * |x| * max|w_e|; the scores it reports for experts it did
    not recompute must lie within that bound of the exact ones (they are in
    fact far inside it)."""
    E, T, H = 128, 3000, 2880
    sh = synth.LayerShape("eb", T, H, 64, E)
    L = bf16_layer(sh, seed=3)
    x = synth.round_bf16(L["x"] * np.random.default_rng(1).uniform(0.1, 30.0, (T, 1)).astype(np.float32))
    m = make_moe(sh, L, T)
    R, score, _ = _check_ids_loose(m, L, x, E)
    gamma = 2.0 * 33.0 * 2.0 ** -23  # router_gamma(1): a hand-over to fp64 after every MFMA
    bound = gamma * np.linalg.norm(x.astype(np.float64), axis=1) * np.linalg.norm(
        L["w_router"].astype(np.float64), axis=1).max()
    ratio = np.abs(R["score"].astype(np.float64) - score).max(axis=1) / bound
    print(f"first-pass error / proven bound: max {ratio.max():.3g}, median {np.median(ratio):.3g}")
    assert ratio.max() < 0.5


def _check_ids_loose(m, L, x, E):
    R = abi.run_layer(m, 0, x, None)
    score, ti, tv = ob.router(x, None, L["w_router"], L["b_router"], 4)
    assert np.array_equal(R["topk_i"], ti), "expert ids differ from the oracle"
    np.testing.assert_allclose(R["topk_v"], tv, rtol=0, atol=2e-5)  # rows scaled by up to 30
    return R, score, ti


def test_router_nan_row():
    """A row of NaN activations: every logit is NaN, no comparison succeeds and
    the reference's stable sort leaves the experts in index order (run.cpp:378-421),
    so the row goes to experts 0..3 and its output is NaN, as in the reference;
    the other rows are not disturbed."""
    sh = synth.LayerShape("nan", 100, 320, 128, 32)
    L = bf16_layer(sh, seed=9)
    m = make_moe(sh, L, sh.tokens)
    clean = abi.run_layer(m, 0, L["x"], None)
    x = L["x"].copy()
    x[37] = np.nan
    R = abi.run_layer(m, 0, x, None)
    _, ti, tv = ob.router(x, None, L["w_router"], L["b_router"], 4)
    assert list(ti[37]) == [0, 1, 2, 3] and np.isnan(tv[37]).all()
    assert np.array_equal(R["topk_i"], ti)
    assert np.isnan(R["topk_v"][37]).all() and np.isnan(R["out"][37]).all()
    keep = np.arange(sh.tokens) != 37
    assert np.array_equal(R["out"][keep], clean["out"][keep])
    off, perm, _ = ob.dispatch(ti, None, sh.experts)
    assert np.array_equal(R["offsets"], off) and np.array_equal(R["perm"][:off[-1]], perm)


# ---------------- repeatability of the large-batch kernels ----------------

def test_large_batches_repeat_bit_for_bit():
    """The GEMMs' main loop waits for its operands by counting outstanding loads
    (loads complete in issue order).  4096 tokens at the 20B shape run every
    tile height and both narrow last column tiles (row split 2 in gate_up, 4 in
    down); twelve calls in a row must give the same bits, with bf16 and with
    MXFP4 weights, so must 7168 tokens under Zipf routing (one expert with 28
    row tiles), and so must the FFN block at 48 tokens."""
    sh = synth.CONFIGS["c2"]
    T = sh.tokens
    wr, br = (synth.round_bf16(a) for a in synth.make_router(sh))
    b1k, s1, b1, b2k, s2, b2 = synth.make_experts_mxfp4(sh)
    w1, w2 = ob.mxfp4_dequant(b1k, s1), ob.mxfp4_dequant(b2k, s2)
    m4 = abi.Moe(sh.hidden, sh.inter, sh.experts, max_tokens=T, swiglu_limit=sh.limit)
    m4.upload_layer_mxfp4(0, wr, br, b1k, s1, b1, b2k, s2, b2)
    m16 = abi.Moe(sh.hidden, sh.inter, sh.experts, max_tokens=T, swiglu_limit=sh.limit)
    m16.upload_layer(0, wr, br, w1, b1, w2, b2)
    del w1, w2
    x = synth.round_bf16(synth.make_activations(sh, seed=1, tokens=T))
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(x))
    dout = abi.DevBuf(T * sh.hidden * 4)
    first = None
    for m in (m16, m4):
        for i in range(12):
            dout.memset(0xFF)
            m.forward(0, dx, None, T, dout)
            abi.sync()
            got = dout.download((T, sh.hidden), np.float32)
            if first is None:
                first = got
                assert np.isfinite(got).all()
            assert np.array_equal(got, first), f"call {i}: a repeated call gave other bits"
    # 7168 tokens with Zipf routing: up to 28 row tiles on one expert, the deepest XCD ranges
    z = synth.CONFIGS["c3b"]
    T3 = z.tokens
    m4.close()
    mz = abi.Moe(z.hidden, z.inter, z.experts, max_tokens=T3, swiglu_limit=z.limit)
    wrz, brz = (synth.round_bf16(a) for a in synth.make_router(z))
    w1, w2 = ob.mxfp4_dequant(b1k, s1), ob.mxfp4_dequant(b2k, s2)
    mz.upload_layer(0, wrz, brz, w1, b1, w2, b2)
    del w1, w2
    xz = synth.round_bf16(synth.make_activations(z))
    dxz = abi.DevBuf.from_numpy(synth.to_bf16_bits(xz))
    doz = abi.DevBuf(T3 * z.hidden * 4)
    firstz = None
    for i in range(12):
        doz.memset(0xFF)
        mz.forward(0, dxz, None, T3, doz)
        abi.sync()
        got = doz.download((T3, z.hidden), np.float32)
        if firstz is None:
            firstz = got
            assert np.isfinite(got).all()
        assert np.array_equal(got, firstz), f"7168 tokens, Zipf routing, call {i}: other bits"
    mz.close()
    del firstz, got
    rw = synth.round_bf16((1 + 0.1 * np.random.default_rng(2).standard_normal(sh.hidden)).astype(np.float32))
    m16.upload_norm(0, rw)
    ref = None
    for i in range(12):
        dxx = abi.DevBuf.from_numpy(synth.to_bf16_bits(x[:48]))
        m16.block_forward(0, dxx, None, 48)
        abi.sync()
        got = dxx.download((48, sh.hidden), np.uint16)
        if ref is None:
            ref = got
        assert np.array_equal(got, ref), f"FFN block, call {i}: other bits"


# ---------------- HIP-graph replay of the paths added later ----------------

@pytest.mark.parametrize("T", [3, 100])
def test_padded_shape_and_split_reduction_replay_from_a_hip_graph(T):
    """moe_forward at a hidden size that needs padding (one more kernel per call,
    the row widening) and, at 3 tokens, with the down GEMM's reduction split over
    two workgroups per tile: captured once, replayed three times with eager
    calls of another size in between, every replay bit-identical to the eager
    result."""
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")

    def ok(rc):
        assert rc == 0, f"HIP call failed with {rc}"

    sh = synth.LayerShape("g", T, 96, 96, 8)
    L = bf16_layer(sh, seed=13)
    m = make_moe(sh, L, 128)
    H = sh.hidden
    dx = abi.DevBuf.from_numpy(synth.to_bf16_bits(L["x"]))
    dout, dref = abi.DevBuf(T * H * 4), abi.DevBuf(T * H * 4)
    stream = C.c_void_p()
    ok(hip.hipStreamCreate(C.byref(stream)))
    m.forward(0, dx, None, T, dref, stream=stream)
    ok(hip.hipStreamSynchronize(stream))
    ref = dref.download((T, H), np.float32)
    want = ob.moe_layer(L["x"], None, *[L[k] for k in W], 4, sh.limit, mode=ob.ROUND_ACT_BF16 | ob.PAR_TOKENS)
    assert np.abs(ref - want).max() <= 2e-2 and np.linalg.norm(ref - want) <= 1e-3 * np.linalg.norm(want)
    graph, gexec = C.c_void_p(), C.c_void_p()
    ok(hip.hipStreamBeginCapture(stream, C.c_int(0)))
    m.forward(0, dx, None, T, dout, stream=stream)
    ok(hip.hipStreamEndCapture(stream, C.byref(graph)))
    ok(hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)))
    try:
        for _ in range(3):
            dout.memset(0)
            abi.sync()
            ok(hip.hipGraphLaunch(gexec, stream))
            ok(hip.hipStreamSynchronize(stream))
            assert np.array_equal(dout.download((T, H), np.float32), ref)
            m.forward(0, dx, None, max(T // 2, 1), dref, stream=stream)  # eager work of another size
            ok(hip.hipStreamSynchronize(stream))
    finally:
        hip.hipGraphExecDestroy(gexec)
        hip.hipGraphDestroy(graph)
        hip.hipStreamDestroy(stream)
