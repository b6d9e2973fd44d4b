"""Pins the CPU oracle (oracle/moe_oracle.c) against the reference's own
outputs (committed vectors made from its forward(), run.cpp:529-758), against
the reference build itself where it is present, and against what the
mathematics fixes.  No GPU."""
import numpy as np
import pytest

from gpt_oss_amd import synth
from oracle import binding as ob

W = ("w_router", "b_router", "w_mlp1", "b_mlp1", "w_mlp2", "b_mlp2")


def rel_l2(a, b):
    return float(np.linalg.norm(a - b) / np.linalg.norm(b))


# ---------------- golden vectors from the reference ----------------

def test_generator_reproduces_fixture_inputs(golden, c1_layer):
    assert synth.digest(c1_layer["x"]) == str(golden["emb_digest"])
    assert synth.digest(*[c1_layer[k] for k in W]) == str(golden["weights_digest"])


def test_layer_matches_reference_forward_c1(golden, c1_layer):
    L = c1_layer
    out, score, ti, tv = ob.moe_layer(golden["t"], None, *[L[k] for k in W], 4, 7.0, mode=0,
                                      want_routing=True)
    assert np.array_equal(ti, golden["topk_i"])
    assert np.array_equal(score, golden["score"])
    np.testing.assert_allclose(tv, golden["topk_v"], rtol=0, atol=1e-7)
    assert np.abs(out - golden["e_agg"]).max() <= 1e-7
    # token-parallel evaluation must not change anything
    out2 = ob.moe_layer(golden["t"], None, *[L[k] for k in W], 4, 7.0, mode=ob.PAR_TOKENS)
    assert np.array_equal(out, out2)


def test_topk_ties_match_reference(golden):
    names = [k[4:-6] for k in golden.files if k.startswith("tie_") and k.endswith("_score")]
    assert len(names) >= 6
    for n in names:
        v, i = ob.topk(golden[f"tie_{n}_score"], 4)
        assert np.array_equal(i, golden[f"tie_{n}_idx"]), n
        assert np.array_equal(v, golden[f"tie_{n}_val"]), n


def test_softmax_matches_reference(golden):
    for row_in, row_out in zip(golden["softmax_in"], golden["softmax_out"]):
        assert np.array_equal(ob.softmax(row_in), row_out)


@pytest.mark.skipif(not ob.ref_available(), reason="reference build (oracle/_ref) not present")
def test_against_reference_build_random_shapes():
    rng = np.random.default_rng(5)
    for (T, H, IM, E) in [(5, 64, 128, 4), (9, 192, 64, 12), (3, 128, 128, 33)]:
        emb = rng.standard_normal((T, H)).astype(np.float32)
        wr = (rng.standard_normal((E, H)) * 0.3).astype(np.float32)
        br = (rng.standard_normal(E) * 0.1).astype(np.float32)
        w1 = (rng.standard_normal((E, 2 * IM, H)) * 0.2).astype(np.float32)
        b1 = (rng.standard_normal((E, 2 * IM)) * 0.5).astype(np.float32)
        w2 = (rng.standard_normal((E, H, IM)) * 0.2).astype(np.float32)
        b2 = (rng.standard_normal((E, H)) * 0.5).astype(np.float32)
        R = ob.ref_moe_forward(emb, wr, br, w1, b1, w2, b2, 4, 7.0)
        out, score, ti, tv = ob.moe_layer(R["t"], None, wr, br, w1, b1, w2, b2, 4, 7.0, want_routing=True)
        assert np.array_equal(ti, R["topk_i"])
        assert np.array_equal(score, R["score"])
        assert np.abs(tv - R["topk_v"]).max() <= 1e-7
        assert rel_l2(out, R["e_agg"]) <= 1e-6
        x = rng.standard_normal(H).astype(np.float32)
        y = np.empty(E, np.float32)
        ob.ref().ref_matmul(y, x.copy(), wr.copy(), H, E)
        assert np.array_equal(y, ob.matmul(x, wr))


def test_rmsnorm_matches_reference_vectors(golden, c1_layer):
    """The fixture's t is the reference's own rmsnorm (unit weight) of the
    embedding rows, taken out of forward()'s state (run.cpp:660)."""
    x = c1_layer["x"]
    assert synth.digest(x) == str(golden["emb_digest"])
    t = ob.rmsnorm(x, np.ones(x.shape[1], np.float32))
    assert np.array_equal(t, golden["t"])


@pytest.mark.skipif(not ob.ref_available(), reason="reference build (oracle/_ref) not present")
def test_rmsnorm_against_reference_build():
    rng = np.random.default_rng(11)
    for H in (64, 2880, 257):
        x = (rng.standard_normal(H) * rng.uniform(0.01, 30)).astype(np.float32)
        w = (1 + 0.2 * rng.standard_normal(H)).astype(np.float32)
        want = np.empty(H, np.float32)
        ob.ref().ref_rmsnorm(want, x.copy(), w.copy(), H)
        assert np.array_equal(ob.rmsnorm(x, w), want)


def test_rmsnorm_closed_forms():
    H = 96
    w = np.linspace(0.5, 1.5, H).astype(np.float32)
    # constant rows: mean square is c^2 exactly
    for c in (1.0, -3.0, 0.25):
        x = np.full(H, c, np.float32)
        scale = np.float32(1.0) / np.sqrt(np.float32(np.float64(c) * c + np.float64(np.float32(1e-5))))
        want = (w.astype(np.float64) * (np.float64(scale) * np.float64(c))).astype(np.float32)
        assert np.array_equal(ob.rmsnorm(x, w), want)
    # the direction survives scaling; the length is sqrt(H) up to the epsilon
    rng = np.random.default_rng(3)
    x = rng.standard_normal(H).astype(np.float32)
    a = ob.rmsnorm(x, np.ones(H, np.float32))
    b = ob.rmsnorm(64 * x, np.ones(H, np.float32))
    np.testing.assert_allclose(a, b, rtol=2e-5)
    np.testing.assert_allclose(np.linalg.norm(a.astype(np.float64)), np.sqrt(H), rtol=1e-4)
    # a zero row stays zero (the epsilon keeps the scale finite)
    assert np.all(ob.rmsnorm(np.zeros(H, np.float32), w) == 0)


def test_ffn_block_composition():
    """x' = bf16(x + layer(bf16(rmsnorm(x) w))); inactive rows keep x."""
    rng = np.random.default_rng(8)
    T, H, IM, E = 6, 64, 64, 8
    x = ob.round_to_bf16((rng.standard_normal((T, H)) * 2).astype(np.float32))
    rw = ob.round_to_bf16((1 + 0.1 * rng.standard_normal(H)).astype(np.float32))
    wr = (rng.standard_normal((E, H)) * 0.3).astype(np.float32)
    br = (rng.standard_normal(E) * 0.1).astype(np.float32)
    w1 = (rng.standard_normal((E, 2 * IM, H)) * 0.1).astype(np.float32)
    b1 = np.zeros((E, 2 * IM), np.float32)
    w2 = np.zeros((E, H, IM), np.float32)       # experts output their bias only
    b2 = np.full((E, H), 0.5, np.float32)
    pos = np.array([0, 0, -1, 0, 0, 0], np.int32)
    xn, t = ob.ffn_block(x, pos, rw, wr, br, w1, b1, w2, b2, 4, 7.0)
    assert np.array_equal(t, ob.round_to_bf16(ob.rmsnorm(x, rw)))
    act = pos >= 0
    # routing weights sum to one, so the layer adds 0.5 to every element
    np.testing.assert_allclose(xn[act], ob.round_to_bf16(x[act] + np.float32(0.5)), rtol=0, atol=2.0 ** -6)
    assert np.array_equal(xn[~act], x[~act])


# ---------------- what the mathematics fixes ----------------

def test_matmul_one_hot_and_double_accumulation():
    rng = np.random.default_rng(0)
    w = rng.standard_normal((7, 33)).astype(np.float32)
    for j in (0, 13, 32):
        x = np.zeros(33, np.float32)
        x[j] = 2.0
        assert np.array_equal(ob.matmul(x, w), 2.0 * w[:, j])
    # a float accumulator would lose the 1.0; a double one keeps it (run.cpp:362)
    x = np.array([1e8, 1.0, -1e8], np.float32)
    assert ob.matmul(x, np.ones((1, 3), np.float32))[0] == 1.0
    # products are rounded to float before the double sum (run.cpp:364)
    a = np.float32(1.0 + 2.0 ** -12)
    x = np.array([a, -1.0], np.float32)
    wrow = np.array([[a, np.float32(a * a)]], np.float32)
    assert ob.matmul(x, wrow)[0] == 0.0
    # against a float64 numpy product on bf16 data, where every product is exact
    xb = synth.round_bf16(rng.standard_normal(512).astype(np.float32))
    wb = synth.round_bf16(rng.standard_normal((9, 512)).astype(np.float32))
    ref = (wb.astype(np.float64) @ xb.astype(np.float64)).astype(np.float32)
    assert np.abs(ob.matmul(xb, wb) - ref).max() <= 1e-6 * np.abs(ref).max()


def test_topk_brute_force():
    rng = np.random.default_rng(1)
    for E in (4, 8, 32, 128):
        for _ in range(50):
            s = rng.integers(-3, 4, E).astype(np.float32)  # many ties
            v, i = ob.topk(s, 4)
            order = sorted(range(E), key=lambda e: (-s[e], e))[:4]
            assert list(i) == order
            assert np.array_equal(v, s[order])


def test_softmax_closed_forms():
    p = ob.softmax(np.zeros(4, np.float32))
    assert np.array_equal(p, np.full(4, 0.25, np.float32))
    x = np.array([1.5, 0.5, -0.25, -2.0], np.float32)
    p = ob.softmax(x)
    assert abs(float(p.sum()) - 1.0) < 1e-6
    np.testing.assert_allclose(p, ob.softmax(x + 3.0), atol=1e-7)
    e = np.exp(x.astype(np.float64) - 1.5)
    np.testing.assert_allclose(p, e / e.sum(), rtol=2e-7)
    assert list(np.argsort(-p)) == [0, 1, 2, 3]


def test_dispatch_brute_force_and_invariants():
    rng = np.random.default_rng(2)
    for (T, E) in [(1, 4), (7, 5), (64, 8), (300, 32), (513, 128)]:
        ti = np.stack([rng.permutation(E)[:4] for _ in range(T)]).astype(np.int32)
        pos = np.where(rng.random(T) < 0.2, -1, 0).astype(np.int32)
        off, perm, inv = ob.dispatch(ti, pos, E)
        active = pos >= 0
        hist = np.bincount(ti[active].reshape(-1), minlength=E)
        assert np.array_equal(off, np.concatenate([[0], np.cumsum(hist)]))
        assert sorted(perm.tolist()) == sorted((np.nonzero(np.repeat(active, 4))[0]).tolist())
        for e in range(E):
            seg = perm[off[e]:off[e + 1]]
            assert np.all(ti.reshape(-1)[seg] == e)
            assert np.all(np.diff(seg // 4) > 0)  # token order, a token at most once
        expect = [a for e in range(E) for a in range(4 * T) if active[a // 4] and ti.reshape(-1)[a] == e]
        assert perm.tolist() == expect
        assert np.all(inv[~active] == -1)
        assert np.array_equal(perm[inv[active].reshape(-1)], np.nonzero(np.repeat(active, 4))[0])
    off, perm, inv = ob.dispatch(np.zeros((3, 4), np.int32), np.full(3, -1, np.int32), 4)
    assert off.tolist() == [0] * 5 and perm.size == 0


def test_bf16_round_known_answers_and_exhaustive():
    kat = [(1.0, 0x3F80), (1.00390625, 0x3F80), (1.01171875, 0x3F82), (1.0078125, 0x3F81),
           (-2.5, 0xC020), (0.0, 0x0000), (3.3895314e38, 0x7F7F), (3.4e38, 0x7F80)]
    for f, bits in kat:
        assert ob.f32_to_bf16(f) == bits, f
    # every float whose low 16 bits sweep all values, for a few exponents
    hi = np.array([0x3F80, 0x3F81, 0x0001, 0x7F7F, 0xBF80, 0x0000], np.uint32)
    lo = np.arange(65536, dtype=np.uint32)
    u = (hi[:, None] << 16 | lo[None, :]).reshape(-1)
    f = u.view(np.float32)
    got = ob.round_to_bf16(f).view(np.uint32) >> 16
    base = u >> 16
    frac = u & 0xFFFF
    up = (frac > 0x8000) | ((frac == 0x8000) & ((base & 1) == 1))
    assert np.array_equal(got, base + up.astype(np.uint32))
    assert np.array_equal(synth.round_bf16(f).view(np.uint32) >> 16, got)


def test_mxfp4_table():
    lut = [0, .5, 1, 1.5, 2, 3, 4, 6, -0.0, -.5, -1, -1.5, -2, -3, -4, -6]
    for scale in range(119, 130):
        blocks = np.zeros((1, 16), np.uint8)
        for b in range(16):
            blocks[0, b] = (b & 0xF) | (((15 - b) & 0xF) << 4)
        out = ob.mxfp4_dequant(blocks, np.array([scale], np.uint8))
        for b in range(16):
            assert out[2 * b] == lut[b] * 2.0 ** (scale - 127)
            assert out[2 * b + 1] == lut[15 - b] * 2.0 ** (scale - 127)
        assert np.array_equal(synth.round_bf16(out), out)  # exactly representable in bf16


def _tiny(rng, T, H, IM, E):
    return dict(x=rng.standard_normal((T, H)).astype(np.float32),
                wr=rng.standard_normal((E, H)).astype(np.float32),
                br=rng.standard_normal(E).astype(np.float32),
                w1=(rng.standard_normal((E, 2 * IM, H)) * 0.3).astype(np.float32),
                b1=(rng.standard_normal((E, 2 * IM)) * 0.3).astype(np.float32),
                w2=(rng.standard_normal((E, H, IM)) * 0.3).astype(np.float32),
                b2=(rng.standard_normal((E, H)) * 0.3).astype(np.float32))


def _swiglu64(o, limit=7.0):
    g = np.minimum(o[..., 0::2], limit)
    u = np.clip(o[..., 1::2], -limit, limit)
    return g / (1.0 + np.exp(-1.702 * g)) * (u + 1.0)


def test_expert_against_float64_textbook_mlp():
    rng = np.random.default_rng(3)
    d = _tiny(rng, 1, 64, 96, 1)
    y = ob.expert_token(d["x"][0], d["w1"][0], d["b1"][0], d["w2"][0], d["b2"][0], 7.0)
    o = d["w1"][0].astype(np.float64) @ d["x"][0] + d["b1"][0]
    ref = d["w2"][0].astype(np.float64) @ _swiglu64(o) + d["b2"][0]
    assert rel_l2(y, ref) < 1e-6


def test_swiglu_clamp_points():
    H = IM = 64
    w1 = np.zeros((2 * IM, H), np.float32)
    w2 = np.eye(H, IM, dtype=np.float32)
    b2 = np.zeros(H, np.float32)
    b1 = np.zeros(2 * IM, np.float32)
    b1[0:2] = (9.0, 0.5)      # gate above the limit -> 7
    b1[2:4] = (1.0, 9.0)      # up above the limit -> 7
    b1[4:6] = (1.0, -9.0)     # up below -limit -> -7
    b1[6:8] = (-30.0, 2.0)    # very negative gate: NOT clamped from below, ~0
    b1[8:10] = (-9.0, 1.0)    # gate below -limit stays -9 (CPU path, run.cpp:714-715)
    y = ob.expert_token(np.zeros(H, np.float32), w1, b1, w2, b2, 7.0)
    sig = lambda g: 1.0 / (1.0 + np.exp(-1.702 * g))
    np.testing.assert_allclose(y[0], 7 * sig(7) * 1.5, rtol=1e-6)
    np.testing.assert_allclose(y[1], 1 * sig(1) * 8.0, rtol=1e-6)
    np.testing.assert_allclose(y[2], 1 * sig(1) * -6.0, rtol=1e-6)
    assert abs(y[3]) < 1e-18
    np.testing.assert_allclose(y[4], -9 * sig(-9) * 2.0, rtol=1e-5)
    assert np.all(y[5:] == 0)


def test_layer_special_cases():
    rng = np.random.default_rng(4)
    T, H, IM, E = 6, 64, 64, 6
    d = _tiny(rng, T, H, IM, E)
    # constant-output experts: W2 = 0, b2 = c_e  ->  out = sum_k w_k c_{e_k}
    w2 = np.zeros_like(d["w2"])
    out, score, ti, tv = ob.moe_layer(d["x"], None, d["wr"], d["br"], d["w1"], d["b1"], w2, d["b2"],
                                      4, 7.0, want_routing=True)
    ref = np.einsum("tk,tkh->th", tv.astype(np.float64), d["b2"][ti].astype(np.float64))
    assert rel_l2(out, ref) < 1e-6
    # all experts share one constant -> that constant, because the weights sum to 1
    b2 = np.tile(d["b2"][0], (E, 1))
    out = ob.moe_layer(d["x"], None, d["wr"], d["br"], d["w1"], d["b1"], w2, b2, 4, 7.0)
    np.testing.assert_allclose(out, np.tile(d["b2"][0], (T, 1)), rtol=2e-6, atol=1e-7)
    # inactive rows produce zeros and do not disturb the others
    pos = np.array([0, -1, 5, -3, 2, 0], np.int32)
    full = ob.moe_layer(d["x"], None, d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], 4, 7.0)
    part = ob.moe_layer(d["x"], pos, d["wr"], d["br"], d["w1"], d["b1"], d["w2"], d["b2"], 4, 7.0)
    assert np.all(part[pos < 0] == 0)
    assert np.array_equal(part[pos >= 0], full[pos >= 0])
    # E = K = 4 with equal router rows -> plain average of the four experts
    d4 = _tiny(rng, 3, 64, 64, 4)
    wr = np.tile(d4["wr"][0], (4, 1))
    br = np.zeros(4, np.float32)
    out, _, ti, tv = ob.moe_layer(d4["x"], None, wr, br, d4["w1"], d4["b1"], d4["w2"], d4["b2"], 4,
                                  7.0, want_routing=True)
    assert np.array_equal(ti, np.tile(np.arange(4, dtype=np.int32), (3, 1)))
    assert np.all(tv == 0.25)
    ys = np.stack([[ob.expert_token(d4["x"][t], d4["w1"][e], d4["b1"][e], d4["w2"][e], d4["b2"][e], 7.0)
                    for e in range(4)] for t in range(3)])
    np.testing.assert_allclose(out, ys.astype(np.float64).mean(axis=1), rtol=1e-5, atol=1e-6)


def test_bf16_activation_rounding_point():
    """ORACLE_ROUND_ACT_BF16 rounds exactly the SwiGLU output (matmul.cpp:1427):
    with W2 = I the unrounded activation is observable, and the rounded mode must
    equal the down projection of its bf16 rounding."""
    rng = np.random.default_rng(6)
    H = IM = 64
    d = _tiny(rng, 1, H, IM, 1)
    eye = np.eye(H, IM, dtype=np.float32)
    zero = np.zeros(H, np.float32)
    act = ob.expert_token(d["x"][0], d["w1"][0], d["b1"][0], eye, zero, 7.0, mode=0)
    y_round = ob.expert_token(d["x"][0], d["w1"][0], d["b1"][0], d["w2"][0], d["b2"][0], 7.0,
                              mode=ob.ROUND_ACT_BF16)
    expect = ob.matmul(synth.round_bf16(act), d["w2"][0]) + d["b2"][0]
    assert np.array_equal(y_round, expect)
    y_plain = ob.expert_token(d["x"][0], d["w1"][0], d["b1"][0], d["w2"][0], d["b2"][0], 7.0)
    assert not np.array_equal(y_round, y_plain)
    # where the activation is already representable the two modes coincide
    b1 = np.zeros(2 * IM, np.float32)  # gate = 0 -> activation exactly 0
    a = ob.expert_token(d["x"][0], np.zeros_like(d["w1"][0]), b1, d["w2"][0], d["b2"][0], 7.0, mode=0)
    b = ob.expert_token(d["x"][0], np.zeros_like(d["w1"][0]), b1, d["w2"][0], d["b2"][0], 7.0,
                        mode=ob.ROUND_ACT_BF16)
    assert np.array_equal(a, b)
