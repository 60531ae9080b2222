"""Pins of the oracle's M = 1 linears (the weight-streaming GEMVs around the attention path). No GPU."""
import numpy as np
import pytest

from linear_cases import order_cases


def _lin(oracle, x, w, bias=None, residual=None):
    out = np.zeros(w.shape[0], dtype=np.uint16)
    assert oracle.linear_m1(x, np.ascontiguousarray(w), bias, residual, out, w.shape[0], w.shape[1]) == 0
    return out


def test_identity_weight_returns_the_input(oracle):
    n = 96
    x = oracle.normal_bf16((n,), 5)
    w = np.zeros((n, n), dtype=np.uint16)
    w[np.arange(n), np.arange(n)] = 0x3f80
    assert np.array_equal(_lin(oracle, x, w), x)


def test_small_integers_are_summed_exactly(oracle):
    rng = np.random.default_rng(3)
    rows, red = 40, 130                      # reduction not a multiple of 32: ragged last step
    xi = rng.integers(-8, 9, size=red)
    wi = rng.integers(-8, 9, size=(rows, red))
    x = oracle.f32_to_bf16(xi.astype(np.float32))
    w = oracle.f32_to_bf16(wi.astype(np.float32).ravel()).reshape(rows, red)
    want = oracle.f32_to_bf16((wi @ xi).astype(np.float32))   # |sum| <= 8320: exact in fp32, rounded once
    assert np.array_equal(_lin(oracle, x, w), want)


def test_random_rows_agree_with_fp64_dot_products(oracle):
    rows, red = 256, 2048
    x = oracle.normal_bf16((red,), 11)
    w = oracle.normal_bf16((rows, red), 12, std=0.02)
    b = oracle.normal_bf16((rows,), 13, std=0.1)
    got = oracle.bf16_to_f32(_lin(oracle, x, w, bias=b)).astype(np.float64)
    exact = oracle.bf16_to_f32(w.ravel()).reshape(rows, red).astype(np.float64) @ oracle.bf16_to_f32(x).astype(np.float64) \
        + oracle.bf16_to_f32(b).astype(np.float64)
    # fp32 accumulation error is far below a bf16 ulp: the result is the correctly rounded one,
    # up to one ulp where the exact value sits next to a rounding boundary
    ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -7
    assert np.all(np.abs(got - exact) <= ulp)
    want = oracle.bf16_to_f32(oracle.f32_to_bf16(exact.astype(np.float32))).astype(np.float64)
    assert np.mean(got == want) > 0.99


def test_linear_rows_against_fp64_and_layout(oracle):
    """qmo_linear_rows / qmo_gate_up_swiglu_rows pinned on their own, not through the scalar they loop over:
    every (row, column) against the fp64 dot product (correctly rounded up to an ulp next to a boundary), the
    bias per column, the residual per (row, column) after the rounding, and the row-major layouts (a
    transposed or strided index would move values between rows)."""
    rows, cols, red = 7, 40, 256
    x = oracle.normal_bf16((rows, red), 21)
    w = oracle.normal_bf16((cols, red), 22, std=0.05)
    b = oracle.normal_bf16((cols,), 23, std=0.1)
    res = oracle.normal_bf16((rows, cols), 24)
    xf, wf = oracle.bf16_to_f32(x).astype(np.float64), oracle.bf16_to_f32(w).astype(np.float64)
    exact = xf @ wf.T + oracle.bf16_to_f32(b).astype(np.float64)[None, :]
    out = np.zeros((rows, cols), dtype=np.uint16)
    assert oracle.linear_rows(x, w, b, None, out, rows, cols, red) == 0
    got = oracle.bf16_to_f32(out).astype(np.float64)
    assert np.all(np.abs(got - exact) <= np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -7)
    rounded = oracle.f32_to_bf16(exact.astype(np.float32))
    assert np.mean(out == rounded) > 0.99
    # residual: bf16(residual + bf16(linear)), per element
    out_r = np.zeros_like(out)
    assert oracle.linear_rows(x, w, b, res, out_r, rows, cols, red) == 0
    want_r = oracle.f32_to_bf16(oracle.bf16_to_f32(res) + oracle.bf16_to_f32(out))
    assert np.array_equal(out_r, want_r)
    # one row at a time gives the same rows (no coupling between rows)
    for r in (0, 3, 6):
        one = np.zeros((1, cols), dtype=np.uint16)
        assert oracle.linear_rows(x[r:r + 1].copy(), w, b, None, one, 1, cols, red) == 0
        assert np.array_equal(one[0], out[r])
    # gate/up/SwiGLU rows against fp64: g = bf16(x.gate), u = bf16(x.up), bf16(bf16(g*sigmoid(g)) * u)
    inter = 24
    gw = oracle.normal_bf16((inter, red), 25, std=0.05)
    uw = oracle.normal_bf16((inter, red), 26, std=0.05)
    act = np.zeros((rows, inter), dtype=np.uint16)
    assert oracle.gate_up_swiglu_rows(x, gw, uw, act, rows, red, inter) == 0
    g = oracle.bf16_to_f32(oracle.f32_to_bf16((xf @ oracle.bf16_to_f32(gw).astype(np.float64).T).astype(np.float32))).astype(np.float64)
    u = oracle.bf16_to_f32(oracle.f32_to_bf16((xf @ oracle.bf16_to_f32(uw).astype(np.float64).T).astype(np.float32))).astype(np.float64)
    silu = oracle.bf16_to_f32(oracle.f32_to_bf16((g / (1.0 + np.exp(-g))).astype(np.float32))).astype(np.float64)
    want = silu * u
    got = oracle.bf16_to_f32(act).astype(np.float64)
    assert np.all(np.abs(got - want) <= np.maximum(np.abs(want), 1e-30) * 2.0 ** -6 + 1e-6)


@pytest.mark.parametrize("case", order_cases(), ids=lambda c: c[0])
def test_evaluation_order(oracle, case):
    _, wrow, bias, residual, expected = case
    x = np.full(96, 0x3f80, dtype=np.uint16)
    w = np.stack([wrow, wrow])
    b = None if bias is None else np.full(2, bias, dtype=np.uint16)
    r = None if residual is None else np.full(2, residual, dtype=np.uint16)
    got = _lin(oracle, x, w, b, r)
    assert got[0] == expected and got[1] == expected


def test_qkv_is_three_linears_over_one_input(oracle):
    hidden, q_dim, kv_dim = 160, 48, 20
    x = oracle.normal_bf16((hidden,), 21)
    ws = [oracle.normal_bf16((n, hidden), 22 + i, std=0.05) for i, n in enumerate((q_dim, kv_dim, kv_dim))]
    bs = [oracle.normal_bf16((n,), 32 + i) for i, n in enumerate((q_dim, kv_dim, kv_dim))]
    outs = [np.zeros(n, dtype=np.uint16) for n in (q_dim, kv_dim, kv_dim)]
    assert oracle.qkv_m1(x, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2], outs[0], outs[1], outs[2],
                         hidden, q_dim, kv_dim) == 0
    for w, b, o in zip(ws, bs, outs):
        assert np.array_equal(o, _lin(oracle, x, w, bias=b))
    # routing: constant weights 1, 2, 3 and x = e_0 make every q, k, v output name its matrix
    e0 = np.zeros(hidden, dtype=np.uint16)
    e0[0] = 0x3f80
    cw = [np.full((n, hidden), v, dtype=np.uint16) for n, v in ((q_dim, 0x3f80), (kv_dim, 0x4000), (kv_dim, 0x4040))]
    assert oracle.qkv_m1(e0, cw[0], None, cw[1], None, cw[2], None, outs[0], outs[1], outs[2],
                         hidden, q_dim, kv_dim) == 0
    assert np.all(outs[0] == 0x3f80) and np.all(outs[1] == 0x4000) and np.all(outs[2] == 0x4040)


def test_argument_errors(oracle):
    x = np.zeros(4, dtype=np.uint16)
    w = np.zeros((2, 4), dtype=np.uint16)
    out = np.zeros(2, dtype=np.uint16)
    assert oracle.linear_m1(None, w, None, None, out, 2, 4) == -1
    assert oracle.linear_m1(x, w, None, None, out, -1, 4) == -5


# ---- the other M = 1 pieces of a decode layer ---------------------------------------------------------
def test_rmsnorm_closed_form_and_rounding_order(oracle):
    dim = 2048
    # constant vector c: inverse rms = 1/sqrt(c^2 + eps) exactly (the sum c^2 * dim is exact for c = 2)
    x = np.full((3, dim), 0x4000, dtype=np.uint16)             # 2.0
    w = oracle.normal_bf16((dim,), 41, mean=1.0, std=0.1)
    out = np.zeros_like(x)
    assert oracle.rmsnorm_rows(x, w, out, 3, dim) == 0
    inv = np.float32(1.0) / np.sqrt(np.float32(4.0) + np.float32(1e-6), dtype=np.float32)
    n = oracle.f32_to_bf16(np.array([np.float32(2.0) * inv], dtype=np.float32))[0]            # first rounding
    want = oracle.f32_to_bf16(oracle.bf16_to_f32(np.full(dim, n, dtype=np.uint16)) * oracle.bf16_to_f32(w))
    assert np.array_equal(out[0], want) and np.array_equal(out[1], want) and np.array_equal(out[2], want)


def test_rmsnorm_random_rows_against_fp64(oracle):
    rows, dim = 5, 2048
    x = oracle.normal_bf16((rows, dim), 42)
    w = oracle.normal_bf16((dim,), 43, mean=1.0, std=0.1)
    out = np.zeros_like(x)
    assert oracle.rmsnorm_rows(x, w, out, rows, dim) == 0
    xf = oracle.bf16_to_f32(x.ravel()).reshape(rows, dim).astype(np.float64)
    exact = xf / np.sqrt((xf ** 2).mean(axis=1, keepdims=True) + 1e-6) * oracle.bf16_to_f32(w).astype(np.float64)
    got = oracle.bf16_to_f32(out.ravel()).reshape(rows, dim).astype(np.float64)
    assert np.all(np.abs(got - exact) <= np.abs(exact) * 2.0 ** -7 + 1e-30)     # two roundings: <= 2 half-ulps


def test_add_postnorm_is_rounded_sum_then_rmsnorm(oracle):
    dim = 2048
    h = oracle.normal_bf16((dim,), 44)
    a = oracle.normal_bf16((dim,), 45)
    w = oracle.normal_bf16((dim,), 46, mean=1.0, std=0.1)
    res = np.zeros(dim, dtype=np.uint16)
    nrm = np.zeros(dim, dtype=np.uint16)
    assert oracle.add_postnorm_m1(h, a, w, res, nrm, dim) == 0
    assert np.array_equal(res, oracle.f32_to_bf16(oracle.bf16_to_f32(h) + oracle.bf16_to_f32(a)))
    again = np.zeros((1, dim), dtype=np.uint16)
    assert oracle.rmsnorm_rows(res.reshape(1, dim), w, again, 1, dim) == 0       # statistic over the rounded residual
    assert np.array_equal(nrm, again[0])


def test_gate_up_swiglu_values(oracle):
    hidden, inter = 64, 40
    x = np.zeros(hidden, dtype=np.uint16)
    x[0] = 0x3f80                                                       # e_0: g = gate[c][0], u = up[c][0]
    g = oracle.normal_bf16((inter,), 47, std=2.0)
    u = oracle.normal_bf16((inter,), 48)
    gw = np.zeros((inter, hidden), dtype=np.uint16)
    uw = np.zeros((inter, hidden), dtype=np.uint16)
    gw[:, 0], uw[:, 0] = g, u
    out = np.zeros(inter, dtype=np.uint16)
    assert oracle.gate_up_swiglu_m1(x, gw, uw, out, hidden, inter) == 0
    gf = oracle.bf16_to_f32(g).astype(np.float64)
    silu = gf / (1.0 + np.exp(-gf))
    act = oracle.bf16_to_f32(oracle.f32_to_bf16(silu.astype(np.float32))).astype(np.float64)    # bf16(silu)
    exact = act * oracle.bf16_to_f32(u).astype(np.float64)
    got = oracle.bf16_to_f32(out).astype(np.float64)
    assert np.all(np.abs(got - exact) <= np.abs(exact) * 2.0 ** -8 + 1e-30)
    # g = 0 gives exactly 0 whatever u is; a large negative gate switches the channel off
    gw[:, 0] = 0
    assert oracle.gate_up_swiglu_m1(x, gw, uw, out, hidden, inter) == 0
    assert np.all((out & 0x7fff) == 0)
    gw[:, 0] = 0xc2c8                                                   # -100
    assert oracle.gate_up_swiglu_m1(x, gw, uw, out, hidden, inter) == 0
    assert np.all(np.abs(oracle.bf16_to_f32(out)) < 1e-30)


# ---- the code predictor's order ----------------------------------------------------------------------
from linear_cases import predictor_order_cases  # noqa: E402


def _plin(oracle, x, w, residual=None):
    out = np.zeros(w.shape[0], dtype=np.uint16)
    assert oracle.predictor_linear_m1(x, np.ascontiguousarray(w), residual, out, w.shape[0], w.shape[1]) == 0
    return out


@pytest.mark.parametrize("case", predictor_order_cases(), ids=lambda c: c[0])
def test_predictor_evaluation_order(oracle, case):
    _, wrow, residual, expected = case
    x = np.full(wrow.shape[0], 0x3f80, dtype=np.uint16)
    w = np.stack([wrow, wrow])
    r = None if residual is None else np.full(2, residual, dtype=np.uint16)
    got = _plin(oracle, x, w, r)
    assert got[0] == expected and got[1] == expected


def test_predictor_linear_small_integers_and_fp64(oracle):
    rng = np.random.default_rng(11)
    rows, red = 24, 200
    xi = rng.integers(-8, 9, size=red)
    wi = rng.integers(-8, 9, size=(rows, red))
    x = oracle.f32_to_bf16(xi.astype(np.float32))
    w = oracle.f32_to_bf16(wi.astype(np.float32))
    want = oracle.f32_to_bf16((wi @ xi).astype(np.float32))          # exact in fp32, any order
    assert np.array_equal(_plin(oracle, x, w), want)
    x = oracle.normal_bf16((1024,), 12)
    w = oracle.normal_bf16((64, 1024), 13, std=0.05)
    got = oracle.bf16_to_f32(_plin(oracle, x, w)).astype(np.float64)
    ref = oracle.bf16_to_f32(w).astype(np.float64) @ oracle.bf16_to_f32(x).astype(np.float64)
    assert np.max(np.abs(got - ref) / (np.abs(ref) + 1.0)) < 1e-2    # one bf16 rounding of a fp32-accurate sum


def test_predictor_qkv_and_gate_up_are_built_from_the_linear(oracle):
    hidden, q_dim, kv_dim, inter = 192, 40, 24, 56
    x = oracle.normal_bf16((hidden,), 41)
    ws = [oracle.normal_bf16((n, hidden), 42 + i, std=0.05) for i, n in enumerate((q_dim, kv_dim, kv_dim))]
    outs = [np.zeros(n, dtype=np.uint16) for n in (q_dim, kv_dim, kv_dim)]
    assert oracle.predictor_qkv_m1(x, ws[0], ws[1], ws[2], outs[0], outs[1], outs[2], hidden, q_dim, kv_dim) == 0
    for w, o in zip(ws, outs):
        assert np.array_equal(o, _plin(oracle, x, w))
    gate = oracle.normal_bf16((inter, hidden), 51, std=0.08)
    up = oracle.normal_bf16((inter, hidden), 52, std=0.08)
    out = np.zeros(inter, dtype=np.uint16)
    assert oracle.predictor_gate_up_swiglu_m1(x, gate, up, out, hidden, inter) == 0
    g = oracle.bf16_to_f32(_plin(oracle, x, gate)).astype(np.float64)
    u = oracle.bf16_to_f32(_plin(oracle, x, up)).astype(np.float64)
    want = g / (1.0 + np.exp(-g)) * u                                  # SiLU(g) * u
    got = oracle.bf16_to_f32(out).astype(np.float64)
    assert np.max(np.abs(got - want) / (np.abs(want) + 1e-3)) < 2e-2   # two bf16 roundings


@pytest.mark.parametrize("seed", [0, 1])
def test_the_predictors_step_0_is_two_m1_steps_in_the_talkers_chain_order(oracle, seed):
    """What lets the frame kernel run step 0 as two more passes of its loop: one predictor layer over the two rows of step 0
    with the reference's row operators (generic linears, per-head RMSNorm, BHSD transpose / RoPE / cache update, staged
    causal attention; R17:13663-13699) leaves, bit for bit, what two M = 1 steps at cache positions 0 and 1 leave with the
    talker-order M = 1 operators (fused Q/K/V, QK-norm + RoPE + append, M = 1 attention, o_proj, add + post-norm,
    gate/up/SwiGLU, down_proj + residual): the layer's output rows, both caches and the attention's context."""
    PH, Q, KV, PI, rows = 1024, 2048, 1024, 3072, 2
    u16 = lambda *s: np.zeros(s, dtype=np.uint16)
    n = [7000 + 100 * seed]

    def rnd(shape, std=1.0, mean=0.0):
        n[0] += 1
        return oracle.normal_bf16(shape, n[0], mean, std, threads=8)

    w = dict(inn=rnd((PH,), 0.1, 1.0), wq=rnd((Q, PH), 0.03), wk=rnd((KV, PH), 0.03), wv=rnd((KV, PH), 0.03),
             gq=rnd((128,), 0.1, 1.0), gk=rnd((128,), 0.1, 1.0), wo=rnd((PH, Q), 0.02), post=rnd((PH,), 0.1, 1.0),
             wg=rnd((PI, PH), 0.03), wu=rnd((PI, PH), 0.03), wd=rnd((PH, PI), 0.02))
    cur = rnd((rows, PH))
    cos, sin = oracle.rope_table(16, 0)
    # the row operators
    kc, vc = u16(8, 16, 128), u16(8, 16, 128)
    norm, q, k, v = u16(rows, PH), u16(rows, Q), u16(rows, KV), u16(rows, KV)
    assert oracle.rmsnorm_rows(cur, w["inn"], norm, rows, PH) == 0
    for name, dst, columns in (("wq", q, Q), ("wk", k, KV), ("wv", v, KV)):
        assert oracle.linear_rows(norm, w[name], None, None, dst, rows, columns, PH, 8) == 0
    qn, kn = u16(rows * 16, 128), u16(rows * 8, 128)
    assert oracle.rmsnorm_rows(q.reshape(rows * 16, 128), w["gq"], qn, rows * 16, 128) == 0
    assert oracle.rmsnorm_rows(k.reshape(rows * 8, 128), w["gk"], kn, rows * 8, 128) == 0
    qb, kb, vb = u16(16, rows, 128), u16(8, rows, 128), u16(8, rows, 128)
    assert oracle.predictor_transpose(qn, qb, rows, 16) == 0
    assert oracle.predictor_transpose(kn, kb, rows, 8) == 0
    assert oracle.predictor_transpose(v, vb, rows, 8) == 0
    qr, kr = u16(16, rows, 128), u16(8, rows, 128)
    assert oracle.predictor_rope_bhsd(qb, cos, sin, qr, rows, 16) == 0
    assert oracle.predictor_rope_bhsd(kb, cos, sin, kr, rows, 8) == 0
    assert oracle.predictor_update_cache(kr, kc, rows, 0) == 0
    assert oracle.predictor_update_cache(vb, vc, rows, 0) == 0
    ctx = u16(rows, Q)
    assert oracle.predictor_attention_staged(qr, kc, vc, ctx.reshape(rows, 16, 128), rows, 2, True) == 0
    res, post, act, out_rows = u16(rows, PH), u16(rows, PH), u16(rows, PI), u16(rows, PH)
    assert oracle.linear_rows(ctx, w["wo"], None, cur, res, rows, PH, Q, 8) == 0
    assert oracle.rmsnorm_rows(res, w["post"], post, rows, PH) == 0
    assert oracle.gate_up_swiglu_rows(post, w["wg"], w["wu"], act, rows, PH, PI, 8) == 0
    assert oracle.linear_rows(act, w["wd"], None, res, out_rows, rows, PH, PI, 8) == 0
    # two M = 1 steps
    kc2, vc2 = u16(8, 16, 128), u16(8, 16, 128)
    for r in range(rows):
        norm1, q1, k1, v1, qrot, ctx1, attn, res1, post1, act1, out1 = (u16(1, PH), u16(Q), u16(KV), u16(KV), u16(Q), u16(Q), u16(PH),
                                                                        u16(PH), u16(PH), u16(PI), u16(PH))
        assert oracle.rmsnorm_rows(cur[r].reshape(1, PH), w["inn"], norm1, 1, PH) == 0
        assert oracle.qkv_m1(norm1[0], w["wq"], None, w["wk"], None, w["wv"], None, q1, k1, v1, PH, Q, KV, 8) == 0
        assert oracle.qk_norm_rope_kv_append(q1, k1, v1, w["gq"], w["gk"], cos[r], sin[r], qrot, oracle.flat_cache(kc2, vc2, 8, 16),
                                             None, 1, 16, r) == 0
        assert oracle.predictor_attention_m1(qrot, kc2, vc2, ctx1, r + 1) == 0
        assert np.array_equal(ctx1, ctx[r])
        assert oracle.linear_m1(ctx1, w["wo"], None, None, attn, PH, Q, 8) == 0
        assert oracle.add_postnorm_m1(cur[r], attn, w["post"], res1, post1, PH) == 0
        assert oracle.gate_up_swiglu_m1(post1, w["wg"], w["wu"], act1, PH, PI, 8) == 0
        assert oracle.linear_m1(act1, w["wd"], None, res1, out1, PH, PI, 8) == 0
        assert np.array_equal(out1, out_rows[r])
    assert np.array_equal(kc, kc2) and np.array_equal(vc, vc2)
    assert np.any(kc[:, :2] != 0) and not np.any(kc[:, 2:] != 0)
