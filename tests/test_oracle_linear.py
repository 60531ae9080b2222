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
