"""GPU parity: M = 1 linear and fused Q/K/V projection through the C ABI — bit-exact against the
oracle (the kernel reproduces the reference's fp32 summation order)."""
import numpy as np
import pytest

from linear_cases import order_cases
from qm_testlib import to_dev, to_u16

pytestmark = pytest.mark.gpu


def _gpu_linear(qm, dev, x, w, bias=None, residual=None):
    import torch
    out = torch.full((w.shape[0],), 0x7fc0, dtype=torch.int16, device=dev)
    qm.linear_m1(to_dev(x, dev), to_dev(np.ascontiguousarray(w), dev), None if bias is None else to_dev(bias, dev),
                 None if residual is None else to_dev(residual, dev), out, w.shape[0], w.shape[1])
    torch.cuda.synchronize()
    return to_u16(out)


def _cpu_linear(oracle, x, w, bias=None, residual=None):
    out = np.zeros(w.shape[0], dtype=np.uint16)
    assert oracle.linear_m1(x, np.ascontiguousarray(w), bias, residual, out, w.shape[0], w.shape[1], 16) == 0
    return out


@pytest.mark.parametrize("rows,red,bias,residual", [
    (2048, 2048, True, False),      # o_proj
    (2048, 6144, False, True),      # down_proj + residual: three register batches and a half
    (1, 2, False, False), (17, 34, True, True), (33, 62, True, False), (5, 66, False, True),
    (100, 2050, True, True), (16, 4096, True, True), (3, 16384, False, False),
])
def test_linear_m1_bit_exact(oracle, qm, dev, rows, red, bias, residual):
    seed = 100 + rows + red
    x = oracle.normal_bf16((red,), seed)
    w = oracle.normal_bf16((rows, red), seed + 1, std=0.02)
    b = oracle.normal_bf16((rows,), seed + 2, std=0.1) if bias else None
    r = oracle.normal_bf16((rows,), seed + 3) if residual else None
    assert np.array_equal(_gpu_linear(qm, dev, x, w, b, r), _cpu_linear(oracle, x, w, b, r))


@pytest.mark.parametrize("hidden,q_dim,kv_dim", [(2048, 2048, 1024), (1024, 2048, 1024), (160, 48, 20), (34, 1, 1)])
def test_qkv_m1_bit_exact(oracle, qm, dev, hidden, q_dim, kv_dim):
    import torch
    seed = 300 + hidden
    x = oracle.normal_bf16((hidden,), seed)
    dims = (q_dim, kv_dim, kv_dim)
    ws = [oracle.normal_bf16((n, hidden), seed + 1 + i, std=0.02) for i, n in enumerate(dims)]
    bs = [oracle.normal_bf16((n,), seed + 5 + i, std=0.1) for i, n in enumerate(dims)]
    want = [np.zeros(n, dtype=np.uint16) for n in dims]
    assert oracle.qkv_m1(x, ws[0], bs[0], ws[1], bs[1], ws[2], bs[2], want[0], want[1], want[2],
                         hidden, q_dim, kv_dim, 16) == 0
    outs = [torch.full((n,), 0x7fc0, dtype=torch.int16, device=dev) for n in dims]
    wd = [to_dev(w, dev) for w in ws]
    bd = [to_dev(b, dev) for b in bs]
    qm.qkv_m1(to_dev(x, dev), wd[0], bd[0], wd[1], bd[1], wd[2], bd[2], outs[0], outs[1], outs[2],
              hidden, q_dim, kv_dim)
    torch.cuda.synchronize()
    for o, w_ in zip(outs, want):
        assert np.array_equal(to_u16(o), w_)
    # without biases
    assert oracle.qkv_m1(x, ws[0], None, ws[1], None, ws[2], None, want[0], want[1], want[2],
                         hidden, q_dim, kv_dim, 16) == 0
    qm.qkv_m1(to_dev(x, dev), wd[0], None, wd[1], None, wd[2], None, outs[0], outs[1], outs[2],
              hidden, q_dim, kv_dim)
    torch.cuda.synchronize()
    for o, w_ in zip(outs, want):
        assert np.array_equal(to_u16(o), w_)


@pytest.mark.parametrize("case", order_cases(), ids=lambda c: c[0])
def test_evaluation_order_on_the_gpu(qm, dev, case):
    _, wrow, bias, residual, expected = case
    x = np.full(96, 0x3f80, dtype=np.uint16)
    w = np.stack([wrow] * 18)      # more than one wave row group
    b = None if bias is None else np.full(18, bias, dtype=np.uint16)
    r = None if residual is None else np.full(18, residual, dtype=np.uint16)
    assert np.all(_gpu_linear(qm, dev, x, w, b, r) == expected)


def test_qkv_step_feeds_norm_rope_append_bit_exactly(oracle, qm, dev):
    """The decode-step front half as the reference chains it (R17:17176-17186): fused Q/K/V
    projection, then QK-RMSNorm + RoPE + append into the flat LayerCache — every bit of q_rotated
    and of both caches equals the oracle's."""
    import torch
    hidden, q_dim, kv_dim, max_cache, pos = 2048, 2048, 1024, 64, 37
    x = oracle.normal_bf16((hidden,), 900)
    ws = [oracle.normal_bf16((n, hidden), 901 + i, std=0.02) for i, n in enumerate((q_dim, kv_dim, kv_dim))]
    gq = oracle.normal_bf16((128,), 905, mean=1.0, std=0.1)
    gk = oracle.normal_bf16((128,), 906, mean=1.0, std=0.1)
    cos, sin = oracle.rope_table(1, pos)
    q, k, v = (np.zeros(n, dtype=np.uint16) for n in (q_dim, kv_dim, kv_dim))
    assert oracle.qkv_m1(x, ws[0], None, ws[1], None, ws[2], None, q, k, v, hidden, q_dim, kv_dim, 16) == 0
    kc = np.zeros((8, max_cache, 128), dtype=np.uint16)
    vc = np.zeros((8, max_cache, 128), dtype=np.uint16)
    qrot = np.zeros(q_dim, dtype=np.uint16)
    assert oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qrot, oracle.flat_cache(kc, vc, 8, max_cache),
                                         None, 1, 16, pos, 1e-6) == 0
    qd, kd, vd = (torch.zeros(n, dtype=torch.int16, device=dev) for n in (q_dim, kv_dim, kv_dim))
    wd = [to_dev(w, dev) for w in ws]
    qm.qkv_m1(to_dev(x, dev), wd[0], None, wd[1], None, wd[2], None, qd, kd, vd, hidden, q_dim, kv_dim)
    kcd = torch.zeros((8, max_cache, 128), dtype=torch.int16, device=dev)
    vcd = torch.zeros((8, max_cache, 128), dtype=torch.int16, device=dev)
    qrd = torch.zeros(q_dim, dtype=torch.int16, device=dev)
    qm.qk_norm_rope_kv_append(qd, kd, vd, to_dev(gq, dev), to_dev(gk, dev), to_dev(cos, dev), to_dev(sin, dev), qrd,
                              qm.flat_cache(kcd, vcd, 8, max_cache), None, 1, 16, pos, 1e-6)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(qrd), qrot)
    assert np.array_equal(to_u16(kcd), kc) and np.array_equal(to_u16(vcd), vc)


def test_linear_argument_errors(qm, dev):
    import torch
    x = torch.zeros(64, dtype=torch.int16, device=dev)
    w = torch.zeros((4, 64), dtype=torch.int16, device=dev)
    out = torch.zeros(4, dtype=torch.int16, device=dev)
    L = qm.lib()
    assert L.qm_linear_m1(None, w.data_ptr(), None, None, out.data_ptr(), 4, 64, None) == -1
    assert L.qm_linear_m1(x.data_ptr(), w.data_ptr(), None, None, out.data_ptr(), 4, 63, None) == -2    # odd reduction
    assert L.qm_linear_m1(x.data_ptr(), w.data_ptr(), None, None, out.data_ptr(), 4, 20000, None) == -2
    assert L.qm_linear_m1(x.data_ptr(), w.data_ptr(), None, None, out.data_ptr(), -1, 64, None) == -5
    assert L.qm_linear_m1(x.data_ptr(), w.data_ptr(), None, None, out.data_ptr(), 0, 64, None) == 0
    assert L.qm_qkv_m1(x.data_ptr(), w.data_ptr(), None, None, None, w.data_ptr(), None, out.data_ptr(),
                       out.data_ptr(), out.data_ptr(), 64, 4, 4, None) == -1
