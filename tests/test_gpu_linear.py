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


@pytest.mark.parametrize("rows,dim", [(1, 2048), (3, 2048), (2, 1024), (5, 130), (1, 16), (2, 6144)])
def test_rmsnorm_rows_bit_exact(oracle, qm, dev, rows, dim):
    import torch
    x = oracle.normal_bf16((rows, dim), 500 + dim)
    w = oracle.normal_bf16((dim,), 501 + dim, mean=1.0, std=0.1)
    want = np.zeros_like(x)
    assert oracle.rmsnorm_rows(x, w, want, rows, dim) == 0
    out = torch.full((rows, dim), 0x7fc0, dtype=torch.int16, device=dev)
    qm.rmsnorm_rows(to_dev(x, dev), to_dev(w, dev), out, rows, dim)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(out), want)


@pytest.mark.parametrize("dim", [2048, 1024, 130, 6])
def test_add_postnorm_bit_exact(oracle, qm, dev, dim):
    import torch
    h = oracle.normal_bf16((dim,), 600 + dim)
    a = oracle.normal_bf16((dim,), 601 + dim)
    w = oracle.normal_bf16((dim,), 602 + dim, mean=1.0, std=0.1)
    res, nrm = np.zeros(dim, dtype=np.uint16), np.zeros(dim, dtype=np.uint16)
    assert oracle.add_postnorm_m1(h, a, w, res, nrm, dim) == 0
    rd = torch.full((dim,), 0x7fc0, dtype=torch.int16, device=dev)
    nd = torch.full((dim,), 0x7fc0, dtype=torch.int16, device=dev)
    qm.add_postnorm_m1(to_dev(h, dev), to_dev(a, dev), to_dev(w, dev), rd, nd, dim)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(rd), res) and np.array_equal(to_u16(nd), nrm)


@pytest.mark.parametrize("hidden,inter", [(2048, 6144), (2048, 3072), (66, 33), (34, 1)])
def test_gate_up_swiglu(oracle, qm, dev, hidden, inter):
    """Bit-identical except where the device's expf and glibc's differ in the last place and the
    two bf16 roundings behind it do not hide that: at most one bf16 ulp, on well under 0.1 % of outputs."""
    import torch
    from qm_testlib import ulp_distance
    x = oracle.normal_bf16((hidden,), 700 + hidden)
    gw = oracle.normal_bf16((inter, hidden), 701 + hidden, std=0.03)
    uw = oracle.normal_bf16((inter, hidden), 702 + hidden, std=0.03)
    want = np.zeros(inter, dtype=np.uint16)
    assert oracle.gate_up_swiglu_m1(x, gw, uw, want, hidden, inter, 16) == 0
    out = torch.full((inter,), 0x7fc0, dtype=torch.int16, device=dev)
    qm.gate_up_swiglu_m1(to_dev(x, dev), to_dev(gw, dev), to_dev(uw, dev), out, hidden, inter)
    torch.cuda.synchronize()
    got = to_u16(out)
    d = ulp_distance(got, want)
    assert d.max() <= 1
    assert np.count_nonzero(d) <= max(1, inter // 1000)


@pytest.mark.parametrize("hidden,q_dim,kv_dim", [(2048, 2048, 1024), (512, 40, 24), (1024, 8, 8)])
def test_fused_rmsnorm_qkv_equals_the_two_operators(oracle, qm, dev, hidden, q_dim, kv_dim):
    import torch
    seed = 1100 + hidden
    x = oracle.normal_bf16((hidden,), seed)
    nw = oracle.normal_bf16((hidden,), seed + 1, mean=1.0, std=0.1)
    dims = (q_dim, kv_dim, kv_dim)
    ws = [oracle.normal_bf16((n, hidden), seed + 2 + i, std=0.02) for i, n in enumerate(dims)]
    bs = [oracle.normal_bf16((n,), seed + 6 + i, std=0.1) for i, n in enumerate(dims)]
    normed = np.zeros((1, hidden), dtype=np.uint16)
    assert oracle.rmsnorm_rows(x.reshape(1, hidden), nw, normed, 1, hidden) == 0
    want = [np.zeros(n, dtype=np.uint16) for n in dims]
    assert oracle.qkv_m1(normed[0], ws[0], bs[0], ws[1], bs[1], ws[2], bs[2], want[0], want[1], want[2],
                         hidden, q_dim, kv_dim, 16) == 0
    outs = [torch.full((n,), 0x7fc0, dtype=torch.int16, device=dev) for n in dims]
    wd = [to_dev(w, dev) for w in ws]
    bd = [to_dev(b, dev) for b in bs]
    qm.rmsnorm_qkv_m1(to_dev(x, dev), to_dev(nw, dev), wd[0], bd[0], wd[1], bd[1], wd[2], bd[2], outs[0], outs[1],
                      outs[2], hidden, q_dim, kv_dim)
    torch.cuda.synchronize()
    for o, w_ in zip(outs, want):
        assert np.array_equal(to_u16(o), w_)


@pytest.mark.parametrize("hidden,inter", [(2048, 6144), (512, 20), (64, 8)])
def test_fused_add_postnorm_gate_up_equals_the_two_operators(oracle, qm, dev, hidden, inter):
    import torch
    from qm_testlib import ulp_distance
    seed = 1200 + hidden
    h = oracle.normal_bf16((hidden,), seed)
    a = oracle.normal_bf16((hidden,), seed + 1)
    nw = oracle.normal_bf16((hidden,), seed + 2, mean=1.0, std=0.1)
    gw = oracle.normal_bf16((inter, hidden), seed + 3, std=0.03)
    uw = oracle.normal_bf16((inter, hidden), seed + 4, std=0.03)
    res, nrm = np.zeros(hidden, dtype=np.uint16), np.zeros(hidden, dtype=np.uint16)
    assert oracle.add_postnorm_m1(h, a, nw, res, nrm, hidden) == 0
    want = np.zeros(inter, dtype=np.uint16)
    assert oracle.gate_up_swiglu_m1(nrm, gw, uw, want, hidden, inter, 16) == 0
    rd = torch.full((hidden,), 0x7fc0, dtype=torch.int16, device=dev)
    out = torch.full((inter,), 0x7fc0, dtype=torch.int16, device=dev)
    qm.add_postnorm_gate_up_swiglu_m1(to_dev(h, dev), to_dev(a, dev), to_dev(nw, dev), rd, to_dev(gw, dev),
                                      to_dev(uw, dev), out, hidden, inter)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(rd), res)
    d = ulp_distance(to_u16(out), want)
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, inter // 1000)


def test_fused_entries_reject_what_the_staged_kernel_cannot_take(qm, dev):
    import torch
    x = torch.zeros(68, dtype=torch.int16, device=dev)
    w = torch.zeros((8, 68), dtype=torch.int16, device=dev)
    o = torch.zeros(8, dtype=torch.int16, device=dev)
    L = qm.lib()
    # hidden = 68 is even (fine for qm_qkv_m1) but not a multiple of 8
    assert L.qm_rmsnorm_qkv_m1(x.data_ptr(), x.data_ptr(), 1e-6, w.data_ptr(), None, w.data_ptr(), None, w.data_ptr(),
                               None, o.data_ptr(), o.data_ptr(), o.data_ptr(), 68, 8, 8, None) == -2
    assert L.qm_add_postnorm_gate_up_swiglu_m1(x.data_ptr(), x.data_ptr(), x.data_ptr(), 1e-6, x.data_ptr(),
                                               w.data_ptr(), w.data_ptr(), o.data_ptr(), 68, 8, None) == -2
    assert L.qm_rmsnorm_qkv_m1(None, x.data_ptr(), 1e-6, w.data_ptr(), None, w.data_ptr(), None, w.data_ptr(),
                               None, o.data_ptr(), o.data_ptr(), o.data_ptr(), 64, 8, 8, None) == -1


# ---- the code predictor's twins (pair order of the chains, no bias) -----------------------------------
from linear_cases import predictor_order_cases  # noqa: E402


def _gpu_plinear(qm, dev, x, w, residual=None):
    import torch
    out = torch.full((w.shape[0],), 0x7fc0, dtype=torch.int16, device=dev)
    qm.predictor_linear_m1(to_dev(x, dev), to_dev(np.ascontiguousarray(w), dev),
                           None if residual is None else to_dev(residual, dev), out, w.shape[0], w.shape[1])
    torch.cuda.synchronize()
    return to_u16(out)


@pytest.mark.parametrize("rows,red,residual", [
    (1024, 2048, True),       # o_proj + residual of the predictor (kQueryDim -> kHidden)
    (1024, 3072, True),       # down_proj + residual
    (2048, 1024, False), (1, 8, False), (5, 72, True), (33, 136, False), (7, 4104, True), (3, 16384, False),
])
def test_predictor_linear_m1_bit_exact(oracle, qm, dev, rows, red, residual):
    seed = 2100 + rows + red
    x = oracle.normal_bf16((red,), seed)
    w = oracle.normal_bf16((rows, red), seed + 1, std=0.02)
    r = oracle.normal_bf16((rows,), seed + 3) if residual else None
    want = np.zeros(rows, dtype=np.uint16)
    assert oracle.predictor_linear_m1(x, w, r, want, rows, red, 16) == 0
    assert np.array_equal(_gpu_plinear(qm, dev, x, w, r), want)


@pytest.mark.parametrize("case", [c for c in predictor_order_cases() if c[1].shape[0] % 8 == 0], ids=lambda c: c[0])
def test_predictor_evaluation_order_on_the_gpu(qm, dev, case):
    _, wrow, residual, expected = case
    x = np.full(wrow.shape[0], 0x3f80, dtype=np.uint16)
    w = np.stack([wrow] * 9)                   # more rows than one block owns
    r = None if residual is None else np.full(9, residual, dtype=np.uint16)
    got = _gpu_plinear(qm, dev, x, w, r)
    assert np.all(got == expected)


@pytest.mark.parametrize("hidden,q_dim,kv_dim", [(1024, 2048, 1024), (200, 40, 24), (8, 1, 1)])
def test_predictor_qkv_m1_bit_exact(oracle, qm, dev, hidden, q_dim, kv_dim):
    import torch
    seed = 2300 + hidden
    x = oracle.normal_bf16((hidden,), seed)
    nw = oracle.normal_bf16((hidden,), seed + 9, mean=1.0, std=0.1)
    dims = (q_dim, kv_dim, kv_dim)
    ws = [oracle.normal_bf16((n, hidden), seed + 1 + i, std=0.02) for i, n in enumerate(dims)]
    wd = [to_dev(w, dev) for w in ws]
    want = [np.zeros(n, dtype=np.uint16) for n in dims]
    assert oracle.predictor_qkv_m1(x, ws[0], ws[1], ws[2], want[0], want[1], want[2], hidden, q_dim, kv_dim, 16) == 0
    outs = [torch.full((n,), 0x7fc0, dtype=torch.int16, device=dev) for n in dims]
    qm.predictor_qkv_m1(to_dev(x, dev), wd[0], wd[1], wd[2], outs[0], outs[1], outs[2], hidden, q_dim, kv_dim)
    torch.cuda.synchronize()
    for o, w_ in zip(outs, want):
        assert np.array_equal(to_u16(o), w_)
    # fused with the RMSNorm in front of it = the two operators
    normed = np.zeros((1, hidden), dtype=np.uint16)
    assert oracle.rmsnorm_rows(x.reshape(1, hidden), nw, normed, 1, hidden) == 0
    assert oracle.predictor_qkv_m1(normed[0], ws[0], ws[1], ws[2], want[0], want[1], want[2], hidden, q_dim, kv_dim,
                                   16) == 0
    outs = [torch.full((n,), 0x7fc0, dtype=torch.int16, device=dev) for n in dims]
    qm.predictor_rmsnorm_qkv_m1(to_dev(x, dev), to_dev(nw, dev), wd[0], wd[1], wd[2], outs[0], outs[1], outs[2],
                                hidden, q_dim, kv_dim)
    torch.cuda.synchronize()
    for o, w_ in zip(outs, want):
        assert np.array_equal(to_u16(o), w_)


@pytest.mark.parametrize("hidden,inter", [(1024, 3072), (200, 33), (8, 1)])
def test_predictor_gate_up_swiglu(oracle, qm, dev, hidden, inter):
    """As for the talker's: identical up to the last place of expf (at most one bf16 ulp, rarely)."""
    import torch
    from qm_testlib import ulp_distance
    seed = 2700 + hidden
    x = oracle.normal_bf16((hidden,), seed)
    gw = oracle.normal_bf16((inter, hidden), seed + 1, std=0.03)
    uw = oracle.normal_bf16((inter, hidden), seed + 2, std=0.03)
    want = np.zeros(inter, dtype=np.uint16)
    assert oracle.predictor_gate_up_swiglu_m1(x, gw, uw, want, hidden, inter, 16) == 0
    out = torch.full((inter,), 0x7fc0, dtype=torch.int16, device=dev)
    qm.predictor_gate_up_swiglu_m1(to_dev(x, dev), to_dev(gw, dev), to_dev(uw, dev), out, hidden, inter)
    torch.cuda.synchronize()
    d = ulp_distance(to_u16(out), want)
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, inter // 1000)
    # fused with residual add + post-norm in front of it = the two operators
    h = oracle.normal_bf16((hidden,), seed + 3)
    a = oracle.normal_bf16((hidden,), seed + 4)
    nw = oracle.normal_bf16((hidden,), seed + 5, mean=1.0, std=0.1)
    res, nrm = np.zeros(hidden, dtype=np.uint16), np.zeros(hidden, dtype=np.uint16)
    assert oracle.add_postnorm_m1(h, a, nw, res, nrm, hidden) == 0
    assert oracle.predictor_gate_up_swiglu_m1(nrm, gw, uw, want, hidden, inter, 16) == 0
    rd = torch.full((hidden,), 0x7fc0, dtype=torch.int16, device=dev)
    out = torch.full((inter,), 0x7fc0, dtype=torch.int16, device=dev)
    qm.predictor_add_postnorm_gate_up_swiglu_m1(to_dev(h, dev), to_dev(a, dev), to_dev(nw, dev), rd, to_dev(gw, dev),
                                                to_dev(uw, dev), out, hidden, inter)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(rd), res)
    d = ulp_distance(to_u16(out), want)
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, inter // 1000)


def test_predictor_linears_reject_what_the_staged_kernel_cannot_take(qm, dev):
    import torch
    x = torch.zeros(68, dtype=torch.int16, device=dev)
    w = torch.zeros((8, 68), dtype=torch.int16, device=dev)
    o = torch.zeros(8, dtype=torch.int16, device=dev)
    L = qm.lib()
    assert L.qm_predictor_linear_m1(x.data_ptr(), w.data_ptr(), None, o.data_ptr(), 8, 68, None) == -2   # 68 % 8 != 0
    assert L.qm_predictor_linear_m1(x.data_ptr(), w.data_ptr(), None, o.data_ptr(), 8, 67, None) == -2   # odd
    assert L.qm_predictor_linear_m1(None, w.data_ptr(), None, o.data_ptr(), 8, 64, None) == -1
    assert L.qm_predictor_qkv_m1(x.data_ptr(), w.data_ptr(), w.data_ptr(), w.data_ptr(), o.data_ptr(), o.data_ptr(),
                                 o.data_ptr(), 68, 8, 8, None) == -2
    assert L.qm_predictor_gate_up_swiglu_m1(x.data_ptr(), w.data_ptr(), w.data_ptr(), o.data_ptr(), 64, -1, None) == -5
