"""GPU parity: linears over token rows (the prompt pass) through the C ABI — bit-exact against
the oracle, which evaluates every (row, column) as the M = 1 linear does."""
import numpy as np
import pytest

from qm_testlib import to_dev, to_u16, ulp_distance

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("rows,cols,red,bias,residual", [
    (1, 8, 8, False, False), (7, 20, 40, True, True), (8, 9, 264, True, False), (9, 33, 1000, False, True),
    (100, 2048, 2048, True, True),      # o_proj of a 100-token prompt + residual
    (37, 2048, 6144, False, True),      # down_proj + residual: four columns per block
    (300, 1024, 2048, True, False),     # k_proj
])
def test_linear_rows_bit_exact(oracle, qm, dev, rows, cols, red, bias, residual):
    import torch
    seed = 4000 + rows + cols + red
    x = oracle.normal_bf16((rows, red), seed)
    w = oracle.normal_bf16((cols, red), seed + 1, std=0.02)
    b = oracle.normal_bf16((cols,), seed + 2, std=0.1) if bias else None
    r = oracle.normal_bf16((rows, cols), seed + 3) if residual else None
    want = np.zeros((rows, cols), dtype=np.uint16)
    assert oracle.linear_rows(x, w, b, r, want, rows, cols, red, 16) == 0
    out = torch.full((rows, cols), 0x7fc0, dtype=torch.int16, device=dev)
    qm.linear_rows(to_dev(x, dev), to_dev(w, dev), None if b is None else to_dev(b, dev),
                   None if r is None else to_dev(r, dev), out, rows, cols, red)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(out), want)


def test_a_prompt_row_equals_the_decode_linear_of_that_row(oracle, qm, dev):
    import torch
    rows, cols, red = 12, 96, 2048
    x = oracle.normal_bf16((rows, red), 1)
    w = oracle.normal_bf16((cols, red), 2, std=0.02)
    b = oracle.normal_bf16((cols,), 3, std=0.1)
    xd, wd, bd = to_dev(x, dev), to_dev(w, dev), to_dev(b, dev)
    out = torch.zeros((rows, cols), dtype=torch.int16, device=dev)
    qm.linear_rows(xd, wd, bd, None, out, rows, cols, red)
    one = torch.zeros(cols, dtype=torch.int16, device=dev)
    for r in (0, 5, 11):
        qm.linear_m1(xd[r], wd, bd, None, one, cols, red)
        torch.cuda.synchronize()
        assert torch.equal(one, out[r])


@pytest.mark.parametrize("rows,hidden,inter", [(1, 8, 1), (9, 200, 33), (64, 2048, 6144), (5, 2048, 512)])
def test_gate_up_swiglu_rows(oracle, qm, dev, rows, hidden, inter):
    import torch
    seed = 5000 + rows + hidden
    x = oracle.normal_bf16((rows, hidden), seed)
    gw = oracle.normal_bf16((inter, hidden), seed + 1, std=0.03)
    uw = oracle.normal_bf16((inter, hidden), seed + 2, std=0.03)
    want = np.zeros((rows, inter), dtype=np.uint16)
    assert oracle.gate_up_swiglu_rows(x, gw, uw, want, rows, hidden, inter, 16) == 0
    out = torch.full((rows, inter), 0x7fc0, dtype=torch.int16, device=dev)
    qm.gate_up_swiglu_rows(to_dev(x, dev), to_dev(gw, dev), to_dev(uw, dev), out, rows, hidden, inter)
    torch.cuda.synchronize()
    d = ulp_distance(to_u16(out), want)                 # (the device's expf: at most one bf16 ulp, rarely)
    assert d.max() <= 1 and np.count_nonzero(d) <= max(1, rows * inter // 1000)


def test_linear_rows_argument_errors(qm, dev):
    import torch
    x = torch.zeros((4, 72), dtype=torch.int16, device=dev)
    w = torch.zeros((8, 72), dtype=torch.int16, device=dev)
    o = torch.zeros((4, 8), dtype=torch.int16, device=dev)
    L = qm.lib()
    assert L.qm_linear_rows(None, w.data_ptr(), None, None, o.data_ptr(), 4, 8, 72, None) == -1
    assert L.qm_linear_rows(x.data_ptr(), w.data_ptr(), None, None, o.data_ptr(), 4, 8, 70, None) == -2
    assert L.qm_linear_rows(x.data_ptr(), w.data_ptr(), None, None, o.data_ptr(), -1, 8, 72, None) == -5
    assert L.qm_linear_rows(x.data_ptr() + 2, w.data_ptr(), None, None, o.data_ptr(), 1, 8, 64, None) == -2
    assert L.qm_linear_rows(x.data_ptr(), w.data_ptr(), None, None, o.data_ptr(), 0, 8, 72, None) == 0
    assert L.qm_gate_up_swiglu_rows(x.data_ptr(), w.data_ptr(), None, o.data_ptr(), 4, 72, 8, None) == -1
