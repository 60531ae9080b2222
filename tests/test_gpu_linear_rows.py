"""GPU parity: linears over token rows (the prompt pass) through the C ABI, against the oracle, which evaluates every
(row, column) as the M = 1 linear does.  Two kernels serve the entry points (QM_OPT_LINEAR_ROWS_KERNEL): the exact chain
(1; also what fewer than 16 rows or shapes off the matrix tiles always run) must be bit-exact; the matrix cores (0,
default) form the same fp32 sum of the same bf16 products in another order, so an output may land on the neighbouring
bf16 value: at most one ulp, and rarely."""
import numpy as np
import pytest

from qm_testlib import to_dev, to_u16, ulp_distance

pytestmark = pytest.mark.gpu

EXACT, MATRIX = 1, 0


@pytest.fixture(autouse=True, params=[EXACT, MATRIX], ids=["exact_chain", "matrix_cores"])
def rows_kernel(request, qm):
    qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, request.param)
    yield request.param
    qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, 0)


def _on_matrix_cores(kernel, rows, cols, red):
    return kernel == MATRIX and rows >= 16 and cols % 128 == 0 and red % 128 == 0


def _check(oracle, got, want, matrix, residual=None):
    if not matrix:
        assert np.array_equal(got, want)
        return
    # one bf16 spacing of the sum (which a residual of the opposite sign can leave standing alone in a small result)
    # and, with a residual, the rounding of the second addition on top: two spacings at the larger magnitude
    g, w = oracle.bf16_to_f32(got).astype(np.float64), oracle.bf16_to_f32(want).astype(np.float64)
    scale = np.abs(w) if residual is None else np.maximum(np.abs(w), np.abs(oracle.bf16_to_f32(residual).astype(np.float64)) + np.abs(w))
    bound = np.maximum(1e-2, scale * 2.0 ** (-7 if residual is None else -6))
    assert np.all(np.abs(g - w) <= bound), float(np.max(np.abs(g - w) / bound))
    assert np.count_nonzero(got != want) <= max(2, got.size // 200), (np.count_nonzero(got != want), got.size)


@pytest.mark.parametrize("rows,cols,red,bias,residual", [
    (1, 8, 8, False, False), (7, 20, 40, True, True), (8, 9, 264, True, False), (9, 33, 1000, False, True),
    (100, 2048, 2048, True, True),      # o_proj of a 100-token prompt + residual
    (37, 2048, 6144, False, True),      # down_proj + residual: four columns per block
    (300, 1024, 2048, True, False),     # k_proj
    (16, 128, 128, True, True), (129, 256, 384, False, False), (255, 384, 1024, True, True), (40, 128, 192, True, False),   # edges of the matrix tiles
    (1024, 2048, 2048, True, True),     # o_proj of a 1024-token prompt + residual
])
def test_linear_rows_against_the_oracle(oracle, qm, dev, rows, cols, red, bias, residual, rows_kernel):
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
    _check(oracle, to_u16(out), want, _on_matrix_cores(rows_kernel, rows, cols, red), r)


def test_a_prompt_row_equals_the_decode_linear_of_that_row(oracle, qm, dev, rows_kernel):
    """(the exact chain; with 64 rows and 128 columns the default kernel is the matrix cores, the other is asked for)"""
    import torch
    rows, cols, red = (12, 96, 2048) if rows_kernel == MATRIX else (64, 128, 2048)
    x = oracle.normal_bf16((rows, red), 1)
    w = oracle.normal_bf16((cols, red), 2, std=0.02)
    b = oracle.normal_bf16((cols,), 3, std=0.1)
    xd, wd, bd = to_dev(x, dev), to_dev(w, dev), to_dev(b, dev)
    out = torch.zeros((rows, cols), dtype=torch.int16, device=dev)
    qm.linear_rows(xd, wd, bd, None, out, rows, cols, red)
    one = torch.zeros(cols, dtype=torch.int16, device=dev)
    for r in (0, 5, rows - 1):
        qm.linear_m1(xd[r], wd, bd, None, one, cols, red)
        torch.cuda.synchronize()
        assert torch.equal(one, out[r])


# (the last two: grids between one and two blocks per CU of 128-column tiles, which take the 192-column tile; 600 rows
# leave the last row tile ragged)
@pytest.mark.parametrize("rows,hidden,inter", [(1, 8, 1), (9, 200, 33), (64, 2048, 6144), (5, 2048, 512), (200, 1024, 3072),
                                               (640, 256, 6912), (600, 320, 6912)])
def test_gate_up_swiglu_rows(oracle, qm, dev, rows, hidden, inter, rows_kernel):
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
    if _on_matrix_cores(rows_kernel, rows, inter, hidden):
        # a gate or up value on the neighbouring bf16 value moves the product by up to two of its spacings; a gate sum
        # that nearly cancels differs by more of ITS spacings, all of them tiny: the bound is absolute + relative
        g, w = oracle.bf16_to_f32(to_u16(out)).astype(np.float64), oracle.bf16_to_f32(want).astype(np.float64)
        assert np.all(np.abs(g - w) <= 1e-3 + np.abs(w) * 2.0 ** -6), float(np.max(np.abs(g - w)))
        assert np.count_nonzero(d) <= rows * inter // 100, np.count_nonzero(d)
    else:
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


@pytest.mark.parametrize("rows,cols,red,bias,residual", [
    (128, 2048, 4096, True, True),      # 32 blocks, 64 steps: eight pieces
    (100, 1024, 4096, False, False),    # 16 blocks
    (37, 2048, 6144, False, True),      # down_proj + residual of a short prompt: 96 steps
    (64, 4096, 4096, True, False),      # 32 blocks: eight pieces
    (200, 1024, 4096, False, True),     # 32 blocks: eight pieces
])
def test_linear_rows_with_the_reduction_shared_between_blocks(oracle, qm, dev, rows, cols, red, bias, residual, rows_kernel):
    """qm_linear_rows_split: few token rows leave most CUs without a block; with a workspace the reduction is cut into pieces
    whose fp32 sums a second launch adds in order.  Held to the bounds of the uncut matrix-core call; the same bits on every
    call; on the exact chain the workspace is not used and the result stays bit-exact."""
    import torch
    seed = 4500 + rows + cols + red
    x = oracle.normal_bf16((rows, red), seed)
    w = oracle.normal_bf16((cols, red), seed + 1, std=0.02)
    b = oracle.normal_bf16((cols,), seed + 2, std=0.1) if bias else None
    r = oracle.normal_bf16((rows, cols), seed + 3) if residual else None
    want = np.zeros((rows, cols), dtype=np.uint16)
    assert oracle.linear_rows(x, w, b, r, want, rows, cols, red, 16) == 0
    nbytes = qm.linear_rows_split_workspace_bytes(rows, cols, red)
    assert nbytes > 0
    ws = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device=dev)
    xd, wd = to_dev(x, dev), to_dev(w, dev)
    bd, rd = None if b is None else to_dev(b, dev), None if r is None else to_dev(r, dev)
    outs = []
    for _ in range(2):
        out = torch.full((rows, cols), 0x7fc0, dtype=torch.int16, device=dev)
        qm.linear_rows_split(xd, wd, bd, rd, out, rows, cols, red, ws, nbytes)
        torch.cuda.synchronize()
        outs.append(to_u16(out))
    assert np.array_equal(outs[0], outs[1])
    _check(oracle, outs[0], want, rows_kernel == MATRIX, r)
    if rows_kernel == MATRIX:
        assert qm.lib().qm_linear_rows_split(xd.data_ptr(), wd.data_ptr(), None, None, out.data_ptr(), rows, cols, red, ws.data_ptr(),
                                             nbytes - 4, None) == -4
    assert qm.linear_rows_split_workspace_bytes(1024, 2048, 6144) == 0      # enough blocks already
    assert qm.linear_rows_split_workspace_bytes(128, 2048, 2048) == 0       # a reduction of 2048 stays whole


@pytest.mark.parametrize("rows,hidden,inter", [(128, 4096, 3072), (48, 4096, 1536)])
def test_gate_up_swiglu_rows_with_the_reduction_shared_between_blocks(oracle, qm, dev, rows, hidden, inter, rows_kernel):
    import torch
    seed = 5500 + rows + hidden
    x = oracle.normal_bf16((rows, hidden), seed)
    gw = oracle.normal_bf16((inter, hidden), seed + 1, std=0.03)
    uw = oracle.normal_bf16((inter, hidden), seed + 2, std=0.03)
    want = np.zeros((rows, inter), dtype=np.uint16)
    assert oracle.gate_up_swiglu_rows(x, gw, uw, want, rows, hidden, inter, 16) == 0
    nbytes = qm.linear_rows_split_workspace_bytes(rows, inter, hidden, True)
    assert nbytes > 0
    ws = torch.full((nbytes // 4,), float("nan"), dtype=torch.float32, device=dev)
    outs = []
    for _ in range(2):
        out = torch.full((rows, inter), 0x7fc0, dtype=torch.int16, device=dev)
        qm.gate_up_swiglu_rows_split(to_dev(x, dev), to_dev(gw, dev), to_dev(uw, dev), out, rows, hidden, inter, ws, nbytes)
        torch.cuda.synchronize()
        outs.append(to_u16(out))
    assert np.array_equal(outs[0], outs[1])
    d = ulp_distance(outs[0], want)
    if rows_kernel == MATRIX:
        g, w = oracle.bf16_to_f32(outs[0]).astype(np.float64), oracle.bf16_to_f32(want).astype(np.float64)
        assert np.all(np.abs(g - w) <= 1e-3 + np.abs(w) * 2.0 ** -6), float(np.max(np.abs(g - w)))
        assert np.count_nonzero(d) <= rows * inter // 100, np.count_nonzero(d)
    else:
        assert d.max() <= 1 and np.count_nonzero(d) <= max(1, rows * inter // 1000)


@pytest.mark.parametrize("rows,q_cols,kv_cols,red", [(1024, 2048, 1024, 2048), (300, 512, 256, 384), (128, 2048, 1024, 2048), (7, 256, 128, 256)])
def test_qkv_rows_is_three_linear_rows(qm, dev, oracle, rows, q_cols, kv_cols, red):
    """qm_qkv_rows: bit for bit what three qm_linear_rows calls give (one grid on the matrix cores where the shapes are
    served; three calls below sixteen rows)."""
    import torch
    x = to_dev(oracle.normal_bf16((rows, red), 77), dev)
    ws = [to_dev(oracle.normal_bf16((c, red), 78 + i, std=0.03), dev) for i, c in enumerate((q_cols, kv_cols, kv_cols))]
    bs = [to_dev(oracle.normal_bf16((c,), 88 + i, std=0.1), dev) for i, c in enumerate((q_cols, kv_cols, kv_cols))]
    for biases in (bs, [bs[0], None, bs[2]]):
        want = [torch.full((rows, c), 0x7fc0, dtype=torch.int16, device=dev) for c in (q_cols, kv_cols, kv_cols)]
        got = [torch.full((rows, c), 0x7fc0, dtype=torch.int16, device=dev) for c in (q_cols, kv_cols, kv_cols)]
        for w, b, o, c in zip(ws, biases, want, (q_cols, kv_cols, kv_cols)):
            qm.linear_rows(x, w, b, None, o, rows, c, red)
        qm.qkv_rows(x, ws, biases, got, rows, q_cols, kv_cols, red)
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w)
    # with a workspace (of whatever size: the one grid never cuts a reduction) the same bits
    wsp = torch.empty(1 << 20, dtype=torch.float32, device=dev)
    got = [torch.full((rows, c), 0x7fc0, dtype=torch.int16, device=dev) for c in (q_cols, kv_cols, kv_cols)]
    qm.qkv_rows(x, ws, bs, got, rows, q_cols, kv_cols, red, wsp, 4 << 20)
    torch.cuda.synchronize()
    for g, w, b, c in zip(got, ws, bs, (q_cols, kv_cols, kv_cols)):
        want = torch.full((rows, c), 0x7fc0, dtype=torch.int16, device=dev)
        qm.linear_rows(x, w, b, None, want, rows, c, red)
        torch.cuda.synchronize()
        assert torch.equal(g, want)


def test_qkv_rows_argument_errors(qm, dev):
    import torch
    x = torch.zeros((16, 128), dtype=torch.int16, device=dev)
    w = torch.zeros((128, 128), dtype=torch.int16, device=dev)
    o = torch.zeros((16, 128), dtype=torch.int16, device=dev)
    f = qm.lib().qm_qkv_rows
    assert f(None, w.data_ptr(), w.data_ptr(), w.data_ptr(), None, None, None, o.data_ptr(), o.data_ptr(), o.data_ptr(), 16, 128, 128, 128, None) == -1
    assert f(x.data_ptr(), w.data_ptr(), w.data_ptr(), w.data_ptr(), None, None, None, o.data_ptr(), o.data_ptr(), None, 16, 128, 128, 128, None) == -1
    assert f(x.data_ptr(), w.data_ptr(), w.data_ptr(), w.data_ptr(), None, None, None, o.data_ptr(), o.data_ptr(), o.data_ptr(), 16, 128, 128, 124, None) == -2
    assert f(x.data_ptr(), w.data_ptr(), w.data_ptr(), w.data_ptr(), None, None, None, o.data_ptr(), o.data_ptr(), o.data_ptr(), -1, 128, 128, 128, None) == -5


def test_qkv_rows_with_an_empty_member(qm, dev, oracle):
    """A linear of no columns among the three leaves the other two as they are alone (the shapes that would share one
    grid: 64 rows, widths in 128s)."""
    import torch
    rows, red = 64, 256
    x = to_dev(oracle.normal_bf16((rows, red), 5), dev)
    for q_cols, kv_cols in ((0, 128), (256, 0)):
        widths = (q_cols, kv_cols, kv_cols)
        ws = [to_dev(oracle.normal_bf16((max(c, 1), red), 6 + i, std=0.03), dev) for i, c in enumerate(widths)]
        got = [torch.full((rows, max(c, 1)), 0x7fc0, dtype=torch.int16, device=dev) for c in widths]
        want = [torch.full((rows, max(c, 1)), 0x7fc0, dtype=torch.int16, device=dev) for c in widths]
        for w, o, c in zip(ws, want, widths):
            qm.linear_rows(x, w, None, None, o, rows, c, red)
        qm.qkv_rows(x, ws, [None, None, None], got, rows, q_cols, kv_cols, red)
        torch.cuda.synchronize()
        for g, w in zip(got, want):
            assert torch.equal(g, w)

