"""GPU parity of qm_decode_attention_ragged_static, the ragged decode whose split records live in a
device array the library owns (for callers that cannot allocate), through the C ABI: its output must
equal qm_decode_attention_ragged's bit for bit and the oracle's within tolerance, on two calls in a
row, the second with a smaller input (the array keeps the first call's records)."""
import numpy as np
import pytest

from qm_testlib import SCALE, PagedPool, max_abs_err, to_dev, to_u16

pytestmark = pytest.mark.gpu

TOL = 1e-2


def _both(oracle, qm, dev, lens, seed):
    import torch
    lens = np.asarray(lens, dtype=np.int32)
    n = len(lens)
    pool = PagedPool(oracle, lens, seed)
    q = oracle.normal_bf16((n, 16, 128), seed + 9)
    want = np.zeros_like(q)
    assert oracle.decode_attention_ragged(q, pool.descriptor(oracle), pool.page_table, pool.max_pages, lens, want, 16,
                                          SCALE, oracle.POLICY_ONLINE, 8) == 0
    kd, vd, cache_d, table_d = pool.device(qm, dev)
    max_len = int(lens.max())
    nbytes = qm.decode_workspace_bytes(n, 16, 8, max_len)
    assert nbytes <= qm.DECODE_STATIC_SCRATCH_BYTES
    ws = torch.zeros(max(nbytes // 4, 1), dtype=torch.float32, device=dev)
    qd, ld = to_dev(q, dev), to_dev(lens, dev)
    ref = torch.full((n, 16, 128), 0x7fc0, dtype=torch.int16, device=dev)
    out = torch.full((n, 16, 128), 0x7fc0, dtype=torch.int16, device=dev)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    qm.decode_attention_ragged(qd, cache_d, table_d, pool.max_pages, ld, n, max_len, ref, 16, SCALE, ws, nbytes, sd)
    qm.decode_attention_ragged_static(qd, cache_d, table_d, pool.max_pages, ld, n, max_len, out, 16, SCALE, sd)
    torch.cuda.synchronize()
    assert int(sd.item()) == 0
    return to_u16(out), to_u16(ref), want


def test_static_scratch_decode_two_calls_second_smaller(oracle, qm, dev):
    big = oracle.uniform_int(24, 606, 256, 4096)
    got, ref, want = _both(oracle, qm, dev, big, seed=61)
    assert np.array_equal(got, ref)
    assert max_abs_err(oracle, got, want) <= TOL
    small = [700, 0, 1, 33, 2048, 17]
    got, ref, want = _both(oracle, qm, dev, small, seed=62)
    assert np.array_equal(got, ref)
    assert max_abs_err(oracle, got, want) <= TOL
    assert not got[1].any()


def test_static_scratch_decode_rejects_shapes_beyond_the_array(oracle, qm, dev):
    import torch
    n, max_len = 64, 4096
    assert qm.decode_workspace_bytes(n, 16, 8, max_len) > qm.DECODE_STATIC_SCRATCH_BYTES
    pool = PagedPool(oracle, [16] * n, 3)
    kd, vd, cache_d, table_d = pool.device(qm, dev)
    z = torch.zeros((n, 16, 128), dtype=torch.int16, device=dev)
    out = torch.full((n, 16, 128), 0x1234, dtype=torch.int16, device=dev)
    lens = torch.full((n,), 16, dtype=torch.int32, device=dev)
    with pytest.raises(qm.QmError) as err:
        qm.decode_attention_ragged_static(z, cache_d, table_d, 256, lens, n, max_len, out, 16, SCALE)
    assert err.value.code == -4
    torch.cuda.synchronize()
    assert (to_u16(out) == 0x1234).all()
