"""GPU parity: causal prefill with a key-split workspace (qm_prefill_attention_causal_split).

Long query tiles are shared by up to three blocks whose partial results are combined by the last
block to finish: another association of the sums than the unsplit kernel's, so the bar is the
operator's tolerance (max abs error <= 1e-2 on bf16 outputs against the scalar fp32 oracle, ONLINE
policy), not equality of bits with the unsplit call; K/V page contents stay bit-exact, the result
may not depend on which block finishes last, and the workspace must come back as it was found.
"""
import numpy as np
import pytest

from qm_testlib import SCALE, PagedPool, max_abs_err, to_dev, to_u16

pytestmark = pytest.mark.gpu

TOL = 1e-2
POISON = 0x7F7F7F7F      # what the workspace holds before its init call


def _workspace(qm, dev, batch, seq, poison=True):
    import torch
    n = qm.prefill_split_workspace_bytes(batch, seq, 8)
    ws = torch.full((max(n, 256) // 4,), POISON if poison else 0, dtype=torch.int32, device=dev)
    if n:
        qm.prefill_split_workspace_init(ws, n)
    return ws, n


def _inputs(oracle, batch, seq, seed):
    return (oracle.normal_bf16((batch, seq, 16, 128), seed), oracle.normal_bf16((batch, seq, 8, 128), seed + 1),
            oracle.normal_bf16((batch, seq, 8, 128), seed + 2))


@pytest.mark.parametrize("batch,seq", [(1, 577), (2, 640), (1, 1024), (3, 700), (1, 1300), (1, 2048)])
def test_split_prefill_against_oracle_and_unsplit(oracle, qm, dev, batch, seq):
    import torch
    q, k, v = _inputs(oracle, batch, seq, 7000 + seq)
    pool = PagedPool(oracle, [seq] * batch, seed=7003 + seq, fill=0x7fc0)
    want = np.zeros_like(q)
    assert oracle.prefill_attention_causal(q, k, v, want, pool.descriptor(oracle), pool.page_table, pool.max_pages,
                                           batch, seq, 16, 8, SCALE, 1, 16) == 0
    qd, kd, vd = to_dev(q, dev), to_dev(k, dev), to_dev(v, dev)
    ws, n = _workspace(qm, dev, batch, seq)
    assert n > 0, "the case is meant to split"
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    outs = []
    for _ in range(3):                       # the second and third call find the workspace as the first left it
        fresh = PagedPool(oracle, [seq] * batch, seed=7003 + seq, fill=0x7fc0)
        k_pages, v_pages, cache_d, table_d = fresh.device(qm, dev)
        out = torch.full((batch, seq, 16, 128), 0x7fc0, dtype=torch.int16, device=dev)
        qm.prefill_attention_causal_split(qd, kd, vd, out, cache_d, table_d, fresh.max_pages, batch, seq, 16, 8, ws, n,
                                          SCALE, sd)
        torch.cuda.synchronize()
        assert int(sd.item()) == 0
        assert np.array_equal(to_u16(k_pages), pool.k) and np.array_equal(to_u16(v_pages), pool.v)
        outs.append(to_u16(out))
    assert max_abs_err(oracle, outs[0], want) <= TOL
    assert np.array_equal(outs[0], outs[1]) and np.array_equal(outs[0], outs[2])   # whoever finishes last
    whole = torch.full((batch, seq, 16, 128), 0x7fc0, dtype=torch.int16, device=dev)
    qm.prefill_attention_causal(qd, kd, vd, whole, None, None, 0, batch, seq, 16, 8, SCALE, sd)
    torch.cuda.synchronize()
    assert max_abs_err(oracle, outs[0], to_u16(whole)) <= TOL
    # rows of query tiles that are not split carry the unsplit kernel's bits (the first 384 rows never split)
    assert np.array_equal(outs[0][:, :384], to_u16(whole)[:, :384])
    # tickets and flags are back at zero (the workspace starts with eight integers per split query tile)
    assert int(ws[: 8 * batch * 8].abs().max().item()) == 0


def test_split_prefill_fp32_scores_option(oracle, qm, dev):
    import torch
    batch, seq = 1, 1024
    q, k, v = _inputs(oracle, batch, seq, 7100)
    qd, kd, vd = to_dev(q, dev), to_dev(k, dev), to_dev(v, dev)
    ws, n = _workspace(qm, dev, batch, seq)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    qm.set_option(qm.OPT_PREFILL_SCORE_ROUNDING, 0)
    try:
        split = torch.zeros((batch, seq, 16, 128), dtype=torch.int16, device=dev)
        whole = torch.zeros_like(split)
        qm.prefill_attention_causal_split(qd, kd, vd, split, None, None, 0, batch, seq, 16, 8, ws, n, SCALE, sd)
        qm.prefill_attention_causal(qd, kd, vd, whole, None, None, 0, batch, seq, 16, 8, SCALE, sd)
        torch.cuda.synchronize()
    finally:
        qm.set_option(qm.OPT_PREFILL_SCORE_ROUNDING, 1)
    assert int(sd.item()) == 0
    assert max_abs_err(oracle, to_u16(split), to_u16(whole)) <= TOL
    assert not np.array_equal(to_u16(split), np.zeros_like(q))


def test_split_workspace_rules(oracle, qm, dev):
    import torch
    assert qm.prefill_split_workspace_bytes(4, 1024, 8) == 0        # two blocks per CU already: nothing to gain
    assert qm.prefill_split_workspace_bytes(1, 384, 8) == 0         # chains too short to pay for the exchange
    assert qm.prefill_split_workspace_bytes(0, 1024, 8) == 0
    n = qm.prefill_split_workspace_bytes(1, 1024, 8)
    assert n > 0 and n % 256 == 0
    q, k, v = _inputs(oracle, 1, 1024, 7200)
    qd, kd, vd = to_dev(q, dev), to_dev(k, dev), to_dev(v, dev)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    ws = torch.zeros(n // 4, dtype=torch.int32, device=dev)
    out = torch.zeros((1, 1024, 16, 128), dtype=torch.int16, device=dev)
    with pytest.raises(qm.QmError) as e:                            # too small for the shape
        qm.prefill_attention_causal_split(qd, kd, vd, out, None, None, 0, 1, 1024, 16, 8, ws, n - 256, SCALE, sd)
    assert e.value.code == -4
    with pytest.raises(qm.QmError) as e:                            # bytes without a pointer
        qm.prefill_attention_causal_split(qd, kd, vd, out, None, None, 0, 1, 1024, 16, 8, None, n, SCALE, sd)
    assert e.value.code == -5
    with pytest.raises(qm.QmError) as e:                            # not 256-byte aligned
        qm.prefill_attention_causal_split(qd, kd, vd, out, None, None, 0, 1, 1024, 16, 8, ws[1:], n, SCALE, sd)
    assert e.value.code == -2
    # no workspace, and a shape that does not split: the unsplit call, bit for bit
    whole = torch.zeros_like(out)
    qm.prefill_attention_causal(qd, kd, vd, whole, None, None, 0, 1, 1024, 16, 8, SCALE, sd)
    qm.prefill_attention_causal_split(qd, kd, vd, out, None, None, 0, 1, 1024, 16, 8, None, 0, SCALE, sd)
    torch.cuda.synchronize()
    assert torch.equal(out, whole)
    q4, k4, v4 = (to_dev(x, dev) for x in _inputs(oracle, 4, 320, 7300))
    out4 = torch.zeros((4, 320, 16, 128), dtype=torch.int16, device=dev)
    whole4 = torch.zeros_like(out4)
    qm.prefill_attention_causal(q4, k4, v4, whole4, None, None, 0, 4, 320, 16, 8, SCALE, sd)
    qm.prefill_attention_causal_split(q4, k4, v4, out4, None, None, 0, 4, 320, 16, 8, ws, n, SCALE, sd)
    torch.cuda.synchronize()
    assert torch.equal(out4, whole4)
    assert int(sd.item()) == 0


def test_split_prefill_other_kernel_choices_ignore_the_workspace(oracle, qm, dev):
    """Only the interleaved kernel splits; with another kernel chosen the workspace is left alone."""
    import torch
    q, k, v = _inputs(oracle, 1, 1024, 7400)
    qd, kd, vd = to_dev(q, dev), to_dev(k, dev), to_dev(v, dev)
    ws, n = _workspace(qm, dev, 1, 1024, poison=False)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    outs = {}
    try:
        for choice in (1,):
            qm.set_option(qm.OPT_PREFILL_KERNEL, choice)
            out = torch.zeros((1, 1024, 16, 128), dtype=torch.int16, device=dev)
            qm.prefill_attention_causal_split(qd, kd, vd, out, None, None, 0, 1, 1024, 16, 8, ws, n, SCALE, sd)
            torch.cuda.synchronize()
            outs[choice] = out
    finally:
        qm.set_option(qm.OPT_PREFILL_KERNEL, 0)
    reference = torch.zeros((1, 1024, 16, 128), dtype=torch.int16, device=dev)
    qm.prefill_attention_causal(qd, kd, vd, reference, None, None, 0, 1, 1024, 16, 8, SCALE, sd)
    torch.cuda.synchronize()
    assert torch.equal(outs[1], reference)
    assert int(ws.abs().max().item()) == 0 and int(sd.item()) == 0


def test_split_prefill_over_flat_layer_cache_in_place(oracle, qm, dev):
    """K/V read in place from the flat [kv_head][max_cache][128] cache (strided rows), 700 tokens: the parts of a
    split query tile start at their own key tiles of the strided layout; against the unsplit call and the oracle."""
    import torch
    seq, max_cache = 700, 733
    q = oracle.normal_bf16((seq, 16, 128), 7501)
    k = oracle.normal_bf16((seq, 8, 128), 7502)
    v = oracle.normal_bf16((seq, 8, 128), 7503)
    kc = np.full((8, max_cache, 128), 0x7fc0, dtype=np.uint16)     # NaN beyond the sequence
    vc = np.full((8, max_cache, 128), 0x7fc0, dtype=np.uint16)
    assert oracle.scatter_kv(k, v, oracle.flat_cache(kc, vc, 8, max_cache), None, 1, seq, 0) == 0
    want = np.zeros_like(q)
    assert oracle.attention(q, oracle.flat_cache(kc, vc, 8, max_cache), None, 1, want, seq, 0, 16, -1, SCALE, 1, 16) == 0
    kd, vd = to_dev(kc, dev), to_dev(vc, dev)
    ws, n = _workspace(qm, dev, 1, seq)
    assert n > 0
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    split = torch.zeros((seq, 16, 128), dtype=torch.int16, device=dev)
    whole = torch.zeros_like(split)
    strides = (128, max_cache * 128, 0)
    qm.prefill_attention_causal_split(to_dev(q, dev), kd, vd, split, None, None, 0, 1, seq, 16, 8, ws, n, SCALE, sd, 0,
                                      strides)
    qm.prefill_attention_causal(to_dev(q, dev), kd, vd, whole, None, None, 0, 1, seq, 16, 8, SCALE, sd, 0, strides)
    torch.cuda.synchronize()
    assert int(sd.item()) == 0
    assert np.array_equal(to_u16(kd), kc)
    assert max_abs_err(oracle, to_u16(split), want) <= TOL
    assert max_abs_err(oracle, to_u16(split), to_u16(whole)) <= TOL
    assert not np.array_equal(to_u16(split)[448:], np.zeros_like(q)[448:])


def _double_bf16(bits):
    """Every finite, normal bf16 value times two: one more in the exponent field, exact."""
    bits = bits.copy()
    normal = ((bits & 0x7F80) != 0) & ((bits & 0x7F80) < 0x7F00)
    bits[normal] += 0x0080
    return bits


@pytest.mark.parametrize("batch,seq,split", [(4, 1024, False), (1, 1024, True), (1, 2048, True)])
def test_prefill_is_exactly_linear_in_v(oracle, qm, dev, batch, seq, split):
    """A property that does not depend on the size, at the benchmark's shapes: doubling every V doubles every
    output bit for bit (P.V on the matrix cores, the rescaling by running maxima, the combination of the parts of
    a split query tile and the final rounding all commute with a power of two)."""
    import torch
    q, k, v = _inputs(oracle, batch, seq, 7600 + seq)
    qd, kd = to_dev(q, dev), to_dev(k, dev)
    ws, n = _workspace(qm, dev, batch, seq) if split else (None, 0)
    assert (n > 0) == split
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    outs = []
    for vv in (v, _double_bf16(v)):
        out = torch.zeros((batch, seq, 16, 128), dtype=torch.int16, device=dev)
        qm.prefill_attention_causal_split(qd, kd, to_dev(vv, dev), out, None, None, 0, batch, seq, 16, 8, ws, n, SCALE, sd)
        torch.cuda.synchronize()
        outs.append(to_u16(out))
    assert int(sd.item()) == 0
    assert np.count_nonzero(outs[0] & 0x7F80) > outs[0].size * 0.99
    assert np.array_equal(outs[1], _double_bf16(outs[0]))


def test_prefill_batch_entries_are_independent(oracle, qm, dev):
    """Every entry of the 4 x 1024 benchmark batch, run alone (another grid, another block order), gives the bits
    it has inside the batch."""
    import torch
    q, k, v = _inputs(oracle, 4, 1024, 7700)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    whole = torch.zeros((4, 1024, 16, 128), dtype=torch.int16, device=dev)
    qm.prefill_attention_causal(to_dev(q, dev), to_dev(k, dev), to_dev(v, dev), whole, None, None, 0, 4, 1024, 16, 8,
                                SCALE, sd)
    torch.cuda.synchronize()
    for b in range(4):
        alone = torch.zeros((1, 1024, 16, 128), dtype=torch.int16, device=dev)
        qm.prefill_attention_causal(to_dev(q[b:b + 1], dev), to_dev(k[b:b + 1], dev), to_dev(v[b:b + 1], dev), alone, None,
                                    None, 0, 1, 1024, 16, 8, SCALE, sd)
        torch.cuda.synchronize()
        assert torch.equal(alone[0], whole[b]), b
    assert int(sd.item()) == 0
