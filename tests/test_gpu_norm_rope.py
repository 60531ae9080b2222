"""GPU parity: fused QK-RMSNorm + RoPE + KV append, prefill rows and scatter, through the C ABI.

Bar: bit-exact against the oracle (every rounding of the chain is elementwise and the sum of
squares is reduced in the same order), including the KV slot / page index.
"""
import numpy as np
import pytest

from qm_testlib import PagedPool, to_dev, to_u16

pytestmark = pytest.mark.gpu


def _inputs(oracle, seed, n=1, q_heads=16, kv_heads=8, std=1.0):
    q = oracle.normal_bf16((n, q_heads, 128), seed, 0.0, std)
    k = oracle.normal_bf16((n, kv_heads, 128), seed + 1, 0.0, std)
    v = oracle.normal_bf16((n, kv_heads, 128), seed + 2, 0.0, std)
    gq = oracle.normal_bf16((128,), seed + 3, 1.0, 0.1)
    gk = oracle.normal_bf16((128,), seed + 4, 1.0, 0.1)
    return q, k, v, gq, gk


@pytest.mark.parametrize("position,max_cache", [(0, 16), (2047, 2052), (29, 37), (511, 512)])
def test_append_flat_bit_exact(oracle, qm, dev, position, max_cache):
    import torch
    q, k, v, gq, gk = _inputs(oracle, 100 + position, std=0.02 * 45)   # projection-scale values
    cos, sin = oracle.rope_table(1, position)
    sentinel = 0x7fc1
    kc = np.full((8, max_cache, 128), sentinel, dtype=np.uint16)
    vc = np.full((8, max_cache, 128), sentinel, dtype=np.uint16)
    qr = np.zeros((16, 128), dtype=np.uint16)
    assert oracle.qk_norm_rope_kv_append(q[0], k[0], v[0], gq, gk, cos[0], sin[0], qr,
                                         oracle.flat_cache(kc, vc, 8, max_cache), None, 1, 16, position) == 0
    kd = to_dev(np.full((8, max_cache, 128), sentinel, dtype=np.uint16), dev)
    vd = to_dev(np.full((8, max_cache, 128), sentinel, dtype=np.uint16), dev)
    qd = torch.zeros((16, 128), dtype=torch.int16, device=dev)
    t = [to_dev(a, dev) for a in (q[0], k[0], v[0], gq, gk, cos[0], sin[0])]
    qm.qk_norm_rope_kv_append(*t, qd, qm.flat_cache(kd, vd, 8, max_cache), None, 1, 16, position)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(qd), qr)
    assert np.array_equal(to_u16(kd), kc)      # value bits and slot index, sentinel elsewhere
    assert np.array_equal(to_u16(vd), vc)


def test_append_flat_errors(oracle, qm, dev):
    import torch
    q, k, v, gq, gk = _inputs(oracle, 1)
    cos, sin = oracle.rope_table(1, 0)
    kd = torch.zeros((8, 32, 128), dtype=torch.int16, device=dev)
    vd = torch.zeros_like(kd)
    qd = torch.zeros((16, 128), dtype=torch.int16, device=dev)
    t = [to_dev(a, dev) for a in (q[0], k[0], v[0], gq, gk, cos[0], sin[0])]
    cache = qm.flat_cache(kd, vd, 8, 32)
    with pytest.raises(qm.QmError) as e:
        qm.qk_norm_rope_kv_append(*t, qd, cache, None, 1, 16, 32)       # overflow (R17:16844)
    assert e.value.code == -3
    with pytest.raises(qm.QmError) as e:
        qm.qk_norm_rope_kv_append(*t, qd, cache, None, 1, 16, -1)
    assert e.value.code == -3
    with pytest.raises(qm.QmError) as e:
        qm.qk_norm_rope_kv_append(None, *t[1:], qd, cache, None, 1, 16, 0)
    assert e.value.code == -1
    bad = qm.flat_cache(kd, vd, 8, 32)
    bad.head_dim = 64
    with pytest.raises(qm.QmError) as e:
        qm.qk_norm_rope_kv_append(*t, qd, bad, None, 1, 16, 0)
    assert e.value.code == -2
    torch.cuda.synchronize()
    assert not kd.any() and not vd.any()


def test_append_ragged_paged_bit_exact(oracle, qm, dev):
    import torch
    n = 64
    lens = oracle.uniform_int(n, 7, 0, 300)            # positions to append at
    pool = PagedPool(oracle, lens, seed=3, extra_tokens=1)
    q, k, v, gq, gk = _inputs(oracle, 50, n=n)
    cos, sin = oracle.rope_table(301, 0)               # table indexed by position
    qr = np.zeros_like(q)
    status = np.zeros(1, dtype=np.uint32)
    kd, vd, cache_d, table_d = pool.device(qm, dev)
    assert oracle.qk_norm_rope_kv_append_ragged(q, k, v, gq, gk, cos, sin, 1, qr, pool.descriptor(oracle),
                                                pool.page_table, pool.max_pages, lens, 16, 1e-6, status) == 0
    assert status[0] == 0
    qd = torch.zeros((n, 16, 128), dtype=torch.int16, device=dev)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    t = [to_dev(a, dev) for a in (q, k, v, gq, gk, cos, sin)]
    qm.qk_norm_rope_kv_append_ragged(*t, 1, qd, cache_d, table_d, pool.max_pages, to_dev(lens, dev), n, 16,
                                     1e-6, sd)
    torch.cuda.synchronize()
    assert int(sd.item()) == 0
    assert np.array_equal(to_u16(qd), qr)
    assert np.array_equal(to_u16(kd), pool.k)
    assert np.array_equal(to_u16(vd), pool.v)
    # per-stream rope rows (rope_by_position = 0) give the same result when the rows are gathered
    cos_g, sin_g = cos[lens].copy(), sin[lens].copy()
    qd2 = torch.zeros_like(qd)
    qm.qk_norm_rope_kv_append_ragged(t[0], t[1], t[2], t[3], t[4], to_dev(cos_g, dev), to_dev(sin_g, dev), 0, qd2,
                                     cache_d, table_d, pool.max_pages, to_dev(lens, dev), n, 16, 1e-6, sd)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(qd2), qr)


def test_append_ragged_bad_streams_are_skipped(oracle, qm, dev):
    import torch
    n = 4
    pos = np.array([3, 1000, 5, 17], dtype=np.int32)        # stream 1 beyond its table
    pool = PagedPool(oracle, [20, 20, 20, 20], seed=3, fill=0)
    pool.page_table[2, 0] = pool.n_pages + 5                    # stream 2: page out of the pool
    q, k, v, gq, gk = _inputs(oracle, 9, n=n)
    cos, sin = oracle.rope_table(n, 0)
    kd, vd, cache_d, table_d = pool.device(qm, dev)
    qd = torch.zeros((n, 16, 128), dtype=torch.int16, device=dev)
    sd = torch.zeros(1, dtype=torch.int32, device=dev)
    t = [to_dev(a, dev) for a in (q, k, v, gq, gk, cos, sin)]
    qm.qk_norm_rope_kv_append_ragged(*t, 0, qd, cache_d, table_d, pool.max_pages, to_dev(pos, dev), n, 16, 1e-6, sd)
    torch.cuda.synchronize()
    assert int(sd.item()) == 3                                  # BAD_PAGE | BAD_POSITION
    qr = np.zeros_like(q)
    status = np.zeros(1, dtype=np.uint32)
    oracle.qk_norm_rope_kv_append_ragged(q, k, v, gq, gk, cos, sin, 0, qr, pool.descriptor(oracle), pool.page_table,
                                         pool.max_pages, pos, 16, 1e-6, status)
    assert status[0] == 3
    assert np.array_equal(to_u16(qd), qr) and not to_u16(qd)[1].any() and not to_u16(qd)[2].any()
    assert np.array_equal(to_u16(kd), pool.k) and np.array_equal(to_u16(vd), pool.v)


@pytest.mark.parametrize("rows,heads,with_norm", [(1, 16, True), (33, 8, True), (64, 16, False), (1024, 24, True)])
def test_norm_rope_rows_bit_exact(oracle, qm, dev, rows, heads, with_norm):
    import torch
    x = oracle.normal_bf16((rows, heads, 128), rows + heads)
    g = oracle.normal_bf16((128,), 5, 1.0, 0.1) if with_norm else None
    cos, sin = oracle.rope_table(rows, 11)
    want = np.zeros_like(x)
    assert oracle.norm_rope_rows(x, g, cos, sin, want, rows, heads) == 0
    out = torch.zeros((rows, heads, 128), dtype=torch.int16, device=dev)
    qm.norm_rope_rows(to_dev(x, dev), to_dev(g, dev) if with_norm else None, to_dev(cos, dev), to_dev(sin, dev),
                      out, rows, heads)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(out), want)


@pytest.mark.parametrize("rows,q_heads,kv_heads,with_norm", [(1, 16, 8, True), (33, 16, 8, True), (130, 8, 8, False), (7, 3, 1, True)])
def test_query_and_key_rows_in_one_launch_are_the_two_calls(oracle, qm, dev, rows, q_heads, kv_heads, with_norm):
    import torch
    q = to_dev(oracle.normal_bf16((rows, q_heads, 128), 600 + rows), dev)
    k = to_dev(oracle.normal_bf16((rows, kv_heads, 128), 601 + rows), dev)
    gq = to_dev(oracle.normal_bf16((128,), 602, 1.0, 0.1), dev) if with_norm else None
    gk = to_dev(oracle.normal_bf16((128,), 603, 1.0, 0.1), dev) if with_norm else None
    cos, sin = (to_dev(a, dev) for a in oracle.rope_table(rows, 5))
    want_q, want_k, got_q, got_k = (torch.full(t.shape, 0x7fc0, dtype=torch.int16, device=dev) for t in (q, k, q, k))
    qm.norm_rope_rows(q, gq, cos, sin, want_q, rows, q_heads)
    qm.norm_rope_rows(k, gk, cos, sin, want_k, rows, kv_heads)
    qm.qk_norm_rope_rows(q, k, gq, gk, cos, sin, got_q, got_k, rows, q_heads, kv_heads)
    torch.cuda.synchronize()
    assert torch.equal(got_q, want_q) and torch.equal(got_k, want_k)
    f = qm.lib().qm_qk_norm_rope_rows
    a = [t.data_ptr() for t in (q, k)] + [None, None] + [cos.data_ptr(), sin.data_ptr(), got_q.data_ptr(), got_k.data_ptr()]
    assert f(*a, -1, q_heads, kv_heads, 1e-6, None) == -5 and f(*a, rows, 0, kv_heads, 1e-6, None) == -5
    assert f(*(a[:1] + [None] + a[2:]), rows, q_heads, kv_heads, 1e-6, None) == -1
    assert f(*a, 0, q_heads, kv_heads, 1e-6, None) == 0


def test_scatter_kv_paged_and_flat(oracle, qm, dev):
    import torch
    rows, first = 75, 9
    key = oracle.normal_bf16((rows, 8, 128), 3)
    val = oracle.normal_bf16((rows, 8, 128), 4)
    pool = PagedPool(oracle, [first + rows], seed=12, fill=0x1234)
    kd, vd, cache_d, table_d = pool.device(qm, dev)
    assert oracle.scatter_kv(key, val, pool.descriptor(oracle), pool.page_table, pool.max_pages, rows, first) == 0
    qm.scatter_kv(to_dev(key, dev), to_dev(val, dev), cache_d, table_d, pool.max_pages, rows, first)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(kd), pool.k) and np.array_equal(to_u16(vd), pool.v)
    # flat layout with a capacity that is not a multiple of 16
    kc = np.zeros((8, 91, 128), dtype=np.uint16)
    vc = np.zeros_like(kc)
    oracle.scatter_kv(key, val, oracle.flat_cache(kc, vc, 8, 91), None, 1, rows, first)
    kf, vf = to_dev(np.zeros_like(kc), dev), to_dev(np.zeros_like(vc), dev)
    qm.scatter_kv(to_dev(key, dev), to_dev(val, dev), qm.flat_cache(kf, vf, 8, 91), None, 1, rows, first)
    torch.cuda.synchronize()
    assert np.array_equal(to_u16(kf), kc) and np.array_equal(to_u16(vf), vc)
    with pytest.raises(qm.QmError) as e:
        qm.scatter_kv(to_dev(key, dev), to_dev(val, dev), qm.flat_cache(kf, vf, 8, 91), None, 1, rows, 20)
    assert e.value.code == -3
    # a page table entry outside the pool: those tokens are skipped and flagged, nothing else changes
    bad = pool.page_table.copy()
    bad[0, 2] = pool.n_pages + 5
    kd2, vd2, cache_d2, _ = pool_fresh = PagedPool(oracle, [first + rows], seed=12, fill=0x1234).device(qm, dev)
    status = torch.zeros(1, dtype=torch.int32, device=dev)
    qm.scatter_kv(to_dev(key, dev), to_dev(val, dev), cache_d2, to_dev(bad, dev), pool.max_pages, rows, first, status)
    torch.cuda.synchronize()
    assert int(status.item()) == 1                                   # QM_STATUS_BAD_PAGE
    skipped = pool.page_table[0, 2]
    keep = np.ones(pool.n_pages, dtype=bool)
    keep[skipped] = False
    assert np.array_equal(to_u16(kd2)[keep], pool.k[keep]) and np.array_equal(to_u16(vd2)[keep], pool.v[keep])
    assert (to_u16(kd2)[skipped] == 0x1234).all()


def test_hardware_bf16_rounding_equals_the_reference_sequence_for_every_float(qm, dev):
    """The kernels round fp32 to bf16 with v_cvt_pk_bf16_f32; the reference (and the oracle) with an integer sequence.  All
    2^32 bit patterns, NaN payloads and denormals included, must give the same bits (compared on the device)."""
    import torch
    bad = torch.zeros(1, dtype=torch.int64, device=dev)
    for quarter in range(4):
        assert qm.lib().qm_selftest_bf16_rounding(quarter << 30, 1 << 30, bad.data_ptr(), None) == 0
    torch.cuda.synchronize()
    assert int(bad.item()) == 0
    assert qm.lib().qm_selftest_bf16_rounding(0, 16, None, None) == -1
