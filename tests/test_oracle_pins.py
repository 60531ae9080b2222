"""Pins of the CPU oracle: closed forms, invariants and brute force chosen so that a dropped
term, a wrong sign/index or a transposed operand fails one of them.  No GPU."""
import math
import struct

import numpy as np
import pytest

from qm_testlib import SCALE, PagedPool


def f32_bits(x):
    return struct.unpack("<I", struct.pack("<f", x))[0]


def bits_f32(b):
    return struct.unpack("<f", struct.pack("<I", b))[0]


# ---- a1: bf16 conversion ------------------------------------------------------------------
def test_bf16_roundtrip_exhaustive(oracle):
    allb = np.arange(65536, dtype=np.uint32).astype(np.uint16)
    f = oracle.bf16_to_f32(allb)
    back = oracle.f32_to_bf16(f)
    nan = np.isnan(f)
    assert np.array_equal(back[~nan], allb[~nan])
    # NaNs keep sign/payload high bits and get the quiet bit
    assert np.array_equal(back[nan], allb[nan] | 0x0040)


def test_bf16_ties_to_even_and_specials(oracle):
    L = oracle.lib()
    assert L.qmo_f32_to_bf16(bits_f32(0x3f808000)) == 0x3f80   # tie, even stays
    assert L.qmo_f32_to_bf16(bits_f32(0x3f818000)) == 0x3f82   # tie, odd rounds up
    assert L.qmo_f32_to_bf16(bits_f32(0x3f808001)) == 0x3f81   # above tie
    assert L.qmo_f32_to_bf16(bits_f32(0x3f807fff)) == 0x3f80   # below tie
    assert L.qmo_f32_to_bf16(float("inf")) == 0x7f80
    assert L.qmo_f32_to_bf16(float("-inf")) == 0xff80
    assert L.qmo_f32_to_bf16(bits_f32(0x7f7fffff)) == 0x7f80   # max float rounds to inf
    assert L.qmo_f32_to_bf16(bits_f32(0x7fa00000)) == 0x7fe0   # NaN quieted
    assert L.qmo_f32_to_bf16(-0.0) == 0x8000


def test_bf16_matches_torch(oracle):
    torch = pytest.importorskip("torch")
    rng = np.random.default_rng(7)
    x = np.concatenate([rng.standard_normal(20000).astype(np.float32) * 37.0,
                        (rng.standard_normal(2000) * 1e-30).astype(np.float32),
                        np.array([0.0, -0.0, 1e38, -1e38, 3.3895e38], dtype=np.float32)])
    ours = oracle.f32_to_bf16(x)
    theirs = torch.from_numpy(x).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    assert np.array_equal(ours, theirs)


# ---- a2: RoPE table --------------------------------------------------------------------------
def test_rope_table_closed_form(oracle):
    cos, sin = oracle.rope_table(5, 0)
    assert np.all(cos[0] == 0x3f80) and np.all(sin[0] == 0)
    assert np.array_equal(cos[:, :64], cos[:, 64:]) and np.array_equal(sin[:, :64], sin[:, 64:])
    pos = 2047
    c, s = oracle.rope_table(1, pos)
    for i in (0, 1, 17, 63):
        inv = 1.0e6 ** (-2.0 * i / 128.0)
        want_c = oracle.f32_to_bf16(np.array([math.cos(pos * inv)], dtype=np.float32))[0]
        want_s = oracle.f32_to_bf16(np.array([math.sin(pos * inv)], dtype=np.float32))[0]
        assert c[0, i] == want_c and s[0, i] == want_s
    inv63 = 1.0e6 ** (-126.0 / 128.0)
    assert abs(oracle.bf16_to_f32(s[0, 63:64])[0] - math.sin(pos * inv63)) < 2e-4 * 2 + 1e-3
    with pytest.raises(ValueError):
        oracle.rope_table(1, 0, head_dim=127)                                 # odd head_dim rejected
    # start offset = row offset
    c2, s2 = oracle.rope_table(3, 100)
    c3, s3 = oracle.rope_table(1, 102)
    assert np.array_equal(c2[2], c3[0]) and np.array_equal(s2[2], s3[0])


# ---- a3: fused norm + RoPE + append ------------------------------------------------------------
def _append_case(oracle, seed, position, max_cache=64, q_heads=16, kv_heads=8):
    q = oracle.normal_bf16((q_heads, 128), seed)
    k = oracle.normal_bf16((kv_heads, 128), seed + 1)
    v = oracle.normal_bf16((kv_heads, 128), seed + 2)
    gq = oracle.normal_bf16((128,), seed + 3, 1.0, 0.1)
    gk = oracle.normal_bf16((128,), seed + 4, 1.0, 0.1)
    cos, sin = oracle.rope_table(1, position)
    return q, k, v, gq, gk, cos[0].copy(), sin[0].copy()


def test_append_flat_slot_index_bit_exact(oracle):
    max_cache, pos = 37, 29
    q, k, v, gq, gk, cos, sin = _append_case(oracle, 11, pos)
    sentinel = 0x7fc1
    kc = np.full((8, max_cache, 128), sentinel, dtype=np.uint16)
    vc = np.full((8, max_cache, 128), sentinel, dtype=np.uint16)
    qr = np.zeros((16, 128), dtype=np.uint16)
    cache = oracle.flat_cache(kc, vc, 8, max_cache)
    assert oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr, cache, None, 1, 16, pos) == 0
    changed_k = np.argwhere(kc != sentinel)
    changed_v = np.argwhere(vc != sentinel)
    assert len(changed_k) == 8 * 128 and len(changed_v) == 8 * 128
    assert np.all(changed_k[:, 1] == pos) and np.all(changed_v[:, 1] == pos)
    # reference index (head*max_cache + pos)*128 + d  (R17:15505-15522)
    flat = kc.reshape(-1)
    for h in (0, 3, 7):
        base = (h * max_cache + pos) * 128
        assert np.all(flat[base:base + 128] != sentinel)
    # V is copied bit-identically
    assert np.array_equal(vc[:, pos, :], v)
    # overflow guard (R17:16844-16847)
    assert oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr, cache, None, 1, 16, max_cache) == -3


def test_append_paged_address_brute_force(oracle):
    n_pages, page_size = 9, 16
    table = np.array([5, 2, 7, 0], dtype=np.int32)
    for pos in (0, 15, 16, 33, 63):
        q, k, v, gq, gk, cos, sin = _append_case(oracle, 100 + pos, pos)
        kp = np.zeros((n_pages, 8, page_size, 128), dtype=np.uint16)
        vp = np.zeros_like(kp)
        qr = np.zeros((16, 128), dtype=np.uint16)
        cache = oracle.paged_cache(kp, vp)
        assert oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr, cache, table, 4, 16, pos) == 0
        where = np.argwhere(vp != 0)
        assert set(where[:, 0]) == {int(table[pos // 16])}
        assert set(where[:, 2]) == {pos % 16}
        assert np.array_equal(vp[table[pos // 16], :, pos % 16, :], v)
        # K equals the flat-layout result for the same inputs (layout independence)
        kc = np.zeros((8, 64, 128), dtype=np.uint16)
        vc = np.zeros_like(kc)
        qr2 = np.zeros_like(qr)
        oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr2, oracle.flat_cache(kc, vc, 8, 64), None, 1, 16, pos)
        assert np.array_equal(kp[table[pos // 16], :, pos % 16, :], kc[:, pos, :])
        assert np.array_equal(qr, qr2)
    # page out of range
    q, k, v, gq, gk, cos, sin = _append_case(oracle, 1, 64)
    assert oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr, cache, table, 4, 16, 64) == -3
    bad = np.array([5, 2, 9, 0], dtype=np.int32)
    assert oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr, cache, bad, 4, 16, 40) == -3


def test_norm_closed_forms(oracle):
    one = oracle.f32_to_bf16(np.ones(128, dtype=np.float32))
    zero_sin = np.zeros(128, dtype=np.uint16)
    for c in (0.5, 3.0, -2.0):
        x = oracle.f32_to_bf16(np.full((1, 128), c, dtype=np.float32))
        out = np.zeros((1, 128), dtype=np.uint16)
        # gamma = 1, position 0 (cos 1, sin 0): out = bf16(bf16(x * r)), r = 1/sqrt(c^2 + eps)
        assert oracle.norm_rope_rows(x, one, one.reshape(1, 128), zero_sin.reshape(1, 128), out, 1, 1) == 0
        cb = oracle.bf16_to_f32(x)[0, 0]
        r = np.float32(1.0) / np.sqrt(np.float32(cb * cb) + np.float32(1e-6), dtype=np.float32)
        want = oracle.f32_to_bf16(np.array([np.float32(cb) * r], dtype=np.float32))[0]
        assert np.all(out == want)
    # sum of squares in reference order equals the exact sum when it is exactly representable
    x = oracle.f32_to_bf16(np.arange(128, dtype=np.float32))
    got = oracle.lib().qmo_head_sum_squares(x.ctypes.data_as(__import__("ctypes").c_void_p))
    assert got == float(sum(i * i for i in range(128)))


def test_rope_sign_and_pairing(oracle):
    # e_0 at position p: out[0] = cos, out[64] = +sin ; e_64: out[0] = -sin, out[64] = cos
    p = 3
    cos, sin = oracle.rope_table(1, p)
    for hot, want0, want64 in ((0, "cos", "sin"), (64, "-sin", "cos")):
        x = np.zeros((1, 128), dtype=np.uint16)
        x[0, hot] = 0x3f80
        out = np.zeros_like(x)
        assert oracle.norm_rope_rows(x, None, cos, sin, out, 1, 1) == 0
        val = {"cos": cos[0, 0], "sin": sin[0, 0], "-sin": sin[0, 0] ^ 0x8000}
        assert out[0, 0] == val[want0] and out[0, 64] == val[want64]
        assert np.count_nonzero(out & 0x7fff) == 2     # (-0.0 entries are zeros)
    # rotation preserves the pair norm up to bf16 rounding
    x = oracle.normal_bf16((4, 2, 128), 5)
    cos, sin = oracle.rope_table(4, 1000)
    out = np.zeros_like(x)
    oracle.norm_rope_rows(x, None, cos, sin, out, 4, 2)
    xf, of = oracle.bf16_to_f32(x), oracle.bf16_to_f32(out)
    n_in = xf[..., :64] ** 2 + xf[..., 64:] ** 2
    n_out = of[..., :64] ** 2 + of[..., 64:] ** 2
    assert np.max(np.abs(n_in - n_out) / (n_in + 1e-3)) < 0.03


def test_norm_rope_rows_equals_fused_append(oracle):
    # cross-operator invariant: the prefill pieces and the decode fused kernel share one chain
    pos = 77
    q, k, v, gq, gk, cos, sin = _append_case(oracle, 21, pos)
    kc = np.zeros((8, 128, 128), dtype=np.uint16)
    vc = np.zeros_like(kc)
    qr = np.zeros((16, 128), dtype=np.uint16)
    oracle.qk_norm_rope_kv_append(q, k, v, gq, gk, cos, sin, qr, oracle.flat_cache(kc, vc, 8, 128), None, 1, 16, pos)
    out_q = np.zeros_like(q)
    out_k = np.zeros_like(k)
    oracle.norm_rope_rows(q.reshape(1, 16, 128), gq, cos.reshape(1, 128), sin.reshape(1, 128), out_q.reshape(1, 16, 128), 1, 16)
    oracle.norm_rope_rows(k.reshape(1, 8, 128), gk, cos.reshape(1, 128), sin.reshape(1, 128), out_k.reshape(1, 8, 128), 1, 8)
    assert np.array_equal(out_q, qr) and np.array_equal(out_k, kc[:, pos, :])


def test_scatter_kv(oracle):
    rows, first = 21, 5
    key = oracle.normal_bf16((rows, 8, 128), 3)
    val = oracle.normal_bf16((rows, 8, 128), 4)
    kc = np.zeros((8, 40, 128), dtype=np.uint16)
    vc = np.zeros_like(kc)
    assert oracle.scatter_kv(key, val, oracle.flat_cache(kc, vc, 8, 40), None, 1, rows, first) == 0
    assert np.array_equal(kc[:, first:first + rows, :], key.transpose(1, 0, 2))
    assert np.array_equal(vc[:, first:first + rows, :], val.transpose(1, 0, 2))
    assert not kc[:, :first].any() and not kc[:, first + rows:].any()
    assert oracle.scatter_kv(key, val, oracle.flat_cache(kc, vc, 8, 40), None, 1, rows, 20) == -3


# ---- a6/a7: attention -------------------------------------------------------------------------
def _flat_attention(oracle, q, kc, vc, ctx, policy, window=-1, q_len=1):
    out = np.zeros_like(q)
    cache = oracle.flat_cache(kc, vc, kc.shape[0], kc.shape[1])
    rc = oracle.attention(q, cache, None, 1, out, q_len, ctx - q_len, q.shape[-2], window, SCALE, policy, 1)
    assert rc == 0
    return out


@pytest.mark.parametrize("policy", [0, 1, 2])
def test_attention_ctx1_is_value(oracle, policy):
    q = oracle.normal_bf16((16, 128), 1)
    kc = oracle.normal_bf16((8, 4, 128), 2)
    vc = oracle.normal_bf16((8, 4, 128), 3)
    out = _flat_attention(oracle, q, kc, vc, 1, policy)
    for h in range(16):
        assert np.array_equal(out[h], vc[h // 2, 0])       # GQA map: q head h -> kv head h // 2


@pytest.mark.parametrize("policy", [0, 1, 2])
def test_attention_equal_keys_gives_mean(oracle, policy):
    ctx = 8
    q = oracle.normal_bf16((16, 128), 1)
    kc = np.repeat(oracle.normal_bf16((8, 1, 128), 2), ctx, axis=1)
    vc = oracle.normal_bf16((8, ctx, 128), 3)
    out = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, vc, ctx, policy))
    mean = oracle.bf16_to_f32(vc).mean(axis=1)
    for h in range(16):
        assert np.max(np.abs(out[h] - mean[h // 2])) < 0.02


def test_attention_dominant_key(oracle):
    ctx = 32
    q = oracle.f32_to_bf16(np.full((16, 128), 1.0, dtype=np.float32))
    kf = np.zeros((8, ctx, 128), dtype=np.float32)
    kf[:, 13, :] = 5.0     # score 640 * scale ~ 56 above the rest
    vc = oracle.normal_bf16((8, ctx, 128), 9)
    for policy in (0, 1, 2):
        out = _flat_attention(oracle, q, oracle.f32_to_bf16(kf), vc, ctx, policy)
        for h in range(16):
            assert np.array_equal(out[h], vc[h // 2, 13])


def test_attention_gqa_map_distinct_constants(oracle):
    ctx = 5
    q = oracle.normal_bf16((16, 128), 4)
    kc = oracle.normal_bf16((8, ctx, 128), 5)
    vf = np.zeros((8, ctx, 128), dtype=np.float32)
    for h in range(8):
        vf[h] = float(h + 1)
    out = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, oracle.f32_to_bf16(vf), ctx, 0))
    for h in range(16):
        assert np.allclose(out[h], h // 2 + 1, atol=0.02)


def _brute_force(oracle, q, kc, vc, ctx, round_scores):
    """float64 softmax(QK^T * scale) V with optional bf16 score roundings, per head."""
    qf = oracle.bf16_to_f32(q).astype(np.float64)
    kf = oracle.bf16_to_f32(kc).astype(np.float64)
    vf = oracle.bf16_to_f32(vc).astype(np.float64)
    out = np.zeros((q.shape[0], 128))
    for h in range(q.shape[0]):
        s = kf[h // 2, :ctx] @ qf[h]
        if round_scores:
            s = oracle.bf16_to_f32(oracle.f32_to_bf16(s.astype(np.float32))).astype(np.float64)
            s = oracle.bf16_to_f32(oracle.f32_to_bf16((s.astype(np.float32) * np.float32(SCALE)))).astype(np.float64)
        else:
            s = s * np.float64(np.float32(SCALE))
        p = np.exp(s - s.max())
        p /= p.sum()
        out[h] = p @ vf[h // 2, :ctx]
    return out


def test_attention_brute_force_fp64(oracle):
    for ctx in (2, 3, 8, 40):
        q = oracle.normal_bf16((16, 128), 10 + ctx)
        kc = oracle.normal_bf16((8, ctx, 128), 20 + ctx)
        vc = oracle.normal_bf16((8, ctx, 128), 30 + ctx)
        exact = _brute_force(oracle, q, kc, vc, ctx, False)
        rounded = _brute_force(oracle, q, kc, vc, ctx, True)
        fp32 = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, vc, ctx, 2))
        online = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, vc, ctx, 1))
        ref = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, vc, ctx, 0))
        ulp = np.maximum(np.abs(exact), 2.0 ** -126) * 2.0 ** -8   # one bf16 ulp bound
        assert np.all(np.abs(fp32 - exact) <= ulp)                  # fp32 policy = textbook softmax
        assert np.all(np.abs(online - rounded) <= np.maximum(np.abs(rounded), 1e-30) * 2.0 ** -8)
        # the reference chain differs from `rounded` only by bf16(P): <= 2^-9 relative per term
        vmax = np.abs(oracle.bf16_to_f32(vc)).max()
        assert np.max(np.abs(ref - rounded)) <= 2.0 ** -8 * vmax + 2.0 ** -7 * np.abs(rounded).max()


def test_attention_matches_torch_sdpa_fp32(oracle):
    torch = pytest.importorskip("torch")
    S, H, KV = 12, 16, 8
    q = oracle.normal_bf16((S, H, 128), 1)
    k = oracle.normal_bf16((S, KV, 128), 2)
    v = oracle.normal_bf16((S, KV, 128), 3)
    out = np.zeros_like(q)
    assert oracle.prefill_attention_causal(q, k, v, out, None, None, 0, 1, S, H, KV, SCALE, 2, 2) == 0
    tq = torch.from_numpy(oracle.bf16_to_f32(q)).permute(1, 0, 2)[None]
    tk = torch.from_numpy(oracle.bf16_to_f32(k)).permute(1, 0, 2)[None].repeat_interleave(2, dim=1)
    tv = torch.from_numpy(oracle.bf16_to_f32(v)).permute(1, 0, 2)[None].repeat_interleave(2, dim=1)
    want = torch.nn.functional.scaled_dot_product_attention(tq, tk, tv, is_causal=True, scale=SCALE)
    want = want[0].permute(1, 0, 2).numpy()
    got = oracle.bf16_to_f32(out)
    assert np.max(np.abs(got - want)) <= 2.0 ** -8 * max(1.0, np.abs(want).max()) + 1e-6


def test_attention_page_permutation_invariance(oracle):
    lens = [1, 15, 16, 17, 100]
    pool_a = PagedPool(oracle, lens, seed=40)
    q = oracle.normal_bf16((len(lens), 16, 128), 41)
    out_a = np.zeros_like(q)
    assert oracle.decode_attention_ragged(q, pool_a.descriptor(oracle), pool_a.page_table, pool_a.max_pages,
                                          pool_a.seq_lens, out_a, 16, SCALE, 0, 2) == 0
    # move the data to other physical pages, update the tables: output must be bit-identical
    perm = oracle.permutation(pool_a.n_pages, 99)
    k_b = np.zeros_like(pool_a.k)
    v_b = np.zeros_like(pool_a.v)
    k_b[perm] = pool_a.k
    v_b[perm] = pool_a.v
    table_b = np.where(pool_a.page_table >= 0, perm[np.maximum(pool_a.page_table, 0)], -1).astype(np.int32)
    out_b = np.zeros_like(q)
    assert oracle.decode_attention_ragged(q, oracle.paged_cache(k_b, v_b), table_b, pool_a.max_pages,
                                          pool_a.seq_lens, out_b, 16, SCALE, 0, 2) == 0
    assert np.array_equal(out_a, out_b)
    # and equals the flat layout
    for s, n in enumerate(lens):
        kc = np.zeros((8, n, 128), dtype=np.uint16)
        vc = np.zeros_like(kc)
        for t in range(n):
            kc[:, t] = pool_a.k[pool_a.page_table[s, t // 16], :, t % 16]
            vc[:, t] = pool_a.v[pool_a.page_table[s, t // 16], :, t % 16]
        assert np.array_equal(_flat_attention(oracle, q[s], kc, vc, n, 0), out_a[s])


def test_attention_sliding_window(oracle):
    ctx, w = 40, 7
    q = oracle.normal_bf16((16, 128), 1)
    kc = oracle.normal_bf16((8, ctx, 128), 2)
    vc = oracle.normal_bf16((8, ctx, 128), 3)
    win = _flat_attention(oracle, q, kc, vc, ctx, 0, window=w)
    # equals full attention over only the last w tokens (R17:16032-16036)
    tail = _flat_attention(oracle, q, kc[:, ctx - w:].copy(), vc[:, ctx - w:].copy(), w, 0)
    assert np.array_equal(win, tail)
    assert np.array_equal(_flat_attention(oracle, q, kc, vc, ctx, 0, window=0),
                          _flat_attention(oracle, q, kc, vc, ctx, 0, window=-1))
    assert np.array_equal(_flat_attention(oracle, q, kc, vc, ctx, 0, window=1000),
                          _flat_attention(oracle, q, kc, vc, ctx, 0, window=-1))


def test_prefill_rows_equal_decode_and_causality(oracle):
    S = 20
    q = oracle.normal_bf16((1, S, 16, 128), 1)
    k = oracle.normal_bf16((1, S, 8, 128), 2)
    v = oracle.normal_bf16((1, S, 8, 128), 3)
    pool = PagedPool(oracle, [S], seed=8, fill=0)
    out = np.zeros_like(q)
    assert oracle.prefill_attention_causal(q, k, v, out, pool.descriptor(oracle), pool.page_table,
                                           pool.max_pages, 1, S, 16, 8, SCALE, 0, 2) == 0
    assert np.array_equal(out[0, 0], np.repeat(v[0, 0], 2, axis=0))     # row 0 = V[0]
    # row i == decode attention at position i over the cache the prefill wrote
    for i in (0, 1, 7, 19):
        o = np.zeros((16, 128), dtype=np.uint16)
        assert oracle.attention(q[0, i].copy(), pool.descriptor(oracle), pool.page_table[0], pool.max_pages,
                                o, 1, i, 16, -1, SCALE, 0, 1) == 0
        assert np.array_equal(o, out[0, i])
    # generic kernel semantics: query_length rows over the cache, cache_before = 0
    o_all = np.zeros((S, 16, 128), dtype=np.uint16)
    assert oracle.attention(q[0].copy(), pool.descriptor(oracle), pool.page_table[0], pool.max_pages, o_all,
                            S, 0, 16, -1, SCALE, 0, 2) == 0
    assert np.array_equal(o_all, out[0])
    # causality: poisoning future keys/values with NaN must not change row i
    k2, v2 = k.copy(), v.copy()
    k2[0, 11:] = 0x7fc0
    v2[0, 11:] = 0x7fc0
    out2 = np.zeros_like(q)
    oracle.prefill_attention_causal(q, k2, v2, out2, None, None, 0, 1, S, 16, 8, SCALE, 0, 2)
    assert np.array_equal(out2[0, :11], out[0, :11])
    # batch entries are independent
    qb = np.concatenate([q, oracle.normal_bf16((1, S, 16, 128), 50)])
    kb = np.concatenate([k, oracle.normal_bf16((1, S, 8, 128), 51)])
    vb = np.concatenate([v, oracle.normal_bf16((1, S, 8, 128), 52)])
    ob = np.zeros_like(qb)
    oracle.prefill_attention_causal(qb, kb, vb, ob, None, None, 0, 2, S, 16, 8, SCALE, 0, 2)
    assert np.array_equal(ob[0], out[0])


def test_reference_vs_online_policy_gap(oracle):
    """Documents how far the reference chain's bf16(P) sits from the online policy."""
    ctx = 512
    q = oracle.normal_bf16((16, 128), 1)
    kc = oracle.normal_bf16((8, ctx, 128), 2)
    vc = oracle.normal_bf16((8, ctx, 128), 3)
    ref = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, vc, ctx, 0))
    onl = oracle.bf16_to_f32(_flat_attention(oracle, q, kc, vc, ctx, 1))
    assert np.max(np.abs(ref - onl)) <= 1e-2


# ---- a8-a10: predictor ---------------------------------------------------------------------------
def test_predictor_m1_vs_talker_chain(oracle):
    # same rounding chain, different fp32 summation topology: equal up to rare 1-ulp flips
    for n in (1, 2, 9, 16):
        q = oracle.normal_bf16((16, 128), n)
        kc = oracle.normal_bf16((8, 16, 128), n + 100)
        vc = oracle.normal_bf16((8, 16, 128), n + 200)
        a = np.zeros_like(q)
        assert oracle.predictor_attention_m1(q, kc, vc, a, n) == 0
        b = _flat_attention(oracle, q, kc, vc, n, 0)
        from qm_testlib import ulp_distance
        assert ulp_distance(a, b).max() <= 1
        assert (a != b).mean() < 0.02
        if n == 1:
            assert np.array_equal(a, np.repeat(vc[:, 0], 2, axis=0))
    assert oracle.predictor_attention_m1(q, kc, vc, a, 17) == -5
    assert oracle.predictor_attention_m1(q, kc, vc, a, 0) == -5


def test_predictor_staged_step0_equals_m1_rows(oracle):
    # the two-row causal staged attention of step 0 equals M=1 attention at key_length 1 and 2
    q = oracle.normal_bf16((2, 16, 128), 5)          # [row][head][128]
    kc = np.zeros((8, 16, 128), dtype=np.uint16)
    vc = np.zeros_like(kc)
    kc[:, :2] = oracle.normal_bf16((8, 2, 128), 6)
    vc[:, :2] = oracle.normal_bf16((8, 2, 128), 7)
    q_bhsd = np.ascontiguousarray(q.transpose(1, 0, 2))
    staged = np.zeros((2, 16, 128), dtype=np.uint16)
    assert oracle.predictor_attention_staged(q_bhsd, kc, vc, staged, 2, 2, True) == 0
    for r in range(2):
        o = np.zeros((16, 128), dtype=np.uint16)
        oracle.predictor_attention_m1(q[r].copy(), kc, vc, o, r + 1)
        assert np.array_equal(o, staged[r])


def test_predictor_step0_layout_operators(oracle):
    """transpose / rope / update_cache of the predictor's step 0 index BHSD [head][row][128]
    (R17:8366-8529).  Pinned without repeating the oracle's index arithmetic: numpy's own transpose,
    a rotation whose result is known in closed form per (head, row), and a sentinel-filled cache."""
    rows, heads = 2, 16
    x = oracle.normal_bf16((rows, heads, 128), 11)
    t = np.zeros((heads, rows, 128), dtype=np.uint16)
    assert oracle.predictor_transpose(x, t, rows, heads) == 0
    assert np.array_equal(t, x.transpose(1, 0, 2))
    # rope: head h, row s must use table row s.  Input = unit vector e_0 everywhere, so the rotated
    # vector is cos_s[0] at dim 0 and +sin_s[64] at dim 64 (rotate_half gives d >= 64 the value +x[d-64]),
    # whatever the head; table rows differ, so a head/row mix-up shows.
    cos, sin = oracle.rope_table(rows, 0)
    cos[1], sin[1] = oracle.rope_table(1, 7)[0][0], oracle.rope_table(1, 7)[1][0]   # row 1 := position 7
    e0 = np.zeros((heads, rows, 128), dtype=np.uint16)
    e0[:, :, 0] = 0x3F80
    out = np.zeros_like(e0)
    assert oracle.predictor_rope_bhsd(e0, cos, sin, out, rows, heads) == 0
    for h in range(heads):
        for s_ in range(rows):
            assert out[h, s_, 0] == cos[s_, 0] and out[h, s_, 64] == sin[s_, 64]
            assert not (out[h, s_, 1:64] & 0x7FFF).any() and not (out[h, s_, 65:] & 0x7FFF).any()   # +-0
    assert out[0, 0, 0] == 0x3F80 and out[0, 0, 64] == 0          # position 0: identity
    assert out[0, 1, 64] != 0                                      # position 7 rotates
    # the rotation of a BHSD tensor is the row-wise rotation (pinned elsewhere) of its BSHD transpose
    y = oracle.normal_bf16((rows, heads, 128), 12)
    y_bhsd = np.ascontiguousarray(y.transpose(1, 0, 2))
    got = np.zeros_like(y_bhsd)
    assert oracle.predictor_rope_bhsd(y_bhsd, cos, sin, got, rows, heads) == 0
    want = np.zeros_like(y)
    assert oracle.norm_rope_rows(y, None, cos, sin, want, rows, heads) == 0
    assert np.array_equal(got, want.transpose(1, 0, 2))
    # e_64 picks the other sign: out[0] = -sin_s[0], out[64] = cos_s[64]
    e64 = np.zeros((heads, rows, 128), dtype=np.uint16)
    e64[:, :, 64] = 0x3F80
    assert oracle.predictor_rope_bhsd(e64, cos, sin, out, rows, heads) == 0
    assert out[3, 1, 0] == (sin[1, 0] ^ 0x8000) and out[3, 1, 64] == cos[1, 64]
    # update_cache: exactly 8 * rows * 128 elements change, head h row s lands at (h*16 + start + s)*128
    for rows_u, start in ((2, 0), (1, 2), (3, 13), (16, 0)):
        src = oracle.normal_bf16((8, rows_u, 128), 13 + start)
        src[src == 0xABCD] = 0
        cache = np.full((8, 16, 128), 0xABCD, dtype=np.uint16)
        assert oracle.predictor_update_cache(src, cache, rows_u, start) == 0
        assert np.count_nonzero(cache != 0xABCD) == 8 * rows_u * 128
        flat = cache.reshape(-1)
        for h in (0, 5, 7):
            for s_ in range(rows_u):
                at = (h * 16 + start + s_) * 128
                assert np.array_equal(flat[at:at + 128], src[h, s_])
    cache = np.full((8, 16, 128), 0xABCD, dtype=np.uint16)
    assert oracle.predictor_update_cache(src, cache, 2, 15) == -3
    assert (cache == 0xABCD).all()


def test_predictor_step0_chain_equals_loop(oracle):
    """The reference's step-0 sequence (R17:13663-13705) — transpose, rope, update_cache, staged causal
    attention — on normed rows gives the loop operator's rows 0 and 1 (first_rows = 2) bit for bit."""
    rows = 2
    q = oracle.normal_bf16((1, rows, 16, 128), 21)
    k = oracle.normal_bf16((1, rows, 8, 128), 22)
    v = oracle.normal_bf16((1, rows, 8, 128), 23)
    gq = oracle.normal_bf16((1, 128), 24, 1.0, 0.1)
    gk = oracle.normal_bf16((1, 128), 25, 1.0, 0.1)
    cos, sin = oracle.rope_table(rows, 0)
    want = np.zeros_like(q)
    kc_want = np.zeros((1, 8, 16, 128), dtype=np.uint16)
    vc_want = np.zeros_like(kc_want)
    assert oracle.predictor_attention_loop(q, k, v, gq, gk, cos, sin, want, kc_want, vc_want, 1, 1, rows, 2) == 0
    from qm_testlib import step0_chain
    got, kc, vc = step0_chain(oracle, oracle, q[0], k[0], v[0], gq[0], gk[0], cos, sin, rows)
    assert np.array_equal(kc, kc_want[0]) and np.array_equal(vc, vc_want[0])
    assert np.array_equal(got, want[0])


def test_predictor_loop_properties(oracle):
    units, layers, rows = 4, 2, 16
    q = oracle.normal_bf16((units, rows, 16, 128), 1)
    k = oracle.normal_bf16((units, rows, 8, 128), 2)
    v = oracle.normal_bf16((units, rows, 8, 128), 3)
    gq = oracle.normal_bf16((layers, 128), 4, 1.0, 0.1)
    gk = oracle.normal_bf16((layers, 128), 5, 1.0, 0.1)
    cos, sin = oracle.rope_table(rows, 0)
    out = np.zeros_like(q)
    kc = np.zeros((units, 8, 16, 128), dtype=np.uint16)
    vc = np.zeros_like(kc)
    assert oracle.predictor_attention_loop(q, k, v, gq, gk, cos, sin, out, kc, vc, units, layers, rows, 1) == 0
    out2 = np.zeros_like(q)
    assert oracle.predictor_attention_loop(q, k, v, gq, gk, cos, sin, out2, None, None, units, layers, rows, 2) == 0
    assert np.array_equal(out, out2)                      # first_rows only renumbers steps
    assert np.array_equal(out[:, 0], np.repeat(v[:, 0], 2, axis=1))   # step 0, ctx 1: out = V
    assert np.array_equal(vc, v.transpose(0, 2, 1, 3))    # V cache = raw V, [unit][head][token]
    # K cache row r = norm+rope of k row r with the unit's layer gamma at position r
    for u in (0, 3):
        want = np.zeros((rows, 8, 128), dtype=np.uint16)
        oracle.norm_rope_rows(k[u], gk[u % layers].copy(), cos, sin, want, rows, 8)
        assert np.array_equal(kc[u], want.transpose(1, 0, 2))
    # step t equals generic attention with context t+1 on the accumulated cache (talker chain, <=1 ulp)
    from qm_testlib import ulp_distance
    u = 1
    qn = np.zeros((rows, 16, 128), dtype=np.uint16)
    oracle.norm_rope_rows(q[u], gq[u % layers].copy(), cos, sin, qn, rows, 16)
    cache = oracle.flat_cache(kc[u], vc[u], 8, 16)
    for t in (0, 5, 15):
        o = np.zeros((16, 128), dtype=np.uint16)
        oracle.attention(qn[t].copy(), cache, None, 1, o, 1, t, 16, -1, SCALE, 0, 1)
        assert ulp_distance(o, out[u, t]).max() <= 1
    assert oracle.predictor_attention_loop(q, k, v, gq, gk, cos, sin, out, None, None, units, layers, 17, 1) == -5
    assert oracle.predictor_attention_loop(q, k, v, gq, gk, cos, sin, out, None, None, units, layers, rows, 3) == -5


# ---- input generator --------------------------------------------------------------------------------
def test_generator_is_thread_independent_and_normal(oracle):
    a = oracle.normal_bf16((100000,), 42, threads=1)
    b = oracle.normal_bf16((100000,), 42, threads=8)
    assert np.array_equal(a, b)
    f = oracle.bf16_to_f32(a)
    assert abs(f.mean()) < 0.02 and abs(f.std() - 1.0) < 0.02
    assert not np.array_equal(a, oracle.normal_bf16((100000,), 43))
    p = oracle.permutation(1000, 3)
    assert sorted(p.tolist()) == list(range(1000))
    u = oracle.uniform_int(5000, 9, 256, 4096)
    assert u.min() >= 256 and u.max() <= 4096 and u.max() > 3900 and u.min() < 400
