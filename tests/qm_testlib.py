"""Shared builders for the parity tests: seeded inputs, paged pools, host<->device copies."""
import numpy as np

SCALE = 0.08838834764831845


def to_dev(a, dev):
    """numpy uint16/int32/uint32 -> device tensor with the same bits."""
    import torch
    if a.dtype == np.uint16:
        return torch.from_numpy(a.view(np.int16).copy()).to(dev)
    if a.dtype == np.uint32:
        return torch.from_numpy(a.view(np.int32).copy()).to(dev)
    return torch.from_numpy(a.copy()).to(dev)


def to_u16(t):
    return t.detach().cpu().numpy().view(np.uint16)


def max_abs_err(oracle, a_bits, b_bits):
    a = oracle.bf16_to_f32(a_bits).astype(np.float64)
    b = oracle.bf16_to_f32(b_bits).astype(np.float64)
    return float(np.max(np.abs(a - b))) if a.size else 0.0


def within_rule(oracle, got_bits, want_bits, tol=1e-2):
    """The one tolerance rule for bf16 outputs, per element: |got - want| <= max(tol, one bf16 ulp of the oracle's
    value).  north_star's bound is tol = 1e-2; from |x| = 2 on a single bf16 step is 1.56e-2, so a result that is the
    neighbouring bf16 value of the oracle's cannot be held to 1e-2 there.  Returns (every element within the rule,
    max abs error, number of elements outside the rule)."""
    want = oracle.bf16_to_f32(want_bits).astype(np.float64)
    err = np.abs(oracle.bf16_to_f32(got_bits).astype(np.float64) - want)
    one_ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -20))) - 7)
    outside = int(np.count_nonzero(err > np.maximum(one_ulp, tol)))
    return outside == 0, float(err.max()) if err.size else 0.0, outside


def ulp_distance(a_bits, b_bits):
    """Distance in bf16 ulps between two arrays of finite same-sign-or-not bf16 bit patterns."""
    def key(x):
        x = x.astype(np.int32)
        return np.where(x & 0x8000, 0x8000 - x, x)
    return np.abs(key(a_bits) - key(b_bits))


class PagedPool:
    """K/V pools in the native [page][kv_head][16][128] layout plus per-stream page tables
    built from a seeded permutation of the physical pages (numpy side)."""

    def __init__(self, oracle, seq_lens, seed, kv_heads=8, page_size=16, slack_pages=3, fill="normal",
                 extra_tokens=0, min_table_pages=0):
        self.kv_heads = kv_heads
        self.page_size = page_size
        seq_lens = np.asarray(seq_lens, dtype=np.int32)
        self.seq_lens = seq_lens
        pages_per = (seq_lens + extra_tokens + page_size - 1) // page_size
        self.max_pages = int(max(1, pages_per.max(), min_table_pages))
        total = int(pages_per.sum())
        self.n_pages = total + slack_pages
        perm = oracle.permutation(self.n_pages, seed ^ 0x5151)
        self.page_table = np.full((len(seq_lens), self.max_pages), -1, dtype=np.int32)
        cur = 0
        for s, n in enumerate(pages_per):
            self.page_table[s, :n] = perm[cur:cur + n]
            cur += n
        shape = (self.n_pages, kv_heads, page_size, 128)
        if fill == "normal":
            self.k = oracle.normal_bf16(shape, seed + 1)
            self.v = oracle.normal_bf16(shape, seed + 2)
        else:
            self.k = np.full(shape, fill, dtype=np.uint16)
            self.v = np.full(shape, fill, dtype=np.uint16)

    def descriptor(self, oracle):
        return oracle.paged_cache(self.k, self.v, self.kv_heads, self.page_size)

    def device(self, qm, dev):
        kd, vd = to_dev(self.k, dev), to_dev(self.v, dev)
        return kd, vd, qm.paged_cache(kd, vd, self.n_pages, self.kv_heads, self.page_size), to_dev(self.page_table, dev)


def step0_chain(oracle, ops, q, k, v, gq, gk, cos, sin, rows):
    """The reference's step-0 attention sequence (R17:13650-13705) on numpy arrays: per-head RMSNorm
    (oracle) -> transpose -> rope -> update_cache -> staged causal attention, the last four through `ops`
    (the oracle binding, or an object with the same five functions that runs them on the device)."""
    ones_c, zeros_s = oracle.rope_table(rows, 0)
    ones_c[:], zeros_s[:] = 0x3F80, 0
    qn, kn = np.zeros_like(q), np.zeros_like(k)
    # per-head RMSNorm alone = norm + RoPE with cos 1, sin 0 (x*1 and +0 are exact)
    assert oracle.norm_rope_rows(q, gq.copy(), ones_c, zeros_s, qn, rows, 16) == 0
    assert oracle.norm_rope_rows(k, gk.copy(), ones_c, zeros_s, kn, rows, 8) == 0
    q_bhsd, k_bhsd, v_bhsd = (np.zeros((16, rows, 128), np.uint16), np.zeros((8, rows, 128), np.uint16),
                              np.zeros((8, rows, 128), np.uint16))
    assert ops.predictor_transpose(qn, q_bhsd, rows, 16) == 0
    assert ops.predictor_transpose(kn, k_bhsd, rows, 8) == 0
    assert ops.predictor_transpose(v, v_bhsd, rows, 8) == 0
    q_rot, k_rot = np.zeros_like(q_bhsd), np.zeros_like(k_bhsd)
    assert ops.predictor_rope_bhsd(q_bhsd, cos, sin, q_rot, rows, 16) == 0
    assert ops.predictor_rope_bhsd(k_bhsd, cos, sin, k_rot, rows, 8) == 0
    kc, vc = np.zeros((8, 16, 128), np.uint16), np.zeros((8, 16, 128), np.uint16)
    assert ops.predictor_update_cache(k_rot, kc, rows, 0) == 0
    assert ops.predictor_update_cache(v_bhsd, vc, rows, 0) == 0
    out = np.zeros((rows, 16, 128), np.uint16)
    assert ops.predictor_attention_staged(q_rot, kc, vc, out, rows, rows, True) == 0
    return out, kc, vc
