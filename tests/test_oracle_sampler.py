"""Pins for the oracle's restatement of the final head's score processing and the top-k sampler
(R17:7353-7518, 14025-14143): SplitMix64 known answers, closed forms of the categorical draw,
the order's tie rule, and the arithmetic of the repetition penalty."""
import numpy as np
import pytest

VOCAB, EOS, TAIL, PENALTY, TOP_K, TEMP = 3072, 2150, 1024, 1.05, 50, 0.9


def _state(seed):
    return np.array([seed], dtype=np.uint64)


def test_splitmix64_known_answers(oracle):
    # the published test vectors of SplitMix64 (Steele, Lea, Flood 2014; Vigna's splitmix64.c)
    raw, _ = oracle.splitmix64(_state(0), 4)
    assert [int(x) for x in raw] == [0xe220a8397b1dcdaf, 0x6e789e6aa1b965f4, 0x06c45d188009454f, 0xf88bb8a8724c81ec]
    raw, _ = oracle.splitmix64(_state(1234567), 5)
    assert [int(x) for x in raw] == [6457827717110365317, 3203168211198807973, 9817491932198370423,
                                     4593380528125082431, 16408922859458223821]


def test_uniform_is_the_top_53_bits(oracle):
    st = _state(42)
    raw, uni = oracle.splitmix64(st, 1000)
    assert np.array_equal(uni, (raw >> np.uint64(11)).astype(np.float64) / 2.0 ** 53)
    assert uni.min() >= 0.0 and uni.max() < 1.0
    assert int(st[0]) == (42 + 1000 * 0x9e3779b97f4a7c15) % 2 ** 64      # the state is a counter


def _sample(oracle, scores, top_k, temp, seed, bf16=False, offset=0, vocab=None):
    st = _state(seed)
    out = np.zeros(1, dtype=np.int32)
    vocab = len(scores) - offset if vocab is None else vocab
    assert oracle.sample_topk(scores, bf16, offset, vocab, top_k, temp, st, out) == 0
    return int(out[0]), int(st[0])


def test_top_1_is_the_argmax_and_draws_once(oracle):
    rng = np.random.default_rng(1)
    scores = rng.standard_normal(VOCAB).astype(np.float32)
    got, state = _sample(oracle, scores, 1, TEMP, 7)
    assert got == int(np.argmax(scores))
    assert state == (7 + 0x9e3779b97f4a7c15) % 2 ** 64
    assert _sample(oracle, scores, 0, TEMP, 7) == (int(np.argmax(scores)), 7)          # arg-max mode: no draw


def test_equal_scores_pick_floor_of_u_times_k_in_id_order(oracle):
    # all scores equal: the order is by id, every exp is 1, the running sums are 1, 2, ..., k, and
    # the first index with u * k < i + 1 is floor(u * k)
    scores = np.full(200, 0.25, dtype=np.float32)
    for seed in range(50):
        _, uni = oracle.splitmix64(_state(seed), 1)
        got, _ = _sample(oracle, scores, 8, TEMP, seed)
        assert got == int(np.floor(uni[0] * 8))


def test_ties_go_to_the_lower_id_and_pads_never_enter(oracle):
    scores = np.full(10, -np.inf, dtype=np.float32)
    scores[[7, 3]] = 1.0
    assert _sample(oracle, scores, 0, TEMP, 0)[0] == 3
    # keep = 2 holds ids 3 and 7, each with probability 1/2
    picks = {_sample(oracle, scores, 2, TEMP, s)[0] for s in range(40)}
    assert picks == {3, 7}
    # keep = 4 > two finite scores: the -inf entries that enter (ids 0, 1) have weight 0
    picks = {_sample(oracle, scores, 4, TEMP, s)[0] for s in range(40)}
    assert picks == {3, 7}


def test_without_a_positive_total_the_first_id_is_returned_and_nothing_is_drawn(oracle):
    scores = np.full(64, -np.inf, dtype=np.float32)          # exp(-inf - -inf) = exp(nan)
    assert _sample(oracle, scores, 5, TEMP, 99) == (0, 99)


def test_frequencies_follow_the_softmax_over_the_top_k(oracle):
    scores = np.array([2.0, 1.0, 0.5, -1.0, 3.0, 0.0], dtype=np.float32)
    k, temp, n = 4, 0.7, 20000
    order = np.argsort(-scores, kind="stable")[:k]
    p = np.exp(scores[order].astype(np.float64) / temp)
    p /= p.sum()
    st = _state(5)
    out = np.zeros(1, dtype=np.int32)
    counts = np.zeros(len(scores))
    for _ in range(n):
        assert oracle.sample_topk(scores, False, 0, len(scores), k, temp, st, out) == 0
        counts[out[0]] += 1
    assert counts[[3, 5]].sum() == 0                          # outside the top 4
    assert np.max(np.abs(counts[order] / n - p)) < 0.012      # ~4 sigma at n = 20000


def test_bf16_logits_with_row_offset(oracle):
    logits = oracle.normal_bf16((3 * 2048,), 8)
    want = _sample(oracle, oracle.bf16_to_f32(logits[2 * 2048:]), TOP_K, TEMP, 3)
    assert _sample(oracle, logits, TOP_K, TEMP, 3, bf16=True, offset=2 * 2048, vocab=2048) == want


def test_reciprocal_of_the_penalty_is_the_reference_constant():
    assert (np.float32(1.0) / np.float32(PENALTY)).view(np.uint32) == 0x3f73cf3e      # R17:14062


def test_score_processing_closed_forms(oracle):
    logits = oracle.normal_bf16((VOCAB,), 21)
    raw = oracle.bf16_to_f32(logits)
    history = np.array([5, 17, 5, EOS, 2047, 3000], dtype=np.int32)
    scores = np.zeros(VOCAB, dtype=np.float32)
    assert oracle.final_head_process(logits, history, len(history), 3, VOCAB, EOS, TAIL, PENALTY, scores) == 0
    want = raw.copy()
    for t in (5, 17, EOS, 2047):
        want[t] = raw[t] * np.float32(PENALTY) if raw[t] < 0 else raw[t] * (np.float32(1.0) / np.float32(PENALTY))
    tail = np.arange(VOCAB - TAIL, VOCAB)
    want[tail[tail != EOS]] = -np.inf
    assert np.array_equal(scores, want)
    assert np.isfinite(scores[EOS]) and np.isfinite(scores[2047]) and scores[2048] == -np.inf
    # only the first history_count entries count; the end-of-sequence token is barred in frames 0 and 1
    assert oracle.final_head_process(logits, history, 1, 1, VOCAB, EOS, TAIL, PENALTY, scores) == 0
    assert scores[17] == raw[17] and scores[EOS] == -np.inf and scores[5] != raw[5]


def test_final_head_sample_appends_to_the_history_it_reads(oracle):
    logits = oracle.normal_bf16((VOCAB,), 33)
    history = np.zeros(16, dtype=np.int32)
    st = _state(11)
    code = np.zeros(1, dtype=np.int32)
    codes = []
    for g in range(6):
        assert oracle.final_head_sample(logits, history, g, VOCAB, EOS, TAIL, PENALTY, TOP_K, TEMP, st, code) == 0
        codes.append(int(code[0]))
        assert history[g] == code[0]
    assert all(0 <= c < VOCAB - TAIL or c == EOS for c in codes)
    assert int(st[0]) == (11 + 6 * 0x9e3779b97f4a7c15) % 2 ** 64
    # with sampling off the most likely token is penalised after it was emitted once
    history[:] = 0
    for g in range(3):
        assert oracle.final_head_sample(logits, history, g, VOCAB, EOS, TAIL, PENALTY, 0, TEMP, None, code) == 0
    scores = np.zeros(VOCAB, dtype=np.float32)
    assert oracle.final_head_process(logits, None, 0, 2, VOCAB, EOS, TAIL, PENALTY, scores) == 0
    assert history[0] == int(np.argmax(scores))
