"""GPU parity: final-head score processing, top-k sampler / arg-max and history append through the
C ABI — the chosen ids, the SplitMix64 state, the history and the processed scores are bit-exact
against the oracle (the device's double exp and glibc's may differ in the last place; a chosen id
could only change if a draw fell within that distance of a boundary of the running sum)."""
import numpy as np
import pytest

from qm_testlib import to_dev

pytestmark = pytest.mark.gpu

VOCAB, EOS, TAIL, PENALTY, TOP_K, TEMP = 3072, 2150, 1024, 1.05, 50, 0.9


def _gpu_sample(qm, dev, logits, bf16, offset, vocab, top_k, temp, seed, draws=1):
    import torch
    st = torch.tensor([seed], dtype=torch.int64, device=dev)
    out = torch.full((1,), -7, dtype=torch.int32, device=dev)
    ld = to_dev(logits, dev) if bf16 else torch.from_numpy(logits).to(dev)
    got = []
    for _ in range(draws):
        qm.sample_topk(ld, bf16, offset, vocab, top_k, temp, st if top_k > 0 else None, out)
        got.append(int(out.item()))
    return got, int(st.item()) % 2 ** 64


def _cpu_sample(oracle, logits, bf16, offset, vocab, top_k, temp, seed, draws=1):
    st = np.array([seed], dtype=np.uint64)
    out = np.zeros(1, dtype=np.int32)
    got = []
    for _ in range(draws):
        assert oracle.sample_topk(logits, bf16, offset, vocab, top_k, temp, st, out) == 0
        got.append(int(out[0]))
    return got, int(st[0])


@pytest.mark.parametrize("vocab,top_k,temp", [(3072, 50, 0.9), (2048, 50, 0.9), (4096, 256, 1.3), (1, 50, 0.9),
                                              (300, 7, 0.5), (77, 200, 2.0), (3072, 1, 0.9), (3072, 0, 0.9)])
def test_sampler_f32_matches_the_oracle_over_many_draws(oracle, qm, dev, vocab, top_k, temp):
    rng = np.random.default_rng(vocab + top_k)
    scores = (rng.standard_normal(vocab) * 3.0).astype(np.float32)
    want = _cpu_sample(oracle, scores, False, 0, vocab, top_k, temp, 1234, draws=64)
    got = _gpu_sample(qm, dev, scores, False, 0, vocab, top_k, temp, 1234, draws=64)
    assert got == want


def test_sampler_bf16_with_row_offset(oracle, qm, dev):
    logits = oracle.normal_bf16((2 * 2048,), 77, std=2.0)
    want = _cpu_sample(oracle, logits, True, 2048, 2048, TOP_K, TEMP, 5, draws=48)
    assert _gpu_sample(qm, dev, logits, True, 2048, 2048, TOP_K, TEMP, 5, draws=48) == want


def test_sampler_order_rules(oracle, qm, dev):
    # many equal scores (bf16-like quantisation), -inf blocks, signed zeros: the order is (score, id)
    rng = np.random.default_rng(9)
    scores = np.round(rng.standard_normal(3072) * 4.0).astype(np.float32) / 4.0
    scores[rng.integers(0, 3072, 900)] = -np.inf
    scores[[10, 20]] = [0.0, -0.0]
    for top_k in (0, 1, 50, 256):
        assert _gpu_sample(qm, dev, scores, False, 0, 3072, top_k, TEMP, 3, draws=32) == \
               _cpu_sample(oracle, scores, False, 0, 3072, top_k, TEMP, 3, draws=32)
    # fewer finite scores than top_k: the -inf entries that enter carry no weight
    few = np.full(512, -np.inf, dtype=np.float32)
    few[[400, 3, 77]] = [1.0, 1.0, 0.5]
    assert _gpu_sample(qm, dev, few, False, 0, 512, 50, TEMP, 8, draws=32) == \
           _cpu_sample(oracle, few, False, 0, 512, 50, TEMP, 8, draws=32)
    # nothing finite: first id, no draw
    none = np.full(100, -np.inf, dtype=np.float32)
    assert _gpu_sample(qm, dev, none, False, 0, 100, 50, TEMP, 99) == ([0], 99)
    # all equal: floor(u * k) in id order
    flat = np.full(1000, 0.5, dtype=np.float32)
    assert _gpu_sample(qm, dev, flat, False, 0, 1000, 8, TEMP, 17, draws=40) == \
           _cpu_sample(oracle, flat, False, 0, 1000, 8, TEMP, 17, draws=40)


def test_final_head_process_bit_exact(oracle, qm, dev):
    import torch
    logits = oracle.normal_bf16((VOCAB,), 21, std=3.0)
    history = np.random.default_rng(2).integers(0, VOCAB, 700).astype(np.int32)
    for count, gen in ((0, 0), (1, 1), (700, 2), (700, 700)):
        want = np.zeros(VOCAB, dtype=np.float32)
        assert oracle.final_head_process(logits, history, count, gen, VOCAB, EOS, TAIL, PENALTY, want) == 0
        got = torch.full((VOCAB,), 123.0, dtype=torch.float32, device=dev)
        qm.final_head_process(to_dev(logits, dev), torch.from_numpy(history).to(dev), count, gen, VOCAB, EOS, TAIL,
                              PENALTY, got)
        torch.cuda.synchronize()
        assert np.array_equal(got.cpu().numpy().view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("top_k", [50, 0])
def test_final_head_sample_sequence(oracle, qm, dev, top_k):
    """Forty frames with fresh logits each: codes, history, generator state and processed scores."""
    import torch
    frames = 40
    hist_cpu = np.zeros(64, dtype=np.int32)
    hist_gpu = torch.zeros(64, dtype=torch.int32, device=dev)
    st_cpu = np.array([2024], dtype=np.uint64)
    st_gpu = torch.tensor([2024], dtype=torch.int64, device=dev)
    code_cpu = np.zeros(1, dtype=np.int32)
    code_gpu = torch.zeros(1, dtype=torch.int32, device=dev)
    scores_cpu = np.zeros(VOCAB, dtype=np.float32)
    scores_gpu = torch.zeros(VOCAB, dtype=torch.float32, device=dev)
    for g in range(frames):
        # a peaked distribution, so that codes repeat and the penalty matters
        logits = oracle.normal_bf16((VOCAB,), 500 + g % 3, std=4.0)
        assert oracle.final_head_sample(logits, hist_cpu, g, VOCAB, EOS, TAIL, PENALTY, top_k, TEMP,
                                        st_cpu if top_k > 0 else None, code_cpu, scores_cpu) == 0
        qm.final_head_sample(to_dev(logits, dev), hist_gpu, g, VOCAB, EOS, TAIL, PENALTY, top_k, TEMP,
                             st_gpu if top_k > 0 else None, code_gpu, scores_gpu)
        torch.cuda.synchronize()
        assert int(code_gpu.item()) == int(code_cpu[0]), g
        assert np.array_equal(scores_gpu.cpu().numpy().view(np.uint32), scores_cpu.view(np.uint32)), g
    assert np.array_equal(hist_gpu.cpu().numpy(), hist_cpu)
    assert int(st_gpu.item()) % 2 ** 64 == int(st_cpu[0])
    assert len(set(hist_cpu[:frames].tolist())) < frames or top_k > 0      # arg-max over 3 logit sets repeats


def test_head_projection_then_sample_is_the_reference_frame_tail(oracle, qm, dev):
    """hidden -> qm_linear_m1 (the head, 3072 x 2048, no bias) -> qm_final_head_sample."""
    import torch
    hidden = oracle.normal_bf16((2048,), 900)
    weight = oracle.normal_bf16((VOCAB, 2048), 901, std=0.05)
    logits = np.zeros(VOCAB, dtype=np.uint16)
    assert oracle.linear_m1(hidden, weight, None, None, logits, VOCAB, 2048, 16) == 0
    hist_cpu = np.array([1, 2, 3, 0], dtype=np.int32)
    st_cpu = np.array([77], dtype=np.uint64)
    code_cpu = np.zeros(1, dtype=np.int32)
    assert oracle.final_head_sample(logits, hist_cpu, 3, VOCAB, EOS, TAIL, PENALTY, TOP_K, TEMP, st_cpu, code_cpu) == 0
    ld = torch.zeros(VOCAB, dtype=torch.int16, device=dev)
    qm.linear_m1(to_dev(hidden, dev), to_dev(weight, dev), None, None, ld, VOCAB, 2048)
    hist_gpu = torch.tensor([1, 2, 3, 0], dtype=torch.int32, device=dev)
    st_gpu = torch.tensor([77], dtype=torch.int64, device=dev)
    code_gpu = torch.zeros(1, dtype=torch.int32, device=dev)
    qm.final_head_sample(ld, hist_gpu, 3, VOCAB, EOS, TAIL, PENALTY, TOP_K, TEMP, st_gpu, code_gpu)
    torch.cuda.synchronize()
    assert int(code_gpu.item()) == int(code_cpu[0])
    assert hist_gpu.cpu().tolist() == hist_cpu.tolist()


def test_sampler_argument_errors(qm, dev):
    import torch
    x = torch.zeros(8192, dtype=torch.float32, device=dev)
    st = torch.zeros(1, dtype=torch.int64, device=dev)
    o = torch.zeros(1, dtype=torch.int32, device=dev)
    L = qm.lib()
    assert L.qm_sample_topk(None, 0, 0, 10, 5, 0.9, st.data_ptr(), o.data_ptr(), None) == -1
    assert L.qm_sample_topk(x.data_ptr(), 0, 0, 10, 5, 0.9, None, o.data_ptr(), None) == -1      # a draw needs the state
    assert L.qm_sample_topk(x.data_ptr(), 0, 0, 10, 0, 0.9, None, o.data_ptr(), None) == 0       # the arg-max does not
    assert L.qm_sample_topk(x.data_ptr(), 0, 0, 4097, 5, 0.9, st.data_ptr(), o.data_ptr(), None) == -2
    assert L.qm_sample_topk(x.data_ptr(), 0, 0, 4096, 257, 0.9, st.data_ptr(), o.data_ptr(), None) == -2
    assert L.qm_sample_topk(x.data_ptr(), 0, 0, 0, 5, 0.9, st.data_ptr(), o.data_ptr(), None) == -5
    assert L.qm_sample_topk(x.data_ptr(), 0, -1, 10, 5, 0.9, st.data_ptr(), o.data_ptr(), None) == -5
    assert L.qm_sample_topk(x.data_ptr(), 0, 0, 10, 5, 0.0, st.data_ptr(), o.data_ptr(), None) == -5
    assert L.qm_final_head_sample(x.data_ptr(), None, 0, 3072, 2150, 1024, 1.05, 50, 0.9, st.data_ptr(), o.data_ptr(),
                                  None, None) == -1
    assert L.qm_final_head_sample(x.data_ptr(), o.data_ptr(), -1, 3072, 2150, 1024, 1.05, 50, 0.9, st.data_ptr(),
                                  o.data_ptr(), None, None) == -5
