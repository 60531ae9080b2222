"""GPU parity of qm_predictor_frame_steps: the steps of a code-predictor frame in one launch.

The launch must leave exactly what the operator-by-operator chain of the same C entry points leaves (sampled codes,
selected embeddings, the next input, the generator state and the appended K/V rows, bit for bit); that chain is held
against the oracle in test_gpu_generate.py, test_gpu_linear.py, test_gpu_predictor.py and test_gpu_sampler.py.
Weights are random in the predictor's real geometry (R17:7951-7964).
"""
import ctypes as C

import numpy as np
import pytest

from qm_testlib import to_dev

pytestmark = pytest.mark.gpu

H, Q, KV, I, OUT, V, LAYERS = 1024, 2048, 1024, 3072, 2048, 2048, 5
SEED = 20240229
FIELDS = dict(in_norm="input_norm", wq="q_weight", wk="k_weight", wv="v_weight", gq="q_norm", gk="k_norm", wo="o_weight",
              post="post_norm", wg="gate_weight", wu="up_weight", wd="down_weight", k="key_cache", v="value_cache")


class _Frame:
    """Weights, the state of a frame after its step 0 (cache rows 0 and 1, the gathered input) and both ways to run on."""

    def __init__(self, oracle, qm, dev, seed=910):
        import torch
        self.qm, self.dev = qm, dev
        n = [seed]

        def rnd(shape, std=1.0, mean=0.0):
            n[0] += 1
            return to_dev(oracle.normal_bf16(shape, n[0], mean, std, threads=16), dev)

        self.proj_w, self.proj_b = rnd((H, OUT), 0.02), rnd((H,), 0.1)
        self.layers = []
        for _ in range(LAYERS):
            k, v = rnd((8, 16, 128)), rnd((8, 16, 128))
            k[:, 2:] = 0                                  # a frame's caches are cleared; step 0 filled rows 0 and 1
            v[:, 2:] = 0
            self.layers.append(dict(in_norm=rnd((H,), 0.1, 1.0), wq=rnd((Q, H), 0.03), wk=rnd((KV, H), 0.03), wv=rnd((KV, H), 0.03),
                                    gq=rnd((128,), 0.1, 1.0), gk=rnd((128,), 0.1, 1.0), wo=rnd((H, Q), 0.02), post=rnd((H,), 0.1, 1.0),
                                    wg=rnd((I, H), 0.03), wu=rnd((I, H), 0.03), wd=rnd((H, I), 0.02), k=k, v=v, k0=k.clone(),
                                    v0=v.clone()))
        self.final_norm = rnd((H,), 0.1, 1.0)
        self.heads = {s: rnd((V, H), 0.05) for s in range(0, 15)}
        self.tables = {s: rnd((V, OUT)) for s in range(0, 15)}
        cos, sin = oracle.rope_table(16, 0, 128, 1.0e6)
        self.cos, self.sin = to_dev(cos, dev), to_dev(sin, dev)
        self.input0 = rnd((OUT,))
        self.step0_rows = rnd((2, OUT))                    # the talker's hidden state, the embedding of the talker's code
        z = lambda *shape: torch.zeros(shape, dtype=torch.int16, device=dev)
        self.free_input, self.selected = self.input0.clone(), z(16, OUT)
        self.codes = torch.zeros(16, dtype=torch.int32, device=dev)
        self.rng = torch.tensor([SEED], dtype=torch.int64, device=dev)
        self.hidden = [z(H), z(H)]
        self.q, self.k_, self.v_, self.ctx = z(Q), z(KV), z(KV), z(Q)
        self.attn, self.res, self.act, self.logits = z(H), z(H), z(I), z(V)
        self.ws_bytes = qm.predictor_frame_workspace_bytes()
        self.ws = torch.zeros(self.ws_bytes // 4, dtype=torch.int32, device=dev)
        qm.predictor_frame_workspace_init(self.ws, self.ws_bytes)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)
        layers = [{FIELDS[key]: layer[key] for key in FIELDS} for layer in self.layers]
        self.frame = qm.predictor_frame(layers, self.proj_w, self.proj_b, self.final_norm, self.heads, self.tables, self.cos,
                                        self.sin, self.free_input, self.selected, self.codes, self.rng, step0_input=self.step0_rows)

    def reset(self):
        self.free_input.copy_(self.input0)
        self.selected.zero_()
        self.codes.zero_()
        self.rng.fill_(SEED)
        for layer in self.layers:
            layer["k"].copy_(layer["k0"])
            layer["v"].copy_(layer["v0"])

    def by_operators(self, first, last, top_k):
        qm = self.qm
        for step in range(first, last + 1):
            position = step + 1
            cur, nxt = self.hidden
            qm.linear_m1(self.free_input, self.proj_w, self.proj_b, None, cur, H, OUT)
            for layer in self.layers:
                qm.predictor_rmsnorm_qkv_m1(cur, layer["in_norm"], layer["wq"], layer["wk"], layer["wv"], self.q, self.k_, self.v_,
                                            H, Q, KV, 1e-6)
                qm.predictor_step_attention_m1(self.q, self.k_, self.v_, layer["gq"], layer["gk"], self.cos[position],
                                               self.sin[position], layer["k"], layer["v"], self.ctx, position, 1e-6)
                qm.predictor_linear_m1(self.ctx, layer["wo"], None, self.attn, H, Q)
                qm.predictor_add_postnorm_gate_up_swiglu_m1(cur, self.attn, layer["post"], self.res, layer["wg"], layer["wu"],
                                                            self.act, H, I, 1e-6)
                qm.predictor_linear_m1(self.act, layer["wd"], self.res, nxt, H, I)
                cur, nxt = nxt, cur
            head = self.heads[step]
            qm.rmsnorm_qkv_m1(cur, self.final_norm, head, None, head, None, head, None, self.logits, self.logits, self.logits,
                              H, V, 0, 1e-6)
            qm.sample_topk(self.logits, True, 0, V, top_k, 0.9, self.rng, self.codes[step + 1:])
            qm.gather_embedding(self.tables[step], V, self.codes, step + 1, OUT, self.selected, self.free_input)

    def step0_by_operators(self, top_k):
        """Step 0 row by row with the talker-order M = 1 operators at cache positions 0 and 1 (what the reference's row
        operators evaluate, row for row); the head, the sampler and the gather after the second row only."""
        qm = self.qm
        for layer in self.layers:
            layer["k"].zero_()
            layer["v"].zero_()
        for position in (0, 1):
            cur, nxt = self.hidden
            qm.linear_m1(self.step0_rows[position], self.proj_w, self.proj_b, None, cur, H, OUT)
            for layer in self.layers:
                qm.rmsnorm_qkv_m1(cur, layer["in_norm"], layer["wq"], None, layer["wk"], None, layer["wv"], None, self.q, self.k_, self.v_,
                                  H, Q, KV, 1e-6)
                qm.predictor_step_attention_m1(self.q, self.k_, self.v_, layer["gq"], layer["gk"], self.cos[position],
                                               self.sin[position], layer["k"], layer["v"], self.ctx, position, 1e-6)
                qm.linear_m1(self.ctx, layer["wo"], None, None, self.attn, H, Q)
                qm.add_postnorm_gate_up_swiglu_m1(cur, self.attn, layer["post"], self.res, layer["wg"], layer["wu"], self.act, H, I, 1e-6)
                qm.linear_m1(self.act, layer["wd"], None, self.res, nxt, H, I)
                cur, nxt = nxt, cur
        head = self.heads[0]
        qm.rmsnorm_qkv_m1(cur, self.final_norm, head, None, head, None, head, None, self.logits, self.logits, self.logits, H, V, 0, 1e-6)
        qm.sample_topk(self.logits, True, 0, V, top_k, 0.9, self.rng, self.codes[1:])
        qm.gather_embedding(self.tables[0], V, self.codes, 1, OUT, self.selected, self.free_input)

    def one_launch(self, first, last, top_k, stream=0):
        self.qm.predictor_frame_steps(self.frame, first, last, top_k, 0.9, self.ws, self.ws_bytes, self.status, stream)

    def snapshot(self):
        import torch
        torch.cuda.synchronize()
        return ([self.codes.clone(), self.selected.clone(), self.free_input.clone(), self.rng.clone()]
                + [layer[name].clone() for layer in self.layers for name in ("k", "v")])


@pytest.fixture(scope="module")
def frame(oracle, qm, dev):
    return _Frame(oracle, qm, dev)


def _same(a, b):
    import torch
    return all(torch.equal(x, y) for x, y in zip(a, b))


@pytest.mark.parametrize("top_k", [50, 0], ids=["top50", "argmax"])
def test_frame_steps_equal_the_operator_chain(frame, top_k):
    frame.reset()
    frame.by_operators(1, 14, top_k)
    want = frame.snapshot()
    codes = want[0].tolist()
    assert codes[:2] == [0, 0] and all(0 <= c < V for c in codes) and len(set(codes[2:])) > 4
    for _ in range(2):                                     # the second launch finds the workspace as the first left it
        frame.reset()
        frame.one_launch(1, 14, top_k)
        got = frame.snapshot()
        assert int(frame.status.item()) == 0
        assert _same(got, want)


@pytest.mark.parametrize("top_k", [50, 0], ids=["top50", "argmax"])
def test_step_0_and_the_whole_frame_in_one_launch(frame, top_k):
    """Step 0 alone leaves what its row-by-row operators leave (caches rows 0 and 1, codes[1], selected[1], the next
    input, the generator state); steps 0..14 in one launch equal step 0 followed by the operator chain of steps 1..14."""
    frame.reset()
    frame.step0_by_operators(top_k)
    want0 = frame.snapshot()
    assert 0 <= want0[0].tolist()[1] < V
    frame.by_operators(1, 14, top_k)
    want = frame.snapshot()
    frame.reset()
    for layer in frame.layers:
        layer["k"].fill_(0x7fc0)                           # whatever a frame before left: step 0 reads none of it
        layer["v"].fill_(0x7fc0)
    frame.one_launch(0, 0, top_k)
    got0 = frame.snapshot()
    assert int(frame.status.item()) == 0
    for layer in frame.layers:                             # (rows 2.. are not step 0's)
        layer["k"][:, 2:] = 0
        layer["v"][:, 2:] = 0
    assert _same(frame.snapshot(), want0) and _same(got0[:4], want0[:4])
    frame.reset()
    frame.one_launch(0, 14, top_k)
    assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
    # and step 0 in one launch, the rest in another
    frame.reset()
    frame.one_launch(0, 0, top_k)
    frame.one_launch(1, 14, top_k)
    assert _same(frame.snapshot(), want)


def test_step_0_after_the_operator_numbers_wrapped_around(frame):
    """The vectors of step 0's second row are written by launches with step 0 only, and the 16-bit operator numbers in their
    words repeat after 128 launches: a launch whose numbers would equal those of the launch that wrote them last takes
    other numbers for that pass (the words then hold another frame's values, which must not be taken for this frame's)."""
    import torch
    frame.reset()
    frame.one_launch(0, 14, 50)
    want = frame.snapshot()
    other = frame.step0_rows.clone()
    try:
        frame.step0_rows.copy_(torch.roll(other, 1, dims=1))   # another frame's step 0 leaves its second-row vectors ...
        frame.reset()
        frame.one_launch(0, 0, 50)
        torch.cuda.synchronize()
        last = int(frame.ws[2].item())                         # (the first operator number of that pass)
        assert last == int(frame.ws[0].item()) - 512
        frame.ws[0] = last + 65536                             # ... and 128 launches later the numbers are the same again
        frame.step0_rows.copy_(other)
        frame.reset()
        frame.one_launch(0, 14, 50)
        assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
        assert int(frame.ws[2].item()) == last + 65536 + 32
    finally:
        frame.step0_rows.copy_(other)
        frame.status.zero_()
        frame.qm.predictor_frame_workspace_init(frame.ws, frame.ws_bytes)
        torch.cuda.synchronize()


def test_frame_steps_in_several_launches(frame):
    """Steps 1..14 as 1..5, 6..6 and 7..14: each launch continues from the caches, the input and the state the one before left."""
    frame.reset()
    frame.one_launch(1, 14, 50)
    want = frame.snapshot()
    frame.reset()
    frame.one_launch(1, 5, 50)
    frame.one_launch(6, 6, 50)
    frame.one_launch(7, 14, 50)
    assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
    # and mixed with the operators: steps 1..3 operator by operator, the rest in one launch
    frame.reset()
    frame.by_operators(1, 3, 50)
    frame.one_launch(4, 14, 50)
    assert _same(frame.snapshot(), want)


def test_frame_steps_from_projected_embedding_tables(frame, qm, dev):
    """With `projected` tables (the input projection of every embedding row, in qm_linear_m1's chain) a step starts from a
    table row instead of projecting the sampled code's embedding: same codes, embeddings, caches and generator state —
    for the whole frame, for launches that start in the middle, and with tables for some steps only."""
    import torch
    tables = {}
    qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, 1)            # the exact chain: row by row what qm_linear_m1 gives
    try:
        for s in range(0, 14):
            tables[s] = torch.zeros((V, H), dtype=torch.int16, device=dev)
            qm.linear_rows(frame.tables[s], frame.proj_w, frame.proj_b, None, tables[s], V, H, OUT)
    finally:
        qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, 0)
    torch.cuda.synchronize()
    # (one row against the M = 1 operator itself)
    one = torch.zeros(H, dtype=torch.int16, device=dev)
    qm.linear_m1(frame.tables[3][77], frame.proj_w, frame.proj_b, None, one, H, OUT)
    assert torch.equal(one, tables[3][77])
    saved = {s: frame.frame.projected[s] for s in range(15)}
    try:
        for given in (range(0, 14), (2, 3, 9)):
            for first, last in ((0, 14), (1, 14), (5, 9)):
                for s in range(15):
                    frame.frame.projected[s] = None
                frame.reset()
                if first > 1:
                    frame.one_launch(1, first - 1, 50)
                frame.one_launch(first, last, 50)
                want = frame.snapshot()
                for s in given:
                    frame.frame.projected[s] = tables[s].data_ptr()
                frame.reset()
                if first > 1:
                    frame.one_launch(1, first - 1, 50)
                frame.one_launch(first, last, 50)
                assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
    finally:
        for s in range(15):
            frame.frame.projected[s] = saved[s]


def test_frame_steps_replayed_from_a_graph(frame):
    """A captured launch is replayed with the operator numbers the workspace has reached by then: every replay, with the
    program's own eager work in between, gives the eager result."""
    import torch
    frame.reset()
    frame.one_launch(1, 14, 50)
    want = frame.snapshot()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    frame.reset()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        frame.one_launch(1, 14, 50, torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        frame.reset()
        torch.cuda.synchronize()
        graph.replay()
        assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
    # an eager launch after the replays
    frame.reset()
    frame.one_launch(1, 14, 50)
    assert _same(frame.snapshot(), want)


def test_frame_steps_abort_word_and_argument_errors(frame, qm, dev):
    import torch
    frame.reset()
    frame.one_launch(1, 14, 0)
    want = frame.snapshot()
    # a workspace whose abort word is set (a launch gave up before): nothing runs, the status says so
    frame.reset()
    before = frame.snapshot()
    frame.ws[1] = 1
    frame.one_launch(1, 14, 0)
    after = frame.snapshot()
    assert int(frame.status.item()) == qm.STATUS_FRAME_TIMEOUT and _same(after, before)
    frame.status.zero_()
    qm.predictor_frame_workspace_init(frame.ws, frame.ws_bytes)
    frame.one_launch(1, 14, 0)
    assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
    # waits cut to one attempt: the launch gives up, every block returns, the status says so
    qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 1)
    try:
        frame.reset()
        frame.one_launch(1, 14, 0)
        torch.cuda.synchronize()
    finally:
        qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 0)
    assert int(frame.status.item()) == qm.STATUS_FRAME_TIMEOUT
    frame.status.zero_()
    qm.predictor_frame_workspace_init(frame.ws, frame.ws_bytes)
    frame.reset()
    frame.one_launch(1, 14, 0)
    assert _same(frame.snapshot(), want) and int(frame.status.item()) == 0
    # arguments
    L = qm.lib()
    call = lambda first, last, top_k, ws, nbytes: L.qm_predictor_frame_steps(C.byref(frame.frame), first, last, top_k, C.c_float(0.9),
                                                                             ws, nbytes, None, None)
    p = frame.ws.data_ptr()
    assert call(-1, 14, 50, p, frame.ws_bytes) == -5 and call(1, 15, 50, p, frame.ws_bytes) == -5 and call(5, 4, 50, p, frame.ws_bytes) == -5
    saved = frame.frame.step0_input
    frame.frame.step0_input = None                         # step 0 needs its two rows
    assert call(0, 14, 50, p, frame.ws_bytes) == -1 and call(1, 14, 50, p, frame.ws_bytes) == 0
    frame.frame.step0_input = saved
    torch.cuda.synchronize()
    assert call(1, 14, 257, p, frame.ws_bytes) == -5
    assert call(1, 14, 50, p, frame.ws_bytes - 256) == -4 and call(1, 14, 50, p + 64, frame.ws_bytes) == -2
    assert call(1, 14, 50, None, frame.ws_bytes) == -1
    saved = frame.frame.final_norm
    frame.frame.final_norm = None
    assert call(1, 14, 50, p, frame.ws_bytes) == -1
    frame.frame.final_norm = saved + 2
    assert call(1, 14, 50, p, frame.ws_bytes) == -2
    frame.frame.final_norm = saved
    assert L.qm_predictor_frame_workspace_init(None, frame.ws_bytes, None) == -1
    assert L.qm_predictor_frame_workspace_init(p, frame.ws_bytes - 1, None) == -4
