"""GPU parity of qm_talker_post_attention_m1: o_proj, residual + post-norm + gate/up/SwiGLU, down_proj + residual of a
talker layer and the RMSNorm + Q/K/V of the next one in one launch.

The launch must leave exactly what the four one-operator entry points leave (bit for bit); those are held against the
oracle in test_gpu_linear.py.  Weights are random in the 1.7B talker's geometry (hidden 2048, R17:14626; the rest from its
checkpoint, R17:14993-15003).
"""
import ctypes as C

import pytest

from qm_testlib import to_dev

pytestmark = pytest.mark.gpu

H, Q, KV, I = 2048, 2048, 1024, 6144


class _Layer:
    def __init__(self, oracle, qm, dev, seed, biases):
        import torch
        self.qm, self.dev = qm, dev
        n = [seed]

        def rnd(shape, std=1.0, mean=0.0):
            n[0] += 1
            return to_dev(oracle.normal_bf16(shape, n[0], mean, std, threads=16), dev)

        self.context, self.hidden = rnd((Q,)), rnd((H,))
        self.wo, self.post = rnd((H, Q), 0.02), rnd((H,), 0.1, 1.0)
        self.wg, self.wu, self.wd = rnd((I, H), 0.03), rnd((I, H), 0.03), rnd((H, I), 0.02)
        self.in_norm = rnd((H,), 0.1, 1.0)
        self.wq, self.wk, self.wv = rnd((Q, H), 0.03), rnd((KV, H), 0.03), rnd((KV, H), 0.03)
        self.bo = rnd((H,), 0.1) if biases else None
        self.bq, self.bk, self.bv = (rnd((Q,), 0.1), rnd((KV,), 0.1), rnd((KV,), 0.1)) if biases else (None, None, None)
        z = lambda n_: torch.full((n_,), 0x7fc0, dtype=torch.int16, device=dev)
        self.attn, self.res, self.act = z(H), z(H), z(I)
        self.want = dict(hidden=z(H), q=z(Q), k=z(KV), v=z(KV))
        self.got = dict(hidden=z(H), q=z(Q), k=z(KV), v=z(KV))
        self.ws_bytes = qm.talker_post_attention_workspace_bytes()
        self.ws = torch.zeros(self.ws_bytes // 4, dtype=torch.int32, device=dev)
        qm.talker_post_attention_workspace_init(self.ws, self.ws_bytes)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)

    def by_operators(self, with_next=True):
        qm, w = self.qm, self.want
        qm.linear_m1(self.context, self.wo, self.bo, None, self.attn, H, Q)
        qm.add_postnorm_gate_up_swiglu_m1(self.hidden, self.attn, self.post, self.res, self.wg, self.wu, self.act, H, I)
        qm.linear_m1(self.act, self.wd, None, self.res, w["hidden"], H, I)
        if with_next:
            qm.rmsnorm_qkv_m1(w["hidden"], self.in_norm, self.wq, self.bq, self.wk, self.bk, self.wv, self.bv, w["q"], w["k"], w["v"],
                              H, Q, KV)

    def descriptor(self, with_next=True):
        g = self.got
        names = dict(context=self.context, hidden=self.hidden, o_weight=self.wo, o_bias=self.bo, post_norm=self.post,
                     gate_weight=self.wg, up_weight=self.wu, down_weight=self.wd, hidden_out=g["hidden"])
        if with_next:
            names.update(next_input_norm=self.in_norm, next_q_weight=self.wq, next_q_bias=self.bq, next_k_weight=self.wk,
                         next_k_bias=self.bk, next_v_weight=self.wv, next_v_bias=self.bv, q_out=g["q"], k_out=g["k"], v_out=g["v"])
        return self.qm.talker_post_attention(**{k: v for k, v in names.items() if v is not None})

    def one_launch(self, with_next=True, stream=0):
        self.qm.talker_post_attention_m1(self.descriptor(with_next), self.ws, self.ws_bytes, self.status, stream)

    def same(self, names=("hidden", "q", "k", "v")):
        import torch
        torch.cuda.synchronize()
        return all(torch.equal(self.got[name], self.want[name]) for name in names)


@pytest.fixture(scope="module", params=[False, True], ids=["no_bias", "biases"])
def layer(request, oracle, qm, dev):
    return _Layer(oracle, qm, dev, 7300 + 50 * int(request.param), request.param)


def test_one_launch_equals_the_four_operators(layer):
    import torch
    layer.by_operators()
    for _ in range(3):                                     # a later launch finds the workspace as the one before left it
        for t in layer.got.values():
            t.fill_(0x7fc0)
        layer.one_launch()
        assert layer.same() and int(layer.status.item()) == 0
    # other inputs, same workspace
    layer.context.copy_(torch.roll(layer.context, 3))
    layer.hidden.copy_(torch.roll(layer.hidden, 5))
    layer.by_operators()
    layer.one_launch()
    assert layer.same() and int(layer.status.item()) == 0


def test_after_the_last_layer_there_is_no_next(layer):
    layer.by_operators(with_next=False)
    for name in ("q", "k", "v"):
        layer.got[name].fill_(0x1234)
    layer.one_launch(with_next=False)
    assert layer.same(("hidden",)) and int(layer.status.item()) == 0
    assert all(bool((layer.got[name] == 0x1234).all()) for name in ("q", "k", "v"))
    layer.by_operators()
    layer.one_launch()
    assert layer.same()


def test_replayed_from_a_graph(layer):
    import torch
    layer.by_operators()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    graph = torch.cuda.CUDAGraph()
    torch.cuda.synchronize()
    with torch.cuda.graph(graph, stream=side):
        layer.one_launch(stream=torch.cuda.current_stream().cuda_stream)
    for _ in range(3):
        for t in layer.got.values():
            t.fill_(0x7fc0)
        torch.cuda.synchronize()
        graph.replay()
        assert layer.same() and int(layer.status.item()) == 0
    layer.one_launch()                                     # an eager launch after the replays
    assert layer.same()


def test_giving_up_and_argument_errors(layer, qm):
    import torch
    layer.by_operators()
    # a workspace whose abort word is set (a launch gave up before): nothing runs, the status says so
    for t in layer.got.values():
        t.fill_(0x7fc0)
    layer.ws[1] = 1
    layer.one_launch()
    torch.cuda.synchronize()
    assert int(layer.status.item()) == qm.STATUS_FRAME_TIMEOUT
    assert all(bool((t == 0x7fc0).all()) for t in layer.got.values())
    layer.status.zero_()
    qm.talker_post_attention_workspace_init(layer.ws, layer.ws_bytes)
    layer.one_launch()
    assert layer.same() and int(layer.status.item()) == 0
    # waits cut to one attempt: the launch gives up, every block returns, the status says so
    qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 1)
    try:
        layer.one_launch()
        torch.cuda.synchronize()
    finally:
        qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 0)
    assert int(layer.status.item()) == qm.STATUS_FRAME_TIMEOUT
    layer.status.zero_()
    qm.talker_post_attention_workspace_init(layer.ws, layer.ws_bytes)
    layer.one_launch()
    assert layer.same() and int(layer.status.item()) == 0
    # arguments
    L = qm.lib()
    op = layer.descriptor()
    p = layer.ws.data_ptr()
    call = lambda ws, nbytes: L.qm_talker_post_attention_m1(C.byref(op), ws, nbytes, None, None)
    assert call(None, layer.ws_bytes) == -1 and call(p, layer.ws_bytes - 256) == -4 and call(p + 64, layer.ws_bytes) == -2
    op.hidden_columns = 1024
    assert call(p, layer.ws_bytes) == -2
    op.hidden_columns = 2048
    saved = op.post_norm
    op.post_norm = None
    assert call(p, layer.ws_bytes) == -1
    op.post_norm = saved
    saved = op.next_k_weight
    op.next_k_weight = None
    assert call(p, layer.ws_bytes) == -1
    op.next_k_weight = saved + 2
    assert call(p, layer.ws_bytes) == -2
    op.next_k_weight = saved
    assert call(p, layer.ws_bytes) == 0
    torch.cuda.synchronize()
    assert L.qm_talker_post_attention_workspace_init(None, layer.ws_bytes, None) == -1
    assert L.qm_talker_post_attention_workspace_init(p, layer.ws_bytes - 1, None) == -4


@pytest.mark.parametrize("ctx,paged", [(1, False), (17, False), (130, True), (300, False), (2048, False), (2048, True), (5000, True)])
def test_layer_step_in_two_launches_equals_attention_then_the_one_launch(oracle, qm, dev, layer, ctx, paged):
    """qm_talker_layer_step_m1 — the attention without its merge launch, its split records combined by the first blocks of
    the launch that follows — leaves what qm_decode_step_fused followed by qm_talker_post_attention_m1 leaves: context,
    rotated query, cache, hidden state and the next layer's Q/K/V, bit for bit (one split at short contexts, up to 32)."""
    import numpy as np
    import torch
    from qm_testlib import SCALE, PagedPool, to_u16
    pos = ctx - 1
    q = to_dev(oracle.normal_bf16((16, 128), 8000 + ctx), dev)
    k = to_dev(oracle.normal_bf16((8, 128), 8001 + ctx), dev)
    v = to_dev(oracle.normal_bf16((8, 128), 8002 + ctx), dev)
    gq = to_dev(oracle.normal_bf16((128,), 8003, mean=1.0, std=0.1), dev)
    gk = to_dev(oracle.normal_bf16((128,), 8004, mean=1.0, std=0.1), dev)
    cos_h, sin_h = oracle.rope_table(1, pos)
    cos, sin = to_dev(cos_h, dev), to_dev(sin_h, dev)

    def make():
        if paged:
            pool = PagedPool(oracle, [ctx], seed=8100 + ctx)
            kd, vd, cache, table = pool.device(qm, dev)
            return kd, vd, cache, table, pool.max_pages
        kd = to_dev(oracle.normal_bf16((8, ctx + 3, 128), 8200 + ctx), dev)
        vd = to_dev(oracle.normal_bf16((8, ctx + 3, 128), 8201 + ctx), dev)
        return kd, vd, qm.flat_cache(kd, vd, 8, ctx + 3), None, 1

    ws_bytes = qm.decode_workspace_bytes(1, 16, 8, ctx)
    ws = torch.zeros(ws_bytes // 4 + 1, dtype=torch.float32, device=dev)
    z = lambda *shape: torch.full(shape, 0x7fc0, dtype=torch.int16, device=dev)
    # three launches
    kd1, vd1, cache1, table1, mp = make()
    qrot1, ctx1 = z(16, 128), z(16, 128)
    qm.decode_step_fused(q, k, v, gq, gk, cos, sin, qrot1, cache1, table1, mp, ctx1, 16, pos, -1, SCALE, 1e-6, ws, ws_bytes,
                         layer.status)
    layer.context.copy_(ctx1.view(-1))
    for t in layer.want.values():
        t.fill_(0x7fc0)
    saved, layer.got = layer.got, layer.want
    layer.one_launch()
    layer.got = saved
    torch.cuda.synchronize()
    # two launches
    kd2, vd2, cache2, table2, _ = make()
    qrot2, ctx2 = z(16, 128), z(16, 128)
    for t in layer.got.values():
        t.fill_(0x7fc0)
    step = qm.talker_layer_step(q, k, v, gq, gk, cos, sin, qrot2, cache2, table2, mp, ctx2, 16, pos, -1, SCALE, 1e-6, ws, ws_bytes,
                                layer.descriptor())
    for turn in range(3):                                  # a second step finds the workspaces as the first left them
        wraps = turn == 2 and int(layer.ws[2].item()) == int(layer.ws[0].item()) - 8 + 3   # (the last launch combined splits)
        if wraps:
            # ... and a third whose 16-bit operator number for the context words would be the one they were last written
            # with (65 536 numbers later) takes its second choice instead of taking the old words for its own: the old
            # words are made wrong here (their numbers kept), so taking them would show
            last = int(layer.ws[2].item())
            layer.ws[0] = last - 3 + 65536
            words = layer.ws[64 + 2048 + 6144 + 2048:][:2048]      # (the context words follow the three handed-over vectors)
            words ^= 0x0101
            for t in layer.got.values():
                t.fill_(0x7fc0)
        qm.talker_layer_step_m1(step, layer.ws, layer.ws_bytes, layer.status)
        torch.cuda.synchronize()
        assert int(layer.status.item()) == 0
        assert np.array_equal(to_u16(ctx2), to_u16(ctx1)) and np.array_equal(to_u16(qrot2), to_u16(qrot1))
        assert np.array_equal(to_u16(kd2), to_u16(kd1)) and np.array_equal(to_u16(vd2), to_u16(vd1))
        assert layer.same()
        if wraps:
            assert int(layer.ws[2].item()) == last + 65536 + 2
    assert wraps or ctx < 130 or qm.get_option(qm.OPT_DECODE_TILES_PER_BLOCK) != 0   # (the case was exercised where splits are combined)


def test_layer_step_with_more_splits_than_one_merge_round(oracle, qm, dev, layer):
    """Blocks of four tiles cut a context of 3000 tokens into 47 splits, more than the 32 records one round of the merge takes:
    the attention then keeps its own merge launch, and the step still leaves the same bits."""
    qm.set_option(qm.OPT_DECODE_TILES_PER_BLOCK, 4)
    try:
        test_layer_step_in_two_launches_equals_attention_then_the_one_launch(oracle, qm, dev, layer, 3000, True)
    finally:
        qm.set_option(qm.OPT_DECODE_TILES_PER_BLOCK, 0)


def test_layer_step_argument_errors(oracle, qm, dev, layer):
    import ctypes as C
    import torch
    from qm_testlib import SCALE
    z = torch.zeros((16, 128), dtype=torch.int16, device=dev)
    kv = torch.zeros((8, 32, 128), dtype=torch.int16, device=dev)
    cache = qm.flat_cache(kv, kv.clone(), 8, 32)
    make = lambda position=3, heads=16: qm.talker_layer_step(z, z, z, z, z, z, z, None, cache, None, 1, z, heads, position, -1, SCALE, 1e-6,
                                                             None, 0, layer.descriptor())
    call = lambda step, ws=layer.ws.data_ptr(), nbytes=layer.ws_bytes: qm.lib().qm_talker_layer_step_m1(C.byref(step), ws, nbytes, None, None)
    assert call(make(32)) == -3 and call(make(heads=8)) == -2
    assert call(make(), None) == -1 and call(make(), nbytes=layer.ws_bytes - 256) == -4
    bad = make()
    bad.post.hidden_columns = 1024
    assert call(bad) == -2                                 # nothing is launched when the second launch's arguments are wrong
    bad = make()
    bad.context = None
    assert call(bad) == -1
    bad = make()
    saved = bad.post.next_v_weight
    bad.post.next_v_weight = None
    assert call(bad) == -1                                 # (the next layer's arguments as well)
    bad.post.next_v_weight = saved + 2
    assert call(bad) == -2
    assert call(make()) == 0
    torch.cuda.synchronize()
    assert qm.lib().qm_talker_layer_step_m1(None, layer.ws.data_ptr(), layer.ws_bytes, None, None) == -1
