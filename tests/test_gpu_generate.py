"""GPU parity of the frame engine (libqm_engine): final head, the code predictor's fifteen-step frame and the
generation loop, on a synthetic checkpoint written here.

The predictor frame and the final head are compared with the oracle's chain of the same operators from the same
inputs: the sampled codes must be identical (the linears are bit-exact, the attention over at most 16 keys is the
exact-chain kernel) and the next talker input with them.  The loop itself is held to the determinism contract of
the reference (CONTRACT.md:148-158): the same request gives the same codec trajectory and hash, also after a reset,
and the loop's codes equal a replay of the same engines step by step from Python.
"""
import ctypes as C
import os

import numpy as np
import pytest

from qm_testlib import to_u16

pytestmark = pytest.mark.gpu

H, Q, KV, I_T, T_LAYERS = 2048, 2048, 1024, 512, 2           # talker (small intermediate: the test is about the loop)
PH, PI, P_LAYERS, V, STEPS = 1024, 3072, 5, 2048, 15            # predictor: its real geometry (the one-launch frame kernel needs it)
HEAD_V, EOS, TABLE_ROWS = 3072, 2150, 3072
SEED = 20240229


def _checkpoint(directory, eos_gain=1.0, intermediate=I_T):
    import torch
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(99)

    def rnd(shape, std=1.0, mean=0.0):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    t = {"talker.model.norm.weight": rnd((H,), 0.1, 1.0), "talker.model.codec_embedding.weight": rnd((TABLE_ROWS, H), 0.5),
         "talker.codec_head.weight": rnd((HEAD_V, H), 0.05)}
    for i in range(T_LAYERS):
        p = f"talker.model.layers.{i}."
        t.update({p + "input_layernorm.weight": rnd((H,), 0.1, 1.0), p + "post_attention_layernorm.weight": rnd((H,), 0.1, 1.0),
                  p + "self_attn.q_proj.weight": rnd((Q, H), 0.02), p + "self_attn.k_proj.weight": rnd((KV, H), 0.02),
                  p + "self_attn.v_proj.weight": rnd((KV, H), 0.02), p + "self_attn.o_proj.weight": rnd((H, Q), 0.02),
                  p + "self_attn.q_norm.weight": rnd((128,), 0.1, 1.0), p + "self_attn.k_norm.weight": rnd((128,), 0.1, 1.0),
                  p + "mlp.gate_proj.weight": rnd((intermediate, H), 0.03), p + "mlp.up_proj.weight": rnd((intermediate, H), 0.03),
                  p + "mlp.down_proj.weight": rnd((H, intermediate), 0.03)})
    c = "talker.code_predictor."
    t.update({c + "small_to_mtp_projection.weight": rnd((PH, H), 0.02), c + "small_to_mtp_projection.bias": rnd((PH,), 0.1),
              c + "model.norm.weight": rnd((PH,), 0.1, 1.0)})
    for i in range(P_LAYERS):
        p = c + f"model.layers.{i}."
        t.update({p + "input_layernorm.weight": rnd((PH,), 0.1, 1.0), p + "post_attention_layernorm.weight": rnd((PH,), 0.1, 1.0),
                  p + "self_attn.q_proj.weight": rnd((Q, PH), 0.03), p + "self_attn.k_proj.weight": rnd((KV, PH), 0.03),
                  p + "self_attn.v_proj.weight": rnd((KV, PH), 0.03), p + "self_attn.o_proj.weight": rnd((PH, Q), 0.02),
                  p + "self_attn.q_norm.weight": rnd((128,), 0.1, 1.0), p + "self_attn.k_norm.weight": rnd((128,), 0.1, 1.0),
                  p + "mlp.gate_proj.weight": rnd((PI, PH), 0.03), p + "mlp.up_proj.weight": rnd((PI, PH), 0.03),
                  p + "mlp.down_proj.weight": rnd((PH, PI), 0.02)})
    for i in range(STEPS):
        t[c + f"lm_head.{i}.weight"] = rnd((V, PH), 0.05)
        t[c + f"model.codec_embedding.{i}.weight"] = rnd((V, H), 0.5)
    if eos_gain != 1.0:
        # the end-of-sequence code wins or loses by a wide margin, depending on the sign of its row's product with the hidden state
        t["talker.codec_head.weight"][EOS] = (t["talker.codec_head.weight"][EOS].float() * eos_gain).to(torch.bfloat16)
    save_file(t, os.path.join(directory, "model.safetensors"))
    return {n: x.view(torch.int16).numpy().view(np.uint16).copy() for n, x in t.items()}


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    directory = str(tmp_path_factory.mktemp("frame_model"))
    return directory, _checkpoint(directory)


def _device_bytes(address, nbytes):
    hip = C.CDLL("libamdhip64.so")
    out = np.zeros(nbytes // 2, dtype=np.uint16)
    assert hip.hipMemcpy(out.ctypes.data_as(C.c_void_p), C.c_void_p(address), C.c_size_t(nbytes), 2) == 0
    return out


def _oracle_predictor_frame(oracle, w, hidden, code0, context, rng, sampling=True):
    """capture_step x 15 and capture_graph's tail (R17:13592-13896) with the oracle's operators."""
    c = "talker.code_predictor."
    u16 = lambda *s: np.zeros(s, dtype=np.uint16)
    cos, sin = oracle.rope_table(16, 0)
    codes = np.zeros(16, dtype=np.int32)
    selected = u16(16, H)
    table = w["talker.model.codec_embedding.weight"]
    free = u16(2, H)
    free[0] = hidden
    codes[0] = code0
    selected[0] = table[code0]
    free[1] = table[code0]
    caches = [(u16(8, 16, 128), u16(8, 16, 128)) for _ in range(P_LAYERS)]
    top_k = 50 if sampling else 0
    # ---- step 0: two rows, the staged path ----
    rows = 2
    cur = u16(rows, PH)
    assert oracle.linear_rows(free, w[c + "small_to_mtp_projection.weight"], w[c + "small_to_mtp_projection.bias"], None, cur,
                              rows, PH, H, 16) == 0
    for layer in range(P_LAYERS):
        p = c + f"model.layers.{layer}."
        kc, vc = caches[layer]
        norm, q, k, v = u16(rows, PH), u16(rows, Q), u16(rows, KV), u16(rows, KV)
        assert oracle.rmsnorm_rows(cur, w[p + "input_layernorm.weight"], norm, rows, PH) == 0
        for name, dst, n in (("q", q, Q), ("k", k, KV), ("v", v, KV)):
            assert oracle.linear_rows(norm, w[p + f"self_attn.{name}_proj.weight"], None, None, dst, rows, n, PH, 16) == 0
        qn, kn = u16(rows * 16, 128), u16(rows * 8, 128)
        assert oracle.rmsnorm_rows(q.reshape(rows * 16, 128), w[p + "self_attn.q_norm.weight"], qn, rows * 16, 128) == 0
        assert oracle.rmsnorm_rows(k.reshape(rows * 8, 128), w[p + "self_attn.k_norm.weight"], kn, rows * 8, 128) == 0
        qb, kb, vb = u16(16, rows, 128), u16(8, rows, 128), u16(8, rows, 128)
        assert oracle.predictor_transpose(qn, qb, rows, 16) == 0
        assert oracle.predictor_transpose(kn, kb, rows, 8) == 0
        assert oracle.predictor_transpose(v, vb, rows, 8) == 0
        qr, kr = u16(16, rows, 128), u16(8, rows, 128)
        assert oracle.predictor_rope_bhsd(qb, cos, sin, qr, rows, 16) == 0
        assert oracle.predictor_rope_bhsd(kb, cos, sin, kr, rows, 8) == 0
        assert oracle.predictor_update_cache(kr, kc, rows, 0) == 0
        assert oracle.predictor_update_cache(vb, vc, rows, 0) == 0
        ctx = u16(rows, Q)
        assert oracle.predictor_attention_staged(qr, kc, vc, ctx.reshape(rows, 16, 128), rows, 2, True) == 0
        res, post, act, nxt = u16(rows, PH), u16(rows, PH), u16(rows, PI), u16(rows, PH)
        assert oracle.linear_rows(ctx, w[p + "self_attn.o_proj.weight"], None, cur, res, rows, PH, Q, 16) == 0
        assert oracle.rmsnorm_rows(res, w[p + "post_attention_layernorm.weight"], post, rows, PH) == 0
        assert oracle.gate_up_swiglu_rows(post, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], act, rows, PH, PI, 16) == 0
        assert oracle.linear_rows(act, w[p + "mlp.down_proj.weight"], None, res, nxt, rows, PH, PI, 16) == 0
        cur = nxt
    fin, logits = u16(rows, PH), u16(rows, V)
    assert oracle.rmsnorm_rows(cur, w[c + "model.norm.weight"], fin, rows, PH) == 0
    assert oracle.linear_rows(fin, w[c + "lm_head.0.weight"], None, None, logits, rows, V, PH, 16) == 0
    out = np.zeros(1, dtype=np.int32)
    assert oracle.sample_topk(logits.reshape(-1), True, (rows - 1) * V, V, top_k, 0.9, rng, out) == 0
    codes[1] = out[0]
    selected[1] = w[c + "model.codec_embedding.0.weight"][out[0]]
    free_input = selected[1].copy()
    # ---- steps 1..14: one row, the M = 1 operators ----
    for step in range(1, STEPS):
        position = step + 1
        cur = u16(PH)
        assert oracle.linear_m1(free_input, w[c + "small_to_mtp_projection.weight"], w[c + "small_to_mtp_projection.bias"], None,
                                cur, PH, H, 16) == 0
        for layer in range(P_LAYERS):
            p = c + f"model.layers.{layer}."
            kc, vc = caches[layer]
            norm, q, k, v, qrot, ctx, attn, res, post, act, nxt = (u16(1, PH), u16(Q), u16(KV), u16(KV), u16(Q), u16(Q),
                                                                   u16(PH), u16(PH), u16(PH), u16(PI), u16(PH))
            assert oracle.rmsnorm_rows(cur.reshape(1, PH), w[p + "input_layernorm.weight"], norm, 1, PH) == 0
            assert oracle.predictor_qkv_m1(norm[0], w[p + "self_attn.q_proj.weight"], w[p + "self_attn.k_proj.weight"],
                                           w[p + "self_attn.v_proj.weight"], q, k, v, PH, Q, KV, 16) == 0
            assert oracle.qk_norm_rope_kv_append(q, k, v, w[p + "self_attn.q_norm.weight"], w[p + "self_attn.k_norm.weight"],
                                                 cos[position], sin[position], qrot, oracle.flat_cache(kc, vc, 8, 16), None, 1,
                                                 16, position) == 0
            assert oracle.predictor_attention_m1(qrot, kc, vc, ctx, position + 1) == 0
            assert oracle.predictor_linear_m1(ctx, w[p + "self_attn.o_proj.weight"], None, attn, PH, Q, 16) == 0
            assert oracle.add_postnorm_m1(cur, attn, w[p + "post_attention_layernorm.weight"], res, post, PH) == 0
            assert oracle.predictor_gate_up_swiglu_m1(post, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], act, PH, PI,
                                                      16) == 0
            assert oracle.predictor_linear_m1(act, w[p + "mlp.down_proj.weight"], res, nxt, PH, PI, 16) == 0
            cur = nxt
        fin, logits = u16(1, PH), u16(V)
        assert oracle.rmsnorm_rows(cur.reshape(1, PH), w[c + "model.norm.weight"], fin, 1, PH) == 0
        assert oracle.linear_m1(fin[0], w[c + f"lm_head.{step}.weight"], None, None, logits, V, PH, 16) == 0
        assert oracle.sample_topk(logits, True, 0, V, top_k, 0.9, rng, out) == 0
        codes[step + 1] = out[0]
        selected[step + 1] = w[c + f"model.codec_embedding.{step}.weight"][out[0]]
        free_input = selected[step + 1].copy()
    total = oracle.bf16_to_f32(selected).astype(np.float32)
    acc = np.zeros(H, dtype=np.float32)
    for group in range(16):
        acc = (acc + total[group]).astype(np.float32)
    summed = oracle.f32_to_bf16(acc)
    nxt_input = oracle.f32_to_bf16(oracle.bf16_to_f32(summed) + oracle.bf16_to_f32(context))
    return codes, nxt_input


@pytest.mark.parametrize("by_operators", [0, 1], ids=["one_launch", "operator_by_operator"])
def test_final_head_and_predictor_frame_match_the_oracle_chain(engine, oracle, qm, dev, model, by_operators):
    """Both ways of running the frame's M = 1 steps (QM_OPT_PREDICTOR_FRAME_OPERATORS) against the oracle's chain."""
    import torch
    directory, w = model
    qm.set_option(qm.OPT_PREDICTOR_FRAME_OPERATORS, by_operators)
    try:
        _frames_against_the_oracle(engine, oracle, dev, directory, w)
    finally:
        qm.set_option(qm.OPT_PREDICTOR_FRAME_OPERATORS, 0)


def _frames_against_the_oracle(engine, oracle, dev, directory, w):
    import torch
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    rng = np.array([SEED], dtype=np.uint64)
    history = np.zeros(32, dtype=np.int32)
    for frame, sampling in ((0, True), (1, True), (2, False)):
        hidden = oracle.normal_bf16((H,), 500 + frame)
        hd = torch.from_numpy(hidden.view(np.int16)).to(dev)
        torch.cuda.synchronize()
        code0 = head.run(hd, frame, sampling)
        # the oracle's final head: codec_head in the talker linear's order, then the sampler with the history so far
        logits = np.zeros(HEAD_V, dtype=np.uint16)
        assert oracle.linear_m1(hidden, w["talker.codec_head.weight"], None, None, logits, HEAD_V, H, 16) == 0
        want = np.zeros(1, dtype=np.int32)
        assert oracle.final_head_sample(logits, history, frame, HEAD_V, EOS, 1024, 1.05, 50 if sampling else 0, 0.9, rng, want) == 0
        assert code0 == int(want[0])
        context = oracle.normal_bf16((H,), 600 + frame, 0.0, 0.5)
        codes = predictor.run_frame(hd, head.device_code, context, sampling)
        want_codes, want_next = _oracle_predictor_frame(oracle, w, hidden, code0, context, rng, sampling)
        assert codes == want_codes.tolist()
        assert np.array_equal(_device_bytes(predictor.next_input, H * 2), want_next)
    predictor.close(); head.close(); talker.close()


def test_predictor_frame_that_gives_up_reports_status_and_recovers(engine, oracle, qm, dev, model):
    """With the frame kernel's waits cut to one attempt (QM_OPT_PREDICTOR_FRAME_SPIN_LIMIT = 1) a frame ends, every block
    returning normally, with QM_ERR_STATUS; the engine sets its workspace up again and the next frame is right."""
    import torch
    directory, w = model
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    hidden = oracle.normal_bf16((H,), 700)
    hd = torch.from_numpy(hidden.view(np.int16)).to(dev)
    context = oracle.normal_bf16((H,), 701, 0.0, 0.5)
    torch.cuda.synchronize()
    code0 = head.run(hd, 0, True)
    good = predictor.run_frame(hd, head.device_code, context, False)          # arg-max: no generator state involved
    qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 1)
    try:
        with pytest.raises(engine.EngineError) as info:
            predictor.run_frame(hd, head.device_code, context, False)
        assert info.value.code == -9
    finally:
        qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 0)
    assert predictor.run_frame(hd, head.device_code, context, False) == good
    assert good[0] == code0
    predictor.close(); head.close(); talker.close()


def _fnv1a64(data):
    value = 1469598103934665603
    for b in data:
        value = ((value ^ b) * 1099511628211) & 0xFFFFFFFFFFFFFFFF
    return value


def test_generation_loop_is_deterministic_and_equals_its_stepwise_replay(engine, oracle, qm, dev, model):
    import torch
    directory, w = model
    prompt_rows, frames = 19, 5
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    prompt = oracle.normal_bf16((prompt_rows, H), 41)
    pd = torch.from_numpy(prompt.view(np.int16)).to(dev)
    torch.cuda.synchronize()
    tts_pad = oracle.normal_bf16((H,), 42, 0.0, 0.5)
    trailing = oracle.normal_bf16((2, H), 43, 0.0, 0.5)
    codes, digest = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, trailing)
    assert codes.shape == (frames, 16) and digest == _fnv1a64(codes.tobytes()) == engine.fnv1a64(codes.tobytes())
    assert codes.min() >= 0 and codes[:, 1:].max() < V
    # the same request again, after a reset: same trajectory, same hash (CONTRACT.md:148-158)
    for _ in range(2):
        head.reset(SEED)
        again, digest2 = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, trailing)
        assert np.array_equal(again, codes) and digest2 == digest
    # another seed gives another trajectory (the samplers do draw)
    head.reset(SEED + 1)
    other, _ = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, trailing)
    assert not np.array_equal(other, codes)
    # the loop, replayed from Python with the same engines: prefill, then per frame head / predictor / decode
    head.reset(SEED)
    cos, sin = engine.rope_rows(prompt_rows, 0)
    dcos, dsin = engine.rope_rows(frames, prompt_rows)
    hidden = talker.prefill(pd, cos, sin, prompt_rows)
    talker.synchronize()
    replay = []
    for frame in range(frames):
        code0 = head.run(hidden, frame)
        context = trailing[frame] if frame < trailing.shape[0] else tts_pad
        frame_codes = predictor.run_frame(hidden, head.device_code, context)
        assert frame_codes[0] == code0
        replay.append(frame_codes)
        if frame + 1 < frames:
            hidden = talker.decode(predictor.next_input, dcos[frame], dsin[frame], frame)
    talker.synchronize()
    assert np.array_equal(np.array(replay, dtype=np.int32), codes)
    # fewer frames: a prefix of the trajectory; argument errors
    head.reset(SEED)
    short, _ = engine.generate(talker, head, predictor, pd, prompt_rows, 2, tts_pad, trailing)
    assert np.array_equal(short, codes[:2])
    with pytest.raises(engine.EngineError):
        engine.generate(talker, head, predictor, pd, 0, 2, tts_pad, trailing)
    predictor.close(); head.close(); talker.close()


def test_generation_stops_at_the_end_of_sequence_code(engine, oracle, qm, dev, tmp_path):
    """A checkpoint whose final head gives the end-of-sequence code for about every other hidden state: the loop stops at
    the first such frame from the third on (R17:22222-22232) without counting it, exactly where the stepwise replay — which
    reads the code before the predictor runs, as the reference does — stops, and leaves the generator state that replay leaves."""
    import torch
    directory = str(tmp_path)
    _checkpoint(directory, eos_gain=60.0)
    prompt_rows, limit = 11, 24
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    pd = torch.from_numpy(oracle.normal_bf16((prompt_rows, H), 51).view(np.int16)).to(dev)
    torch.cuda.synchronize()
    tts_pad = oracle.normal_bf16((H,), 52, 0.0, 0.5)
    codes, digest = engine.generate(talker, head, predictor, pd, prompt_rows, limit, tts_pad, None)
    state_after_generate = _device_bytes(head.rng_state, 8).copy()
    assert 2 <= codes.shape[0] < limit, "the checkpoint is meant to end the sequence early, from the third frame on"
    assert digest == _fnv1a64(codes.tobytes())
    assert not (codes[2:, 0] == EOS).any()                   # the frame that carries the code is not part of the output
    # the stepwise replay
    head.reset(SEED)
    cos, sin = engine.rope_rows(prompt_rows, 0)
    dcos, dsin = engine.rope_rows(limit, prompt_rows)
    hidden = talker.prefill(pd, cos, sin, prompt_rows)
    talker.synchronize()
    replay = []
    for frame in range(limit):
        code0 = head.run(hidden, frame)
        if code0 == EOS and frame >= 2:
            break
        replay.append(predictor.run_frame(hidden, head.device_code, tts_pad))
        if frame + 1 < limit:
            hidden = talker.decode(predictor.next_input, dcos[frame], dsin[frame], frame)
    talker.synchronize()
    assert np.array_equal(np.array(replay, dtype=np.int32), codes)
    assert np.array_equal(_device_bytes(head.rng_state, 8), state_after_generate)
    # and again through the loop: the same trajectory
    head.reset(SEED)
    again, digest2 = engine.generate(talker, head, predictor, pd, prompt_rows, limit, tts_pad, None)
    assert np.array_equal(again, codes) and digest2 == digest
    predictor.close(); head.close(); talker.close()


def _masked_stream(compute_units):
    """A HIP stream confined to the first `compute_units` compute units (hipExtStreamCreateWithCUMask), as the
    reference's generation stream is (R17:7733-7792)."""
    hip = C.CDLL("libamdhip64.so")
    words = (compute_units + 31) // 32
    mask = (C.c_uint32 * words)(*[0xFFFFFFFF if 32 * (i + 1) <= compute_units else (1 << (compute_units - 32 * i)) - 1
                                  for i in range(words)])
    stream = C.c_void_p()
    assert hip.hipExtStreamCreateWithCUMask(C.byref(stream), C.c_uint32(words), mask) == 0
    return hip, stream


def test_a_stream_confined_to_part_of_the_chip_takes_the_operators_one_by_one(engine, oracle, qm, dev, tmp_path):
    """The two one-launch kernels (a talker layer between two attentions, the predictor's frame) need all 256 compute
    units at once.  On a stream with a CU mask of half the chip the library says so without launching (…_fits = 0, the
    launch entry returns QM_ERR_NO_DEVICE), and engines created on that stream run operator by operator: the same codes
    and hash as engines on an unconfined stream."""
    import torch
    directory = str(tmp_path)
    _checkpoint(directory, intermediate=6144)                # the geometry the talker's one launch per layer serves
    prompt_rows, frames = 13, 4
    prompt = oracle.normal_bf16((prompt_rows, H), 61)
    pd = torch.from_numpy(prompt.view(np.int16)).to(dev)
    tts_pad = oracle.normal_bf16((H,), 62, 0.0, 0.5)
    torch.cuda.synchronize()
    assert qm.talker_chain_fits(0) and qm.predictor_frame_fits(0)
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    want, want_digest = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, None)
    predictor.close(); head.close(); talker.close()

    hip, stream = _masked_stream(128)
    try:
        assert not qm.talker_chain_fits(stream.value) and not qm.predictor_frame_fits(stream.value)
        ws_bytes = qm.talker_post_attention_workspace_bytes()
        ws = torch.zeros(ws_bytes // 4 + 64, dtype=torch.int32, device=dev)
        z = torch.zeros(8192, dtype=torch.int16, device=dev)
        big = torch.zeros((6144, 2048), dtype=torch.int16, device=dev)
        op = qm.talker_post_attention(context=z, hidden=z, o_weight=big, post_norm=z, gate_weight=big, up_weight=big,
                                      down_weight=big, hidden_out=z)
        with pytest.raises(qm.QmError) as info:
            qm.talker_post_attention_m1(op, ws, ws_bytes, None, stream.value)
        assert info.value.code == -6
        talker = engine.Talker(directory, 64, stream.value)
        head = engine.FinalHead(directory, 32, SEED, talker.stream)
        predictor = engine.Predictor(directory, head.rng_state, talker.stream)
        got, digest = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, None)
        assert np.array_equal(got, want) and digest == want_digest
        predictor.close(); head.close(); talker.close()
    finally:
        torch.cuda.synchronize()
        assert hip.hipStreamDestroy(stream) == 0


def test_a_talker_launch_that_gives_up_ends_the_generation_at_once_and_the_engine_recovers(engine, oracle, qm, dev, tmp_path):
    """With the hand-off waits cut to one attempt the talker's one launch per layer gives up (every block returns
    normally, QM_STATUS_FRAME_TIMEOUT in the engine's status word).  The loop reads that word back with every frame's
    codes: the generation ends with QM_ERR_STATUS after the first frame that sees it instead of running to the frame
    limit on a stale hidden state, and the next generation (operator by operator from then on) is right."""
    import torch
    directory = str(tmp_path)
    _checkpoint(directory, intermediate=6144)                # the geometry the talker's one launch per layer serves
    prompt_rows, frames = 13, 6
    pd = torch.from_numpy(oracle.normal_bf16((prompt_rows, H), 71).view(np.int16)).to(dev)
    tts_pad = oracle.normal_bf16((H,), 72, 0.0, 0.5)
    torch.cuda.synchronize()
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    want, want_digest = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, None)
    head.reset(SEED)
    qm.set_option(qm.OPT_PREDICTOR_FRAME_OPERATORS, 1)       # the predictor by operators: only the talker's launch gives up
    qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 1)
    try:
        with pytest.raises(engine.EngineError) as info:
            engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, None)
        assert info.value.code == -9
    finally:
        qm.set_option(qm.OPT_PREDICTOR_FRAME_SPIN_LIMIT, 0)
        qm.set_option(qm.OPT_PREDICTOR_FRAME_OPERATORS, 0)
    head.reset(SEED)
    got, digest = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, None)
    assert np.array_equal(got, want) and digest == want_digest
    predictor.close(); head.close(); talker.close()


def test_prompt_pass_on_the_matrix_cores_against_the_exact_chain(engine, oracle, qm, dev, model, capsys):
    """From 16 prompt rows on the prompt pass's linears take their sums on the matrix cores (QM_OPT_LINEAR_ROWS_KERNEL 0,
    the default): tolerance parity with the reference's linear_bf16 chain (R17:126-245), not bit parity, and the codes
    are sampled, so a trajectory may part from the exact chain's (option value 1) at any frame.  What is held: the
    prompt pass's last hidden state of the two settings agrees to two bf16 steps of its largest value, either setting is
    deterministic, and the test reports whether this checkpoint's trajectories agree and from which frame they do not."""
    import torch
    directory, w = model
    prompt_rows, frames = 40, 6
    pd = torch.from_numpy(oracle.normal_bf16((prompt_rows, H), 81).view(np.int16)).to(dev)
    tts_pad = oracle.normal_bf16((H,), 82, 0.0, 0.5)
    torch.cuda.synchronize()
    talker = engine.Talker(directory, 64)
    head = engine.FinalHead(directory, 32, SEED, talker.stream)
    predictor = engine.Predictor(directory, head.rng_state, talker.stream)
    cos, sin = engine.rope_rows(prompt_rows, 0)
    runs, hiddens = {}, {}
    for setting in (0, 1, 0):
        qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, setting)
        try:
            hidden = talker.prefill(pd, cos, sin, prompt_rows)
            talker.synchronize()
            bits = _device_bytes(hidden, H * 2).copy()
            head.reset(SEED)
            codes, digest = engine.generate(talker, head, predictor, pd, prompt_rows, frames, tts_pad, None)
        finally:
            qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, 0)
        if setting in runs:
            assert np.array_equal(runs[setting][0], codes) and runs[setting][1] == digest      # deterministic
            assert np.array_equal(hiddens[setting], bits)
        runs[setting], hiddens[setting] = (codes, digest), bits
    a, b = oracle.bf16_to_f32(hiddens[0]).astype(np.float64), oracle.bf16_to_f32(hiddens[1]).astype(np.float64)
    step = 2.0 ** (np.floor(np.log2(np.abs(b).max())) - 7)
    assert np.abs(a - b).max() <= 2 * step
    same = np.array_equal(runs[0][0], runs[1][0])
    differ = np.nonzero((runs[0][0] != runs[1][0]).any(axis=1))[0]
    with capsys.disabled():
        print("\n[prompt pass: matrix cores vs exact chain] hidden max abs diff %.4g (one bf16 step of the largest value: %.4g); "
              "trajectories %s" % (np.abs(a - b).max(), step, "agree" if same else "part at frame %d" % differ[0]))
    predictor.close(); head.close(); talker.close()
