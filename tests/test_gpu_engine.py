"""GPU parity of the engine shell: a synthetic talker checkpoint (safetensors, written here with
torch) is loaded by qm_talker_create, a prompt's K/V is placed in the caches, and decode steps run
through every layer; the final hidden vector of each step is compared with the oracle's chain of
the same operators (bit-exact, as for the single-layer step), and the trajectory hash of the
outputs with the hash of the oracle's bytes."""
import os

import numpy as np
import pytest

from qm_testlib import SCALE, to_u16

pytestmark = pytest.mark.gpu

H, Q, KV, I, LAYERS, MAX_CACHE, PREFILL = 2048, 2048, 1024, 512, 3, 48, 21


def _checkpoint(directory, with_bias, inter=I, layers=LAYERS):
    import torch
    from safetensors.torch import save_file
    g = torch.Generator().manual_seed(17 + with_bias)

    def rnd(shape, std=1.0, mean=0.0):
        return (torch.randn(shape, generator=g) * std + mean).to(torch.bfloat16)

    tensors = {"talker.model.norm.weight": rnd((H,), 0.1, 1.0), "talker.model.codec_embedding.weight": rnd((8, 16))}
    for i in range(layers):
        p = f"talker.model.layers.{i}."
        tensors.update({
            p + "input_layernorm.weight": rnd((H,), 0.1, 1.0), p + "post_attention_layernorm.weight": rnd((H,), 0.1, 1.0),
            p + "self_attn.q_proj.weight": rnd((Q, H), 0.02), p + "self_attn.k_proj.weight": rnd((KV, H), 0.02),
            p + "self_attn.v_proj.weight": rnd((KV, H), 0.02), p + "self_attn.o_proj.weight": rnd((H, Q), 0.02),
            p + "self_attn.q_norm.weight": rnd((128,), 0.1, 1.0), p + "self_attn.k_norm.weight": rnd((128,), 0.1, 1.0),
            p + "mlp.gate_proj.weight": rnd((inter, H), 0.03), p + "mlp.up_proj.weight": rnd((inter, H), 0.03),
            p + "mlp.down_proj.weight": rnd((H, inter), 0.03),
        })
        if with_bias:
            tensors.update({p + "self_attn.q_proj.bias": rnd((Q,), 0.1), p + "self_attn.k_proj.bias": rnd((KV,), 0.1),
                            p + "self_attn.v_proj.bias": rnd((KV,), 0.1), p + "self_attn.o_proj.bias": rnd((H,), 0.1)})
    # two files, as a sharded checkpoint: the reader takes the union
    names = sorted(tensors)
    save_file({n: tensors[n] for n in names[::2]}, os.path.join(directory, "model-00001-of-00002.safetensors"))
    save_file({n: tensors[n] for n in names[1::2]}, os.path.join(directory, "model-00002-of-00002.safetensors"))
    return {n: t.view(torch.int16).numpy().view(np.uint16).copy() for n, t in tensors.items()}


@pytest.mark.parametrize("with_bias", [False, True])
def test_engine_decode_steps_match_the_oracle_chain(engine, oracle, qm, dev, tmp_path, with_bias):
    import torch
    w = _checkpoint(str(tmp_path), with_bias)
    talker = engine.Talker(str(tmp_path), MAX_CACHE)
    assert (talker.layers, talker.q_heads, talker.kv_heads, talker.q_dim, talker.kv_dim, talker.intermediate,
            talker.max_cache) == (LAYERS, 16, 8, Q, KV, I, MAX_CACHE)
    talker.reset(PREFILL)
    # a prompt's K/V, placed as the prefill would leave it: [kv_heads][max_cache][128], zero elsewhere
    caches = []
    for layer in range(LAYERS):
        k = np.zeros((8, MAX_CACHE, 128), dtype=np.uint16)
        v = np.zeros((8, MAX_CACHE, 128), dtype=np.uint16)
        k[:, :PREFILL] = oracle.normal_bf16((8, PREFILL, 128), 100 + layer)
        v[:, :PREFILL] = oracle.normal_bf16((8, PREFILL, 128), 200 + layer)
        caches.append((k, v))
    talker.synchronize()
    import ctypes as C
    hip = C.CDLL("libamdhip64.so")
    for layer, (k, v) in enumerate(caches):
        ka, va = talker.cache_addresses(layer)
        assert hip.hipMemcpy(C.c_void_p(ka), k.ctypes.data_as(C.c_void_p), C.c_size_t(k.nbytes), 1) == 0
        assert hip.hipMemcpy(C.c_void_p(va), v.ctypes.data_as(C.c_void_p), C.c_size_t(v.nbytes), 1) == 0

    def tensor(name):
        return w.get(name)

    trajectory_gpu, trajectory_cpu = b"", b""
    for step in range(4):
        x = oracle.normal_bf16((H,), 900 + step)
        cos, sin = engine.rope_rows(1, PREFILL + step)
        xd = torch.from_numpy(x.view(np.int16)).to(dev)
        address = talker.decode(xd, cos[0], sin[0], step)
        talker.synchronize()
        out = torch.empty(H, dtype=torch.int16, device=dev)
        assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(address), C.c_size_t(H * 2), 3) == 0
        got = to_u16(out)
        # the oracle's chain (R17:17155-17252)
        cur = x.copy()
        u16 = lambda n: np.zeros(n, dtype=np.uint16)
        for layer in range(LAYERS):
            p = f"talker.model.layers.{layer}."
            k, v = caches[layer]
            cache = oracle.flat_cache(k, v, 8, MAX_CACHE)
            norm, q, kk, vv, qrot, ctxv, attn, res, post, act, nxt = (u16(H).reshape(1, H), u16(Q), u16(KV), u16(KV),
                                                                     u16(Q), u16(Q), u16(H), u16(H), u16(H), u16(I), u16(H))
            assert oracle.rmsnorm_rows(cur.reshape(1, H), tensor(p + "input_layernorm.weight"), norm, 1, H) == 0
            assert oracle.qkv_m1(norm[0], tensor(p + "self_attn.q_proj.weight"), tensor(p + "self_attn.q_proj.bias"),
                                 tensor(p + "self_attn.k_proj.weight"), tensor(p + "self_attn.k_proj.bias"),
                                 tensor(p + "self_attn.v_proj.weight"), tensor(p + "self_attn.v_proj.bias"),
                                 q, kk, vv, H, Q, KV, 16) == 0
            assert oracle.qk_norm_rope_kv_append(q, kk, vv, tensor(p + "self_attn.q_norm.weight"),
                                                 tensor(p + "self_attn.k_norm.weight"), cos[0], sin[0], qrot, cache,
                                                 None, 1, 16, PREFILL + step) == 0
            assert oracle.attention(qrot, cache, None, 1, ctxv, 1, PREFILL + step, 16, -1, SCALE, oracle.POLICY_ONLINE,
                                    16) == 0
            assert oracle.linear_m1(ctxv, tensor(p + "self_attn.o_proj.weight"), tensor(p + "self_attn.o_proj.bias"),
                                    None, attn, H, Q, 16) == 0
            assert oracle.add_postnorm_m1(cur, attn, tensor(p + "post_attention_layernorm.weight"), res, post, H) == 0
            assert oracle.gate_up_swiglu_m1(post, tensor(p + "mlp.gate_proj.weight"), tensor(p + "mlp.up_proj.weight"),
                                            act, H, I, 16) == 0
            assert oracle.linear_m1(act, tensor(p + "mlp.down_proj.weight"), None, res, nxt, H, I, 16) == 0
            cur = nxt
        final = u16(H).reshape(1, H)
        assert oracle.rmsnorm_rows(cur.reshape(1, H), tensor("talker.model.norm.weight"), final, 1, H) == 0
        err = np.max(np.abs(oracle.bf16_to_f32(final[0]).astype(np.float64) - oracle.bf16_to_f32(got).astype(np.float64)))
        assert err <= 0.0625, (step, err)          # (the layer step is bit-exact in practice; attention's budget is 1e-2)
        trajectory_gpu += got.tobytes()
        trajectory_cpu += final[0].tobytes()
    if trajectory_gpu == trajectory_cpu:
        assert engine.fnv1a64(trajectory_gpu) == engine.fnv1a64(trajectory_cpu)
    # the caches now hold the four appended rows exactly as the oracle's do
    for layer, (k, v) in enumerate(caches):
        ka, va = talker.cache_addresses(layer)
        kd = np.zeros_like(k)
        assert hip.hipMemcpy(kd.ctypes.data_as(C.c_void_p), C.c_void_p(ka), C.c_size_t(k.nbytes), 2) == 0
        if layer == 0:
            assert np.array_equal(kd, k)           # norm, projection and append are bit-exact operators
        else:
            # deeper layers see the attention of the layers before them (judged to 1e-2, not to the bit)
            assert np.max(np.abs(oracle.bf16_to_f32(kd).astype(np.float64) - oracle.bf16_to_f32(k).astype(np.float64))) <= 0.0625
    # overflow guard (the reference throws "Talker device decode cache overflow")
    with pytest.raises(engine.EngineError) as err:
        talker.decode(xd, cos[0], sin[0], MAX_CACHE - PREFILL)
    assert err.value.code == -3
    talker.close()


@pytest.mark.parametrize("with_bias", [False, True])
def test_engine_decode_in_the_talkers_geometry_takes_one_launch_between_attentions(engine, qm, dev, tmp_path, with_bias):
    """With the talker's real intermediate size (6144) a layer of the decode step is two launches (qm_talker_layer_step_m1;
    three with QM_OPT_TALKER_LAYER_OPERATORS = 2: the attention with its merge, then qm_talker_post_attention_m1); the final
    hidden vectors and the caches equal, bit for bit, what the operator-by-operator step (held against the oracle above) leaves."""
    import ctypes as C
    import torch
    layers = 3
    _checkpoint(str(tmp_path), with_bias, inter=6144, layers=layers)
    hip = C.CDLL("libamdhip64.so")
    results = []
    for by_operators in (1, 0, 2):
        qm.set_option(qm.OPT_TALKER_LAYER_OPERATORS, by_operators)
        try:
            talker = engine.Talker(str(tmp_path), MAX_CACHE)
            assert talker.intermediate == 6144
            talker.reset(PREFILL)
            talker.synchronize()
            g = torch.Generator().manual_seed(5)
            for layer in range(layers):
                ka, va = talker.cache_addresses(layer)
                for address in (ka, va):
                    rows = torch.zeros((8, MAX_CACHE, 128), dtype=torch.bfloat16)
                    rows[:, :PREFILL] = torch.randn((8, PREFILL, 128), generator=g).to(torch.bfloat16)
                    rows = rows.view(torch.int16).numpy()
                    assert hip.hipMemcpy(C.c_void_p(address), rows.ctypes.data_as(C.c_void_p), C.c_size_t(rows.nbytes), 1) == 0
            outputs = []
            for step in range(3):
                x = (torch.randn(H, generator=g)).to(torch.bfloat16).view(torch.int16).to(dev)
                cos, sin = engine.rope_rows(1, PREFILL + step)
                address = talker.decode(x, cos[0], sin[0], step)
                talker.synchronize()
                out = torch.empty(H, dtype=torch.int16, device=dev)
                assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(address), C.c_size_t(H * 2), 3) == 0
                outputs.append(out.cpu())
            for layer in range(layers):
                for address in talker.cache_addresses(layer):
                    rows = np.zeros((8, MAX_CACHE, 128), dtype=np.uint16)
                    assert hip.hipMemcpy(rows.ctypes.data_as(C.c_void_p), C.c_void_p(address), C.c_size_t(rows.nbytes), 2) == 0
                    outputs.append(torch.from_numpy(rows.view(np.int16)))
            talker.close()
            results.append(outputs)
        finally:
            qm.set_option(qm.OPT_TALKER_LAYER_OPERATORS, 0)
    assert len(results[0]) == len(results[1]) == len(results[2]) == 3 + 2 * layers
    assert all(torch.equal(a, b) and torch.equal(a, c) for a, b, c in zip(*results))
    assert len({bytes(o.numpy().tobytes()) for o in results[0][:3]}) == 3          # (three different steps)


def test_engine_rejects_a_checkpoint_with_the_wrong_geometry(engine, dev, tmp_path):
    import torch
    from safetensors.torch import save_file
    bad = {"talker.model.layers.0.input_layernorm.weight": torch.ones(100, dtype=torch.bfloat16)}
    save_file(bad, os.path.join(str(tmp_path), "m.safetensors"))
    with pytest.raises(engine.EngineError) as err:
        engine.Talker(str(tmp_path), 32)
    assert err.value.code == -8


def test_engine_prefill_of_a_long_prompt_shares_query_tiles_between_blocks(engine, oracle, qm, dev, tmp_path):
    """A 650-token prompt: qm_talker_prefill hands the attention a key-split workspace (long query tiles are
    shared by two blocks).  Judged against the same prompt with the uniform-waves prefill kernel chosen, which
    ignores the workspace: layer 0 caches to the bit, last-row hidden vector and deeper caches within the
    budget the oracle chain is given below (two association orders of the same sums)."""
    import ctypes as C
    import torch
    _checkpoint(str(tmp_path), True)
    long_cache, S = 704, 650
    assert qm.prefill_split_workspace_bytes(1, S, 8) > 0
    hip = C.CDLL("libamdhip64.so")
    x = oracle.normal_bf16((S, H), 131)
    cos, sin = engine.rope_rows(S, 0)
    xd = torch.from_numpy(x.view(np.int16)).to(dev)
    runs = {}
    try:
        for choice in (0, 1):
            qm.set_option(qm.OPT_PREFILL_KERNEL, choice)
            talker = engine.Talker(str(tmp_path), long_cache)
            hidden = []
            for _ in range(2):                      # the second prompt finds the workspace as the first left it
                address = talker.prefill(xd, cos, sin, S)
                talker.synchronize()
                out = torch.empty(H, dtype=torch.int16, device=dev)
                assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(address), C.c_size_t(H * 2), 3) == 0
                hidden.append(to_u16(out))
            assert np.array_equal(hidden[0], hidden[1])
            caches = []
            for layer in range(LAYERS):
                ka, va = talker.cache_addresses(layer)
                kd = np.zeros((8, long_cache, 128), dtype=np.uint16)
                vd = np.zeros_like(kd)
                assert hip.hipMemcpy(kd.ctypes.data_as(C.c_void_p), C.c_void_p(ka), C.c_size_t(kd.nbytes), 2) == 0
                assert hip.hipMemcpy(vd.ctypes.data_as(C.c_void_p), C.c_void_p(va), C.c_size_t(vd.nbytes), 2) == 0
                caches.append((kd, vd))
            runs[choice] = (hidden[0], caches)
            del talker
    finally:
        qm.set_option(qm.OPT_PREFILL_KERNEL, 0)

    def gap(a, b):
        return np.max(np.abs(oracle.bf16_to_f32(a).astype(np.float64) - oracle.bf16_to_f32(b).astype(np.float64)))

    assert gap(runs[0][0], runs[1][0]) <= 0.0625
    for layer in range(LAYERS):
        for a, b in zip(runs[0][1][layer], runs[1][1][layer]):
            assert not a[:, S:].any()
            if layer == 0:
                assert np.array_equal(a, b)
            else:
                assert gap(a, b) <= 0.0625


@pytest.mark.parametrize("rows_kernel", [1, 0], ids=["exact_chain_linears", "matrix_core_linears"])
def test_engine_prefill_then_decode_matches_the_oracle_chain(engine, oracle, qm, dev, tmp_path, rows_kernel):
    """A 37-token prompt through qm_talker_prefill, then two decoded tokens: last-row hidden vectors,
    and the caches the prompt leaves behind, against the oracle's chain of the same operators.  With the prompt's
    linears on the exact chain (QM_OPT_LINEAR_ROWS_KERNEL = 1) layer 0's K/V are the oracle's to the bit; on the matrix
    cores (default) a projection may land on the neighbouring bf16 value, so they are held to the attention budget."""
    qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, rows_kernel)
    try:
        _prefill_then_decode(engine, oracle, qm, dev, tmp_path, rows_kernel == 1)
    finally:
        qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, 0)


def _prefill_then_decode(engine, oracle, qm, dev, tmp_path, exact):
    import ctypes as C
    import torch
    w = _checkpoint(str(tmp_path), True)
    talker = engine.Talker(str(tmp_path), MAX_CACHE)
    hip = C.CDLL("libamdhip64.so")
    S = 37
    x = oracle.normal_bf16((S, H), 31)
    cos, sin = engine.rope_rows(S + 2, 0)
    xd = torch.from_numpy(x.view(np.int16)).to(dev)
    address = talker.prefill(xd, cos[:S], sin[:S], S)
    talker.synchronize()
    out = torch.empty(H, dtype=torch.int16, device=dev)
    assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(address), C.c_size_t(H * 2), 3) == 0
    got = to_u16(out)

    u16 = lambda *shape: np.zeros(shape, dtype=np.uint16)
    caches = [(u16(8, MAX_CACHE, 128), u16(8, MAX_CACHE, 128)) for _ in range(LAYERS)]
    cur = x.copy()
    for layer in range(LAYERS):
        p = f"talker.model.layers.{layer}."
        k_cache, v_cache = caches[layer]
        cache = oracle.flat_cache(k_cache, v_cache, 8, MAX_CACHE)
        norm, q, k, v, qrot, krot, ctxv, res, post, act, nxt = (u16(S, H), u16(S, Q), u16(S, KV), u16(S, KV), u16(S, Q),
                                                               u16(S, KV), u16(S, Q), u16(S, H), u16(S, H), u16(S, I),
                                                               u16(S, H))
        assert oracle.rmsnorm_rows(cur, w[p + "input_layernorm.weight"], norm, S, H) == 0
        for name, dst, n in (("q", q, Q), ("k", k, KV), ("v", v, KV)):
            assert oracle.linear_rows(norm, w[p + f"self_attn.{name}_proj.weight"], w[p + f"self_attn.{name}_proj.bias"],
                                      None, dst, S, n, H, 16) == 0
        assert oracle.norm_rope_rows(q, w[p + "self_attn.q_norm.weight"], cos[:S], sin[:S], qrot, S, 16) == 0
        assert oracle.norm_rope_rows(k, w[p + "self_attn.k_norm.weight"], cos[:S], sin[:S], krot, S, 8) == 0
        assert oracle.prefill_attention_causal(qrot, krot, v, ctxv, cache, None, 1, 1, S, 16, 8, SCALE,
                                               oracle.POLICY_ONLINE, 16) == 0
        assert oracle.linear_rows(ctxv, w[p + "self_attn.o_proj.weight"], w[p + "self_attn.o_proj.bias"], cur, res, S, H,
                                  Q, 16) == 0
        assert oracle.rmsnorm_rows(res, w[p + "post_attention_layernorm.weight"], post, S, H) == 0
        assert oracle.gate_up_swiglu_rows(post, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], act, S, H, I,
                                          16) == 0
        assert oracle.linear_rows(act, w[p + "mlp.down_proj.weight"], None, res, nxt, S, H, I, 16) == 0
        cur = nxt
    final = u16(1, H)
    assert oracle.rmsnorm_rows(cur[S - 1:S], w["talker.model.norm.weight"], final, 1, H) == 0
    err = np.max(np.abs(oracle.bf16_to_f32(final[0]).astype(np.float64) - oracle.bf16_to_f32(got).astype(np.float64)))
    assert err <= 0.0625, err
    # the prompt's K/V in the caches: layer 0 to the bit, deeper layers within the attention budget
    for layer, (k_cache, v_cache) in enumerate(caches):
        ka, va = talker.cache_addresses(layer)
        kd, vd = np.zeros_like(k_cache), np.zeros_like(v_cache)
        assert hip.hipMemcpy(kd.ctypes.data_as(C.c_void_p), C.c_void_p(ka), C.c_size_t(kd.nbytes), 2) == 0
        assert hip.hipMemcpy(vd.ctypes.data_as(C.c_void_p), C.c_void_p(va), C.c_size_t(vd.nbytes), 2) == 0
        assert not kd[:, S:].any() and not vd[:, S:].any()
        if layer == 0 and exact:
            assert np.array_equal(kd, k_cache) and np.array_equal(vd, v_cache)
        else:
            for a, b in ((kd, k_cache), (vd, v_cache)):
                assert np.max(np.abs(oracle.bf16_to_f32(a).astype(np.float64) - oracle.bf16_to_f32(b).astype(np.float64))) <= 0.0625
    # decoding continues at position S over those caches
    for step in range(2):
        token = oracle.normal_bf16((H,), 77 + step)
        td = torch.from_numpy(token.view(np.int16)).to(dev)
        address = talker.decode(td, cos[S + step], sin[S + step], step)
        talker.synchronize()
        assert hip.hipMemcpy(C.c_void_p(out.data_ptr()), C.c_void_p(address), C.c_size_t(H * 2), 3) == 0
        got = to_u16(out)
        cur1 = token.copy()
        for layer in range(LAYERS):
            p = f"talker.model.layers.{layer}."
            cache = oracle.flat_cache(caches[layer][0], caches[layer][1], 8, MAX_CACHE)
            norm, q, k, v, qrot, ctxv, attn, res, post, act, nxt = (u16(1, H), u16(Q), u16(KV), u16(KV), u16(Q), u16(Q),
                                                                    u16(H), u16(H), u16(H), u16(I), u16(H))
            assert oracle.rmsnorm_rows(cur1.reshape(1, H), w[p + "input_layernorm.weight"], norm, 1, H) == 0
            assert oracle.qkv_m1(norm[0], w[p + "self_attn.q_proj.weight"], w[p + "self_attn.q_proj.bias"],
                                 w[p + "self_attn.k_proj.weight"], w[p + "self_attn.k_proj.bias"],
                                 w[p + "self_attn.v_proj.weight"], w[p + "self_attn.v_proj.bias"], q, k, v, H, Q, KV, 16) == 0
            assert oracle.qk_norm_rope_kv_append(q, k, v, w[p + "self_attn.q_norm.weight"], w[p + "self_attn.k_norm.weight"],
                                                 cos[S + step], sin[S + step], qrot, cache, None, 1, 16, S + step) == 0
            assert oracle.attention(qrot, cache, None, 1, ctxv, 1, S + step, 16, -1, SCALE, oracle.POLICY_ONLINE, 16) == 0
            assert oracle.linear_m1(ctxv, w[p + "self_attn.o_proj.weight"], w[p + "self_attn.o_proj.bias"], None, attn, H,
                                    Q, 16) == 0
            assert oracle.add_postnorm_m1(cur1, attn, w[p + "post_attention_layernorm.weight"], res, post, H) == 0
            assert oracle.gate_up_swiglu_m1(post, w[p + "mlp.gate_proj.weight"], w[p + "mlp.up_proj.weight"], act, H, I,
                                            16) == 0
            assert oracle.linear_m1(act, w[p + "mlp.down_proj.weight"], None, res, nxt, H, I, 16) == 0
            cur1 = nxt
        assert oracle.rmsnorm_rows(cur1.reshape(1, H), w["talker.model.norm.weight"], final, 1, H) == 0
        err = np.max(np.abs(oracle.bf16_to_f32(final[0]).astype(np.float64) - oracle.bf16_to_f32(got).astype(np.float64)))
        assert err <= 0.0625, (step, err)
    with pytest.raises(engine.EngineError) as e:
        talker.prefill(xd, cos[:S], sin[:S], MAX_CACHE + 1)
    assert e.value.code == -3
    talker.close()
