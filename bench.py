#!/usr/bin/env python3
"""Benchmark of the attention / KV-cache hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--headline-only] [--all] [--rows TEXT] [--only NAME [--layers N]]

A step is one pass of the hot path over one batch of synthetic input that is already resident
in HBM.  The headline workload is the ragged multi-stream decode (64 streams, context lengths
uniform in [256, 4096], 16-token pages behind a shuffled page table): the one decode
configuration whose working set (~0.57 GB) exceeds the caches, so that "HBM GB/s" means HBM.
The other four configurations and the four widened rows that make up a generated frame are timed too;
`--all` adds every variant row, `--rows TEXT` times exactly the rows whose name contains TEXT, `--only NAME` times one row
alone (for a profiler).  The full record of
every row goes to stdout on a line that starts with `per_config ` and to the file PER_CONFIG_FILE names;
the LAST stdout line is one compact JSON object (metric, value, roofline, cpu_baseline and a
`summary` of {row: [us per step, fraction of the bounding peak]}), short enough to survive a tail.

Inputs come from the seeded SplitMix64 -> Box-Muller stream that the parity tests use (class Synthetic,
evaluated on the device); the CPU baseline leg copies the same tensors to the host and times the
scalar oracle (oracle/, test infrastructure) on them, and also checks the GPU result against it.
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

# HBM bytes per launch of decode_split_kernel<2, false, true, false> on the headline workload, from rocprofv3 --pmc
# FETCH_SIZE and WRITE_SIZE (KiB per dispatch), each scaled by what the same counter reads for a
# plain 512 MiB copy (FETCH_SIZE reads half the copied bytes: factor 2.0; WRITE_SIZE: 1.0).
# Summary and commands: profiles/decode_split_kernel_ragged64_traffic.txt
HEADLINE_TRAFFIC_BYTES = int((289789.3 * 2.0 + 3317.0 * 1.0) * 1024)

HBM_PEAK_GBPS = 8000.0          # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
SCALE = 0.08838834764831845


_GOLDEN = 0x9E3779B97F4A7C15
_MIX_A = 0xBF58476D1CE4E5B9
_MIX_B = 0x94D049BB133111EB
_MASK64 = (1 << 64) - 1


def _signed64(x):
    x &= _MASK64
    return x - (1 << 64) if x >> 63 else x


def _splitmix_at(seed, k):
    """k-th output (k >= 1) of the SplitMix64 stream seeded with `seed` (Python integers)."""
    z = (seed + k * _GOLDEN) & _MASK64
    z = ((z ^ (z >> 30)) * _MIX_A) & _MASK64
    z = ((z ^ (z >> 27)) * _MIX_B) & _MASK64
    return z ^ (z >> 31)


class Synthetic:
    """The seeded inputs of every workload: SplitMix64 -> Box-Muller, element i of a tensor from stream
    outputs 2i+1 and 2i+2 of that tensor's seed (the generator the parity tests draw from, evaluated here
    on the device in int64 / float64), and integer draws / Fisher-Yates permutations from the same stream
    on the host.  Each tensor drawn from one Synthetic takes the next seed."""

    def __init__(self, dev, seed):
        self.dev, self.seed = dev, seed

    def _next_seed(self):
        self.seed += 1
        return self.seed

    @staticmethod
    def _lsr(z, n):
        return (z >> n) & ((1 << (64 - n)) - 1)

    def _mix(self, seed, k):
        z = k * _signed64(_GOLDEN) + _signed64(seed)
        z = (z ^ self._lsr(z, 30)) * _signed64(_MIX_A)
        z = (z ^ self._lsr(z, 27)) * _signed64(_MIX_B)
        return z ^ self._lsr(z, 31)

    def normal(self, shape, std=1.0, mean=0.0):
        import torch
        seed = self._next_seed()
        n = int(np.prod(shape))
        out = torch.empty(n, dtype=torch.bfloat16, device=self.dev)
        std64, mean64 = float(np.float32(std)), float(np.float32(mean))
        chunk = 1 << 24
        for lo in range(0, n, chunk):
            i = torch.arange(lo, min(n, lo + chunk), dtype=torch.int64, device=self.dev)
            a, b = self._mix(seed, 2 * i + 1), self._mix(seed, 2 * i + 2)
            u1 = (self._lsr(a, 11).double() + 1.0) * (1.0 / 9007199254740992.0)
            u2 = self._lsr(b, 11).double() * (1.0 / 9007199254740992.0)
            z = torch.sqrt(-2.0 * torch.log(u1)) * torch.cos(6.283185307179586477 * u2)
            out[lo:lo + chunk] = (mean64 + std64 * z).float().to(torch.bfloat16)
        return out.view(shape)

    def integers(self, n, lo, hi):
        """n integers uniform in [lo, hi] (host, int32)."""
        seed = self._next_seed()
        return np.array([lo + _splitmix_at(seed, i + 1) % (hi - lo + 1) for i in range(n)], dtype=np.int32)

    def permutation(self, n):
        """Seeded Fisher-Yates permutation of 0..n-1 (host, int32)."""
        seed = self._next_seed()
        out = list(range(n))
        for i in range(n - 1, 0, -1):
            j = _splitmix_at(seed, n - i) % (i + 1)
            out[i], out[j] = out[j], out[i]
        return np.array(out, dtype=np.int32)


def _bits(t):
    """bf16 tensor -> numpy uint16 bit patterns (host)."""
    import torch
    return t.detach().view(torch.int16).cpu().numpy().view(np.uint16)


def _time_steps(fn, steps, warmup):
    """Average milliseconds per call over `steps` back-to-back calls on torch's current stream
    (the stream handed to the library), bracketed by device synchronisation."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def _time_graph(fn, reps=20, replays=20):
    """Average milliseconds per step when `reps` steps are captured into one HIP graph and the graph is
    replayed `replays` times: device-side time without per-launch host overhead (the reference runs its
    predictor loop as a HIP graph for the same reason, R17:13856-13896)."""
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
        for _ in range(reps):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / (reps * replays)


class RaggedDecode:
    """configs[2]: 64 streams, L ~ U{256..4096}, paged KV, split-K decode attention."""
    name = "ragged_decode_64x[256,4096]_paged16"
    bound = "hbm"

    def __init__(self, qm, dev, seed=2024, n_streams=64, lo=256, hi=4096):
        import torch
        syn = Synthetic(dev, seed)
        self.qm, self.dev, self.n = qm, dev, n_streams
        self.lens = torch.from_numpy(syn.integers(n_streams, lo, hi))
        pages_per = (self.lens + 15) // 16
        self.max_pages = int(pages_per.max())
        self.n_pages = int(pages_per.sum()) + 7
        perm = torch.from_numpy(syn.permutation(self.n_pages))
        table = torch.full((n_streams, self.max_pages), -1, dtype=torch.int32)
        cur = 0
        for s in range(n_streams):
            k = int(pages_per[s])
            table[s, :k] = perm[cur:cur + k]
            cur += k
        shape = (self.n_pages, 8, 16, 128)
        self.k, self.v, self.q = syn.normal(shape), syn.normal(shape), syn.normal((n_streams, 16, 128))
        self.out = torch.zeros_like(self.q)
        self.table = table.to(dev)
        self.lens_d = self.lens.to(dev)
        self.max_len = int(self.lens.max())
        self.ws_bytes = qm.decode_workspace_bytes(n_streams, 16, 8, self.max_len)
        self.ws = torch.empty(self.ws_bytes // 4 + 1, dtype=torch.float32, device=dev)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)
        self.cache = qm.paged_cache(self.k, self.v, self.n_pages)
        total = int(self.lens.sum())
        # K+V of every context token, q + out, page table entries actually used
        self.bytes = 4096 * total + n_streams * 8192 + 4 * int(pages_per.sum())
        self.flops = 8192 * total
        self.tokens = total

    def step(self):
        import torch
        self.qm.decode_attention_ragged(self.q, self.cache, self.table, self.max_pages, self.lens_d, self.n,
                                        self.max_len, self.out, 16, SCALE, self.ws, self.ws_bytes, self.status,
                                        torch.cuda.current_stream().cuda_stream)

    def cpu_baseline(self, oracle, threads):
        k, v, q = _bits(self.k), _bits(self.v), _bits(self.q)
        table = self.table.cpu().numpy()
        lens = self.lens.numpy()
        cache = oracle.paged_cache(k, v)
        out = np.zeros_like(q)
        res = {}
        for label, th in (("single", 1), ("all", threads)):
            t0 = time.perf_counter()
            rc = oracle.decode_attention_ragged(q, cache, table, self.max_pages, lens, out, 16, SCALE,
                                                oracle.POLICY_ONLINE, th)
            res[label] = time.perf_counter() - t0
            assert rc == 0
        err = float(np.max(np.abs(oracle.bf16_to_f32(out).astype(np.float64)
                                  - oracle.bf16_to_f32(_bits(self.out)).astype(np.float64))))
        return res, err, "whole workload (all 64 streams)"


class SingleDecode:
    """configs[0] / configs[1]: batch-1 decode over a flat [8][max_cache][128] cache; configs[1]
    also runs the fused norm + RoPE + append at the last position first."""
    bound = "hbm"

    def __init__(self, qm, dev, ctx, fused_append, seed, copies=1, one_launch=True):
        import torch
        self.qm, self.dev, self.ctx, self.fused = qm, dev, ctx, fused_append
        self.one_launch = one_launch     # append folded into the attention launch (qm_decode_step_fused)
        self.name = ("talker_fused_step_ctx%d" if fused_append else "gqa_decode_ctx%d") % ctx
        if fused_append and not one_launch:
            self.name += "_append_and_decode_launches"
        syn = Synthetic(dev, seed)
        self.max_cache = ctx + 4
        self.copies = copies

        rnd = syn.normal

        self.k = [rnd((8, self.max_cache, 128)) for _ in range(copies)]
        self.v = [rnd((8, self.max_cache, 128)) for _ in range(copies)]
        self.caches = [qm.flat_cache(k, v, 8, self.max_cache) for k, v in zip(self.k, self.v)]
        self.q = rnd((16, 128))
        self.out = torch.zeros_like(self.q)
        if fused_append:
            # hidden 2048 -> Q [16,128], K/V [8,128] with N(0, 0.02) hidden and weights: the
            # projection is outside the judged region and done once here with torch.
            hidden = rnd((2048,), 0.02).float()
            wq, wk, wv = rnd((2048, 2048), 0.02).float(), rnd((1024, 2048), 0.02).float(), rnd((1024, 2048), 0.02).float()
            self.q_lin = (wq @ hidden).to(torch.bfloat16).view(16, 128).contiguous()
            self.k_lin = (wk @ hidden).to(torch.bfloat16).view(8, 128).contiguous()
            self.v_lin = (wv @ hidden).to(torch.bfloat16).view(8, 128).contiguous()
            self.gq, self.gk = rnd((128,), 0.1, 1.0), rnd((128,), 0.1, 1.0)
            pos = ctx - 1
            inv = 1.0e6 ** (-2.0 * np.arange(64, dtype=np.float64) / 128.0)
            ang = np.concatenate([pos * inv, pos * inv])
            self.cos = torch.tensor(np.cos(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
            self.sin = torch.tensor(np.sin(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        self.ws_bytes = qm.decode_workspace_bytes(1, 16, 8, ctx)
        self.ws = torch.empty(self.ws_bytes // 4 + 1, dtype=torch.float32, device=dev)
        self.bytes = 2 * 8 * ctx * 128 * 2 + 4096 + 4096
        if fused_append:
            self.bytes = 2 * 8 * ctx * 128 * 2 + 4096 + 8192 + 1024 + 4096
        self.flops = 16 * ctx * 128 * 2 * 2
        self.i = 0

    def step(self):
        import torch
        s = torch.cuda.current_stream().cuda_stream
        c = self.caches[self.i % self.copies]
        self.i += 1
        q = self.q
        if self.fused and self.one_launch:
            self.qm.decode_step_fused(self.q_lin, self.k_lin, self.v_lin, self.gq, self.gk, self.cos, self.sin, self.q,
                                      c, None, 1, self.out, 16, self.ctx - 1, -1, SCALE, 1e-6, self.ws, self.ws_bytes,
                                      None, s)
            return
        if self.fused:
            self.qm.qk_norm_rope_kv_append(self.q_lin, self.k_lin, self.v_lin, self.gq, self.gk, self.cos, self.sin,
                                           self.q, c, None, 1, 16, self.ctx - 1, 1e-6, s)
        self.qm.decode_attention(q, c, None, 1, self.out, 16, self.ctx - 1, -1, SCALE, self.ws, self.ws_bytes, s)

    def cpu_baseline(self, oracle, threads):
        self.i = 0
        self.step()
        import torch
        torch.cuda.synchronize()
        k, v = _bits(self.k[0]).copy(), _bits(self.v[0]).copy()
        cache = oracle.flat_cache(k, v, 8, self.max_cache)
        q = _bits(self.q).copy()
        out = np.zeros_like(q)
        res = {}
        for label, th in (("single", 1), ("all", threads)):
            t0 = time.perf_counter()
            if self.fused:
                rc = oracle.qk_norm_rope_kv_append(_bits(self.q_lin), _bits(self.k_lin), _bits(self.v_lin),
                                                   _bits(self.gq), _bits(self.gk), _bits(self.cos), _bits(self.sin),
                                                   q, cache, None, 1, 16, self.ctx - 1)
                assert rc == 0
            rc = oracle.attention(q, cache, None, 1, out, 1, self.ctx - 1, 16, -1, SCALE, oracle.POLICY_ONLINE, th)
            res[label] = time.perf_counter() - t0
            assert rc == 0
        err = float(np.max(np.abs(oracle.bf16_to_f32(out).astype(np.float64)
                                  - oracle.bf16_to_f32(_bits(self.out)).astype(np.float64))))
        return res, err, "whole workload"


class QkvGemv:
    """The next row after the attention path: the fused M = 1 Q/K/V projection that feeds the
    norm + RoPE + append (hidden 2048 -> q 2048, k 1024, v 1024).  `copies` weight sets are used in
    rotation (64 sets = 1 GB, as the layers of a real decode step never find their weights cached)."""
    bound = "hbm"

    def __init__(self, qm, dev, seed=77, copies=1):
        import torch
        self.qm, self.copies = qm, copies
        self.name = "qkv_gemv_m1_hidden2048" + ("_rotating%d" % copies if copies > 1 else "")
        syn = Synthetic(dev, seed)

        rnd = syn.normal

        self.x = rnd((2048,))
        self.w = [(rnd((2048, 2048), 0.02), rnd((1024, 2048), 0.02), rnd((1024, 2048), 0.02)) for _ in range(copies)]
        self.b = (rnd((2048,), 0.1), rnd((1024,), 0.1), rnd((1024,), 0.1))
        self.q = torch.zeros(2048, dtype=torch.bfloat16, device=dev)
        self.k = torch.zeros(1024, dtype=torch.bfloat16, device=dev)
        self.v = torch.zeros(1024, dtype=torch.bfloat16, device=dev)
        self.bytes = 2 * 4096 * 2048 + 2 * 2048 + 2 * 4096 + 2 * 4096     # weights, input, biases, outputs
        self.flops = 2 * 4096 * 2048
        self.i = 0

    def step(self):
        import torch
        w = self.w[self.i % self.copies]
        self.i += 1
        self.qm.qkv_m1(self.x, w[0], self.b[0], w[1], self.b[1], w[2], self.b[2], self.q, self.k, self.v,
                       2048, 2048, 1024, torch.cuda.current_stream().cuda_stream)

    def cpu_baseline(self, oracle, threads):
        import torch
        self.i = 0
        self.step()
        torch.cuda.synchronize()
        w = [_bits(t).copy() for t in self.w[0]]
        b = [_bits(t).copy() for t in self.b]
        outs = [np.zeros(n, dtype=np.uint16) for n in (2048, 1024, 1024)]
        t0 = time.perf_counter()
        rc = oracle.qkv_m1(_bits(self.x).copy(), w[0], b[0], w[1], b[1], w[2], b[2], outs[0], outs[1], outs[2],
                           2048, 2048, 1024, threads)
        dt = time.perf_counter() - t0
        assert rc == 0
        exact = all(np.array_equal(o, _bits(t)) for o, t in zip(outs, (self.q, self.k, self.v)))
        return {"all": dt}, 0.0 if exact else 1.0, "whole workload (bit-exact comparison)"


class TalkerLayerStep:
    """Beyond the five configurations: one whole decode step of a talker layer as the reference chains
    it (R17:17155-17248) — RMSNorm, fused Q/K/V projection, QK-norm + RoPE + append, GQA decode over a
    2048-token flat cache, o_proj, residual add + post-norm, gate/up/SwiGLU, down_proj + residual —
    with `layers` distinct weight sets and caches used in rotation (hidden 2048, intermediate 6144 as
    in Qwen3-1.7B; the reference reads it from the checkpoint, R17:14862)."""
    bound = "hbm"
    # the layer's output is a hidden state of magnitude up to ~8, where one bf16 ulp is 0.03-0.06: the
    # attention's 1e-2 budget surfaces as at most a couple of ulps there
    tolerance = 0.125

    def __init__(self, qm, dev, layers=28, ctx=2048, seed=91, fused=True, chained=False, two_launches=False):
        import torch
        chained = chained or two_launches
        self.qm, self.layers, self.ctx, self.fused, self.chained, self.two_launches = qm, layers, ctx, fused, chained, two_launches
        self.name = "talker_layer_decode_step_ctx%d_x%dlayers%s" % (
            ctx, layers, "_two_launches" if two_launches else "_one_launch_between_attentions" if chained else
            "" if fused else "_reference_launch_sequence")
        self.copies = layers
        syn = Synthetic(dev, seed)
        H, I = 2048, 6144
        self.H, self.I = H, I

        rnd = syn.normal

        self.max_cache = ctx + 4
        self.w = []
        for _ in range(layers):
            k, v = rnd((8, self.max_cache, 128)), rnd((8, self.max_cache, 128))
            self.w.append(dict(
                in_norm=rnd((H,), 0.1, 1.0), wq=rnd((H, H), 0.02), wk=rnd((1024, H), 0.02), wv=rnd((1024, H), 0.02),
                gq=rnd((128,), 0.1, 1.0), gk=rnd((128,), 0.1, 1.0), wo=rnd((H, H), 0.02), post=rnd((H,), 0.1, 1.0),
                wg=rnd((I, H), 0.02), wu=rnd((I, H), 0.02), wd=rnd((H, I), 0.02), k=k, v=v,
                cache=qm.flat_cache(k, v, 8, self.max_cache)))
        pos = ctx - 1
        inv = 1.0e6 ** (-2.0 * np.arange(64, dtype=np.float64) / 128.0)
        ang = np.concatenate([pos * inv, pos * inv])
        self.cos = torch.tensor(np.cos(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        self.sin = torch.tensor(np.sin(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        z = lambda n: torch.zeros(n, dtype=torch.bfloat16, device=dev)
        self.x = rnd((H,))
        self.norm, self.q, self.k_, self.v_, self.qrot = z(H), z(H), z(1024), z(1024), z(H)
        self.ctxv, self.attn, self.res, self.post, self.act, self.out = z(H), z(H), z(H), z(H), z(I), z(H)
        self.ws_bytes = qm.decode_workspace_bytes(1, 16, 8, ctx)
        self.ws = torch.empty(self.ws_bytes // 4 + 1, dtype=torch.float32, device=dev)
        weights = 2 * (H * H + 2 * 1024 * H + H * H + 2 * I * H + H * I)
        self.bytes = weights + 2 * 8 * ctx * 128 * 2 + 4096 + 2 * (6 * H + 2 * I)   # + KV + append + activations
        self.flops = weights + 16 * ctx * 128 * 2 * 2
        self.i = 0
        if chained:
            # o_proj ... down_proj of a layer and the Q/K/V of the layer after it are one launch
            # (qm_talker_post_attention_m1): a step is the attention of layer i and that launch
            self.chain_ws_bytes = qm.talker_post_attention_workspace_bytes()
            self.chain_ws = torch.zeros(self.chain_ws_bytes // 4, dtype=torch.int32, device=dev)
            qm.talker_post_attention_workspace_init(self.chain_ws, self.chain_ws_bytes)
            self.status = torch.zeros(1, dtype=torch.int32, device=dev)
            self.ops = []
            for i, L in enumerate(self.w):
                N = self.w[(i + 1) % layers]
                self.ops.append(qm.talker_post_attention(
                    context=self.ctxv, hidden=self.x, o_weight=L["wo"], post_norm=L["post"], gate_weight=L["wg"], up_weight=L["wu"],
                    down_weight=L["wd"], hidden_out=self.out, next_input_norm=N["in_norm"], next_q_weight=N["wq"],
                    next_k_weight=N["wk"], next_v_weight=N["wv"], q_out=self.q, k_out=self.k_, v_out=self.v_))
            # ... and with the attention's merge folded into that launch a layer is two launches (qm_talker_layer_step_m1)
            self.steps = [qm.talker_layer_step(self.q, self.k_, self.v_, L["gq"], L["gk"], self.cos, self.sin, self.qrot, L["cache"],
                                               None, 1, self.ctxv, 16, ctx - 1, -1, SCALE, 1e-6, self.ws, self.ws_bytes, op)
                          for L, op in zip(self.w, self.ops)] if two_launches else None
            self.primed = False

    def step(self):
        import torch
        s = torch.cuda.current_stream().cuda_stream
        L = self.w[self.i % self.layers]
        qm, H, I = self.qm, self.H, self.I
        if self.chained:
            if not self.primed:       # the first layer's Q/K/V (later ones come out of the launch before)
                qm.rmsnorm_qkv_m1(self.x, L["in_norm"], L["wq"], None, L["wk"], None, L["wv"], None, self.q, self.k_,
                                  self.v_, H, H, 1024, 1e-6, s)
                self.primed = True
            if self.two_launches:
                qm.talker_layer_step_m1(self.steps[self.i % self.layers], self.chain_ws, self.chain_ws_bytes, self.status, s)
                self.i += 1
                return
            qm.decode_step_fused(self.q, self.k_, self.v_, L["gq"], L["gk"], self.cos, self.sin, self.qrot, L["cache"],
                                 None, 1, self.ctxv, 16, self.ctx - 1, -1, SCALE, 1e-6, self.ws, self.ws_bytes, None, s)
            qm.talker_post_attention_m1(self.ops[self.i % self.layers], self.chain_ws, self.chain_ws_bytes, self.status, s)
            self.i += 1
            return
        self.i += 1
        if self.fused:
            qm.rmsnorm_qkv_m1(self.x, L["in_norm"], L["wq"], None, L["wk"], None, L["wv"], None, self.q, self.k_,
                              self.v_, H, H, 1024, 1e-6, s)
        else:
            qm.rmsnorm_rows(self.x, L["in_norm"], self.norm, 1, H, 1e-6, s)
            qm.qkv_m1(self.norm, L["wq"], None, L["wk"], None, L["wv"], None, self.q, self.k_, self.v_, H, H, 1024, s)
        if self.fused:
            qm.decode_step_fused(self.q, self.k_, self.v_, L["gq"], L["gk"], self.cos, self.sin, self.qrot, L["cache"],
                                 None, 1, self.ctxv, 16, self.ctx - 1, -1, SCALE, 1e-6, self.ws, self.ws_bytes, None, s)
        else:
            qm.qk_norm_rope_kv_append(self.q, self.k_, self.v_, L["gq"], L["gk"], self.cos, self.sin, self.qrot,
                                      L["cache"], None, 1, 16, self.ctx - 1, 1e-6, s)
            qm.decode_attention(self.qrot, L["cache"], None, 1, self.ctxv, 16, self.ctx - 1, -1, SCALE, self.ws,
                                self.ws_bytes, s)
        qm.linear_m1(self.ctxv, L["wo"], None, None, self.attn, H, H, s)
        if self.fused:
            qm.add_postnorm_gate_up_swiglu_m1(self.x, self.attn, L["post"], self.res, L["wg"], L["wu"], self.act, H, I,
                                              1e-6, s)
        else:
            qm.add_postnorm_m1(self.x, self.attn, L["post"], self.res, self.post, H, 1e-6, s)
            qm.gate_up_swiglu_m1(self.post, L["wg"], L["wu"], self.act, H, I, s)
        qm.linear_m1(self.act, L["wd"], None, self.res, self.out, H, I, s)

    def cpu_baseline(self, oracle, threads):
        """One layer on the host; the comparison is on that layer's output hidden state."""
        import torch
        self.i = 0
        self.primed = False
        self.step()
        torch.cuda.synchronize()
        if self.chained:
            assert int(self.status.item()) == 0
        L = {k: (_bits(v).copy() if hasattr(v, "detach") else v) for k, v in self.w[0].items()}
        H, I = self.H, self.I
        x = _bits(self.x).copy()
        u16 = lambda n: np.zeros(n, dtype=np.uint16)
        norm, q, k, v, qrot, ctxv, attn, res, post, act, out = (u16(H).reshape(1, H), u16(H), u16(1024), u16(1024),
                                                                u16(H), u16(H), u16(H), u16(H), u16(H), u16(I), u16(H))
        # the GPU step already appended position ctx-1 to layer 0's cache: the oracle overwrites it with the same bits
        cache = oracle.flat_cache(L["k"], L["v"], 8, self.max_cache)
        t0 = time.perf_counter()
        assert oracle.rmsnorm_rows(x.reshape(1, H), L["in_norm"], norm, 1, H) == 0
        assert oracle.qkv_m1(norm[0], L["wq"], None, L["wk"], None, L["wv"], None, q, k, v, H, H, 1024, threads) == 0
        assert oracle.qk_norm_rope_kv_append(q, k, v, L["gq"], L["gk"], _bits(self.cos), _bits(self.sin), qrot, cache,
                                             None, 1, 16, self.ctx - 1) == 0
        assert oracle.attention(qrot, cache, None, 1, ctxv, 1, self.ctx - 1, 16, -1, SCALE, oracle.POLICY_ONLINE,
                                threads) == 0
        assert oracle.linear_m1(ctxv, L["wo"], None, None, attn, H, H, threads) == 0
        assert oracle.add_postnorm_m1(x, attn, L["post"], res, post, H) == 0
        assert oracle.gate_up_swiglu_m1(post, L["wg"], L["wu"], act, H, I, threads) == 0
        assert oracle.linear_m1(act, L["wd"], None, res, out, H, I, threads) == 0
        dt = time.perf_counter() - t0
        err = float(np.max(np.abs(oracle.bf16_to_f32(out).astype(np.float64)
                                  - oracle.bf16_to_f32(_bits(self.out)).astype(np.float64))))
        return {"all": dt}, err, "one layer step"


class PromptLinears:
    """Beyond the five configurations: the seven linears of one talker layer over a prompt of `rows` tokens as the
    prompt pass chains them (NativeTalkerEngine::prefill, R17:16646-16790): q, k, v projections with bias (one call), o_proj +
    residual, gate/up/SwiGLU, down_proj + residual (hidden 2048, intermediate 6144).  kernel 0: the matrix cores
    (default); 1: every sum in the reference's order (QM_OPT_LINEAR_ROWS_KERNEL)."""
    bound = "mfma"

    def __init__(self, qm, dev, rows=1024, kernel=0, seed=313, split=False, copies=1):
        import torch
        self.qm, self.rows, self.kernel, self.split = qm, rows, kernel, split
        self.name = "prompt_linears_%d_tokens_one_talker_layer%s%s" % (rows, "_exact_chain" if kernel else "",
                                                                      "_reductions_shared_between_blocks" if split else "")
        syn = Synthetic(dev, seed)
        H, KV, I = 2048, 1024, 6144
        self.H, self.KV, self.I = H, KV, I
        rnd = syn.normal
        self.x, self.res = rnd((rows, H)), rnd((rows, H))
        self.wq, self.wk, self.wv, self.wo = rnd((H, H), 0.02), rnd((KV, H), 0.02), rnd((KV, H), 0.02), rnd((H, H), 0.02)
        self.bq, self.bk, self.bv = rnd((H,), 0.1), rnd((KV,), 0.1), rnd((KV,), 0.1)
        self.wg, self.wu, self.wd = rnd((I, H), 0.02), rnd((I, H), 0.02), rnd((H, I), 0.02)
        z = lambda n: torch.zeros((rows, n), dtype=torch.bfloat16, device=dev)
        self.q, self.k, self.v, self.o, self.act, self.out = z(H), z(KV), z(KV), z(H), z(I), z(H)
        self.flops = 2 * rows * (H * H + 2 * KV * H + H * H + 2 * I * H + H * I)
        self.bytes = 2 * (H * H + 2 * KV * H + H * H + 2 * I * H + H * I) + 2 * rows * (6 * H + 2 * KV + 2 * I)
        # outputs of magnitude 1 to 4: one bf16 spacing there
        self.tolerance = 0.0625
        # short prompts: a workspace lets the linears cut their reductions (qm_linear_rows_split)
        self.ws_bytes = max(qm.linear_rows_split_workspace_bytes(rows, c, r, p) for c, r, p in
                            ((H, H, False), (KV, H, False), (I, H, True), (H, I, False))) if split else 0
        self.ws = torch.empty(max(self.ws_bytes, 256) // 4, dtype=torch.float32, device=dev)

    def step(self):
        import torch
        qm, s, R, H, KV, I = self.qm, torch.cuda.current_stream().cuda_stream, self.rows, self.H, self.KV, self.I
        qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, self.kernel)
        try:
            if self.split:
                ws, nb = self.ws, self.ws_bytes
                qm.qkv_rows(self.x, (self.wq, self.wk, self.wv), (self.bq, self.bk, self.bv), (self.q, self.k, self.v), R, H, KV, H,
                            ws, nb, s)
                qm.linear_rows_split(self.q, self.wo, None, self.res, self.o, R, H, H, ws, nb, s)
                qm.gate_up_swiglu_rows_split(self.o, self.wg, self.wu, self.act, R, H, I, ws, nb, s)
                qm.linear_rows_split(self.act, self.wd, None, self.o, self.out, R, H, I, ws, nb, s)
                return
            qm.qkv_rows(self.x, (self.wq, self.wk, self.wv), (self.bq, self.bk, self.bv), (self.q, self.k, self.v), R, H, KV, H,
                        None, 0, s)
            qm.linear_rows(self.q, self.wo, None, self.res, self.o, R, H, H, s)
            qm.gate_up_swiglu_rows(self.o, self.wg, self.wu, self.act, R, H, I, s)
            qm.linear_rows(self.act, self.wd, None, self.o, self.out, R, H, I, s)
        finally:
            qm.set_option(qm.OPT_LINEAR_ROWS_KERNEL, 0)

    def cpu_baseline(self, oracle, threads):
        """Sample: the first 8 token rows through the same chain."""
        n = min(8, self.rows)
        B = lambda t: _bits(t).copy()
        u16 = lambda c: np.zeros((n, c), dtype=np.uint16)
        x, res = B(self.x[:n]), B(self.res[:n])
        q, k, v, o, act, out = u16(self.H), u16(self.KV), u16(self.KV), u16(self.H), u16(self.I), u16(self.H)
        t0 = time.perf_counter()
        assert oracle.linear_rows(x, B(self.wq), B(self.bq), None, q, n, self.H, self.H, threads) == 0
        assert oracle.linear_rows(x, B(self.wk), B(self.bk), None, k, n, self.KV, self.H, threads) == 0
        assert oracle.linear_rows(x, B(self.wv), B(self.bv), None, v, n, self.KV, self.H, threads) == 0
        assert oracle.linear_rows(q, B(self.wo), None, res, o, n, self.H, self.H, threads) == 0
        assert oracle.gate_up_swiglu_rows(o, B(self.wg), B(self.wu), act, n, self.H, self.I, threads) == 0
        assert oracle.linear_rows(act, B(self.wd), None, o, out, n, self.H, self.I, threads) == 0
        dt = time.perf_counter() - t0
        err = float(np.max(np.abs(oracle.bf16_to_f32(out).astype(np.float64)
                                  - oracle.bf16_to_f32(_bits(self.out[:n])).astype(np.float64))))
        return {"all": dt * self.rows / n}, err, "first %d of %d token rows, time scaled" % (n, self.rows)


class PredictorFrameSteps:
    """Beyond the five configurations: the fourteen M = 1 steps of one code-predictor frame as the
    reference chains them (PersistentPredictor::capture_step, R17:13592-13854): input projection,
    five layers (RMSNorm + Q/K/V, QK-norm + RoPE + append + attention over the [8][16][128] cache,
    o_proj, residual add + post-norm + gate/up/SwiGLU, down_proj + residual), final norm + that
    step's head, top-k sampler, embedding gather feeding the next step.  29 launches per step with
    the fused operators (the reference: 46 graph nodes per M = 1 step).  Geometry R17:7951-7962;
    weights random.  One `step()` is the whole frame."""
    bound = "hbm"
    name = "predictor_frame_14_m1_steps_5layers"
    tolerance = 0.125

    def __init__(self, qm, dev, seed=77, one_launch=False):
        import torch
        self.qm, self.dev, self.one_launch = qm, dev, one_launch
        if one_launch:
            self.name += "_one_launch"
        syn = Synthetic(dev, seed)
        H, Q, KV, I, OUT, V = 1024, 2048, 1024, 3072, 2048, 2048
        self.dims = (H, Q, KV, I, OUT, V)

        rnd = syn.normal

        self.proj_w, self.proj_b = rnd((H, OUT), 0.02), rnd((H,), 0.1)
        self.layers = []
        for _ in range(5):
            k, v = rnd((8, 16, 128)), rnd((8, 16, 128))
            self.layers.append(dict(
                in_norm=rnd((H,), 0.1, 1.0), wq=rnd((Q, H), 0.03), wk=rnd((KV, H), 0.03), wv=rnd((KV, H), 0.03),
                gq=rnd((128,), 0.1, 1.0), gk=rnd((128,), 0.1, 1.0), wo=rnd((H, Q), 0.02), post=rnd((H,), 0.1, 1.0),
                wg=rnd((I, H), 0.03), wu=rnd((I, H), 0.03), wd=rnd((H, I), 0.02), k=k, v=v, k0=k.clone(), v0=v.clone(),
                cache=qm.flat_cache(k, v, 8, 16)))
        self.final_norm = rnd((H,), 0.1, 1.0)
        self.heads = [rnd((V, H), 0.05) for _ in range(14)]
        self.tables = [rnd((V, OUT)) for _ in range(14)]
        inv = 1.0e6 ** (-2.0 * np.arange(64, dtype=np.float64) / 128.0)
        ang = np.arange(16, dtype=np.float64)[:, None] * np.concatenate([inv, inv])[None, :]
        self.cos = torch.tensor(np.cos(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        self.sin = torch.tensor(np.sin(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        z = lambda n: torch.zeros(n, dtype=torch.bfloat16, device=dev)
        self.input0 = rnd((OUT,))
        self.free_input = self.input0.clone()
        self.hidden = [z(H), z(H)]
        self.q, self.k_, self.v_, self.qrot, self.ctxv = z(Q), z(KV), z(KV), z(Q), z(Q)
        self.attn, self.res, self.act, self.logits = z(H), z(H), z(I), z(V)
        self.first_logits = z(V)
        self.selected = torch.zeros((16, OUT), dtype=torch.bfloat16, device=dev)
        self.codes = torch.zeros(16, dtype=torch.int32, device=dev)
        self.rng = torch.tensor([20240229], dtype=torch.int64, device=dev)
        self.ws_bytes = qm.decode_workspace_bytes(1, 16, 8, 16)
        self.ws = torch.empty(self.ws_bytes // 4 + 1, dtype=torch.float32, device=dev)
        layer_w = 2 * (Q * H + 2 * KV * H + H * Q + 2 * I * H + H * I)
        self.launches_per_step = 1 + 5 * 5 + 3
        if one_launch:
            # qm_predictor_frame_steps: 256 resident blocks run all fourteen steps and hand the operators' outputs to
            # one another through a workspace
            self.launches_per_step = 1.0 / 14
            names = dict(in_norm="input_norm", wq="q_weight", wk="k_weight", wv="v_weight", gq="q_norm", gk="k_norm",
                         wo="o_weight", post="post_norm", wg="gate_weight", wu="up_weight", wd="down_weight", k="key_cache",
                         v="value_cache")
            self.frame = qm.predictor_frame([{names[k]: L[k] for k in names} for L in self.layers], self.proj_w, self.proj_b,
                                            self.final_norm, {s: self.heads[s - 1] for s in range(1, 15)},
                                            {s: self.tables[s - 1] for s in range(1, 15)}, self.cos, self.sin, self.free_input,
                                            self.selected, self.codes, self.rng)
            self.frame_ws_bytes = qm.predictor_frame_workspace_bytes()
            self.frame_ws = torch.zeros(self.frame_ws_bytes // 4, dtype=torch.int32, device=dev)
            qm.predictor_frame_workspace_init(self.frame_ws, self.frame_ws_bytes)
            self.frame_status = torch.zeros(1, dtype=torch.int32, device=dev)
        self.bytes = 14 * (5 * layer_w + 2 * H * OUT + 2 * V * H + 2 * OUT)          # weights streamed once per step
        self.flops = self.bytes
        self.copies = 14

    def one_step(self, step, s):
        qm = self.qm
        H, Q, KV, I, OUT, V = self.dims
        position = step + 1                      # cache_before of an M = 1 step (R17:13594-13596)
        cur, nxt = self.hidden
        qm.linear_m1(self.free_input, self.proj_w, self.proj_b, None, cur, H, OUT, s)
        for L in self.layers:
            qm.predictor_rmsnorm_qkv_m1(cur, L["in_norm"], L["wq"], L["wk"], L["wv"], self.q, self.k_, self.v_, H, Q, KV,
                                        1e-6, s)
            # append at `position` + attention on the reference's exact chain, one launch (the fused decode step
            # orders its sums differently: a sampled code must not depend on that)
            qm.predictor_step_attention_m1(self.q, self.k_, self.v_, L["gq"], L["gk"], self.cos[position],
                                           self.sin[position], L["k"], L["v"], self.ctxv, position, 1e-6, s)
            qm.predictor_linear_m1(self.ctxv, L["wo"], None, self.attn, H, Q, s)
            qm.predictor_add_postnorm_gate_up_swiglu_m1(cur, self.attn, L["post"], self.res, L["wg"], L["wu"], self.act,
                                                        H, I, 1e-6, s)
            qm.predictor_linear_m1(self.act, L["wd"], self.res, nxt, H, I, s)
            cur, nxt = nxt, cur
        head = self.heads[step - 1]
        # final RMSNorm + this step's head (the talker linear's order, no bias): the fused Q/K/V entry with no K/V rows
        qm.rmsnorm_qkv_m1(cur, self.final_norm, head, None, head, None, head, None, self.logits, self.logits,
                          self.logits, H, V, 0, 1e-6, s)
        qm.sample_topk(self.logits, True, 0, V, 50, 0.9, self.rng, self.codes[step + 1:], s)
        qm.gather_embedding(self.tables[step - 1], V, self.codes, step + 1, OUT, self.selected, self.free_input, s)

    def step(self):
        import torch
        s = torch.cuda.current_stream().cuda_stream
        if self.one_launch:
            self.qm.predictor_frame_steps(self.frame, 1, 14, 50, 0.9, self.frame_ws, self.frame_ws_bytes, self.frame_status, s)
            return
        for step in range(1, 15):
            self.one_step(step, s)

    def reset(self):
        self.free_input.copy_(self.input0)
        self.rng.fill_(20240229)
        self.codes.zero_()
        for L in self.layers:
            L["k"].copy_(L["k0"])
            L["v"].copy_(L["v0"])

    def cpu_baseline(self, oracle, threads):
        """The whole frame on the host from the same start state: the fourteen sampled codes."""
        import torch
        self.reset()
        self.step()
        torch.cuda.synchronize()
        gpu_codes = self.codes.cpu().numpy().copy()
        H, Q, KV, I, OUT, V = self.dims
        u16 = lambda n: np.zeros(n, dtype=np.uint16)
        B = lambda t: _bits(t).copy()
        layers = [{k: (B(v) if hasattr(v, "detach") else v) for k, v in L.items() if k != "cache"} for L in self.layers]
        for L in layers:
            L["k"], L["v"] = L["k0"].copy(), L["v0"].copy()
        cos, sin = B(self.cos), B(self.sin)
        free_input = B(self.input0)
        rng = np.array([20240229], dtype=np.uint64)
        codes = np.zeros(16, dtype=np.int32)
        proj_w, proj_b, final_norm = B(self.proj_w), B(self.proj_b), B(self.final_norm)
        t0 = time.perf_counter()
        worst = 0.0
        for step in range(1, 15):
            position = step + 1
            cur = u16(H)
            assert oracle.linear_m1(free_input, proj_w, proj_b, None, cur, H, OUT, threads) == 0
            for L in layers:
                norm, q, k, v, qrot, ctxv, attn, res, post, act, nxt = (u16(H).reshape(1, H), u16(Q), u16(KV), u16(KV),
                                                                        u16(Q), u16(Q), u16(H), u16(H), u16(H), u16(I),
                                                                        u16(H))
                cache = oracle.flat_cache(L["k"], L["v"], 8, 16)
                assert oracle.rmsnorm_rows(cur.reshape(1, H), L["in_norm"], norm, 1, H) == 0
                assert oracle.predictor_qkv_m1(norm[0], L["wq"], L["wk"], L["wv"], q, k, v, H, Q, KV, threads) == 0
                assert oracle.qk_norm_rope_kv_append(q, k, v, L["gq"], L["gk"], cos[position], sin[position], qrot, cache,
                                                     None, 1, 16, position) == 0
                assert oracle.predictor_attention_m1(qrot, L["k"], L["v"], ctxv, position + 1) == 0
                assert oracle.predictor_linear_m1(ctxv, L["wo"], None, attn, H, Q, threads) == 0
                assert oracle.add_postnorm_m1(cur, attn, L["post"], res, post, H) == 0
                assert oracle.predictor_gate_up_swiglu_m1(post, L["wg"], L["wu"], act, H, I, threads) == 0
                assert oracle.predictor_linear_m1(act, L["wd"], res, nxt, H, I, threads) == 0
                cur = nxt
            fin, logits = u16(H).reshape(1, H), u16(V)
            assert oracle.rmsnorm_rows(cur.reshape(1, H), final_norm, fin, 1, H) == 0
            assert oracle.linear_m1(fin[0], B(self.heads[step - 1]), None, None, logits, V, H, threads) == 0
            if step == 14 and not self.one_launch:
                # (the one launch keeps its logits in its workspace: there the codes, the selected embeddings and the
                # next input below are what is compared)
                worst = float(np.max(np.abs(oracle.bf16_to_f32(logits).astype(np.float64)
                                            - oracle.bf16_to_f32(_bits(self.logits)).astype(np.float64))))
            out = np.zeros(1, dtype=np.int32)
            assert oracle.sample_topk(logits, True, 0, V, 50, 0.9, rng, out) == 0
            codes[step + 1] = out[0]
            free_input = B(self.tables[step - 1])[out[0]].copy()
        dt = time.perf_counter() - t0
        # the input of the next frame step is the embedding of the last code
        worst = max(worst, float(np.max(np.abs(oracle.bf16_to_f32(free_input).astype(np.float64)
                                               - oracle.bf16_to_f32(_bits(self.free_input)).astype(np.float64)))))
        self.codes_match = bool(np.array_equal(codes, gpu_codes))
        # a code that differs redirects every later step: the logits of the last step are compared only then
        return {"all": dt}, (worst if self.codes_match else 1.0e9), "one frame (14 steps); all sampled codes equal"


def generate_end_to_end(qm, dev, frames=96, prompt_rows=128, seed=20240229):
    """Beyond the five configurations: the engine shell's generation loop (prefill of a prompt, then per frame the
    final head, the code predictor's fifteen steps and the talker's decode step; R17:21887-22538) on a synthetic
    checkpoint of the 1.7B model's real geometry (28 talker layers of hidden 2048 / intermediate 6144, the code
    predictor's five layers, fifteen heads and tables), written to a temporary directory as sharded safetensors.
    Reports the time per generated frame for the default paths and with the talker layers and the predictor frame
    operator by operator; the codec trajectories of all four must be identical."""
    import importlib
    import shutil
    import tempfile
    import torch
    from safetensors.torch import save_file
    engine = importlib.import_module("qingming-qwen3-tts_amd.engine")
    H, Q, KV, I, LAYERS = 2048, 2048, 1024, 6144, 28
    PH, PI, P_LAYERS, V, STEPS = 1024, 3072, 5, 2048, 15
    HEAD_V, TABLE_ROWS = 3072, 3072
    g = torch.Generator().manual_seed(7)

    def rnd(shape, std=1.0, mean=0.0):
        # (host generator: the files are what the engine reads; drawn in fp32 and rounded once)
        return torch.empty(shape, dtype=torch.float32).normal_(mean, std, generator=g).to(torch.bfloat16)

    directory = tempfile.mkdtemp(prefix="qm_generate_")
    try:
        t0 = time.perf_counter()
        shard = 0

        def write(tensors):
            nonlocal shard
            shard += 1
            save_file(tensors, os.path.join(directory, "model-%05d.safetensors" % shard))

        write({"talker.model.norm.weight": rnd((H,), 0.1, 1.0), "talker.model.codec_embedding.weight": rnd((TABLE_ROWS, H), 0.5),
               "talker.codec_head.weight": rnd((HEAD_V, H), 0.05)})
        for i in range(LAYERS):
            p = "talker.model.layers.%d." % i
            write({p + "input_layernorm.weight": rnd((H,), 0.1, 1.0), p + "post_attention_layernorm.weight": rnd((H,), 0.1, 1.0),
                   p + "self_attn.q_proj.weight": rnd((Q, H), 0.02), p + "self_attn.k_proj.weight": rnd((KV, H), 0.02),
                   p + "self_attn.v_proj.weight": rnd((KV, H), 0.02), p + "self_attn.o_proj.weight": rnd((H, Q), 0.02),
                   p + "self_attn.q_norm.weight": rnd((128,), 0.1, 1.0), p + "self_attn.k_norm.weight": rnd((128,), 0.1, 1.0),
                   p + "mlp.gate_proj.weight": rnd((I, H), 0.02), p + "mlp.up_proj.weight": rnd((I, H), 0.02),
                   p + "mlp.down_proj.weight": rnd((H, I), 0.02)})
        c = "talker.code_predictor."
        t = {c + "small_to_mtp_projection.weight": rnd((PH, H), 0.02), c + "small_to_mtp_projection.bias": rnd((PH,), 0.1),
             c + "model.norm.weight": rnd((PH,), 0.1, 1.0)}
        for i in range(P_LAYERS):
            p = c + "model.layers.%d." % i
            t.update({p + "input_layernorm.weight": rnd((PH,), 0.1, 1.0), p + "post_attention_layernorm.weight": rnd((PH,), 0.1, 1.0),
                      p + "self_attn.q_proj.weight": rnd((Q, PH), 0.03), p + "self_attn.k_proj.weight": rnd((KV, PH), 0.03),
                      p + "self_attn.v_proj.weight": rnd((KV, PH), 0.03), p + "self_attn.o_proj.weight": rnd((PH, Q), 0.02),
                      p + "self_attn.q_norm.weight": rnd((128,), 0.1, 1.0), p + "self_attn.k_norm.weight": rnd((128,), 0.1, 1.0),
                      p + "mlp.gate_proj.weight": rnd((PI, PH), 0.03), p + "mlp.up_proj.weight": rnd((PI, PH), 0.03),
                      p + "mlp.down_proj.weight": rnd((PH, PI), 0.02)})
        for i in range(STEPS):
            t[c + "lm_head.%d.weight" % i] = rnd((V, PH), 0.05)
            t[c + "model.codec_embedding.%d.weight" % i] = rnd((V, H), 0.5)
        write(t)
        del t
        wrote = time.perf_counter() - t0

        t0 = time.perf_counter()
        talker = engine.Talker(directory, prompt_rows + frames + 16)
        head = engine.FinalHead(directory, frames + 16, seed, talker.stream)
        predictor = engine.Predictor(directory, head.rng_state, talker.stream)
        loaded = time.perf_counter() - t0
        prompt = rnd((prompt_rows, H)).view(torch.int16).to(dev)
        tts_pad = rnd((H,), 0.5).view(torch.int16).numpy().view(np.uint16)
        torch.cuda.synchronize()
        rows = {}
        reference = None
        for name, talker_ops, frame_ops in (("default", 0, 0), ("talker_layers_in_three_launches", 2, 0),
                                            ("talker_layers_by_operators", 1, 0),
                                            ("predictor_frame_by_operators", 0, 1), ("both_by_operators", 1, 1)):
            qm.set_option(qm.OPT_TALKER_LAYER_OPERATORS, talker_ops)
            qm.set_option(qm.OPT_PREDICTOR_FRAME_OPERATORS, frame_ops)
            try:
                best = None
                quickest_first = None      # (the first run of the first path also loads code objects: each figure is its best of three)
                for _ in range(3):
                    head.reset(seed)
                    # one frame alone = prefill + first frame; the difference to the full run is the steady state
                    t0 = time.perf_counter()
                    engine.generate(talker, head, predictor, prompt, prompt_rows, 1, tts_pad)
                    first = time.perf_counter() - t0
                    quickest_first = first if quickest_first is None else min(quickest_first, first)
                    head.reset(seed)
                    t0 = time.perf_counter()
                    codes, digest = engine.generate(talker, head, predictor, prompt, prompt_rows, frames, tts_pad)
                    whole = time.perf_counter() - t0
                    made = int(codes.shape[0])
                    per_frame = (whole - first) / max(made - 1, 1)
                    if best is None or per_frame < best[0]:
                        best = (per_frame, first, made, digest)
                if reference is None:
                    reference = (codes.copy(), digest)
                elif not (np.array_equal(codes, reference[0]) and digest == reference[1]):
                    raise RuntimeError("generate: the codec trajectory of '%s' differs from the default paths'" % name)
                rows[name] = {"ms_per_frame": best[0] * 1e3, "ms_prefill_and_first_frame": quickest_first * 1e3, "frames": best[2],
                              "codec_fnv1a64": "%016x" % best[3]}
            finally:
                qm.set_option(qm.OPT_TALKER_LAYER_OPERATORS, 0)
                qm.set_option(qm.OPT_PREDICTOR_FRAME_OPERATORS, 0)
        predictor.close(); head.close(); talker.close()
        return {"workload": "generate_%d_frames_after_a_%d_token_prompt_1p7b_geometry_synthetic_checkpoint" % (frames, prompt_rows),
                "paths": rows, "seconds_to_write_checkpoint": wrote, "seconds_to_load": loaded,
                "audio_ms_per_frame": 80.0, "real_time_factor_default": rows["default"]["ms_per_frame"] / 80.0}
    finally:
        shutil.rmtree(directory, ignore_errors=True)


class Prefill:
    """configs[3]: causal GQA prefill, batch 4 x seq 1024, K/V also written to shuffled 16-token pages."""
    name = "causal_prefill_b4_s1024_paged16"
    bound = "mfma"

    def __init__(self, qm, dev, seed=44, batch=4, seq=1024, split=False, score_rounding=1):
        import torch
        self.qm, self.batch, self.seq, self.score_rounding = qm, batch, seq, score_rounding
        if (batch, seq) != (4, 1024):
            self.name = "causal_prefill_b%d_s%d_paged16%s" % (batch, seq, "_key_split" if split else "")
        if not score_rounding:
            # scores stay fp32 between Q.K^T and the softmax (the fp32-accumulate formulation); the default
            # rounds them to bf16 twice as the reference's operator does
            self.name += "_fp32_scores"
        # key split: a workspace lets up to three blocks share a long query tile (shapes that leave CUs idle)
        self.workspace, self.workspace_bytes = None, 0
        if split:
            self.workspace_bytes = qm.prefill_split_workspace_bytes(batch, seq, 8)
            self.workspace = torch.zeros(max(self.workspace_bytes, 256) // 4, dtype=torch.int32, device=dev)
            qm.prefill_split_workspace_init(self.workspace, self.workspace_bytes,
                                            torch.cuda.current_stream().cuda_stream)
        syn = Synthetic(dev, seed)

        rnd = syn.normal

        self.q, self.k, self.v = rnd((batch, seq, 16, 128)), rnd((batch, seq, 8, 128)), rnd((batch, seq, 8, 128))
        self.out = torch.zeros_like(self.q)
        per = (seq + 15) // 16
        self.max_pages = per
        self.n_pages = batch * per + 5
        perm = torch.from_numpy(syn.permutation(self.n_pages))
        self.table = perm[:batch * per].view(batch, per).contiguous().to(dev)
        self.kp = torch.zeros((self.n_pages, 8, 16, 128), dtype=torch.bfloat16, device=dev)
        self.vp = torch.zeros_like(self.kp)
        self.cache = qm.paged_cache(self.kp, self.vp, self.n_pages)
        self.status = torch.zeros(1, dtype=torch.int32, device=dev)
        self.flops = batch * 16 * (seq * (seq + 1) // 2) * 128 * 2 * 2
        qo = batch * seq * 16 * 128 * 2
        kv = batch * seq * 8 * 128 * 2
        self.bytes = 2 * qo + 2 * kv + 2 * kv      # Q + O, K + V read, K + V written to pages

    def step(self):
        import torch
        self.qm.set_option(self.qm.OPT_PREFILL_SCORE_ROUNDING, self.score_rounding)
        try:
            self._launch(torch.cuda.current_stream().cuda_stream)
        finally:
            self.qm.set_option(self.qm.OPT_PREFILL_SCORE_ROUNDING, 1)

    def _launch(self, stream):
        if self.workspace is not None:
            self.qm.prefill_attention_causal_split(self.q, self.k, self.v, self.out, self.cache, self.table,
                                                   self.max_pages, self.batch, self.seq, 16, 8, self.workspace,
                                                   self.workspace_bytes, SCALE, self.status, stream)
            return
        self.qm.prefill_attention_causal(self.q, self.k, self.v, self.out, self.cache, self.table, self.max_pages,
                                         self.batch, self.seq, 16, 8, SCALE, self.status, stream)

    def cpu_baseline(self, oracle, threads):
        """Sample: batch entry 0 (a quarter of the flops)."""
        q, k, v = _bits(self.q[:1]).copy(), _bits(self.k[:1]).copy(), _bits(self.v[:1]).copy()
        out = np.zeros_like(q)
        t0 = time.perf_counter()
        rc = oracle.prefill_attention_causal(q, k, v, out, None, None, 0, 1, self.seq, 16, 8, SCALE,
                                             oracle.POLICY_ONLINE if self.score_rounding else oracle.POLICY_FP32,
                                             threads)
        dt = time.perf_counter() - t0
        assert rc == 0
        err = float(np.max(np.abs(oracle.bf16_to_f32(out).astype(np.float64)
                                  - oracle.bf16_to_f32(_bits(self.out[:1])).astype(np.float64))))
        return {"all": dt * self.batch}, err, "batch entry 0 of %d, time scaled by %d" % (self.batch, self.batch)


class PrefillChunk:
    """A prompt continued in chunks (the reference's generic attention branch with cache_before > 0): 256 rows at
    position 2048 of one sequence over the reference's flat LayerCache, on the matrix cores or row by row."""
    bound = "mfma"

    def __init__(self, qm, dev, seed=46, rows=256, before=2048, by_rows=False, split=True, paged=False, q_heads=16):
        import torch
        self.qm, self.rows, self.before, self.by_rows, self.paged, self.q_heads = qm, rows, before, by_rows, paged, q_heads
        self.name = "prefill_chunk_%d_rows_at_%d_%s%s%s" % (
            rows, before, "paged_cache" if paged else "flat_cache", "" if q_heads == 16 else "_%d_query_heads" % q_heads,
            "_row_by_row" if by_rows else "" if split else "_one_block_per_query_tile")
        syn = Synthetic(dev, seed)
        self.max_cache = before + rows
        self.q = syn.normal((rows, q_heads, 128))
        self.k, self.v = syn.normal((8, self.max_cache, 128)), syn.normal((8, self.max_cache, 128))
        self.out = torch.zeros_like(self.q)
        if paged:
            # the same keys behind a shuffled page table: pool [n_pages, 8, 16, 128]
            self.n_pages = (self.max_cache + 15) // 16
            order = torch.randperm(self.n_pages, generator=torch.Generator().manual_seed(seed)).to(torch.int32)
            pad = self.n_pages * 16 - self.max_cache
            def pool_of(t):
                t = torch.nn.functional.pad(t, (0, 0, 0, pad)).view(8, self.n_pages, 16, 128).permute(1, 0, 2, 3).contiguous()
                pool = torch.empty_like(t)
                pool[order.to(dev).long()] = t
                return pool
            self.k_pool, self.v_pool = pool_of(self.k), pool_of(self.v)
            self.table = order.to(dev)
            self.cache = qm.paged_cache(self.k_pool, self.v_pool, self.n_pages)
        else:
            self.cache = qm.flat_cache(self.k, self.v, 8, self.max_cache)
        self.ws_bytes = qm.attention_rows_workspace_bytes(rows, q_heads, 8, self.max_cache) if by_rows else \
            qm.prefill_chunk_workspace_bytes(1, rows, before, 8) if split else 0
        self.ws = torch.empty(self.ws_bytes // 4 + 64, dtype=torch.float32, device=dev)
        keys = sum(before + i + 1 for i in range(rows))
        self.flops = q_heads * keys * 128 * 2 * 2
        self.bytes = 2 * rows * q_heads * 128 * 2 + 2 * self.max_cache * 8 * 128 * 2     # Q + O, K + V read once

    def step(self):
        import torch
        stream = torch.cuda.current_stream().cuda_stream
        ws = self.ws if self.ws_bytes else None
        if self.by_rows:
            self.qm.attention_rows(self.q, self.cache, self.table if self.paged else None, self.n_pages if self.paged else 1,
                                   self.out, self.rows, self.before, self.q_heads, -1, SCALE, self.ws, self.ws_bytes, None, stream)
        elif self.paged:
            self.qm.prefill_attention_chunk_paged(self.q, self.cache, self.table, self.n_pages, self.out, 1, self.rows,
                                                  self.before, self.q_heads, 8, SCALE, ws, self.ws_bytes, None, stream)
        else:
            self.qm.prefill_attention_chunk(self.q, self.k, self.v, self.out, 1, self.rows, self.before, self.q_heads, 8, SCALE,
                                            stream, (128, self.max_cache * 128, 0), ws, self.ws_bytes)

    def cpu_baseline(self, oracle, threads):
        """Sample: the first 32 rows."""
        n = 32
        q, k, v = _bits(self.q[:n]).copy(), _bits(self.k).copy(), _bits(self.v).copy()
        out = np.zeros_like(q)
        t0 = time.perf_counter()
        rc = oracle.attention(q, oracle.flat_cache(k, v, 8, self.max_cache), None, 1, out, n, self.before, self.q_heads, -1,
                              SCALE, oracle.POLICY_ONLINE, threads)
        dt = time.perf_counter() - t0
        assert rc == 0
        err = float(np.max(np.abs(oracle.bf16_to_f32(out).astype(np.float64)
                                  - oracle.bf16_to_f32(_bits(self.out[:n])).astype(np.float64))))
        return {"all": dt * self.rows / n}, err, "first %d of %d rows, time scaled" % (n, self.rows)


class PredictorLoop:
    """configs[4]: 256 frames x 5 layers, 16 steps each (context 1 -> 16), one launch."""
    name = "predictor_loop_256frames_5layers_16steps"
    bound = "hbm"

    def __init__(self, qm, dev, seed=55, frames=256, layers=5, rows=16, write_cache=False, kernel=0):
        import torch
        self.qm, self.units, self.layers, self.rows, self.frames = qm, frames * layers, layers, rows, frames
        self.kernel = kernel      # 0: products on the matrix cores; 1: every fp32 sum in the reference's order
        # bf16 outputs of magnitude >= 2 are 0.0156 apart: a sum taken in another order can land one
        # output spacing away, which is what the gate below allows the matrix-core kernel
        syn = Synthetic(dev, seed)

        rnd = syn.normal

        u = self.units
        self.q, self.k, self.v = rnd((u, rows, 16, 128)), rnd((u, rows, 8, 128)), rnd((u, rows, 8, 128))
        self.gq, self.gk = rnd((layers, 128), 0.1, 1.0), rnd((layers, 128), 0.1, 1.0)
        inv = 1.0e6 ** (-2.0 * np.arange(64, dtype=np.float64) / 128.0)
        ang = np.arange(rows, dtype=np.float64)[:, None] * np.concatenate([inv, inv])[None, :]
        self.cos = torch.tensor(np.cos(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        self.sin = torch.tensor(np.sin(ang), dtype=torch.float32).to(torch.bfloat16).to(dev)
        self.out = torch.zeros_like(self.q)
        self.kc = torch.zeros((u, 8, 16, 128), dtype=torch.bfloat16, device=dev) if write_cache else None
        self.vc = torch.zeros((u, 8, 16, 128), dtype=torch.bfloat16, device=dev) if write_cache else None
        per_unit = 3 * 65536 + (65536 if write_cache else 0)
        self.bytes = per_unit * u
        self.flops = 1114112 * u
        if write_cache:
            self.name += "_cache_writeback"
        if kernel:
            self.name += "_exact_chain"

    def step(self):
        import torch
        self.qm.set_option(self.qm.OPT_PREDICTOR_LOOP_KERNEL, self.kernel)
        try:
            self.qm.predictor_attention_loop(self.q, self.k, self.v, self.gq, self.gk, self.cos, self.sin, self.out,
                                             self.kc, self.vc, self.units, self.layers, self.rows, 1, 1e-6,
                                             torch.cuda.current_stream().cuda_stream)
        finally:
            self.qm.set_option(self.qm.OPT_PREDICTOR_LOOP_KERNEL, 0)

    def cpu_baseline(self, oracle, threads):
        """Sample: the first 160 units (32 frames)."""
        n = min(160, self.units)
        q, k, v = _bits(self.q[:n]).copy(), _bits(self.k[:n]).copy(), _bits(self.v[:n]).copy()
        out = np.zeros_like(q)
        t0 = time.perf_counter()
        rc = oracle.predictor_attention_loop(q, k, v, _bits(self.gq), _bits(self.gk), _bits(self.cos), _bits(self.sin),
                                             out, None, None, n, self.layers, self.rows, 1, 1e-6, threads)
        dt = time.perf_counter() - t0
        assert rc == 0
        # (the matrix-core kernel's other order of summation moves a bf16-rounded score across a rounding boundary about
        # once in 10^6 outputs: the same allowance as tests/test_gpu_predictor.py, none for the exact chain)
        err, outside = _within_rule(oracle, _bits(self.out[:n]), out)
        ok = outside == 0 if self.kernel else (outside <= 4 and err <= 2e-2)
        return {"all": dt * self.units / n}, err, "first %d of %d units, time scaled" % (n, self.units), ok


def _within_rule(oracle, got_bits, want_bits, tol=1e-2):
    """The tolerance rule of the parity tests, per element: |got - want| <= max(tol, one bf16 ulp of the oracle's
    value) (beyond |x| = 2 one bf16 step is 1.56e-2, more than tol).  Returns (max abs error, elements outside the
    rule)."""
    want = oracle.bf16_to_f32(want_bits).astype(np.float64)
    err = np.abs(oracle.bf16_to_f32(got_bits).astype(np.float64) - want)
    one_ulp = 2.0 ** (np.floor(np.log2(np.maximum(np.abs(want), 2.0 ** -20))) - 7)
    return float(err.max()) if err.size else 0.0, int(np.count_nonzero(err > np.maximum(one_ulp, tol)))


def _report(w, ms):
    rep = {"workload": w.name, "us_per_step": ms * 1e3, "algorithmic_bytes": w.bytes, "algorithmic_flops": w.flops,
           "GBps": w.bytes / (ms * 1e-3) / 1e9, "TFLOPps": w.flops / (ms * 1e-3) / 1e12}
    rep["frac_hbm_peak"] = rep["GBps"] / HBM_PEAK_GBPS
    rep["frac_mfma_peak"] = rep["TFLOPps"] / MFMA_BF16_PEAK_TFLOPS
    return rep


def _summary(per_config):
    """{row: [microseconds per step (graph replay where taken), fraction of the peak that bounds the row]}."""
    out = {}
    for key, r in per_config.items():
        if "us_per_step" not in r:
            if "us_per_frame" in r:
                out[key] = [round(r["us_per_frame"], 1), None]
            continue
        # (the headline row is the timed region the record's `value` comes from: K eager steps between events)
        us = r["us_per_step"] if r.get("headline") else r.get("us_per_step_graph", r["us_per_step"])
        work, peak = (r["algorithmic_flops"], MFMA_BF16_PEAK_TFLOPS * 1e12) if r.get("bound") == "mfma" \
            else (r["algorithmic_bytes"], HBM_PEAK_GBPS * 1e9)
        out[key] = [round(us, 2), round(work / (us * 1e-6) / peak, 4)]
    return out


FINAL_LINE_LIMIT = 4000  # bytes; the last stdout line must survive a tail of a few KB
PER_CONFIG_FILE = "gpurun_out/bench_per_config.json"   # the full per-row record, relative to the repository root


def compact_line(line):
    """The last stdout line: the record as JSON, with the summary's row names shortened and, if still too
    long, dropped, so that it stays below FINAL_LINE_LIMIT bytes."""
    text = json.dumps(line, separators=(",", ":"))
    if len(text) > FINAL_LINE_LIMIT:
        line = dict(line)
        line["summary"] = {k: v for k, v in line.get("summary", {}).items() if k.startswith("cfg")}
        text = json.dumps(line, separators=(",", ":"))
    if len(text) > FINAL_LINE_LIMIT:
        line.pop("summary", None)
        text = json.dumps(line, separators=(",", ":"))
    return text


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--headline-only", action="store_true", help="time only the headline workload")
    ap.add_argument("--all", action="store_true", help="time every variant row, not only the five configurations and "
                                                       "the four rows of a generated frame")
    ap.add_argument("--only", choices=["decode512", "talker2048", "prefill", "prefill1", "prefill1split", "prefillfp32", "chunk", "chunkwhole", "chunkrows", "predictor", "predictorexact",
                                      "qkv", "layer", "layer1", "layer2", "frame", "frame1", "linears", "linearsexact", "linears128", "linears128split", "generate"], default=None,
                    help="time just one of the other configurations and print its record (for profiling one "
                         "kernel under rocprofv3); the headline line is not produced")
    ap.add_argument("--rows", default=None, metavar="TEXT",
                    help="beside the headline, time exactly the rows whose name contains TEXT (cfg4c, paged, group_4 ...), "
                         "default or not; the generation loop is left out")
    ap.add_argument("--layers", type=int, default=28,
                    help="with --only layer / layer1 / layer2: distinct weight sets and caches in rotation (a profiler that "
                         "records counters for every dispatch is spared most of the input generation with a small number)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run three plain 512 MiB device-to-device copies (for scaling rocprofv3's "
                         "FETCH_SIZE / WRITE_SIZE counters against a kernel of known traffic)")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one MI355X: this path shards without communication (streams / batch / frames), "
              "and no multi-GPU figure is produced; run with --gpus 1", file=sys.stderr)
        sys.exit(2)

    import torch
    if not torch.cuda.is_available():
        print("bench.py needs a GPU (there is no CPU fallback for the product path)", file=sys.stderr)
        sys.exit(3)
    qm = importlib.import_module("qingming-qwen3-tts_amd").binding
    qm.lib()
    dev = torch.device("cuda:0")
    props = torch.cuda.get_device_properties(0)

    if args.calibrate_copy:
        src = torch.empty(512 * 1024 * 1024 // 4, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
        torch.cuda.empty_cache()

    if args.only == "generate":
        print(json.dumps(generate_end_to_end(qm, dev)))
        return
    if args.only:
        make = {"decode512": lambda: SingleDecode(qm, dev, 512, False, 11),
                "talker2048": lambda: SingleDecode(qm, dev, 2048, True, 12),
                "prefill": lambda: Prefill(qm, dev), "prefill1": lambda: Prefill(qm, dev, batch=1),
                "prefill1split": lambda: Prefill(qm, dev, batch=1, split=True),
                "prefillfp32": lambda: Prefill(qm, dev, score_rounding=0),
                "chunk": lambda: PrefillChunk(qm, dev), "chunkwhole": lambda: PrefillChunk(qm, dev, split=False), "chunkrows": lambda: PrefillChunk(qm, dev, by_rows=True),
                "predictor": lambda: PredictorLoop(qm, dev),
                "predictorexact": lambda: PredictorLoop(qm, dev, kernel=1),
                "qkv": lambda: QkvGemv(qm, dev, copies=64), "layer": lambda: TalkerLayerStep(qm, dev, layers=args.layers), "layer1": lambda: TalkerLayerStep(qm, dev, layers=args.layers, chained=True),
                "layer2": lambda: TalkerLayerStep(qm, dev, layers=args.layers, two_launches=True),
                "frame": lambda: PredictorFrameSteps(qm, dev),
                "frame1": lambda: PredictorFrameSteps(qm, dev, one_launch=True),
                "linears": lambda: PromptLinears(qm, dev), "linearsexact": lambda: PromptLinears(qm, dev, kernel=1),
                "linears128": lambda: PromptLinears(qm, dev, rows=128), "linears128split": lambda: PromptLinears(qm, dev, rows=128, split=True)}[args.only]
        w = make()
        r = _report(w, _time_steps(w.step, args.steps, args.warmup))
        r["bound"] = w.bound
        print(json.dumps(r))
        return

    head = RaggedDecode(qm, dev)
    ms = _time_steps(head.step, args.steps, args.warmup)
    torch.cuda.synchronize()
    if int(head.status.item()) != 0:
        raise RuntimeError("device status flagged a bad page/position")
    rep = _report(head, ms)

    per_config = {}
    oracle = None
    threads = min(os.cpu_count() or 1, 16)
    if not args.no_cpu:
        from oracle import binding as oracle
        oracle.build()
    if not args.headline_only:
        # (row name, constructor, in the default run?)  The default run holds the five configurations and the rows
        # that make up a generated frame; the variants come with --all.
        rows = [
            ("cfg1_decode_ctx512", lambda: SingleDecode(qm, dev, 512, False, 11), True),
            ("cfg2_talker_fused_step_ctx2048", lambda: SingleDecode(qm, dev, 2048, True, 12), True),
            # the same step over 64 distinct KV caches in rotation (0.54 GB): defeats L2 / MALL
            # residency, as consecutive layers of a real decode step do
            ("cfg2_talker_fused_step_ctx2048_rotating64", lambda: SingleDecode(qm, dev, 2048, True, 12, copies=64), False),
            # the same step as the reference launches it: append kernel, then attention
            ("cfg2_talker_step_ctx2048_two_operators", lambda: SingleDecode(qm, dev, 2048, True, 12, one_launch=False), False),
            ("cfg4_causal_prefill", lambda: Prefill(qm, dev), True),
            # scores kept fp32 between Q.K^T and the softmax (the fp32-accumulate formulation; not the reference's two roundings)
            ("cfg4_causal_prefill_fp32_scores", lambda: Prefill(qm, dev, score_rounding=0), True),
            # one prompt, as the talker's prefill runs it: 128 blocks for 256 CUs; the key-split entry fills them
            ("cfg4b_causal_prefill_one_prompt_1024", lambda: Prefill(qm, dev, batch=1), False),
            ("cfg4b_causal_prefill_one_prompt_1024_key_split", lambda: Prefill(qm, dev, batch=1, split=True), False),
            # a prompt continued in chunks: 256 rows at position 2048 (matrix cores; and row by row through the decode kernels,
            # which also serves sliding windows)
            ("cfg4c_prefill_chunk_256_rows_at_2048", lambda: PrefillChunk(qm, dev), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_one_block_per_query_tile", lambda: PrefillChunk(qm, dev, split=False), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_row_by_row", lambda: PrefillChunk(qm, dev, by_rows=True), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_paged", lambda: PrefillChunk(qm, dev, paged=True), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_paged_row_by_row", lambda: PrefillChunk(qm, dev, paged=True, by_rows=True), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_group_1", lambda: PrefillChunk(qm, dev, q_heads=8), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_group_4", lambda: PrefillChunk(qm, dev, q_heads=32), False),
            ("cfg4c_prefill_chunk_256_rows_at_2048_group_4_paged", lambda: PrefillChunk(qm, dev, q_heads=32, paged=True), False),
            ("cfg5_predictor_loop", lambda: PredictorLoop(qm, dev), True),
            ("cfg5_predictor_loop_exact_chain", lambda: PredictorLoop(qm, dev, kernel=1), False),
            ("cfg5_predictor_loop_cache_writeback", lambda: PredictorLoop(qm, dev, write_cache=True), True),
            # beyond the five configurations: the M = 1 projection in front of configuration 2
            ("next_qkv_gemv_m1", lambda: QkvGemv(qm, dev), False),
            ("next_qkv_gemv_m1_rotating64", lambda: QkvGemv(qm, dev, copies=64), False),
            # the whole decode step of one talker layer, 28 layers' weights and caches in rotation (2.8 GB)
            ("next_talker_layer_decode_step", lambda: TalkerLayerStep(qm, dev), False),
            ("next_talker_layer_decode_step_unfused", lambda: TalkerLayerStep(qm, dev, fused=False), False),
            ("next_talker_layer_decode_step_one_launch", lambda: TalkerLayerStep(qm, dev, chained=True), False),
            # the attention's merge launch folded into that launch: two launches per layer
            ("next_talker_layer_decode_step_two_launches", lambda: TalkerLayerStep(qm, dev, two_launches=True), True),
            # the seven linears of a talker layer over a 1024-token prompt: matrix cores, and the exact chain
            ("next_prompt_linears_1024_tokens", lambda: PromptLinears(qm, dev), True),
            ("next_prompt_linears_1024_tokens_exact_chain", lambda: PromptLinears(qm, dev, kernel=1), False),
            # a short prompt (what a sentence of text is): 32 to 96 blocks per linear; with a workspace the reductions are cut
            ("next_prompt_linears_128_tokens", lambda: PromptLinears(qm, dev, rows=128), False),
            ("next_prompt_linears_128_tokens_reductions_shared", lambda: PromptLinears(qm, dev, rows=128, split=True), False),
            # the fourteen M = 1 steps of one code-predictor frame, operator by operator (406 launches)
            ("next_predictor_frame_m1_steps", lambda: PredictorFrameSteps(qm, dev), False),
            # the same fourteen steps as ONE launch of 256 resident blocks (same codes bit for bit)
            ("next_predictor_frame_m1_steps_one_launch", lambda: PredictorFrameSteps(qm, dev, one_launch=True), True),
        ]
        extra = [(key, make) for key, make, default in rows if (args.rows in key if args.rows else default or args.all)]
        for key, make in extra:
            w = make()
            r = _report(w, _time_steps(w.step, max(args.steps, 100), max(args.warmup, 10)))
            copies = getattr(w, "copies", 1)
            r["us_per_step_graph"] = _time_graph(w.step, reps=2 if isinstance(w, PredictorFrameSteps) else
                                                 64 if copies > 1 else 20) * 1e3
            r["GBps_graph"] = w.bytes / (r["us_per_step_graph"] * 1e-6) / 1e9
            r["TFLOPps_graph"] = w.flops / (r["us_per_step_graph"] * 1e-6) / 1e12
            r["bound"] = w.bound
            r["cache_resident"] = copies == 1 and w.bytes < 256e6
            if isinstance(w, PredictorLoop):
                r["us_per_predictor_step"] = r["us_per_step_graph"] / w.rows
                r["us_per_frame"] = r["us_per_step_graph"] / w.frames
            if isinstance(w, PredictorFrameSteps):
                r["us_per_frame"] = r["us_per_step_graph"]
                r["us_per_predictor_step"] = r["us_per_step_graph"] / 14
                r["launches_per_predictor_step"] = w.launches_per_step
            if oracle is not None and not (isinstance(w, PredictorLoop) and w.kc is not None) \
                    and (copies == 1 or isinstance(w, (TalkerLayerStep, PredictorFrameSteps))):
                res, err, sample, *rule = w.cpu_baseline(oracle, threads)
                if not (rule[0] if rule else err <= getattr(w, "tolerance", 1e-2)):
                    raise RuntimeError(f"{key}: GPU result differs from the oracle: max abs err {err}")
                r["cpu_oracle"] = {"seconds": res["all"], "cores": threads, "sample": sample,
                                   "gpu_vs_oracle_max_abs_err": err,
                                   "speedup_vs_cpu": res["all"] / (r["us_per_step_graph"] * 1e-6)}
            per_config[key] = r
            del w
            torch.cuda.empty_cache()
        rep["us_per_step_graph"] = _time_graph(head.step, reps=5, replays=10) * 1e3
        per_config["cfg3_ragged_decode"] = dict(rep, headline=True)
        # the generation loop end to end on a synthetic checkpoint of the real size (3.2 GB written to a temporary
        # directory): skipped, with the reason, where that cannot be written
        try:
            if not args.rows:
                per_config["next_generate_end_to_end"] = generate_end_to_end(qm, dev)
        except OSError as e:
            per_config["next_generate_end_to_end"] = {"skipped": "%s: %s" % (type(e).__name__, e)}

    cpu = None
    if oracle is not None:
        res, err, sample = head.cpu_baseline(oracle, threads)
        if err > 1e-2:
            raise RuntimeError(f"GPU result differs from the oracle: max abs err {err}")
        cpu = {"value": head.bytes / res["all"] / 1e9, "unit": "GB/s", "cores": threads, "kind": "port",
               "sample": sample, "single_thread_value": head.bytes / res["single"] / 1e9,
               "seconds": res["all"], "seconds_single_thread": res["single"], "gpu_vs_oracle_max_abs_err": err}

    line = {
        "metric": "decode_attn_hbm_GBps", "value": rep["GBps"], "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16 storage, f32 accumulate", "data": "synthetic",
        "config": {"workload": head.name, "streams": head.n, "context_tokens_total": head.tokens,
                   "q_heads": 16, "kv_heads": 8, "head_dim": 128, "page_size": 16,
                   "device": props.name, "compute_units": props.multi_processor_count},
        "roofline": {"bound": "hbm", "achieved": rep["GBps"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": rep["GBps"] / HBM_PEAK_GBPS, "traffic": HEADLINE_TRAFFIC_BYTES,
                     "traffic_source": "profiles/decode_split_kernel_ragged64_traffic.txt (rocprofv3 --pmc FETCH_SIZE / "
                                       "WRITE_SIZE of this workload; not measured in this run)",
                     "kernel": "decode_split_kernel<2, false, true, false> (+ decode_merge_kernel<2, false>, both inside the timed step)",
                     "algorithmic_bytes_per_launch": head.bytes, "avg_launch_us": ms * 1e3},
        "cpu_baseline": cpu,
        "summary": _summary(per_config),
    }
    if per_config:
        full = json.dumps(per_config)
        print("per_config " + full, flush=True)
        try:
            os.makedirs(os.path.dirname(os.path.join(ROOT, PER_CONFIG_FILE)), exist_ok=True)
            with open(os.path.join(ROOT, PER_CONFIG_FILE), "w") as f:
                f.write(full + "\n")
            line["per_config_file"] = PER_CONFIG_FILE
        except OSError:
            pass
    print(compact_line(line), flush=True)


if __name__ == "__main__":
    main()
