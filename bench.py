#!/usr/bin/env python3
"""Throughput of the fused softmax + rotary hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one pass of the hot path over one batch of synthetic input, through
the drop-in extension modules (which call libneox_hotpath.so):

  pythia-1.4b (default; the configuration the headline metric is quoted on)
      rotary fwd on q and k  [s=2048, b=8, h=16, d=128] bf16, rotary_pct 0.25 (both tensors in one
                             launch; --rope-per-tensor: one launch each, the reference's call style)
      causal softmax fwd     [b*h=128, 2048, 2048] bf16, scale 1/sqrt(128)
      causal softmax bwd     same shape, in place on the upstream gradient
      rotary bwd on dq, dk
  masked-c3      padding-masked softmax fwd+bwd [16,32,1024,2048] fp16
  rope-c4        rotary fwd+bwd on q,k [4096,4,32,128] bf16, rotary_pct 1.0 and 0.25
  llama2-7b-c5   rotary on q,k [8192,2,32,128] + causal softmax fwd+bwd [64,8192,8192] bf16
  rope-c4-qkv-view  rotary fwd+bwd on q,k given as views of one fused [4096,4,32,3*128] bf16 buffer (the layout
                 the attention layer slices q and k from), rotary_pct 1.0; one launch per tensor, then q and k
                 in one launch
  rope-qk-1.4b   rotary fwd+bwd on q,k [2048,8,16,128] bf16, rotary_pct 0.25, q and k in one launch
  rope-neox-20b  rotary fwd+bwd on q,k [2048,4,64,96] bf16 with 24 rotary dimensions (the reference's 20B configuration):
                 half the rotary dimension is not a whole number of 16-byte chunks
  rope-freqs-1.4b  the same tensors through the entry points that take the angles (fp32) and evaluate sin/cos on the
                 device, per tensor and q and k in one launch
  rope-kgrad-1.4b  rotary bwd on a gradient [2048,8,16,128] bf16 that is contiguous along the sequence (strides
                 (1, h*d*s, d*s, s)): the layout of the key gradient behind the score GEMM's backward
  mistral-window causal softmax fwd+bwd [64,8192,8192] bf16 with a 4096-key sliding window applied by index
  causal-blocks-1.4b  causal softmax fwd+bwd [128,2048,2048] bf16 writing only the 512-column blocks on and below the
                 diagonal (what the blocked attention GEMMs read); causal-blocks-7b: [32,4096,4096], 1024-column blocks;
                 mistral-window-blocks: the same for mistral-window, 1024-column blocks
  alibi-1.4b     causal softmax fwd+bwd [128,2048,2048] bf16 with the AliBi bias of 16 heads added in the kernel
  attn-dropout-1.4b  causal softmax + attention dropout (p = 0.1) in one kernel, fwd+bwd [128,2048,2048] bf16
  masked-dropout-c3  padding-masked softmax + attention dropout (p = 0.1) in one kernel, fwd+bwd on the masked-c3 tensors
  rpe-bias-1.4b  causal softmax fwd+bwd [128,2048,2048] bf16 with a bias tensor [16,2048,2048] added in the kernel

  hbm-probes     kernels that only move data (bench_probes/libneox_probe.so): a plain streaming copy of 16 MiB, 64 MiB,
                 128 MiB and 1 GiB tensors, and the causal softmax forward's access pattern (lower-triangle reads, dense writes)
                 at [128,2048,2048] and [64,8192,8192], and the layout change of the transposing rotary kernel
                 ([128,128,2048] contiguous along the sequence -> [2048,128,128]): what the memory system gives for
                 those patterns and sizes

  mlp-gelu-1.4b  bias + tanh-GeLU fwd and bwd (with the bias gradient) on the MLP activation [2048*8, 8192] bf16
  swiglu-7b      SwiGLU forward and backward on the Llama-2 7B MLP activation [4096*4, 2*11008] -> [4096*4, 11008] bf16
  bias-residual-1.4b  residual + (x + bias) on the hidden state [2048*8, 2048] bf16
  bias-dropout-add-1.4b  residual + dropout(x + bias) with p = 0.1, and the dropout backward, same shape
  bias-residual-pair-1.4b  residual + ((x1 + bias1) + (x2 + bias2)): the parallel-residual layer's three additions in one pass
  layernorm-1.4b  LayerNorm fwd and bwd (with the parameter gradients, and for frozen parameters without) on the hidden
                 state [2048*8, 2048] bf16
  layernorm-pair-1.4b  the two LayerNorms of the parallel-residual layer in one launch each way, same hidden state
  rmsnorm-7b     RMSNorm fwd and bwd on [4096*4, 4096] bf16 (the Llama-2 7B hidden size)

`value` is algorithmic bytes per step / wall time per step (inputs resident in
HBM, K steps bracketed by device synchronisation). Algorithmic bytes: softmax
forward reads the lower triangle and writes the dense result; backward reads
two triangles and writes dense; rotary reads and writes every element once plus
the cos/sin tables. `roofline` is the same ratio for the dominant kernel alone,
timed with events on the launch stream. `cpu_baseline` times the reference's
torch fallback (oracle/fallback_semantics.py) on this machine's host cores on a
bounded sample of the default workload.

One GPU only: there is no multi-GPU mode, `--gpus N` with N > 1 exits.
"""
import argparse
import json
import math
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "gpt-neo-x_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)

METRIC = "achieved HBM GB/s (% of MI355X peak), causal softmax+rotary fwd/bwd, 1.4B shape"
HBM_PEAK_GBS = 8000.0

TRAFFIC_TABLE = os.path.join(ROOT, "profiles", "hbm_traffic.json")
# Workloads whose dominant kernel has no geometry query: a revision label that is changed by hand whenever
# that kernel's launch shape or data flow changes, so that a traffic figure measured before is dropped.
KERNEL_REVISIONS = {"mlp-gelu-1.4b": "bias_gelu_bwd r1", "swiglu-7b": "gated_bwd r1", "layernorm-1.4b": "norm_bwd r2",
                    "rope-c4": "rope_lean r2", "layernorm-pair-1.4b": "norm_pair_bwd r1",
                    "bias-residual-pair-1.4b": "bias_add_residual_pair r1"}


def measured_traffic(workload, signature):
    """HBM bytes per launch of the workload's dominant kernel as measured with rocprofv3 --pmc
    (FETCH_SIZE, WRITE_SIZE), from the tracked table profiles/hbm_traffic.json. A figure belongs to
    one kernel instantiation: it is returned only when the table's signature for the workload equals
    the signature of the kernel that runs now (None otherwise, and when the workload is not listed)."""
    try:
        with open(TRAFFIC_TABLE) as f:
            entry = json.load(f)["workloads"].get(workload)
    except (OSError, ValueError, KeyError):
        return None
    if not entry or entry.get("signature") != signature:
        return None
    return entry["bytes"]


def softmax_signature(lib, row_len, kind):
    """'L<lanes> K<chunks per lane> W<waves per row>' of the kernel the library launches for such rows."""
    import ctypes

    l, k, w = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    if lib.nhp_softmax_geometry(row_len, kind, ctypes.byref(l), ctypes.byref(k), ctypes.byref(w)) != 0:
        return "scalar"
    return f"L{l.value} K{k.value} W{w.value}"


def tri(n):
    return n * (n + 1) // 2


def causal_bytes(a, s, e=2):
    fwd = a * tri(s) * e + a * s * s * e
    bwd = 2 * a * tri(s) * e + a * s * s * e
    return fwd, bwd


def rope_bytes(s, b, h, d, d2, e=2, e_cs=2):
    return 2 * s * b * h * d * e + 2 * s * d2 * e_cs


class Timer:
    """Event-times named kernels on the current stream. `only` restricts the
    bracketing to one name (the others run unbracketed, without event records).
    `chain`: a kernel that directly follows a bracketed one takes that bracket's closing
    event as its opening event (one event record between two kernels instead of two: every
    record is a packet the GPU has to process between them, about 2 us). The workload
    must then issue nothing else between two run() calls; `unchain()` says that it did."""

    def __init__(self, torch, only=None, chain=False):
        self.torch = torch
        self.only = only
        self.chain = chain
        self.last = None
        self.pairs = {}

    def unchain(self):
        self.last = None

    def run(self, name, fn):
        if self.only is not None and name != self.only:
            self.last = None
            return fn()
        a = self.last if (self.chain and self.last is not None) else None
        if a is None:
            a = self.torch.cuda.Event(enable_timing=True)
            a.record()
        b = self.torch.cuda.Event(enable_timing=True)
        out = fn()
        b.record()
        self.last = b
        self.pairs.setdefault(name, []).append((a, b))
        return out

    def averages_ms(self):
        return {k: sum(a.elapsed_time(b) for a, b in v) / len(v) for k, v in self.pairs.items()}

    def spread_ms(self, name):
        """(min, median, max) of the bracketed launches of `name`."""
        t = sorted(a.elapsed_time(b) for a, b in self.pairs[name])
        return t[0], t[len(t) // 2], t[-1]

    def reset(self):
        self.pairs = {}
        self.last = None


def grad_ring(torch, pristine, launches):
    """Copies of the upstream gradient for an in-place backward, made before the timed region: launch i works on
    copy i, so every backward sees the same pristine values instead of the shrinking results of its predecessors
    (dx ~ 0.09 * y * dy: after a few generations the buffer holds zeros, which a plain copy moves ~3 % faster than
    data). Every launch also meets another placement of its gradient buffer, so the average is one over placements.
    As many copies as `launches`, or as fit into the free device memory beside a reserve for the step's own
    results (then the ring wraps and later launches see once-processed data)."""
    free, _ = torch.cuda.mem_get_info(pristine.device)
    per = pristine.numel() * pristine.element_size()
    reserve = max(16 << 30, 6 * per)
    budget = min(free - reserve, 160 << 30)
    count = max(1, min(launches, budget // per))
    ring = [pristine] + [pristine.clone() for _ in range(int(count) - 1)]
    return ring


def make_workload(name, torch, dev, fresh_dy=False, rope_per_tensor=False, launches=1, decaying_dy=False):
    import fused_rotary_positional_embedding as rope_ext
    import scaled_masked_softmax_cuda as masked_ext
    import scaled_upper_triang_masked_softmax_cuda as causal_ext
    from megatron.model.positional_embeddings import RotaryEmbedding

    gen = torch.Generator(device=dev)

    def randn(shape, seed, dtype, std=1.0):
        gen.manual_seed(seed)
        return (torch.randn(shape, generator=gen, device=dev) * std).to(dtype)

    def rope_setup(s, b, h, d, d2, seed):
        q = randn((s, b, h, d), seed, torch.bfloat16)
        k = randn((s, b, h, d), seed + 1, torch.bfloat16)
        dq = randn((s, b, h, d), seed + 2, torch.bfloat16)
        dk = randn((s, b, h, d), seed + 3, torch.bfloat16)
        cos, sin = RotaryEmbedding(d2, s, base=10000, precision=torch.bfloat16)(q, seq_len=s)
        return q, k, dq, dk, cos.contiguous(), sin.contiguous()

    if name in ("pythia-1.4b", "llama2-7b-c5"):
        if name == "pythia-1.4b":
            s, b, h, d, d2 = 2048, 8, 16, 128, 32
        else:
            s, b, h, d, d2 = 8192, 2, 32, 128, 128
        a = b * h
        scale = 1.0 / math.sqrt(d)
        q, k, dq, dk, cos, sin = rope_setup(s, b, h, d, d2, 10)
        x = randn((a, s, s), 0, torch.bfloat16, 2.0)
        dy = randn((a, s, s), 1, torch.bfloat16)
        fwd_b, bwd_b = causal_bytes(a, s)
        rb = rope_bytes(s, b, h, d, d2)
        # q and k share one launch and one read of the tables (--rope-per-tensor: one launch per tensor,
        # the reference's call style, each reading the tables)
        rope_b = 2 * rb if rope_per_tensor else 2 * rb - 2 * s * d2 * 2
        kernel_bytes = {"rope_fwd": rope_b, "causal_softmax_fwd": fwd_b, "causal_softmax_bwd": bwd_b,
                        "rope_bwd": rope_b}
        dense = {"causal_softmax_fwd": 2 * a * s * s * 2, "causal_softmax_bwd": 3 * a * s * s * 2}

        # The backward works in place. By default every launch gets a pristine copy of the upstream gradient from a
        # ring filled beforehand (--decaying-dy: one buffer, each launch works on its predecessor's result).
        ring = [dy] if (decaying_dy or fresh_dy) else grad_ring(torch, dy, launches)
        ring_state = {"i": 0}
        # --fresh-dy: the backward works in place, so without this its input shrinks from step to step
        # (dx ~ 0.09 * y * dy); with it the upstream gradient is restored from a pristine copy before
        # every backward, outside the backward's event bracket (the copy is part of the step's wall time)
        dy0 = dy.clone() if fresh_dy else None

        def step(t):
            def rope_f():
                if rope_per_tensor:
                    rope_ext.forward_cached(q, cos, sin, False)
                    rope_ext.forward_cached(k, cos, sin, False)
                else:
                    rope_ext.forward_cached_qk(q, k, cos, sin, False)

            def rope_b():
                if rope_per_tensor:
                    rope_ext.backward_cached(dq, cos, sin, False)
                    rope_ext.backward_cached(dk, cos, sin, False)
                else:
                    rope_ext.backward_cached_qk(dq, dk, cos, sin, False)

            t.run("rope_fwd", rope_f)
            y = t.run("causal_softmax_fwd", lambda: causal_ext.forward(x, scale))
            g = ring[ring_state["i"] % len(ring)]
            ring_state["i"] += 1
            if fresh_dy:
                g.copy_(dy0)
                t.unchain()
            # in place on the gradient buffer, as the reference does
            t.run("causal_softmax_bwd", lambda: causal_ext.backward(g, y, scale))
            t.run("rope_bwd", rope_b)

        from megatron.fused_kernels import _hotpath as hp

        cfg = {"workload": name, "scores": [a, s, s], "qk": [s, b, h, d], "rotary_dim": d2,
               "scale": "1/sqrt(%d)" % d, "bytes_convention": "causal-min (reads of the lower triangle, dense writes)",
               "dominant_kernel_signature": "softmax_bwd causal " + softmax_signature(hp.lib(), s, 2)}
        cfg["rotary_launches"] = "one per tensor" if rope_per_tensor else "q and k in one launch"
        cfg["upstream_gradient"] = ("restored by a copy before every backward" if fresh_dy else
                                    "one buffer, results fed back (decays to zeros)" if len(ring) == 1 else
                                    f"ring of {len(ring)} pristine copies for {launches} launches")
        return step, kernel_bytes, dense, "causal_softmax_bwd", "bf16", cfg

    if name == "attn-dropout-1.4b":
        a, s = 128, 2048
        scale = 1.0 / math.sqrt(128)
        x = torch.empty((a, s, s), dtype=torch.bfloat16, device=dev)
        dy = torch.empty_like(x)
        for i in range(0, a, 8):
            x[i:i + 8] = randn((8, s, s), i, torch.bfloat16, 2.0)
            dy[i:i + 8] = randn((8, s, s), 1000 + i, torch.bfloat16)
        n = a * s * s
        fwd_b = a * tri(s) * 2 + 2 * n * 2          # triangle read, probabilities and dropped probabilities written
        bwd_b = 2 * a * tri(s) * 2 + n * 2
        kernel_bytes = {"softmax_dropout_fwd": fwd_b, "softmax_dropout_bwd": bwd_b}
        state = {"i": 0}
        ring = [dy] if decaying_dy else grad_ring(torch, dy, launches)

        def step(t):
            state["i"] += 1
            seed = state["i"]
            dropped, y = t.run("softmax_dropout_fwd", lambda: causal_ext.forward_dropout(x, scale, 0.1, seed))
            g = ring[state["i"] % len(ring)]
            t.run("softmax_dropout_bwd", lambda: causal_ext.backward_dropout(g, y, scale, 0.1, seed))

        cfg = {"workload": name, "scores": [a, s, s], "dropout": 0.1, "mask": "regenerated (Philox4x32-10), not stored",
               "bytes_convention": "lower-triangle reads, dense writes (two dense outputs in the forward)"}
        return step, kernel_bytes, {}, "softmax_dropout_fwd", "bf16", cfg

    if name in ("mistral-window", "alibi-1.4b", "rpe-bias-1.4b", "causal-blocks-1.4b", "causal-blocks-7b",
                "mistral-window-blocks"):
        from megatron.model.positional_embeddings import AliBi

        bias = None
        zero_block = 0
        if name in ("mistral-window", "mistral-window-blocks"):
            a, s, window, heads = 64, 8192, 4096, None
            zero_block = 1024 if name.endswith("blocks") else 0
        elif name == "causal-blocks-1.4b":
            a, s, window, heads, zero_block = 128, 2048, None, None, 512
        elif name == "causal-blocks-7b":
            a, s, window, heads, zero_block = 32, 4096, None, None, 1024
        else:
            a, s, window, heads = 128, 2048, None, 16
        scale = 1.0 / math.sqrt(128)
        slopes = None if heads is None else AliBi(heads, mp_size=1, mp_rank=0).slopes.float().to(dev)
        if name == "rpe-bias-1.4b":
            slopes = None
            bias = randn((heads, s, s), 77, torch.bfloat16, 1.0)
        x = torch.empty((a, s, s), dtype=torch.bfloat16, device=dev)
        dy = torch.empty_like(x)
        for i in range(0, a, 8):
            x[i:i + 8] = randn((8, s, s), i, torch.bfloat16, 2.0)
            dy[i:i + 8] = randn((8, s, s), 1000 + i, torch.bfloat16)
        w = s if window is None else window
        band = sum(min(q, w) + 1 for q in range(s))  # keys read per matrix
        written = s * s                               # elements written per matrix
        if zero_block:
            # every row from the block of the first key its block's first row sees to the block of the diagonal
            written = sum((q // zero_block + 1) * zero_block - max(0, q // zero_block * zero_block - w) // zero_block * zero_block
                          for q in range(s))
        fwd_b = a * band * 2 + a * written * 2
        bwd_b = 2 * a * band * 2 + a * written * 2
        if bias is not None:
            fwd_b += heads * band * 2  # each head's bias triangle once; the batch re-reads it from cache
        kernel_bytes = {"causal_softmax_fwd": fwd_b, "causal_softmax_bwd": bwd_b}

        ring = [dy] if decaying_dy else grad_ring(torch, dy, launches)
        ring_state = {"i": 0}

        def step(t):
            y = t.run("causal_softmax_fwd", lambda: causal_ext.forward(x, scale, window, slopes, bias, None, zero_block))
            g = ring[ring_state["i"] % len(ring)]
            ring_state["i"] += 1
            t.run("causal_softmax_bwd", lambda: causal_ext.backward(g, y, scale, window, None, zero_block))

        cfg = {"workload": name, "scores": [a, s, s], "window": window,
               "alibi_heads": None if slopes is None else heads, "bias": None if bias is None else list(bias.shape),
               "bytes_convention": "reads of the attended band, dense writes" if not zero_block else
               f"reads of the attended band, writes of the {zero_block}-column blocks a block-wise caller reads"}
        if zero_block:
            cfg["zero_block"] = zero_block
        from megatron.fused_kernels import _hotpath as hp

        cfg["dominant_kernel_signature"] = "softmax_bwd causal " + softmax_signature(hp.lib(), s, 2) + \
            (f" blocks{zero_block}" if zero_block else "")
        return step, kernel_bytes, {}, "causal_softmax_bwd", "bf16", cfg

    if name == "masked-extras-1.4b":
        # The padding-mask kernel doing what its caller otherwise does in passes of its own: relative-position bias,
        # AliBi and the padding keys of right-padded sequences, under the decoder's causal mask given as a tensor.
        from megatron.model.positional_embeddings import AliBi

        b, np_, s = 8, 16, 2048
        scale = 1.0 / math.sqrt(128)
        x = torch.empty((b, np_, s, s), dtype=torch.bfloat16, device=dev)
        dy = torch.empty_like(x)
        for i in range(b):
            x[i] = randn((np_, s, s), i, torch.bfloat16, 2.0)
            dy[i] = randn((np_, s, s), 1000 + i, torch.bfloat16)
        bias = randn((np_, s, s), 77, torch.bfloat16, 1.0)
        slopes = AliBi(np_, mp_size=1, mp_rank=0).slopes.float().to(dev)
        idx = torch.arange(s, device=dev)
        mask = (idx[None, :] > idx[:, None]).view(1, 1, s, s).contiguous()
        lengths = torch.tensor([2048, 1900, 1024, 2048, 1500, 2000, 777, 2048], dtype=torch.int32, device=dev)
        n = x.numel()
        # 8-key groups with a visible key: those of the triangle that start below the sequence's length
        starts = torch.arange(0, s, 8, device=dev)
        live = ((starts[None, None, :] <= idx[None, :, None]) & (starts[None, None, :] < lengths[:, None, None].long()))
        live_chunks = int(live.sum().item())
        bias_chunks = int((starts[None, :] <= idx[:, None]).sum().item())
        fwd_b = live_chunks * 16 * np_ + bias_chunks * 16 * np_ + mask.numel() + n * 2
        kernel_bytes = {"masked_softmax_ex_fwd": fwd_b, "masked_softmax_bwd": 3 * n * 2}

        ring = [dy] if decaying_dy else grad_ring(torch, dy, launches)
        ring_state = {"i": 0}

        def step(t):
            y = t.run("masked_softmax_ex_fwd", lambda: masked_ext.forward(x, mask, scale, slopes, bias, lengths))
            g = ring[ring_state["i"] % len(ring)]
            ring_state["i"] += 1
            t.run("masked_softmax_bwd", lambda: masked_ext.backward(g, y, scale))

        cfg = {"workload": name, "scores": [b, np_, s, s], "mask": [1, 1, s, s], "alibi_heads": np_, "bias": [np_, s, s],
               "key_lengths": lengths.tolist(),
               "bytes_convention": "forward: 8-key groups with a visible key read + each head's bias groups once + "
                                   "mask once + dense write; backward: 3x tensor"}
        return step, kernel_bytes, {}, "masked_softmax_bwd", "bf16", cfg

    if name in ("masked-c3", "masked-dropout-c3"):
        b, np_, sq, sk = 16, 32, 1024, 2048
        scale = 1.0 / math.sqrt(128)
        x = randn((b, np_, sq, sk), 0, torch.float16, 3.0)
        gen.manual_seed(5)
        hit = torch.rand(x.shape, generator=gen, device=dev) < 0.01
        sign = torch.where(torch.rand(x.shape, generator=gen, device=dev) < 0.5, -60.0, 60.0).half()
        x = torch.where(hit, sign, x)
        del hit, sign
        g = torch.Generator().manual_seed(0)
        valid = torch.randint(512, sk + 1, (b,), generator=g)
        kk = torch.arange(sk)
        mask = (kk[None, :] >= valid[:, None])[:, None, None, :].expand(b, 1, sq, sk).contiguous()
        mask[7] = True
        mask = mask.to(dev)
        dy = randn(x.shape, 1, torch.float16)
        n = x.numel()
        kernel_bytes = {"masked_softmax_fwd": 2 * n * 2 + mask.numel(), "masked_softmax_bwd": 3 * n * 2}
        # what the forward has to move: groups of 8 keys that are all padding are never read
        live_chunks = int((~mask.view(b, sq, sk // 8, 8).all(dim=-1)).sum().item())
        needed = {"masked_softmax_fwd": ("GB/s_unmasked_reads_only", live_chunks * 16 * np_ + mask.numel() + n * 2)}

        ring = [dy] if decaying_dy else grad_ring(torch, dy, launches)
        ring_state = {"i": 0}

        def step(t):
            y = t.run("masked_softmax_fwd", lambda: masked_ext.forward(x, mask, scale))
            g = ring[ring_state["i"] % len(ring)]
            ring_state["i"] += 1
            t.run("masked_softmax_bwd", lambda: masked_ext.backward(g, y, scale))

        if name == "masked-dropout-c3":
            kernel_bytes = {"masked_softmax_dropout_fwd": 3 * n * 2 + mask.numel(), "masked_softmax_dropout_bwd": 3 * n * 2}
            state = {"i": 0}

            def step_dropout(t):
                state["i"] += 1
                seed = 1000 + state["i"]
                _, y = t.run("masked_softmax_dropout_fwd", lambda: masked_ext.forward_dropout(x, mask, scale, 0.1, seed))
                g = ring[state["i"] % len(ring)]
                t.run("masked_softmax_dropout_bwd", lambda: masked_ext.backward_dropout(g, y, scale, 0.1, seed))

            cfg = {"workload": name, "scores": [b, np_, sq, sk], "mask": [b, 1, sq, sk], "dropout": 0.1,
                   "bytes_convention": "dense (tensor read + mask once + probabilities and dropped probabilities written; "
                                       "3x tensor backward)"}
            return step_dropout, kernel_bytes, {}, "masked_softmax_dropout_bwd", "f16", cfg
        from megatron.fused_kernels import _hotpath as hp

        # The forward never reads a group of 8 keys that is all padding (37 % of this workload's keys):
        # its bytes are the reads of the live groups + the mask once + the dense write, which is what the
        # kernel moves; the dense convention (2x tensor) is printed beside it.
        dense_fwd = kernel_bytes["masked_softmax_fwd"]
        kernel_bytes["masked_softmax_fwd"] = needed["masked_softmax_fwd"][1]
        needed = {"masked_softmax_fwd": ("GB/s_dense_convention", dense_fwd)}
        cfg = {"workload": name, "scores": [b, np_, sq, sk], "mask": [b, 1, sq, sk],
               "upstream_gradient": f"ring of {len(ring)} pristine copies for {launches} launches" if len(ring) > 1 else
               "one buffer, results fed back (decays to zeros)",
               "bytes_convention": "forward: unmasked 8-key groups read + mask once + dense write; backward: 3x tensor",
               "dominant_kernel_signature": "softmax_bwd plain " + softmax_signature(hp.lib(), sk, 4)}
        return step, kernel_bytes, needed, "masked_softmax_bwd", "f16", cfg

    if name == "hbm-probes":
        import ctypes

        from megatron.fused_kernels import _hotpath as hp

        path = os.path.join(ROOT, "bench_probes", "libneox_probe.so")
        plib = ctypes.CDLL(path)
        vp, i64 = ctypes.c_void_p, ctypes.c_int64
        plib.nhp_probe_copy.argtypes = [vp, vp, i64, ctypes.c_int, vp]
        plib.nhp_probe_causal_pattern.argtypes = [vp, vp, i64, i64, vp]
        kernel_bytes = {}
        runs = []
        for mib in (16, 64, 128, 1024):  # 16 MiB: the tensor size of the [4,8,512,512] configuration
            nsets = max(2, 1024 // mib)  # rotate over more than the last-level cache holds
            # random data: what the bytes hold changes the time measurably (a copy of zeros is ~3 % faster)
            bufs = [(randn((mib << 19,), 300 + j, torch.bfloat16),
                     torch.empty((mib << 19,), dtype=torch.bfloat16, device=dev)) for j in range(nsets)]
            key = f"copy_{mib}MiB"
            kernel_bytes[key] = 2 * (mib << 20)
            runs.append((key, bufs, mib))
        pat = []
        for a, s in ((128, 2048), (64, 8192)):
            x = torch.empty((a, s, s), dtype=torch.bfloat16, device=dev)
            for j in range(a):
                x[j] = randn((s, s), 400 + j, torch.bfloat16)
            y = torch.empty_like(x)
            key = f"causal_pattern_{a}x{s}x{s}"
            kernel_bytes[key] = causal_bytes(a, s)[0]
            pat.append((key, x, y, a, s))
        plib.nhp_probe_causal_bwd_pattern.argtypes = [vp, vp, i64, i64, vp]
        for _, _, _, a, s in pat:
            kernel_bytes[f"causal_bwd_pattern_{a}x{s}x{s}"] = causal_bytes(a, s)[1]
        # the padding-mask forward's pattern on the tensors of masked-c3 (scores [16,32,1024,2048], 37 % padding keys)
        plib.nhp_probe_masked_pattern.argtypes = [vp, vp, vp, i64, i64, i64, vp]
        mb, mnp, msq, msk = 16, 32, 1024, 2048
        g0 = torch.Generator().manual_seed(0)
        mvalid = torch.randint(512, msk + 1, (mb,), generator=g0)
        mmask = (torch.arange(msk)[None, :] >= mvalid[:, None])[:, None, None, :].expand(mb, 1, msq, msk).contiguous()
        mmask[7] = True
        mmask = mmask.to(dev)
        mlive = int((~mmask.view(mb, msq, msk // 8, 8).all(dim=-1)).sum().item())
        mx = pat[1][1].view(-1)[: mb * mnp * msq * msk].view(mb, mnp, msq, msk)   # 2 GiB of the 8 GiB random tensor
        my = pat[1][2].view(-1)[: mb * mnp * msq * msk].view(mb, mnp, msq, msk)
        kernel_bytes["masked_pattern_16x32x1024x2048"] = mlive * 16 * mnp + mmask.numel() + mx.numel() * 2
        plib.nhp_probe_seq_major_pattern.argtypes = [vp, vp, i64, i64, vp]
        plib.nhp_probe_streams.argtypes = [vp, vp, vp, vp, i64, ctypes.c_int, ctypes.c_int, vp]
        # 64 MiB streams (the hidden state [16384, 2048] bf16 of the layer kernels): n inputs -> one or no output
        mixes = [("read_64MiB", 1, 0), ("write_64MiB", 0, 1), ("read2_write1_64MiB", 2, 1), ("read3_write1_64MiB", 3, 1)]
        mix_bufs = [[randn((64 << 19,), 600 + 4 * i + j, torch.bfloat16) for j in range(4)] for i in range(4)]
        for key, n_in, w in mixes:
            kernel_bytes[key] = (n_in + w) * (64 << 20)
        # the backward's stream mix at its real footprints: two inputs, the result written over the first
        # (on the tensors of the pattern probes: 1 GiB each, and 4 and 8 GiB of the 8 GiB ones)
        inplace = [("read2_write1_in_place_1GiB", 0, 1 << 30), ("read2_write1_in_place_4GiB", 1, 4 << 30),
                   ("read2_write1_in_place_8GiB", 1, 8 << 30)]
        for key, _, nbytes in inplace:
            kernel_bytes[key] = 3 * nbytes
        # the key gradient's layout change at the Pythia-1.4B shape: [b*h = 128, d = 128, s = 2048] -> [s, b*h, d]
        tr_rows, tr_s = 128, 2048
        tr_bufs = [(randn((tr_rows, 128, tr_s), 500 + j, torch.bfloat16),
                    torch.empty((tr_s, tr_rows, 128), dtype=torch.bfloat16, device=dev)) for j in range(8)]
        kernel_bytes["seq_major_pattern_128x128x2048"] = 2 * tr_rows * 128 * tr_s * 2
        # q and k as slices of a fused projection buffer [4096, 4, 32, 3 * 128] bf16: 256-byte head vectors 768 bytes
        # apart copied to one contiguous tensor (one tensor per launch), and 512-byte (q|k) runs split over two
        plib.nhp_probe_strided_runs.argtypes = [vp, vp, vp, i64, ctypes.c_int, i64, ctypes.c_int, vp]
        qkv_rows = 4096 * 4 * 32
        qkv_bufs = [(randn((qkv_rows, 384), 650 + j, torch.bfloat16),
                     torch.empty((qkv_rows, 128), dtype=torch.bfloat16, device=dev),
                     torch.empty((qkv_rows, 128), dtype=torch.bfloat16, device=dev)) for j in range(3)]
        kernel_bytes["strided_256_of_768_bytes_128MiB"] = 2 * qkv_rows * 256
        kernel_bytes["strided_512_of_768_bytes_split_2x128MiB"] = 4 * qkv_rows * 256
        state = {"i": 0}
        stream = hp.stream_of(pat[0][1])

        def step(t):
            state["i"] += 1
            src, o0, o1 = qkv_bufs[state["i"] % len(qkv_bufs)]
            t.run("strided_256_of_768_bytes_128MiB", lambda: hp.check(plib.nhp_probe_strided_runs(
                o0.data_ptr(), None, src.data_ptr(), qkv_rows, 16, 48, 0, stream), "strided runs"))
            t.run("strided_512_of_768_bytes_split_2x128MiB", lambda: hp.check(plib.nhp_probe_strided_runs(
                o0.data_ptr(), o1.data_ptr(), src.data_ptr(), qkv_rows, 32, 48, 1, stream), "strided runs, split"))
            for key, bufs, mib in runs:
                src, dst = bufs[state["i"] % len(bufs)]
                t.run(key, lambda: hp.check(plib.nhp_probe_copy(dst.data_ptr(), src.data_ptr(), mib << 20, 256, stream), key))
            for key, x, y, a, s in pat:
                t.run(key, lambda: hp.check(plib.nhp_probe_causal_pattern(y.data_ptr(), x.data_ptr(), a, s, stream), key))
            for _, x, y, a, s in pat:
                # two triangles read, the first tensor's rows overwritten (XOR of random data stays random)
                t.run(f"causal_bwd_pattern_{a}x{s}x{s}", lambda: hp.check(
                    plib.nhp_probe_causal_bwd_pattern(y.data_ptr(), x.data_ptr(), a, s, stream), "causal bwd pattern"))
            t.run("masked_pattern_16x32x1024x2048", lambda: hp.check(plib.nhp_probe_masked_pattern(
                my.data_ptr(), mx.data_ptr(), mmask.data_ptr(), mb, mnp, msq, stream), "masked pattern"))
            bufs4 = mix_bufs[state["i"] % len(mix_bufs)]
            for key, n_in, w in mixes:
                t.run(key, lambda: hp.check(plib.nhp_probe_streams(bufs4[3].data_ptr(), bufs4[0].data_ptr(), bufs4[1].data_ptr(),
                                                                   bufs4[2].data_ptr(), 64 << 20, n_in, w, stream), key))
            for key, which, nbytes in inplace:
                _, x, y, _, _ = pat[which]
                t.run(key, lambda: hp.check(plib.nhp_probe_streams(y.data_ptr(), y.data_ptr(), x.data_ptr(), x.data_ptr(),
                                                                   nbytes, 2, 1, stream), key))
            src, dst = tr_bufs[state["i"] % len(tr_bufs)]
            t.run("seq_major_pattern_128x128x2048", lambda: hp.check(
                plib.nhp_probe_seq_major_pattern(dst.data_ptr(), src.data_ptr(), tr_rows, tr_s, stream), "seq_major_pattern"))

        cfg = {"workload": name, "what": "data movement only; bytes as the kernels they stand for are priced"}
        return step, kernel_bytes, {}, "copy_1024MiB", "u8", cfg

    if name == "causal-c1":
        # scores [b=4, h=8, 512, 512] bf16 ~ N(0, 4), scale 1/sqrt(64): 16 MiB per tensor, so the launches rotate over
        # 16 buffer pairs (512 MiB in all, twice the last-level cache). A launch lasts a few microseconds, less
        # than the host needs to issue it: each bracket holds 16 launches issued while the GPU is still busy
        # with a 1 GiB copy, so that they run back to back and the bracket measures the GPU's time.
        a, s = 32, 512
        scale = 1.0 / math.sqrt(64)
        sets = [randn((a, s, s), 700 + i, torch.bfloat16, 2.0) for i in range(16)]
        filler = (torch.empty(1 << 29, dtype=torch.bfloat16, device=dev), torch.empty(1 << 29, dtype=torch.bfloat16, device=dev))
        fwd_b, _ = causal_bytes(a, s)
        kernel_bytes = {"causal_softmax_fwd": 16 * fwd_b}

        def step(t):
            filler[1].copy_(filler[0])
            t.run("causal_softmax_fwd", lambda: [causal_ext.forward(x, scale) for x in sets])

        cfg = {"workload": name, "scores": [a, s, s], "scale": "1/sqrt(64)", "launches_per_bracket": 16,
               "bytes_convention": "causal-min (reads of the lower triangle, dense writes)"}
        return step, kernel_bytes, {"causal_softmax_fwd": 16 * 2 * a * s * s * 2}, "causal_softmax_fwd", "bf16", cfg

    if name == "rope-styles-1.4b":
        # the rotary leg of the default workload in both call styles: one launch per tensor (the reference's
        # fused_apply_rotary_pos_emb_cached, called for q and then for k) and q and k in one launch
        s, b, h, d, d2 = 2048, 8, 16, 128, 32
        sets = [rope_setup(s, b, h, d, d2, 50 + 10 * i) for i in range(4)]
        rb = rope_bytes(s, b, h, d, d2)
        one = 2 * rb - 2 * s * d2 * 2
        kernel_bytes = {"rope_fwd_per_tensor": 2 * rb, "rope_bwd_per_tensor": 2 * rb, "rope_fwd_one_launch": one,
                        "rope_bwd_one_launch": one}
        state = {"i": 0}

        def step(t):
            q, k, dq, dk, cos, sin = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("rope_fwd_per_tensor", lambda: (rope_ext.forward_cached(q, cos, sin, False),
                                                  rope_ext.forward_cached(k, cos, sin, False)))
            t.run("rope_bwd_per_tensor", lambda: (rope_ext.backward_cached(dq, cos, sin, False),
                                                  rope_ext.backward_cached(dk, cos, sin, False)))
            t.run("rope_fwd_one_launch", lambda: rope_ext.forward_cached_qk(q, k, cos, sin, False))
            t.run("rope_bwd_one_launch", lambda: rope_ext.backward_cached_qk(dq, dk, cos, sin, False))

        cfg = {"workload": name, "qk": [s, b, h, d], "rotary_dim": d2}
        return step, kernel_bytes, {}, "rope_fwd_per_tensor", "bf16", cfg

    if name == "rope-qk-1.4b":
        s, b, h, d, d2 = 2048, 8, 16, 128, 32
        sets = [rope_setup(s, b, h, d, d2, 50 + 10 * i) for i in range(4)]  # rotate buffers: 64 MiB tensors fit the cache
        rb = rope_bytes(s, b, h, d, d2)
        kernel_bytes = {"rope_qk_fwd": 2 * rb - 2 * s * d2 * 2, "rope_qk_bwd": 2 * rb - 2 * s * d2 * 2}
        state = {"i": 0}

        def step(t):
            q, k, dq, dk, cos, sin = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("rope_qk_fwd", lambda: rope_ext.forward_cached_qk(q, k, cos, sin, False))
            t.run("rope_qk_bwd", lambda: rope_ext.backward_cached_qk(dq, dk, cos, sin, False))

        cfg = {"workload": name, "qk": [s, b, h, d], "rotary_dim": d2}
        return step, kernel_bytes, {}, "rope_qk_fwd", "bf16", cfg

    if name == "rope-neox-20b":
        # the 20B configuration of the reference (configs/20B.yml): 64 heads of 96, rotary_pct 0.25 -> 24 rotary
        # dimensions, whose half (12) is not a whole number of 16-byte chunks
        s, b, h, d, d2 = 2048, 4, 64, 96, 24
        sets = [rope_setup(s, b, h, d, d2, 70 + 10 * i) for i in range(4)]
        rb = rope_bytes(s, b, h, d, d2)
        kernel_bytes = {"rope_fwd": rb, "rope_bwd": rb, "rope_qk_fwd": 2 * rb - 2 * s * d2 * 2, "rope_qk_bwd": 2 * rb - 2 * s * d2 * 2}
        state = {"i": 0}

        def step(t):
            q, k, dq, dk, cos, sin = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("rope_fwd", lambda: rope_ext.forward_cached(q, cos, sin, False))
            t.run("rope_bwd", lambda: rope_ext.backward_cached(dq, cos, sin, False))
            t.run("rope_qk_fwd", lambda: rope_ext.forward_cached_qk(q, k, cos, sin, False))
            t.run("rope_qk_bwd", lambda: rope_ext.backward_cached_qk(dq, dk, cos, sin, False))

        cfg = {"workload": name, "qk": [s, b, h, d], "rotary_dim": d2}
        return step, kernel_bytes, {}, "rope_qk_fwd", "bf16", cfg

    if name == "rope-freqs-1.4b":
        # the entry points that take the angles and evaluate sin/cos on the device (fused_apply_rotary_pos_emb)
        s, b, h, d, d2 = 2048, 8, 16, 128, 32
        sets = [rope_setup(s, b, h, d, d2, 50 + 10 * i) for i in range(4)]
        inv_freq = 1.0 / (10000 ** (torch.arange(0, d2, 2, device=dev, dtype=torch.float32) / d2))
        ang = torch.outer(torch.arange(s, device=dev, dtype=torch.float32), inv_freq)
        freqs = torch.cat((ang, ang), dim=-1).view(s, 1, 1, d2).contiguous()
        per = 2 * s * b * h * d * 2 + s * d2 * 4  # tensor in and out + the fp32 angles
        kernel_bytes = {"rope_freqs_fwd": per, "rope_freqs_bwd": per, "rope_freqs_qk_fwd": 2 * per - s * d2 * 4,
                        "rope_freqs_qk_bwd": 2 * per - s * d2 * 4, "rope_freqs_bwd_seq_major": per}
        # a gradient that is contiguous along the sequence, as in rope-kgrad-1.4b
        gsm = [randn((b, h, d, s), 120 + i, torch.bfloat16).permute(3, 0, 1, 2) for i in range(4)]
        state = {"i": 0}

        def step(t):
            q, k, dq, dk, _, _ = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("rope_freqs_fwd", lambda: rope_ext.forward(q, freqs, False))
            t.run("rope_freqs_bwd", lambda: rope_ext.backward(dq, freqs, False))
            t.run("rope_freqs_qk_fwd", lambda: rope_ext.forward_qk(q, k, freqs, False))
            t.run("rope_freqs_qk_bwd", lambda: rope_ext.backward_qk(dq, dk, freqs, False))
            g = gsm[state["i"] % len(gsm)]
            t.run("rope_freqs_bwd_seq_major", lambda: rope_ext.backward(g, freqs, False))

        cfg = {"workload": name, "t": [s, b, h, d], "rotary_dim": d2, "angles": "fp32 [s,1,1,rotary_dim], sin/cos on the device"}
        return step, kernel_bytes, {}, "rope_freqs_qk_fwd", "bf16", cfg

    if name == "mlp-gelu-1.4b":
        # through the C ABI with preallocated outputs and workspace
        from megatron.fused_kernels import _hotpath as hp

        lib = hp.lib()
        rows, cols = 2048 * 8, 8192
        sets = []
        for i in range(2):  # two buffer sets: a 256 MiB tensor alone would sit in the last-level cache
            y = torch.empty((rows, cols), dtype=torch.bfloat16, device=dev)
            g = torch.empty_like(y)
            for r in range(0, rows, 2048):
                y[r:r + 2048] = randn((2048, cols), 100 * i + r, torch.bfloat16, 2.0)
                g[r:r + 2048] = randn((2048, cols), 100 * i + r + 1, torch.bfloat16)
            sets.append((y, g))
        bias = randn((cols,), 5, torch.bfloat16, 0.5)
        out = torch.empty_like(sets[0][0])
        dbias = torch.empty_like(bias)
        ws = torch.empty(max(lib.nhp_bias_gelu_bwd_workspace_bytes(rows, cols, hp.BF16), 16), dtype=torch.uint8, device=dev)
        n = rows * cols
        kernel_bytes = {"bias_gelu_fwd": 2 * n * 2 + cols * 2, "bias_gelu_bwd": 3 * n * 2 + 2 * cols * 2}
        state = {"i": 0}
        stream = hp.stream_of(out)

        def fwd(y):
            hp.check(lib.nhp_bias_gelu_fwd(out.data_ptr(), y.data_ptr(), bias.data_ptr(), rows, cols, hp.BF16, stream),
                     "bias_gelu forward")

        def bwd(y, g):
            hp.check(lib.nhp_bias_gelu_bwd(out.data_ptr(), g.data_ptr(), y.data_ptr(), bias.data_ptr(), dbias.data_ptr(),
                                           ws.data_ptr(), rows, cols, hp.BF16, stream), "bias_gelu backward")

        def step(t):
            y, g = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("bias_gelu_fwd", lambda: fwd(y))
            t.run("bias_gelu_bwd", lambda: bwd(y, g))

        cfg = {"workload": name, "activation": [rows, cols], "bias_gradient": "fused column sums",
               "bytes_convention": "every tensor element read or written once"}
        return step, kernel_bytes, {}, "bias_gelu_bwd", "bf16", cfg

    if name == "swiglu-7b":
        from megatron.fused_kernels import _hotpath as hp

        lib = hp.lib()
        rows, f = 4096 * 4, 11008
        inp = torch.empty((rows, 2 * f), dtype=torch.bfloat16, device=dev)   # 688 MiB: larger than the last-level cache
        for r in range(0, rows, 2048):
            inp[r:r + 2048] = randn((2048, 2 * f), r, torch.bfloat16, 2.0)
        dy = randn((rows, f), 3, torch.bfloat16)
        out = torch.empty((rows, f), dtype=torch.bfloat16, device=dev)
        din = torch.empty_like(inp)
        n = rows * f
        kernel_bytes = {"swiglu_fwd": 3 * n * 2, "swiglu_bwd": 5 * n * 2}
        stream = hp.stream_of(out)

        def step(t):
            t.run("swiglu_fwd", lambda: hp.check(lib.nhp_gated_act_fwd(out.data_ptr(), inp.data_ptr(), None, rows, f, 0,
                                                                       hp.BF16, stream), "swiglu forward"))
            t.run("swiglu_bwd", lambda: hp.check(lib.nhp_gated_act_bwd(din.data_ptr(), dy.data_ptr(), inp.data_ptr(), None,
                                                                       rows, f, 0, hp.BF16, stream), "swiglu backward"))

        cfg = {"workload": name, "input": [rows, 2 * f], "output": [rows, f],
               "bytes_convention": "every tensor element read or written once"}
        return step, kernel_bytes, {}, "swiglu_bwd", "bf16", cfg

    if name in ("layernorm-1.4b", "rmsnorm-7b"):
        # through the C ABI with preallocated outputs: these kernels run for a few tens of
        # microseconds, less than the autograd bookkeeping around a module call
        from megatron.fused_kernels import _hotpath as hp

        lib = hp.lib()
        layer = name == "layernorm-1.4b"
        rows, cols = (2048 * 8, 2048) if layer else (4096 * 4, 4096)
        nsets = 6 if layer else 3  # rotate buffers so that they come from HBM
        sets = [(randn((rows, cols), 10 * i, torch.bfloat16, 2.0), randn((rows, cols), 10 * i + 1, torch.bfloat16))
                for i in range(nsets)]
        gamma = randn((cols,), 91, torch.bfloat16) + 1
        beta = randn((cols,), 92, torch.bfloat16)
        y = torch.empty_like(sets[0][0])
        dx = torch.empty_like(y)
        mean = torch.empty(rows, dtype=torch.float32, device=dev)
        rstd = torch.empty_like(mean)
        dgamma, dbeta = torch.empty_like(gamma), torch.empty_like(beta)
        ws = torch.empty(max(lib.nhp_norm_bwd_workspace_bytes(rows, cols, hp.BF16), 16), dtype=torch.uint8, device=dev)
        n = rows * cols
        stats = rows * 4 * (2 if layer else 1)
        nparam = 2 if layer else 1
        kernel_bytes = {"norm_fwd": 2 * n * 2 + nparam * cols * 2 + stats,
                        "norm_bwd": 3 * n * 2 + stats + (1 + nparam) * cols * 2,
                        "norm_bwd_frozen_parameters": 3 * n * 2 + stats + cols * 2}
        state = {"i": 0}
        stream = hp.stream_of(y)

        def fwd(x):
            if layer:
                rc = lib.nhp_layernorm_fwd(y.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), gamma.data_ptr(),
                                           beta.data_ptr(), 1e-5, rows, cols, hp.BF16, hp.BF16, stream)
            else:
                rc = lib.nhp_rmsnorm_fwd(y.data_ptr(), rstd.data_ptr(), x.data_ptr(), gamma.data_ptr(), None, 1e-8, 1,
                                         rows, cols, hp.BF16, hp.BF16, stream)
            hp.check(rc, "norm forward")

        def bwd(x, g, params=True):
            # params = False: the gradient of the input alone (frozen or absent parameters): another instantiation,
            # one row block per workgroup, no column sums
            dg, db = (dgamma.data_ptr(), dbeta.data_ptr()) if params else (None, None)
            if layer:
                rc = lib.nhp_layernorm_bwd(dx.data_ptr(), dg, db, g.data_ptr(), x.data_ptr(),
                                           mean.data_ptr(), rstd.data_ptr(), gamma.data_ptr(), ws.data_ptr(), rows, cols,
                                           hp.BF16, hp.BF16, stream)
            else:
                rc = lib.nhp_rmsnorm_bwd(dx.data_ptr(), dg, None, g.data_ptr(), x.data_ptr(), rstd.data_ptr(),
                                         gamma.data_ptr(), ws.data_ptr(), 1e-8, 1, rows, cols, hp.BF16, hp.BF16, stream)
            hp.check(rc, "norm backward")

        def step(t):
            x, g = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("norm_fwd", lambda: fwd(x))
            t.run("norm_bwd", lambda: bwd(x, g))
            t.run("norm_bwd_frozen_parameters", lambda: bwd(x, g, False))

        cfg = {"workload": name, "hidden_state": [rows, cols], "parameters": "bf16", "parameter_gradients": True,
               "bytes_convention": "every tensor element read or written once, plus the fp32 row statistics"}
        return step, kernel_bytes, {}, "norm_bwd", "bf16", cfg

    if name == "layernorm-pair-1.4b":
        from megatron.fused_kernels import _hotpath as hp

        lib = hp.lib()
        rows, cols = 2048 * 8, 2048
        sets = [(randn((rows, cols), 10 * i, torch.bfloat16, 2.0), randn((rows, cols), 10 * i + 1, torch.bfloat16),
                 randn((rows, cols), 10 * i + 2, torch.bfloat16)) for i in range(5)]
        gammas = [randn((cols,), 91 + i, torch.float32) + 1 for i in range(2)]
        betas = [randn((cols,), 95 + i, torch.float32) for i in range(2)]
        y1, y2, dx = (torch.empty_like(sets[0][0]) for _ in range(3))
        mean = torch.empty(rows, dtype=torch.float32, device=dev)
        rstd = torch.empty_like(mean)
        grads = [torch.empty_like(gammas[0]) for _ in range(4)]
        ws = torch.empty(max(lib.nhp_layernorm_pair_bwd_workspace_bytes(rows, cols, hp.BF16), 16), dtype=torch.uint8,
                         device=dev)
        n = rows * cols
        kernel_bytes = {"norm_pair_fwd": 3 * n * 2 + 4 * cols * 4 + rows * 8,
                        "norm_pair_bwd": 4 * n * 2 + rows * 8 + 6 * cols * 4}
        state = {"i": 0}
        stream = hp.stream_of(y1)

        def step(t):
            x, g1, g2 = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("norm_pair_fwd", lambda: hp.check(lib.nhp_layernorm_pair_fwd(
                y1.data_ptr(), y2.data_ptr(), mean.data_ptr(), rstd.data_ptr(), x.data_ptr(), gammas[0].data_ptr(),
                betas[0].data_ptr(), gammas[1].data_ptr(), betas[1].data_ptr(), 1e-5, rows, cols, hp.BF16, hp.F32, stream),
                "LayerNorm pair forward"))
            t.run("norm_pair_bwd", lambda: hp.check(lib.nhp_layernorm_pair_bwd(
                dx.data_ptr(), grads[0].data_ptr(), grads[1].data_ptr(), grads[2].data_ptr(), grads[3].data_ptr(),
                g1.data_ptr(), g2.data_ptr(), x.data_ptr(), mean.data_ptr(), rstd.data_ptr(), gammas[0].data_ptr(),
                gammas[1].data_ptr(), ws.data_ptr(), rows, cols, hp.BF16, hp.F32, stream), "LayerNorm pair backward"))

        cfg = {"workload": name, "hidden_state": [rows, cols], "parameters": "fp32", "parameter_gradients": True,
               "bytes_convention": "every tensor element read or written once, plus the fp32 row statistics"}
        return step, kernel_bytes, {}, "norm_pair_bwd", "bf16", cfg

    if name == "bias-dropout-add-1.4b":
        from megatron.fused_kernels import _hotpath as hp

        lib = hp.lib()
        rows, cols = 2048 * 8, 2048
        sets = [(randn((rows, cols), 10 * i, torch.bfloat16, 2.0), randn((rows, cols), 10 * i + 1, torch.bfloat16, 2.0))
                for i in range(6)]
        bias = randn((cols,), 7, torch.bfloat16)
        out = torch.empty_like(sets[0][0])
        n = rows * cols
        kernel_bytes = {"bias_dropout_add": 3 * n * 2 + cols * 2, "dropout_bwd": 2 * n * 2}
        state = {"i": 0}
        stream = hp.stream_of(out)

        def step(t):
            x, res = sets[state["i"] % len(sets)]
            state["i"] += 1
            seed = 1000 + state["i"]
            t.run("bias_dropout_add", lambda: hp.check(lib.nhp_bias_dropout_add(
                out.data_ptr(), x.data_ptr(), bias.data_ptr(), res.data_ptr(), rows, cols, 0.1, seed, 0, hp.BF16, stream),
                "bias_dropout_add"))
            t.run("dropout_bwd", lambda: hp.check(lib.nhp_dropout_bwd(out.data_ptr(), res.data_ptr(), rows, cols, 0.1, seed,
                                                                      0, hp.BF16, stream), "dropout_bwd"))

        cfg = {"workload": name, "hidden_state": [rows, cols], "dropout": 0.1, "mask": "regenerated (Philox4x32-10), not stored"}
        return step, kernel_bytes, {}, "bias_dropout_add", "bf16", cfg

    if name == "bias-residual-pair-1.4b":
        from megatron.fused_kernels import _hotpath as hp

        lib = hp.lib()
        rows, cols = 2048 * 8, 2048
        sets = [tuple(randn((rows, cols), 10 * i + j, torch.bfloat16, 2.0) for j in range(3)) for i in range(5)]
        b1, b2 = randn((cols,), 7, torch.bfloat16), randn((cols,), 8, torch.bfloat16)
        out = torch.empty_like(sets[0][0])
        kernel_bytes = {"bias_add_residual_pair": 4 * rows * cols * 2 + 2 * cols * 2}
        state = {"i": 0}
        stream = hp.stream_of(out)

        def step(t):
            x1, x2, res = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("bias_add_residual_pair", lambda: hp.check(lib.nhp_bias_add_residual_pair(
                out.data_ptr(), x1.data_ptr(), b1.data_ptr(), x2.data_ptr(), b2.data_ptr(), res.data_ptr(), rows, cols,
                hp.BF16, stream), "bias_add_residual_pair"))

        cfg = {"workload": name, "hidden_state": [rows, cols],
               "bytes_convention": "three tensors read, one written, the two biases"}
        return step, kernel_bytes, {}, "bias_add_residual_pair", "bf16", cfg

    if name == "bias-residual-1.4b":
        from megatron.model.fused_bias_dropout import bias_dropout_add_fused_inference

        rows, cols = 2048 * 8, 2048
        sets = [(randn((rows, cols), 10 * i, torch.bfloat16, 2.0), randn((rows, cols), 10 * i + 1, torch.bfloat16, 2.0))
                for i in range(6)]  # 64 MiB tensors: rotate so that they come from HBM
        bias = randn((cols,), 7, torch.bfloat16)
        kernel_bytes = {"bias_add_residual": 3 * rows * cols * 2 + cols * 2}
        state = {"i": 0}

        def step(t):
            x, res = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("bias_add_residual", lambda: bias_dropout_add_fused_inference(x, bias, res, 0.0))

        cfg = {"workload": name, "hidden_state": [rows, cols]}
        return step, kernel_bytes, {}, "bias_add_residual", "bf16", cfg

    if name == "rope-c4-qkv-view":
        s, b, h, d, d2 = 4096, 4, 32, 128, 128
        sets = []
        for i in range(3):  # rotate through distinct buffers
            qkv = randn((s, b, h, 3 * d), 80 + i, torch.bfloat16)
            dqkv = randn((s, b, h, 3 * d), 90 + i, torch.bfloat16)
            cos, sin = RotaryEmbedding(d2, s, base=10000, precision=torch.bfloat16)(qkv, seq_len=s)
            sets.append((qkv[..., :d], qkv[..., d:2 * d], dqkv[..., :d], dqkv[..., d:2 * d], cos.contiguous(), sin.contiguous()))
        rb = rope_bytes(s, b, h, d, d2)
        one_launch = 2 * rb - 2 * s * d2 * 2   # the tables are read once for q and k
        kernel_bytes = {"rope_fwd_view": 2 * rb, "rope_bwd_view": 2 * rb, "rope_qk_fwd_view": one_launch,
                        "rope_qk_bwd_view": one_launch}
        state = {"i": 0}

        def step(t):
            q, k, dq, dk, cos, sin = sets[state["i"] % len(sets)]
            state["i"] += 1

            def f():
                rope_ext.forward_cached(q, cos, sin, False)
                rope_ext.forward_cached(k, cos, sin, False)

            def bw():
                rope_ext.backward_cached(dq, cos, sin, False)
                rope_ext.backward_cached(dk, cos, sin, False)

            t.run("rope_fwd_view", f)
            t.run("rope_bwd_view", bw)
            # the same through the two-tensor entry point: q and k in one launch
            t.run("rope_qk_fwd_view", lambda: rope_ext.forward_cached_qk(q, k, cos, sin, False))
            t.run("rope_qk_bwd_view", lambda: rope_ext.backward_cached_qk(dq, dk, cos, sin, False))

        cfg = {"workload": name, "qk": [s, b, h, d], "qk_strides": list(sets[0][0].stride()), "rotary_dim": d2}
        return step, kernel_bytes, {}, "rope_fwd_view", "bf16", cfg

    if name == "rope-kgrad-1.4b":
        s, b, h, d, d2 = 2048, 8, 16, 128, 32
        sets = []
        for i in range(4):  # rotate buffers: 64 MiB tensors fit the cache
            g = randn((b, h, d, s), 120 + i, torch.bfloat16).permute(3, 0, 1, 2)   # [s, b, h, d], contiguous along s
            cos, sin = RotaryEmbedding(d2, s, base=10000, precision=torch.bfloat16)(g, seq_len=s)
            sets.append((g, cos.contiguous(), sin.contiguous()))
        kernel_bytes = {"rope_bwd_seq_major": rope_bytes(s, b, h, d, d2)}
        state = {"i": 0}

        def step(t):
            g, cos, sin = sets[state["i"] % len(sets)]
            state["i"] += 1
            t.run("rope_bwd_seq_major", lambda: rope_ext.backward_cached(g, cos, sin, False))

        cfg = {"workload": name, "grad": [s, b, h, d], "grad_strides": list(sets[0][0].stride()), "rotary_dim": d2}
        return step, kernel_bytes, {}, "rope_bwd_seq_major", "bf16", cfg

    if name == "rope-c4":
        s, b, h, d = 4096, 4, 32, 128
        sets = []
        for i, d2 in enumerate((128, 32, 128, 32)):  # rotate through distinct buffers: 128 MiB tensors fit the 256 MB cache
            sets.append((d2,) + rope_setup(s, b, h, d, d2, 20 + 10 * i))
        kernel_bytes = {"rope_fwd_d2_128": 2 * rope_bytes(s, b, h, d, 128), "rope_bwd_d2_128": 2 * rope_bytes(s, b, h, d, 128),
                        "rope_fwd_d2_32": 2 * rope_bytes(s, b, h, d, 32), "rope_bwd_d2_32": 2 * rope_bytes(s, b, h, d, 32)}
        state = {"i": 0}

        def step(t):
            for _ in range(2):
                d2, q, k, dq, dk, cos, sin = sets[state["i"] % len(sets)]
                state["i"] += 1

                def f():
                    rope_ext.forward_cached(q, cos, sin, False)
                    rope_ext.forward_cached(k, cos, sin, False)

                def bw():
                    rope_ext.backward_cached(dq, cos, sin, False)
                    rope_ext.backward_cached(dk, cos, sin, False)

                t.run(f"rope_fwd_d2_{d2}", f)
                t.run(f"rope_bwd_d2_{d2}", bw)

        cfg = {"workload": name, "qk": [s, b, h, d], "rotary_dims": [128, 32]}
        return step, kernel_bytes, {}, "rope_fwd_d2_128", "bf16", cfg

    raise SystemExit(f"unknown workload {name}")


def cpu_baseline(torch):
    """The reference's torch fallback on the host cores, on 1/8 of the default
    workload (one batch entry: scores [1,16,2048,2048], q/k [2048,1,16,128])."""
    from oracle import fallback_semantics as fb

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    s, h, d, d2 = 2048, 16, 128, 32
    scale = 1.0 / math.sqrt(d)
    g = torch.Generator().manual_seed(0)
    x = (torch.randn((1, h, s, s), generator=g) * 2).bfloat16()
    dy = torch.randn((1, h, s, s), generator=g).bfloat16()
    q = torch.randn((s, 1, h, d), generator=g).bfloat16()
    k = torch.randn((s, 1, h, d), generator=g).bfloat16()
    dq = torch.randn((s, 1, h, d), generator=g).bfloat16()
    cos, sin, _ = fb.rotary_tables(d2, s, 10000, torch.bfloat16)
    mask = fb.causal_mask(s)

    def one():
        qq = q.clone().requires_grad_(True)
        kk = k.clone().requires_grad_(True)
        oq = fb.eager_rotary_partial(qq, cos, sin)
        ok = fb.eager_rotary_partial(kk, cos, sin)
        xx = x.clone().requires_grad_(True)
        y = fb.torch_softmax_fallback(xx, mask, scale)
        y.backward(dy)
        torch.autograd.backward([oq, ok], [dq, dq])

    one()  # warm-up
    times = []
    t_end = time.perf_counter() + 12.0  # about 12 s of CPU work
    while len(times) < 3 or time.perf_counter() < t_end:
        t0 = time.perf_counter()
        one()
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    fwd_b, bwd_b = causal_bytes(h, s)
    nbytes = fwd_b + bwd_b + 4 * rope_bytes(s, 1, h, d, d2)
    model = "unknown CPU"
    try:
        with open("/proc/cpuinfo") as f:
            model = next((line.split(":", 1)[1].strip() for line in f if line.startswith("model name")), model)
    except OSError:
        pass
    return {"value": round(nbytes / med / 1e9, 3), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "cpu": f"{model} ({os.cpu_count()} logical cores visible)",
            "sample": "reference torch fallback (fp32 softmax via autograd, eager rotary) on 1/8 of the default "
                      f"workload: scores [1,16,2048,2048], q,k [2048,1,16,128] bf16; median of {len(times)} runs, "
                      f"{med * 1e3:.1f} ms each, same algorithmic-byte convention"}


def measure_workload(name, torch, dev, steps, warmup):
    """Event-brackets every kernel of a workload over `steps` steps after `warmup`: per kernel the algorithmic
    bytes, mean and median bracket in microseconds, GB/s and the fraction of the HBM peak. The workload's tensors
    are released afterwards."""
    import gc

    step, kernel_bytes, other, _, dtype, cfg = make_workload(name, torch, dev, launches=warmup + steps)
    timer = Timer(torch, chain=True)
    for _ in range(warmup):
        timer.unchain()  # a step may begin with work of its own (picking buffers, a copy)
        step(timer)
    torch.cuda.synchronize()
    timer.reset()
    for _ in range(steps):
        timer.unchain()
        step(timer)
    torch.cuda.synchronize()
    avg = timer.averages_ms()
    per = cfg.get("launches_per_bracket", 1)
    out = {}
    for key, nbytes in kernel_bytes.items():
        gbs = nbytes / (avg[key] * 1e-3) / 1e9
        out[key] = {"bytes": nbytes // per, "us": round(avg[key] * 1e3 / per, 2),
                    "median_us": round(timer.spread_ms(key)[1] * 1e3 / per, 2), "GB/s": round(gbs, 1),
                    "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)}
        if key in other:
            label, nb = other[key] if isinstance(other[key], tuple) else ("GB/s_dense_convention", other[key])
            out[key][label] = round(nb / (avg[key] * 1e-3) / 1e9, 1)
    del step, timer
    gc.collect()
    torch.cuda.empty_cache()
    return {"dtype": dtype, "workload": cfg, "steps": steps, "warmup": warmup, "kernels": out}


def cpu_fallback_c1(torch):
    """The first configuration as the reference runs it without its kernels: forward_torch_softmax on the host cores,
    scores [4,8,512,512] bf16 ~ N(0,4), scale 1/sqrt(64), causal mask, seed 0."""
    from oracle import fallback_semantics as fb

    torch.set_num_threads(os.cpu_count() or 1)
    g = torch.Generator().manual_seed(0)
    x = (torch.randn((4, 8, 512, 512), generator=g) * 2).bfloat16()
    mask = fb.causal_mask(512)
    scale = 1.0 / math.sqrt(64)
    fb.torch_softmax_fallback(x, mask, scale)
    times = []
    for _ in range(9):
        t0 = time.perf_counter()
        fb.torch_softmax_fallback(x, mask, scale)
        times.append(time.perf_counter() - t0)
    times.sort()
    med = times[len(times) // 2]
    nbytes = causal_bytes(32, 512)[0]
    return {"ms": round(med * 1e3, 3), "min_ms": round(times[0] * 1e3, 3), "bytes": nbytes,
            "GB/s": round(nbytes / med / 1e9, 2), "cores": torch.get_num_threads(), "kind": "port",
            "what": "reference torch branch (fp32 softmax, masked_fill with the dtype minimum), median of 9 runs"}


def baseline_configs(torch, dev, with_cpu):
    """Every configuration of the benchmark set beside the headline one, each kernel event-bracketed on its
    real tensors: C1 (HIP kernel, and the torch branch on the host cores), the rotary leg of C2 in both call
    styles, C3, C4 (both rotary fractions, one launch per tensor; and q, k as views of one fused projection
    buffer, per tensor and in one launch), C5, and the sliding-window variant of C5's scores."""
    out = {}
    c1 = measure_workload("causal-c1", torch, dev, steps=10, warmup=3)
    if with_cpu:
        c1["cpu_fallback"] = cpu_fallback_c1(torch)
    out["C1 causal fwd [4,8,512,512] bf16"] = c1
    out["C2 rotary leg, both call styles [2048,8,16,128] rotary_pct 0.25"] = measure_workload(
        "rope-styles-1.4b", torch, dev, steps=20, warmup=5)
    out["C3 padding-mask softmax fwd+bwd [16,32,1024,2048] fp16"] = measure_workload("masked-c3", torch, dev, steps=12, warmup=3)
    out["C4 rotary fwd+bwd [4096,4,32,128] rotary_pct 1.0 and 0.25, one launch per tensor"] = measure_workload(
        "rope-c4", torch, dev, steps=20, warmup=5)
    out["C4 rotary on q,k sliced from a fused [4096,4,32,384] buffer"] = measure_workload(
        "rope-c4-qkv-view", torch, dev, steps=20, warmup=5)
    out["C5 rotary [8192,2,32,128] + causal fwd+bwd [64,8192,8192] bf16"] = measure_workload(
        "llama2-7b-c5", torch, dev, steps=8, warmup=2)
    out["C5 scores with a 4096-key sliding window"] = measure_workload("mistral-window", torch, dev, steps=8, warmup=2)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--workload", default="pythia-1.4b")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-configs", action="store_true",
                    help="default workload: leave out the `configs` object (the other configurations of the benchmark set, "
                         "measured after the timed region)")
    ap.add_argument("--fresh-dy", action="store_true",
                    help="pythia-1.4b / llama2-7b-c5: restore the upstream gradient from a pristine copy before every "
                         "in-place backward (the copy runs outside the backward's event bracket but inside the step)")
    ap.add_argument("--decaying-dy", action="store_true",
                    help="workloads with an in-place softmax backward: one gradient buffer, every in-place backward works on "
                         "the result of the one before (the data decay to zeros); default: a ring of pristine copies "
                         "filled before the timed region, one per launch as far as device memory allows")
    ap.add_argument("--rope-per-tensor", action="store_true",
                    help="pythia-1.4b / llama2-7b-c5: rotate q and k with one launch each (the reference's call style) "
                         "instead of both in one launch")
    ap.add_argument("--calibration-copy", action="store_true",
                    help="run one plain 1 GiB device copy first (reference for scaling rocprofv3 --pmc byte counters)")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        raise SystemExit("bench.py measures one GPU; this hot path has no multi-GPU mode (run with --gpus 1)")

    import torch

    if not torch.cuda.is_available():
        raise SystemExit("bench.py needs a GPU")
    from megatron.fused_kernels import load

    load()  # raises if libneox_hotpath.so cannot be loaded; there is no fallback
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibration_copy:
        # 2^29 bf16 elements: the copy kernel reads 1 GiB and writes 1 GiB
        src = torch.ones(1 << 29, dtype=torch.bfloat16, device=dev)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst

    step, kernel_bytes, dense_bytes, dominant, dtype, cfg = make_workload(
        args.workload, torch, dev, args.fresh_dy, args.rope_per_tensor,
        launches=args.warmup + args.steps + min(args.steps, 20), decaying_dy=args.decaying_dy)
    signature = cfg.get("dominant_kernel_signature", KERNEL_REVISIONS.get(args.workload))
    # Timed region: K steps; only the dominant kernel is bracketed by events
    # (every event record is one more packet between the kernels).
    timer = Timer(torch, only=dominant)
    for _ in range(args.warmup):
        step(timer)
    torch.cuda.synchronize()
    timer.reset()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step(timer)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    dominant_ms = timer.averages_ms()[dominant]
    dominant_spread = timer.spread_ms(dominant)

    # Untimed extra pass for the per-kernel breakdown.
    full = Timer(torch)
    for _ in range(min(args.steps, 20)):
        step(full)
    torch.cuda.synchronize()

    ms_per_step = elapsed * 1e3 / args.steps
    step_bytes = sum(kernel_bytes.values())
    value = step_bytes / (ms_per_step * 1e-3) / 1e9
    avg = full.averages_ms()
    avg[dominant] = dominant_ms
    kernels = {}
    for name, nbytes in kernel_bytes.items():
        gbs = nbytes / (avg[name] * 1e-3) / 1e9
        # "ms" is the mean (for the dominant kernel over the timed steps, for the others over the breakdown pass);
        # the median beside it is not moved by a single stalled launch
        kernels[name] = {"ms": round(avg[name], 4), "median_ms": round((timer if name == dominant else full).spread_ms(name)[1], 4),
                         "bytes": nbytes, "GB/s": round(gbs, 1), "frac_of_peak": round(gbs / HBM_PEAK_GBS, 4)}
        if name in dense_bytes:  # the same time under a second byte convention: dense, or (label, bytes)
            other = dense_bytes[name]
            label, nb = other if isinstance(other, tuple) else ("GB/s_dense_convention", other)
            kernels[name][label] = round(nb / (avg[name] * 1e-3) / 1e9, 1)
    dom = kernels[dominant]
    out = {
        "metric": METRIC,
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": dtype,
        "data": "synthetic",
        "config": cfg,
        "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4),
        "bytes_per_step": step_bytes,
        "kernels": kernels,
        "roofline": {"bound": "hbm", "kernel": dominant, "achieved": dom["GB/s"], "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": dom["frac_of_peak"], "traffic": measured_traffic(args.workload, signature),
                     "algorithmic_bytes": kernel_bytes[dominant], "avg_launch_ms": dom["ms"],
                     "min_launch_ms": round(dominant_spread[0], 4), "median_launch_ms": round(dominant_spread[1], 4),
                     "max_launch_ms": round(dominant_spread[2], 4)},
    }
    if args.workload == "pythia-1.4b" and not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(torch)
    if args.workload == "pythia-1.4b" and not args.no_configs:
        import gc

        del step, timer, full
        gc.collect()
        torch.cuda.empty_cache()
        out["configs"] = baseline_configs(torch, dev, not args.no_cpu_baseline)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
