#!/usr/bin/env python3
"""Writes tests/golden/hotpath_golden.npz (softmax and rotary entry points) and
tests/golden/layer_golden.npz (the window / AliBi / bias / key-length variants of
the causal softmax, bias + GeLU, bias + residual add, gated activations, LayerNorm, RMSNorm): small
seeded inputs and the outputs of the CPU oracle (oracle/*.c), stored as raw bit
patterns. The oracle itself is pinned by tests/test_oracle_*.py; these
vectors freeze its answers so that the GPU path (and any later change to the
oracle) is compared against fixed data.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path[:0] = [ROOT, os.path.join(ROOT, "tests")]

import oracle  # noqa: E402
import util  # noqa: E402


def bits(t):
    t = t.contiguous()
    if t.dtype == torch.float32:
        return t.view(torch.int32).numpy()
    if t.dtype in (torch.float16, torch.bfloat16):
        return t.view(torch.int16).numpy()
    return t.numpy()


def main():
    out = {}

    def put(prefix, **tensors):
        for k, v in tensors.items():
            out[f"{prefix}.{k}"] = bits(v) if isinstance(v, torch.Tensor) else np.asarray(v)

    for name, dtype, a, s, scale, seed in (("causal_bf16", torch.bfloat16, 2, 24, 0.125, 1),
                                           ("causal_fp16", torch.float16, 2, 40, 0.0883883461356163, 2)):
        x = util.randn((a, s, s), dtype, seed, std=2.0)
        dy = util.randn((a, s, s), dtype, seed + 100)
        y = oracle.causal_softmax_fwd(x, scale)
        put(name, x=x, dy=dy, y=y, dx=oracle.softmax_bwd(dy, y, scale, True), scale=np.float32(scale))

    for name, dtype, b, np_, sq, sk, pb, scale, seed in (("masked_fp16", torch.float16, 2, 2, 4, 40, 2, 0.0883883461356163, 3),
                                                         ("masked_bf16", torch.bfloat16, 2, 2, 4, 24, 1, 0.5, 4)):
        x = util.randn((b, np_, sq, sk), dtype, seed, std=3.0)
        x[0, 0, 0, 3] = 60.0
        x[1, 1, 2, 5] = -60.0
        mask = util.padding_mask(pb, sq, sk, seed, full_batch=1 if pb > 1 else None)
        if pb == 1:
            mask[0, 0, 1, :] = True
        dy = util.randn((b, np_, sq, sk), dtype, seed + 100)
        y = oracle.masked_softmax_fwd(x, mask, scale)
        put(name, x=x, mask=mask.to(torch.uint8), dy=dy, y=y, dx=oracle.softmax_bwd(dy, y, scale, False),
            scale=np.float32(scale))

    for name, dtype, s, b, h, d, d2, seed in (("rope_bf16", torch.bfloat16, 6, 2, 2, 16, 8, 5),
                                              ("rope_fp16", torch.float16, 5, 1, 3, 16, 16, 6),
                                              ("rope_fp32", torch.float32, 4, 2, 1, 8, 8, 7)):
        t = util.randn((s, b, h, d), dtype, seed)
        g = torch.Generator().manual_seed(seed)
        ang = (torch.rand((s, 1, 1, d2), generator=g) * 20.0 - 10.0).contiguous()
        cos, sin = ang.cos().to(dtype), ang.sin().to(dtype)
        put(name, t=t, cos=cos, sin=sin, freqs=ang, fwd=oracle.rope_cached(t, cos, sin),
            bwd=oracle.rope_cached(t, cos, sin, backward=True),
            fwd_freqs=oracle.rope_freqs(t, ang), bwd_freqs=oracle.rope_freqs(t, ang, backward=True))

    path = os.path.join(HERE, "hotpath_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")

    out.clear()
    for name, dtype, seed in (("ex_bf16", torch.bfloat16, 11), ("ex_fp16", torch.float16, 12)):
        batch, heads, s, window, scale = 2, 2, 24, 5, 0.25
        x = util.randn((batch * heads, s, s), dtype, seed, std=2.0)
        dy = util.randn((batch * heads, s, s), dtype, seed + 100)
        bias = util.randn((heads, s, s), dtype, seed + 200)
        slopes = torch.tensor([0.5, 0.0625], dtype=torch.float32)
        lengths = torch.tensor([24, 9], dtype=torch.int32)
        y = oracle.causal_softmax_fwd(x, scale, window=window, alibi_slopes=slopes, bias=bias, key_lengths=lengths)
        dx = oracle.softmax_bwd(dy, y, scale, True, window=window, key_lengths=lengths)
        put(name, x=x, dy=dy, bias=bias, slopes=slopes, lengths=lengths, y=y, dx=dx, window=np.int64(window),
            scale=np.float32(scale))

    for name, dtype, seed in (("gelu_bf16", torch.bfloat16, 21), ("gelu_fp16", torch.float16, 22),
                              ("gelu_fp32", torch.float32, 23)):
        y = util.randn((6, 16), dtype, seed, std=3.0)
        bias = util.randn((16,), dtype, seed + 1, std=0.5)
        g = util.randn((6, 16), dtype, seed + 2)
        res = util.randn((6, 16), dtype, seed + 3, std=2.0)
        dx = oracle.bias_gelu_bwd(g, y, bias)
        put(name, y=y, bias=bias, g=g, res=res, out=oracle.bias_gelu_fwd(y, bias), dx=dx, dbias=oracle.column_sum(dx),
            added=oracle.bias_add_residual(y, bias, res),
            # attention branch y + bias, MLP branch g + bias, residual res (the parallel-residual layer's join)
            added_pair=oracle.bias_add_residual_pair(y, bias, g, bias, res))

    for name, dtype, seed in (("norm_bf16", torch.bfloat16, 31), ("norm_fp16", torch.float16, 32),
                              ("norm_fp32", torch.float32, 33)):
        x = util.randn((5, 24), dtype, seed, std=2.0) + 0.5
        dy = util.randn((5, 24), dtype, seed + 1)
        g = torch.Generator().manual_seed(seed)
        gamma = (1 + 0.3 * torch.randn(24, generator=g)).to(dtype)
        beta = (0.2 * torch.randn(24, generator=g)).to(dtype)
        y, mean, rstd = oracle.layernorm_fwd(x, gamma, beta, 1e-5)
        dx, dg, db = oracle.layernorm_bwd(dy, x, mean, rstd, gamma)
        put(name, x=x, dy=dy, gamma=gamma, beta=beta, ln_y=y, ln_mean=mean, ln_rstd=rstd, ln_dx=dx, ln_dgamma=dg,
            ln_dbeta=db)
        for mode, eps in ((0, 1e-5), (1, 1e-2)):
            ry, inv = oracle.rmsnorm_fwd(x, gamma, beta, eps, mode)
            rdx, rds, rdo = oracle.rmsnorm_bwd(dy, x, inv, gamma, eps, mode)
            put(name, **{f"rms{mode}_y": ry, f"rms{mode}_inv": inv, f"rms{mode}_dx": rdx, f"rms{mode}_dscale": rds,
                         f"rms{mode}_doffset": rdo, f"rms{mode}_eps": np.float32(eps)})
        # partial RMSNorm (statistic over the first 7 of 24 columns) and ScaleNorm (g = 1.25)
        py, pinv = oracle.rmsnorm_fwd(x, gamma, beta, 1e-2, 1, stat_cols=7)
        pdx, pds, pdo = oracle.rmsnorm_bwd(dy, x, pinv, gamma, 1e-2, 1, stat_cols=7)
        gvec = torch.full((24,), 1.25, dtype=dtype)
        sy, sinv = oracle.rmsnorm_fwd(x, gvec, None, 1e-2, 2)
        sdx, sds, _ = oracle.rmsnorm_bwd(dy, x, sinv, gvec, 1e-2, 2)
        put(name, part_y=py, part_inv=pinv, part_dx=pdx, part_dscale=pds, part_doffset=pdo, sn_y=sy, sn_inv=sinv,
            sn_dx=sdx, sn_dscale=sds)
        # a second LayerNorm of the same input (the parallel-residual layer): one dx for both
        gamma2 = (1 - 0.3 * torch.randn(24, generator=g)).to(dtype)
        beta2 = (0.2 * torch.randn(24, generator=g)).to(dtype)
        dy2 = util.randn((5, 24), dtype, seed + 2)
        _, y2, _, _ = oracle.layernorm_pair_fwd(x, gamma, beta, gamma2, beta2, 1e-5)
        pair_dx, _, _, pdg2, pdb2 = oracle.layernorm_pair_bwd(dy, dy2, x, mean, rstd, gamma, gamma2)
        put(name, gamma2=gamma2, beta2=beta2, dy2=dy2, pair_y2=y2, pair_dx=pair_dx, pair_dgamma2=pdg2, pair_dbeta2=pdb2)

    for name, dtype, seed in (("gated_bf16", torch.bfloat16, 41), ("gated_fp16", torch.float16, 42),
                              ("gated_fp32", torch.float32, 43)):
        inp = util.randn((5, 32), dtype, seed, std=2.5)
        bias = util.randn((32,), dtype, seed + 1, std=0.5)
        dy = util.randn((5, 16), dtype, seed + 2)
        put(name, inp=inp, bias=bias, dy=dy)
        for act in sorted(oracle.GATE_ACTS):
            put(name, **{f"{act}_out": oracle.gated_act_fwd(inp, act, bias), f"{act}_din": oracle.gated_act_bwd(dy, inp, act, bias)})

    for name, dtype, seed in (("drop_bf16", torch.bfloat16, 51), ("drop_fp16", torch.float16, 52)):
        x = util.randn((3, 24, 24), dtype, seed, std=2.0)
        dy = util.randn((3, 24, 24), dtype, seed + 1)
        bias = util.randn((24,), dtype, seed + 2)
        p, sd, scale = 0.25, 1234567890123 + seed, 0.25
        dropped, y = oracle.causal_softmax_dropout_fwd(x, scale, p, sd)
        put(name, x=x, dy=dy, bias=bias, p=np.float32(p), seed=np.int64(sd), scale=np.float32(scale),
            keep=oracle.dropout_mask(x.numel(), p, sd).to(torch.uint8), y=y, dropped=dropped,
            dx=oracle.causal_softmax_dropout_bwd(dy, y, scale, p, sd),
            bda=oracle.bias_dropout_add(x.view(-1, 24), bias, dy.view(-1, 24), p, sd))
        # the same through the padding-mask softmax: x as [b = 3, np = 1, sq = 24, sk = 24], the last entry fully masked
        pad = util.padding_mask(3, 24, 24, seed=seed, full_batch=2, lo=6)
        mdropped, my = oracle.masked_softmax_dropout_fwd(x.view(3, 1, 24, 24), pad, scale, p, sd)
        put(name, pad=pad.to(torch.uint8), m_y=my, m_dropped=mdropped,
            m_dx=oracle.masked_softmax_dropout_bwd(dy.view(3, 1, 24, 24), my, scale, p, sd))

    path = os.path.join(HERE, "layer_golden.npz")
    np.savez_compressed(path, **out)
    print(path, os.path.getsize(path), "bytes,", len(out), "arrays")


if __name__ == "__main__":
    main()
