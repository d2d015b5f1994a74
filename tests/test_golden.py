"""Committed golden vectors (tests/golden/hotpath_golden.npz, written by
tests/golden/make_golden.py from the CPU oracle). Without a GPU: the oracle
still reproduces them bit for bit. With a GPU: the HIP path, called through the
C ABI, matches them to the stated tolerance."""
import os

import numpy as np
import pytest
import torch

import oracle
import util

GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "hotpath_golden.npz"))
DT = {"bf16": torch.bfloat16, "fp16": torch.float16, "fp32": torch.float32}


def get(prefix, key):
    arr = GOLDEN[f"{prefix}.{key}"]
    t = torch.from_numpy(np.ascontiguousarray(arr))
    if key in ("mask",):
        return t
    if key in ("scale",):
        return float(arr)
    if key == "freqs":
        return t.view(torch.float32)
    dtype = DT[prefix.split("_")[-1]]
    return t.view(dtype)


CAUSAL = ["causal_bf16", "causal_fp16"]
MASKED = ["masked_fp16", "masked_bf16"]
ROPE = ["rope_bf16", "rope_fp16", "rope_fp32"]


@pytest.mark.parametrize("name", CAUSAL)
def test_oracle_reproduces_causal_golden(name):
    x, dy, y, dx, scale = (get(name, k) for k in ("x", "dy", "y", "dx", "scale"))
    assert torch.equal(util.raw_bits(oracle.causal_softmax_fwd(x, scale)), util.raw_bits(y))
    assert torch.equal(util.raw_bits(oracle.softmax_bwd(dy, y, scale, True)), util.raw_bits(dx))


@pytest.mark.parametrize("name", MASKED)
def test_oracle_reproduces_masked_golden(name):
    x, mask, dy, y, dx, scale = (get(name, k) for k in ("x", "mask", "dy", "y", "dx", "scale"))
    assert torch.equal(util.raw_bits(oracle.masked_softmax_fwd(x, mask, scale)), util.raw_bits(y))
    assert torch.equal(util.raw_bits(oracle.softmax_bwd(dy, y, scale, False)), util.raw_bits(dx))


@pytest.mark.parametrize("name", ROPE)
def test_oracle_reproduces_rope_golden(name):
    t, cos, sin, freqs = (get(name, k) for k in ("t", "cos", "sin", "freqs"))
    assert torch.equal(util.raw_bits(oracle.rope_cached(t, cos, sin)), util.raw_bits(get(name, "fwd")))
    assert torch.equal(util.raw_bits(oracle.rope_cached(t, cos, sin, backward=True)), util.raw_bits(get(name, "bwd")))
    assert torch.equal(util.raw_bits(oracle.rope_freqs(t, freqs)), util.raw_bits(get(name, "fwd_freqs")))
    assert torch.equal(util.raw_bits(oracle.rope_freqs(t, freqs, backward=True)), util.raw_bits(get(name, "bwd_freqs")))


@pytest.mark.gpu
@pytest.mark.parametrize("name", CAUSAL)
def test_gpu_matches_causal_golden(hotpath, name):
    x, dy, y, dx, scale = (get(name, k) for k in ("x", "dy", "y", "dx", "scale"))
    got = util.abi_causal_fwd(hotpath, x.cuda(), scale).cpu()
    s = x.size(-1)
    upper = torch.triu(torch.ones(s, s, dtype=torch.bool), diagonal=1)
    assert int(util.raw_bits(got)[:, upper].abs().max()) == 0  # masked: bit-exact +0
    util.assert_ulp_close(got, y, 2, name)  # 2 ulp of the storage dtype
    gdx = util.abi_causal_bwd(hotpath, dy.cuda(), y.cuda(), scale).cpu()
    assert int(util.raw_bits(gdx)[:, upper].abs().max()) == 0
    util.assert_softmax_bwd_close(gdx, dx, dy, y, scale, name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", MASKED)
def test_gpu_matches_masked_golden(hotpath, name):
    x, mask, dy, y, dx, scale = (get(name, k) for k in ("x", "mask", "dy", "y", "dx", "scale"))
    got = util.abi_masked_fwd(hotpath, x.cuda(), mask.cuda(), scale).cpu()
    util.assert_ulp_close(got, y, 2, name)
    full = mask.bool().all(-1).expand(x.size(0), 1, x.size(2)).expand(x.size(0), x.size(1), x.size(2))
    assert full.any() and torch.equal(util.raw_bits(got)[full], util.raw_bits(y)[full])  # fully masked rows: identical
    gdx = util.abi_masked_bwd(hotpath, dy.cuda(), y.cuda(), scale).cpu()
    util.assert_softmax_bwd_close(gdx, dx, dy, y, scale, name)


@pytest.mark.gpu
@pytest.mark.parametrize("name", ROPE)
def test_gpu_matches_rope_golden(hotpath, name):
    t, cos, sin, freqs = (get(name, k) for k in ("t", "cos", "sin", "freqs"))
    for backward, key in ((False, "fwd"), (True, "bwd")):
        got = util.abi_rope_cached(hotpath, t.cuda(), cos.cuda(), sin.cuda(), backward).cpu()
        assert torch.equal(util.raw_bits(got), util.raw_bits(get(name, key)))  # bit-exact
        gotf = util.abi_rope_freqs(hotpath, t.cuda(), freqs.cuda(), backward).cpu()
        want = get(name, key + "_freqs")
        # bit-identical wherever the table entries are clear of a rounding boundary of the data dtype
        util.assert_rope_freqs_close(gotf, want, t, freqs, backward, f"{name} {key}")
