"""Rotary cache, the eager (unfused) rotary functions and the AliBi slopes, with
the public surface of GPT-NeoX's ``megatron/model/positional_embeddings.py``
(RotaryEmbedding :38-97, rotate_half :103-107, apply_rotary_pos_emb :110-116,
apply_rotary_pos_emb_torch :119-126, AliBi :129-257).
"""
import math

import torch


class RotaryEmbedding(torch.nn.Module):
    """Precomputed cos/sin tables for rotary position embedding.

    The tables are built once, in fp32, for ``max_seq_len`` positions and cast
    to ``precision``; ``forward`` hands out the first ``seq_len`` rows on the
    device of ``x``. The reference copies the host tables to the device on
    every call; here each device's copy is made once and kept.
    """

    def __init__(self, dim, max_seq_len, base=10000, precision=torch.half, save_inv_freqs=False):
        super().__init__()
        self.seq_len_cached = None
        self.precision = precision
        self.max_seq_len = max_seq_len
        self.base = base
        self.dim = dim

        cos_cached, sin_cached, inv_freq = self._prepare_cache(max_seq_len, precision, base)
        # as in the reference, the buffer that survives is the one cast to `precision`
        self.register_buffer("inv_freq", inv_freq, persistent=save_inv_freqs)
        self.cos_cached = cos_cached
        self.sin_cached = sin_cached
        self._on_device = {}

    def _prepare_cache(self, seq_len, precision, base):
        inv_freq = 1.0 / (base ** (torch.arange(0, self.dim, 2).float() / self.dim))
        t = torch.arange(seq_len).type_as(inv_freq)
        freqs = torch.einsum("i,j->ij", t, inv_freq)
        emb = torch.cat((freqs, freqs), dim=-1)
        self.emb = emb.reshape(emb.size(0), 1, 1, emb.size(1))
        cos_cached = emb.cos()[:, None, None, :]
        sin_cached = emb.sin()[:, None, None, :]
        return cos_cached.to(precision), sin_cached.to(precision), inv_freq.to(precision)

    def get_emb(self):
        return self.emb.to(self.precision).cuda()

    def _tables_on(self, device):
        device = torch.device(device)
        if device == self.cos_cached.device:
            return self.cos_cached, self.sin_cached
        key = str(device)
        hit = self._on_device.get(key)
        if hit is None or hit[0] is not self.cos_cached:
            hit = (self.cos_cached, self.cos_cached.to(device), self.sin_cached.to(device))
            self._on_device[key] = hit
        return hit[1], hit[2]

    def forward(self, x, seq_dim=0, seq_len=None):
        if seq_len is None:
            seq_len = x.shape[seq_dim]
        assert seq_len <= self.max_seq_len
        cos, sin = self._tables_on(x.device)
        if seq_len != self.max_seq_len:
            return cos[:seq_len, ...], sin[:seq_len, ...]
        return cos, sin


# rotary pos emb helpers:


def rotate_half(x):
    half = x.shape[-1] // 2
    x1, x2 = x[..., :half], x[..., half:]
    return torch.cat((-x2, x1), dim=x1.ndim - 1)


def apply_rotary_pos_emb(q, k, cos, sin, offset: int = 0):
    cos = cos[offset : q.shape[0] + offset, ...]
    sin = sin[offset : q.shape[0] + offset, ...]
    return (q * cos) + (rotate_half(q) * sin), (k * cos) + (rotate_half(k) * sin)


def apply_rotary_pos_emb_torch(q, k, cos, sin, offset: int = 0):
    # identical to apply_rotary_pos_emb; the reference keeps two names because
    # its first variant is TorchScript-compiled and that fails for bf16
    return apply_rotary_pos_emb(q, k, cos, sin, offset)


class AliBi(torch.nn.Module):
    """Attention with linear biases: head h adds -(q - k) * slope_h to the score of
    query q and key k <= q.

    Same constructor, ``slopes`` buffer, ``bias`` and ``forward`` as the reference
    class. ``forward(x)`` is the eager path (one extra pass over the scores);
    handing ``alibi.slopes`` to ``FusedScaleMaskSoftmax(alibi_slopes=...)`` adds
    the same bias inside the causal softmax kernel instead.
    """

    def __init__(self, num_heads, mp_size=1, mp_rank=1):
        super().__init__()
        # heads are split across model-parallel ranks: each rank keeps its slice of the slopes
        assert mp_size <= num_heads and mp_rank <= mp_size
        self.mp_size = mp_size
        self.mp_rank = mp_rank
        self.num_heads = num_heads
        self.slice_size = num_heads // mp_size
        self.cached_matrix = None
        self.cached_seq_len = None
        slopes = torch.Tensor(self._get_slopes(num_heads))[mp_rank * self.slice_size : (mp_rank + 1) * self.slice_size]
        self.register_buffer("slopes", slopes)

    def _get_slopes(self, n):
        """Geometric sequence 2^(-8/n), 2^(-16/n), ... for a power-of-two n; other n
        take the sequence of the next lower power of two plus every other slope of
        the next higher one."""

        def power_of_2(m):
            start = 2 ** (-(2 ** -(math.log2(m) - 3)))
            return [start * start**i for i in range(m)]

        if math.log2(n).is_integer():
            return power_of_2(n)
        closest = 2 ** math.floor(math.log2(n))
        return power_of_2(closest) + self._get_slopes(2 * closest)[0::2][: n - closest]

    def bias(self, seq_len_q, seq_len_k, device, dtype):
        """The [np, sq, sk] bias matrix (cached; it grows fourfold when a longer key length shows up)."""
        if self.cached_seq_len is None or self.cached_seq_len < seq_len_k:
            target = seq_len_k if self.cached_seq_len is None else self.cached_seq_len * 4
            i = torch.arange(target)
            a = -torch.tril(i.view(target, 1).repeat(1, target) + torch.arange(0, -target, -1))
            a = a.to(device).to(dtype)
            slopes = self.slopes.to(a.device).to(a.dtype)
            self.cached_matrix = a * slopes.view(self.slopes.shape[0], 1, 1)
            self.cached_seq_len = target
        a = self.cached_matrix
        if self.cached_seq_len > seq_len_k:
            a = a[:, :seq_len_k, :seq_len_k]
        if seq_len_q != seq_len_k:
            # decoding with a key/value cache: one query, the last position
            assert seq_len_q == 1, "assumption sq == sk unless at inference time with cache in layer_past with sq == 1"
            a = a[:, seq_len_k - 1, :].view(a.shape[0], 1, a.shape[2])
        return a

    def forward(self, x):
        # x: [b, np, sq, sk]
        return x + self.bias(x.shape[-2], x.shape[-1], x.device, x.dtype)
