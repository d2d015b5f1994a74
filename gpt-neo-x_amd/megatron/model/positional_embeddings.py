"""Rotary cache, the eager (unfused) rotary functions, the AliBi slopes and the
sinusoidal table, with the public surface of GPT-NeoX's
``megatron/model/positional_embeddings.py`` (SinusoidalPositionalEmbedding :19-35,
RotaryEmbedding :38-97, rotate_half :103-107, apply_rotary_pos_emb :110-116,
apply_rotary_pos_emb_torch :119-126, AliBi :129-257).
"""
import math

import torch


def _rotary_angles(dim, seq_len, base):
    """fp32 angles ``position * base^(-2j/dim)``; the two halves of the feature axis share them."""
    inv_freq = 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim))
    positions = torch.arange(seq_len).type_as(inv_freq)
    half = torch.einsum("i,j->ij", positions, inv_freq)
    return inv_freq, torch.cat((half, half), dim=-1)


class SinusoidalPositionalEmbedding(torch.nn.Module):
    """``[1, seq, dim]`` table ``cat(sin(p * f_j), cos(p * f_j))`` with ``f_j = base^(-2j/dim)``, added to the
    token embeddings once per forward pass (not a per-layer operation, so plain torch here as in the reference)."""

    def __init__(self, dim, base=10000, precision=torch.half):
        super().__init__()
        self.register_buffer("inv_freq", 1.0 / (base ** (torch.arange(0, dim, 2).float() / dim)))
        self.precision = precision

    def forward(self, x, seq_dim=1):
        positions = torch.arange(x.shape[seq_dim], device=x.device).type_as(self.inv_freq)
        angles = torch.einsum("i,j->ij", positions, self.inv_freq)
        if self.precision == torch.bfloat16:
            angles = angles.float()
        sin, cos = angles.sin(), angles.cos()
        if self.precision == torch.bfloat16:
            sin, cos = sin.bfloat16(), cos.bfloat16()
        return torch.cat((sin, cos), dim=-1)[None, :, :]


class RotaryEmbedding(torch.nn.Module):
    """cos / sin tables for rotary position embedding.

    Built once in fp32 for ``max_seq_len`` positions, then cast to ``precision``;
    ``forward`` returns the first ``seq_len`` rows on the device of ``x``. The
    reference copies its host tables to the device on every call; here each
    device gets its copy once.

    Attributes kept from the reference: ``cos_cached``, ``sin_cached``
    (``[max_seq_len, 1, 1, dim]`` in ``precision``), ``emb`` (fp32 angles of the same
    shape), the buffer ``inv_freq`` (cast to ``precision``; in the state dict only
    with ``save_inv_freqs``), ``dim``, ``base``, ``max_seq_len``, ``precision``.
    """

    def __init__(self, dim, max_seq_len, base=10000, precision=torch.half, save_inv_freqs=False):
        super().__init__()
        self.dim = dim
        self.base = base
        self.max_seq_len = max_seq_len
        self.precision = precision
        self.seq_len_cached = None
        self.cos_cached, self.sin_cached, inv_freq = self._prepare_cache(max_seq_len, precision, base)
        self.register_buffer("inv_freq", inv_freq, persistent=save_inv_freqs)
        self._per_device = {}

    def _prepare_cache(self, seq_len, precision, base):
        inv_freq, angles = _rotary_angles(self.dim, seq_len, base)
        self.emb = angles.reshape(seq_len, 1, 1, angles.size(1))
        shape4 = (slice(None), None, None, slice(None))
        return angles.cos()[shape4].to(precision), angles.sin()[shape4].to(precision), inv_freq.to(precision)

    def get_emb(self):
        return self.emb.to(self.precision).cuda()

    def _tables_on(self, device):
        device = torch.device(device)
        if device == self.cos_cached.device:
            return self.cos_cached, self.sin_cached
        entry = self._per_device.get(str(device))
        if entry is None or entry[0] is not self.cos_cached:  # first use, or the host tables were replaced
            entry = (self.cos_cached, self.cos_cached.to(device), self.sin_cached.to(device))
            self._per_device[str(device)] = entry
        return entry[1], entry[2]

    def forward(self, x, seq_dim=0, seq_len=None):
        if seq_len is None:
            seq_len = x.shape[seq_dim]
        assert seq_len <= self.max_seq_len
        cos, sin = self._tables_on(x.device)
        if seq_len == self.max_seq_len:
            return cos, sin
        return cos[:seq_len, ...], sin[:seq_len, ...]


# rotary pos emb helpers:


def rotate_half(x):
    """``(-x2, x1)`` for ``x = (x1, x2)`` split in halves along the last dimension."""
    mid = x.shape[-1] // 2
    return torch.cat((-x[..., mid:], x[..., :mid]), dim=x.ndim - 1)


def _rotate(t, cos, sin):
    return (t * cos) + (rotate_half(t) * sin)


def apply_rotary_pos_emb(q, k, cos, sin, offset: int = 0):
    """Eager RoPE of q and k ``[s, b, h, d]`` with tables ``[S, 1, 1, d]``; row i of
    q/k takes table row ``offset + i``."""
    rows = slice(offset, q.shape[0] + offset)
    cos, sin = cos[rows, ...], sin[rows, ...]
    return _rotate(q, cos, sin), _rotate(k, cos, sin)


def apply_rotary_pos_emb_torch(q, k, cos, sin, offset: int = 0):
    # the reference keeps two names: its first variant is TorchScript-compiled, which fails for bf16
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


class RelativePositionBias(torch.nn.Module):
    """T5 relative position bias: ``bias[0, h, q, k] = weight[bucket(k - q), h] * scale``
    (``ParallelRelativePositionBias``, megatron/mpu/layers.py:215-381, for all heads on one GPU; built with
    ``scale = sqrt(head_dim)`` by megatron/model/gpt2_model.py:228-240). ``forward(q_len, k_len)`` returns
    ``[1, heads, q_len, k_len]``, the ``rpe`` argument of ``CoreAttention``, which hands it to the softmax kernel
    as its bias operand.

    Buckets (causal): distance ``n = max(q - k, 0)``; ``n`` itself below ``num_buckets / 2``, then logarithmic steps
    up to ``max_distance``, the last bucket for everything beyond. Non-causal: half of the buckets per direction.
    """

    def __init__(self, scale, causal=True, num_buckets=32, max_distance=128, heads=8, init_method=None, neox_args=None):
        super().__init__()
        self.scale = scale
        self.causal = causal
        self.num_buckets = num_buckets
        self.max_distance = max_distance
        self.heads = heads
        self.weight = torch.nn.Parameter(torch.empty(num_buckets, heads))
        (init_method or torch.nn.init.xavier_normal_)(self.weight)
        self._cached_lengths = None
        self._cached_buckets = None

    def relative_position_bucket(self, relative_position):
        """Bucket index of ``relative_position = k - q`` (an integer tensor)."""
        buckets = self.num_buckets
        distance = -relative_position
        base = torch.zeros_like(distance)
        if self.causal:
            distance = distance.clamp(min=0)
        else:
            buckets //= 2
            base = (distance < 0).long() * buckets
            distance = distance.abs()
        exact = buckets // 2
        # logarithmic part, in fp32 with the operation order of the reference (log of the ratio, divided by the
        # log of the range, times the number of logarithmic buckets, truncated)
        steps = torch.log(distance.float() / exact) / math.log(self.max_distance / exact) * (buckets - exact)
        far = (exact + steps.long()).clamp(max=buckets - 1)
        return base + torch.where(distance < exact, distance, far)

    def buckets(self, q_len, k_len, device):
        if self._cached_lengths != (q_len, k_len) or self._cached_buckets.device != torch.device(device):
            q_pos = torch.arange(q_len, dtype=torch.long, device=device)
            k_pos = torch.arange(k_len, dtype=torch.long, device=device)
            self._cached_buckets = self.relative_position_bucket(k_pos[None, :] - q_pos[:, None])
            self._cached_lengths = (q_len, k_len)
        return self._cached_buckets

    def forward(self, q_len, k_len):
        values = torch.nn.functional.embedding(self.buckets(q_len, k_len, self.weight.device), self.weight)  # [q, k, h]
        return values.movedim(2, 0).unsqueeze(0) * self.scale


ParallelRelativePositionBias = RelativePositionBias
