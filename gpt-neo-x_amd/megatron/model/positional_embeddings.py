"""Rotary cache and the eager (unfused) rotary functions, with the public
surface of the rotary part of GPT-NeoX's
``megatron/model/positional_embeddings.py`` (RotaryEmbedding :38-97,
rotate_half :103-107, apply_rotary_pos_emb :110-116,
apply_rotary_pos_emb_torch :119-126).
"""
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
