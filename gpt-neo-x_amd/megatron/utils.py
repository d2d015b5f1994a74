"""The producers of the attention mask the fused softmax consumes.

``get_attn_mask`` and ``get_ltor_masks_and_position_ids`` with the semantics of megatron/utils.py:67-110 of
the reference: a boolean ``[1, 1, s, s]`` tensor, True where a query must not see a key (the future, and with a
sliding window the keys more than ``sliding_window_width`` positions back). The causal kernel derives the same
mask from the indices and never reads the tensor; the padding-mask kernel and the torch branch of
``FusedScaleMaskSoftmax`` read it.
"""
import torch


def get_attn_mask(seq_length, device, sliding_window_width):
    """``[1, 1, s, s]`` bool, True = masked: key ``k`` is hidden from query ``q`` when ``k > q`` or, with a window,
    when ``k < q - sliding_window_width`` (megatron/utils.py:67-80)."""
    q = torch.arange(seq_length, device=device).view(seq_length, 1)
    k = torch.arange(seq_length, device=device).view(1, seq_length)
    hidden = k > q
    if sliding_window_width is not None:
        hidden = hidden | (k < q - sliding_window_width)
    return hidden.view(1, 1, seq_length, seq_length)


def get_ltor_masks_and_position_ids(data, eod_token, eod_mask_loss=False, sliding_window_width=None):
    """Attention mask, loss mask and position ids for a left-to-right model (megatron/utils.py:83-110):
    ``data`` ``[b, s]`` token ids; the loss mask is 0 at end-of-document tokens when ``eod_mask_loss``."""
    batch_size, seq_length = data.size()
    attention_mask = get_attn_mask(seq_length, data.device, sliding_window_width)
    loss_mask = torch.ones(data.size(), dtype=torch.float, device=data.device)
    if eod_mask_loss:
        loss_mask[data == eod_token] = 0.0
    position_ids = torch.arange(seq_length, dtype=torch.long, device=data.device).unsqueeze(0).expand_as(data)
    return attention_mask, loss_mask, position_ids
