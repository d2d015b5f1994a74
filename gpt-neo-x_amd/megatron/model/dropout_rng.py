"""Seeds for the dropout masks of the fused kernels.

The kernels generate their keep masks with a counter-based generator (Philox4x32-10 over the
element index) from one 64-bit seed per call. That seed is taken from the device's default CUDA
generator the way torch's own dropout kernels take theirs: the generator's seed and its current
Philox offset are read on the host and the offset is advanced, without touching the device and
without drawing from torch's CPU generator. Consequences, all as for ``torch.nn.functional.dropout``
in the reference (megatron/model/transformer.py:592-593, megatron/model/fused_bias_dropout.py:28-39):

* ``torch.manual_seed`` / ``torch.cuda.manual_seed`` restart the sequence of masks;
* ``torch.cuda.get_rng_state`` / ``set_rng_state`` save and restore it (checkpointing, activation
  recomputation), and a region that swaps the CUDA generator state, like the reference's
  ``mpu.get_cuda_rng_tracker().fork()``, gives the fused dropout inside it that region's stream;
* the CPU generator, hence data order, is not affected;
* a seed is a host value fixed at call time, so it cannot be drawn while a HIP graph is being
  captured (every replay would reuse the one mask): ``next_seed`` raises there. Capture the
  kernels through their extension functions with a seed of the caller's choosing instead.

Which elements are dropped for a given seed is the library's own definition (see
``nhp_bias_dropout_add`` in include/neox_hotpath.h), not torch's.
"""
import torch

_MASK = (1 << 64) - 1


def _mix(seed, offset):
    """splitmix64 of the (seed, offset) pair: one well-spread 63-bit value."""
    z = (seed * 0x9E3779B97F4A7C15 + offset + 0x632BE59BD9B4E019) & _MASK
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _MASK
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _MASK
    return (z ^ (z >> 31)) & ((1 << 63) - 1)


def next_seed(device=None):
    """A fresh seed for one dropout call on ``device`` (default: the current device)."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index
    if index is None:
        index = torch.cuda.current_device()
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError("dropout seeds are drawn on the host and cannot be drawn during graph capture: "
                           "every replay would repeat one mask; pass an explicit seed to the extension functions")
    gen = torch.cuda.default_generators[index]
    seed, offset = gen.initial_seed(), gen.get_offset()
    gen.set_offset(offset + 4)  # Philox offsets advance in steps of four
    return _mix(seed, offset)
