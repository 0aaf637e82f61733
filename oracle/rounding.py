"""Sources of rounding noise for the oracle (test infrastructure; see oracle/__init__.py).

The reference's stochastic sites are
  * ``torch.rand_like(scaled)``            one fp32 uniform per element per ECC encode (heavyball/utils.py:1316)
  * ``torch.randint_like(x, 0, 1 << 16)``  16 bits per element per bf16 stochastic round (heavyball/utils.py:2352)

A ``Rounding`` object answers both for a given (stream, tensor index, shape).  Three modes:

  HalfRounding    uniform = 0.5, noise = 0x8000: every stochastic rounding becomes round-half-up on
                  the magnitude; this is "rounding disabled" and needs no RNG.
  PhiloxRounding  the counter-based stream the kernels use (oracle/philox.py); ``base`` gives each
                  tensor's first flat index in the slab so that element e of tensor t uses counter
                  base[t] + e.  The tensor index may be a pair (t, offsets): the elements of a block of
                  tensor t, each with its own offset e.
  TorchRounding   torch's global generator in call order: what the reference itself does.
"""

import numpy as np
import torch

from . import philox


class HalfRounding:
    mode = "half"

    def uniform(self, stream, tensor_index, shape):
        return torch.full(shape, 0.5, dtype=torch.float32)

    def noise16(self, stream, tensor_index, shape):
        return torch.full(shape, 1 << 15, dtype=torch.int32)

    def at_step(self, step):
        return self


class PhiloxRounding:
    mode = "philox"

    def __init__(self, seed: int, step: int = 0, base=None):
        self.seed = int(seed)
        self.step = int(step)
        self.base = base  # sequence of flat slab offsets, one per tensor; None -> all zero

    def at_step(self, step):
        return PhiloxRounding(self.seed, step, self.base)

    def _bits(self, stream, tensor_index, shape):
        n = int(np.prod(shape)) if len(shape) else 1
        if isinstance(tensor_index, tuple):  # (tensor, offsets of the elements inside it): a block of a tensor that is cut up
            tensor_index, offsets = tensor_index
            b = 0 if self.base is None else int(self.base[tensor_index])
            idx = np.uint64(b) + np.asarray(offsets, dtype=np.uint64)
            assert idx.size == n
        else:
            b = 0 if self.base is None else int(self.base[tensor_index])
            idx = np.arange(b, b + n, dtype=np.uint64)
        return philox.bits16(self.seed, self.step, stream, idx).reshape(tuple(shape))

    def uniform(self, stream, tensor_index, shape):
        # 16-bit uniform on the grid k / 65536; exact in fp32
        bits = self._bits(stream, tensor_index, shape)
        return torch.from_numpy(bits.astype(np.float32)) * (1.0 / 65536.0)

    def noise16(self, stream, tensor_index, shape):
        return torch.from_numpy(self._bits(stream, tensor_index, shape).astype(np.int32))


class TorchRounding:
    mode = "torch"

    def uniform(self, stream, tensor_index, shape):
        return torch.rand(shape, dtype=torch.float32)

    def noise16(self, stream, tensor_index, shape):
        return torch.randint(0, 1 << 16, shape, dtype=torch.int32)

    def at_step(self, step):
        return self
