"""Per-module cache of the packed ternary weights.

The reference re-runs ``ternary_quantize`` on the master weights in every forward
(``bittorch/nn/ternary_linear.py:196-200``, ``bittorch/nn/ternary_linear_cuda.py:52-54``).
The result depends on the weights only, so a forward that cannot be a training step (gradient
mode off, or frozen weights) keeps it until the weights change: the key is the parameter's
version counter (every tracked in-place update, ``load_state_dict`` or optimizer step bumps it),
its storage address, dtype and device, and the quantizer's two settings.  Such a forward then
reads K*N/4 bytes of packed weights instead of 4*K*N bytes of masters -- and reads them from a decode-tiled copy
built next to the packed bytes (``_C.retile_weights``; whole-cache-line loads: what ``TernaryLinearInference`` runs
on), which such a module then holds as well, another K*N/4 bytes.  Up to 32 rows the output is the training forward's
bit for bit; a larger batch may be routed to another kernel on the tiled copy than on the row-major bytes, and the two
sum in fp32 in different orders (a difference in the last bits of the sums).

A training forward (gradient mode on and ``weight.requires_grad``) never uses the cache and
quantizes every time, exactly as the reference does: training code is where weights get written
through ``.data`` (``w.data.clamp_()``, ``p.data.add_(...)``, EMA copies), and writes through
``.data`` do not bump the version counter.  The one case that remains the caller's is an
evaluation-time write through ``.data``; ``module.invalidate_packed_cache()`` (or any tracked
write, e.g. ``with torch.no_grad(): w.copy_(...)``) makes the next forward re-quantize.
"""

from __future__ import annotations

from typing import Optional, Tuple

import torch
from torch import Tensor


class PackedWeightCache:
    __slots__ = ("key", "value")

    def __init__(self) -> None:
        self.key = None
        self.value: Optional[Tuple[Tensor, Tensor, Optional[Tensor]]] = None

    def get(self, weight: Tensor, threshold_factor: float, per_channel: bool) -> Tuple[Tensor, Tensor, Optional[Tensor]]:
        """``(packed_T uint8 [ceil(K/4), N], scale fp32 [N] or 0-dim, tiled)`` of the current weights; ``tiled`` is
        the decode-tiled copy of ``packed_T`` (``_C.retile_weights``), or None where the tiled kernels' 32-bit
        offsets do not reach."""
        from .. import _C

        key = (weight._version, weight.data_ptr(), weight.dtype, weight.device, float(threshold_factor),
               bool(per_channel))
        if key != self.key:
            with torch.no_grad():
                packed, scale, _ = _C.ternary_quantize_pack(weight.detach(), threshold_factor, per_channel)
                n, k = weight.shape
                tiled_bytes = ((n + 15) // 16) * ((((k + 3) // 4) + 15) // 16) * 256
                tiled = _C.retile_weights(packed, k) if tiled_bytes < 2 ** 32 else None
            self.key, self.value = key, (packed, scale, tiled)
        return self.value

    def clear(self) -> None:
        self.key, self.value = None, None


def cache_usable(x: Tensor, weight: Tensor) -> bool:
    """The cache holds the quantization of the stored weights in their own dtype.  A training forward
    re-quantizes (see above).  Under autocast the autograd function quantizes an fp16 copy instead
    (reference semantics), and float64 runs on the dense entry point, so neither uses it."""
    if torch.is_grad_enabled() and weight.requires_grad:
        return False
    return (not torch.is_autocast_enabled() and weight.dtype != torch.float64 and x.dtype != torch.float64)
