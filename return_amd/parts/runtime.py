"""What every part is given at construction: device, precision, the kernels."""
from __future__ import annotations

from typing import Dict, Optional

import torch

_TORCH_DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32}


class ScaledRows:
    """Rows whose RMSNorm is not finished: ``tensor`` [M, size] holds h * w_norm in the compute dtype,
    ``partials`` [M, n] fp32 hold shares of each row's sum of squares of h. The norm's 1/rms is a
    number per row, so a product may multiply its result rows by rsqrt(sum(partials) / size + eps)
    instead of its operand: norm(h) W^T = rstd * ((h * w_norm) W^T). A kernel set that offers
    ``linear_add_norm`` makes such rows in the epilogue of the product that feeds the residual
    stream, and takes them in ``linear`` and ``linear_silu_mul``; ``norm`` is the norm part they
    were made for, which hands them on as its output."""
    __slots__ = ("tensor", "partials", "size", "eps", "norm")

    def __init__(self, tensor, partials, size, eps, norm=None):
        self.tensor, self.partials, self.size, self.eps, self.norm = tensor, partials, int(size), float(eps), norm

    @property
    def shape(self):
        return self.tensor.shape

    @property
    def dtype(self):
        return self.tensor.dtype


class Slabs:
    """A product's result left as shares: ``tensor`` [n, M, N] fp32, the result being their sum in order
    (a product whose K was cut into n pieces, one share each). A norm that takes them adds them up,
    rounds the sum as the one product's result would have been rounded, and adds it into the residual
    stream."""
    __slots__ = ("tensor",)

    def __init__(self, tensor):
        self.tensor = tensor

    @property
    def shape(self):
        return self.tensor.shape[1:]


class ResidualSink:
    """Given to a part for its last product when what the product makes goes nowhere but into the
    residual stream, through a norm that takes every form of it: ``project(x, w)`` is x @ w^T in
    whichever form the kernel set forms fastest for that (``linear_residual``: plain rows or Slabs)."""

    def __init__(self, ops):
        self.ops = ops

    def project(self, x, w):
        if hasattr(self.ops, "linear_residual"):
            return self.ops.linear_residual(x, w)
        return self.ops.linear(x, w)


class NormSink(ResidualSink):
    """The sink when the kernel set can finish the step's next norm inside the product: ``project(x, w)``
    adds x @ w^T into ``h`` and returns the next part's input as ScaledRows, in place of the product's
    result that the next norm would add."""

    def __init__(self, ops, h, norm):
        self.ops, self.h, self.norm = ops, h, norm

    def project(self, x, w):
        rows = self.ops.linear_add_norm(x, w, self.h, self.norm.weight, self.norm.eps)
        rows.norm = self.norm
        return rows


class Runtime:
    """Device, compute dtype and kernel set of one engine.

    dtype "bfloat16": matrices, activations and the cache are bfloat16; the residual
    stream, norm statistics, softmax, rotation and logits are 32-bit.
    dtype "float32": everything is 32-bit and no reduced-precision matrix mode is used.

    ``ops`` is the kernel set (return_amd.kernels.hip_ops.HipOps when none is given;
    constructing that fails loudly if the HIP library cannot be built or loaded).
    """

    def __init__(self, device="cuda:0", dtype="bfloat16", ops=None):
        self.device = torch.device(device)
        self.dtype_name = dtype
        self.dtype = _TORCH_DTYPES[dtype]
        if ops is None:
            from ..kernels.hip_ops import HipOps
            ops = HipOps(self.device)
        self.ops = ops
        self._cast: Dict[int, torch.Tensor] = {}
        self.products = []                  # (weight, gated, result dtype) of the parts' matrix products
        self.norm_pairs = []                # (weight before, norm weight, eps, weight after, gated) of norms between two products

    # ---- weight preparation -------------------------------------------------
    def matrix(self, t: torch.Tensor) -> torch.Tensor:
        """A matrix operand (projection, embedding table) in the compute dtype, on the device.

        The same stored tensor gives the same prepared tensor (tied weights stay one copy).
        """
        key = (t.data_ptr(), tuple(t.shape), t.dtype)
        hit = self._cast.get(key)
        if hit is None:
            # the stored tensor is kept too: while it lives, its address cannot go to another tensor
            hit = (t, t.to(device=self.device, dtype=self.dtype).contiguous())
            self._cast[key] = hit
        return hit[1]

    def product(self, w: torch.Tensor, gated: bool = False, out_dtype: Optional[torch.dtype] = None,
                residual: bool = False) -> torch.Tensor:
        """Notes that the part will multiply by w (ops.linear, or ops.linear_silu_mul when gated; residual:
        through a sink, as the product whose result goes into the residual stream) and returns w. The
        kernel set may measure, once the model is built, which of its ways to form the products of these
        shapes is fastest; a part that does not note its weights is served by rules."""
        self.products.append((w, gated, "residual" if residual else out_dtype))
        return w

    def vector32(self, t: torch.Tensor) -> torch.Tensor:
        """A small vector (norm weight) as 32-bit floats; bf16 values convert exactly."""
        return t.to(device=self.device, dtype=torch.float32).contiguous()

    def forget_casts(self) -> None:
        self._cast.clear()

    # ---- scratch ------------------------------------------------------------
    def empty(self, *shape, dtype: Optional[torch.dtype] = None) -> torch.Tensor:
        return torch.empty(*shape, dtype=dtype or self.dtype, device=self.device)
