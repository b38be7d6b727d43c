"""The residual stream of a step: float32 rows plus at most one pending branch
output.  The sum is applied by the next norm (one kernel does add and norm) or
when the value is asked for."""
from __future__ import annotations

import torch


class Residual:
    def __init__(self, x: torch.Tensor) -> None:
        assert x.dtype == torch.float32
        self._x = x
        self._deferred = None  # a norm (with its addition) that its consumer has been left to compute
        self.pending = None

    @property
    def x(self) -> torch.Tensor:
        if self._deferred is not None:
            self._x, self._deferred = self._deferred.residual(), None
        return self._x

    def add(self, delta: torch.Tensor) -> None:
        if self.pending is not None:
            raise AssertionError("a branch output is already pending on the residual")
        if delta.shape != self.x.shape:
            raise ValueError(f"branch output {tuple(delta.shape)} does not match residual {tuple(self.x.shape)}")
        self.pending = delta

    def normed(self, ctx, weight, eps: float, want32: bool = False, defer: bool = False):
        """``defer``: the part that takes the rows has said it accepts rows that are not computed yet (the
        kernel set's ``defer_norm``): it may then do addition and norm inside a launch of its own."""
        if defer and hasattr(ctx.ops, "defer_norm"):
            p = ctx.ops.defer_norm(self.x, self.pending, weight, eps, ctx.dtype)
            self.pending, self._deferred = None, p
            return p, (p if want32 else None)
        h, h32 = ctx.ops.add_rmsnorm(self.x, self.pending, weight, eps, ctx.dtype, want32)
        self.pending = None
        return h, h32

    def value(self, ctx) -> torch.Tensor:
        if self.pending is not None:
            ctx.ops.add_residual(self.x, self.pending)
            self.pending = None
        return self.x

    def rows(self, ctx, idx: torch.Tensor) -> "Residual":
        """The residual of the chosen rows only (what is pending stays pending)."""
        r = Residual(ctx.ops.gather_rows(self.x, idx))
        if self.pending is not None:
            r.pending = ctx.ops.gather_rows(self.pending, idx)
        return r
