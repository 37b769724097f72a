"""Root-mean-square normalisation over the residual stream."""

from __future__ import annotations

from ..hostcore import core
from ..kernels import ops
from .base import Norm, TensorSpec
from .lowering import OneOp


class NoNorm(Norm):
    """No norm at all: a sublayer that reads the residual stream itself.  y = x in the output
    dtype (after the partial sums before it have been added into the stream)."""

    graph_safe = True
    lowerable = True

    def __init__(self, size: int):
        self.size = int(size)
        self._alone = None

    def forward(self, h, out_dtype, rows=None, partials=None):
        if rows is not None:
            raise ValueError("the stream as it stands is read whole")
        if self._alone is None:
            self._alone = OneOp(out_dtype, self.size, 0, self.lower)
        _logits, x, _pending = self._alone.run(None, h, pending=partials)
        return x

    def lower(self, program, select_rows: bool = False) -> None:
        if select_rows:
            raise ValueError("the stream as it stands is read whole")
        program.append("stream_cast", core.stream_cast_params())


class RMSNorm(Norm):
    """y = (x * rsqrt(mean(x^2) + eps)) * weight, statistics in float32.

    `eps` is added to the mean of squares, inside the root; the normalised value is rounded
    to the output dtype before the weight multiplies it
    (reference: mercury/model/qwen2.py:27-31).  The residual sum the reference folds into the
    norm (`x + residual`, mercury/model/qwen2.py:27-28) arrives here as `partials`: partial
    sums of the preceding projection that are added into the float32 stream in the same pass.

    `one_plus`: the stored weight lies around zero and 1 + weight multiplies (the sum is
    made once, at load, in float32).  `round_once`: x * rstd * weight is computed in float32
    and rounded to the output dtype once, instead of the normalised value first.
    """

    graph_safe = True
    lowerable = True

    def __init__(self, size: int, eps: float, one_plus: bool = False, round_once: bool = False):
        self.size = int(size)
        self.eps = float(eps)
        self.one_plus, self.round_once = bool(one_plus), bool(round_once)
        self.weight = None
        self._alone = None

    def param_specs(self) -> dict:
        return {"weight": TensorSpec((self.size,), role="vector",
                                     init="normal" if self.one_plus else "one_plus_normal")}

    def bind(self, params, dtype, device) -> None:
        self.weight = params["weight"]
        if self.one_plus:
            self.weight = (1.0 + self.weight.float()).contiguous()
        self._alone = None

    def forward(self, h, out_dtype, rows=None, partials=None):
        if self.round_once:
            # the operation `lower` appends, as a program of its own
            if rows is not None:
                raise ValueError("a norm that rounds once runs over selected rows inside a model's program only")
            if self._alone is None:
                self._alone = OneOp(out_dtype, self.size, 0, self.lower)
            _logits, x, _pending = self._alone.run(None, h, pending=partials)
            return x
        # one kernel; its launch is the one the lowered operation makes
        return ops.rmsnorm(h, self.weight, self.eps, out_dtype, rows=rows, partials=partials)

    def lower(self, program, select_rows: bool = False) -> None:
        """`select_rows`: normalise the step's wanted rows only (before an output head)."""
        program.append("norm_once" if self.round_once else "norm", core.norm_params(
            self.weight.data_ptr(), ops.dtype_code(self.weight.dtype), self.eps, select_rows,
            self.round_once))

    def weight_bytes(self) -> int:
        return self.weight.numel() * self.weight.element_size()
