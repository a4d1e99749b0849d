"""Transforms of the residual stream between runs of layers.

joined_projection: x <- W [x; x0] + b, with x0 the embedding's output (kept by an embedding built
with ``keep_origin``), W ``weight`` [width, 2 * width] (the stream's columns first) and b row
``row`` of ``shift`` [rows, width] (a model that runs a stretch of layers several times enters every
pass through such a part, each pass with a row of its own).  The two streams are laid side by side
in the products' type, one product leaves the new stream in 32-bit, the shift added.
"""

from ..kernels import library as K
from .base import Transform, operand_columns, pad_columns
from .registry import register


@register("transform", "joined_projection")
class JoinedProjection(Transform):
    only_launches_kernels = True

    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        self.width, self.row = params["width"], int(params.get("row", 0))
        weight, shift = tensors["weight"], tensors.get("shift")
        if tuple(weight.shape) != (self.width, 2 * self.width):
            raise ValueError(f"joined projection: the matrix is {tuple(weight.shape)}, expected {(self.width, 2 * self.width)}")
        self.columns = operand_columns(2 * self.width, weight.dtype)
        self.weight = pad_columns(weight, self.columns)
        self.shift = None
        if shift is not None:
            if shift.dim() != 2 or shift.shape[1] != self.width or not (0 <= self.row < shift.shape[0]):
                raise ValueError(f"joined projection: row {self.row} of a shift of shape {tuple(shift.shape)}")
            self.shift = shift[self.row].contiguous()
        self.packed = K.PackedWeight(self.weight) if self.weight.is_cuda else None

    def kernel_modules(self, dtype):
        return ("sublayer",)

    def forward(self, stream, step):
        if stream.origin is None:
            raise ValueError("joined projection: the embedding does not keep its output (keep_origin)")
        stream.flush()
        tokens = stream.x.shape[0]
        joined = step.buffer("reentry.joined", tokens, self.columns, step.dtype)
        K.join_rows(stream.x, stream.origin, joined)
        stream.cast = None
        K.gemm(joined, self.weight, K.epilogue_f32(stream.x, self.shift), packed=self.packed)
