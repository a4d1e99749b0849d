"""Recurrent mixers with a state of fixed size per sequence (selective state-space layers).

selective_scan ("mamba1" wiring): parameters width, inner, state, dt_rank, taps.  Tensors:
in_weight [2*inner, width] (x, then the gate z), conv_weight [inner, taps], conv_bias [inner],
x_weight [dt_rank + 2*state, inner] (dt, B, C), dt_weight [inner, dt_rank], dt_bias [inner],
A_log [inner, state], D [inner], out_weight [width, inner].
    x <- silu(conv(x));  dt = softplus(dt_weight dt_low + dt_bias);  A = -exp(A_log)
    S[c, n] <- exp(dt_c A[c, n]) S[c, n] + dt_c x_c B_n;   y_c = sum_n S[c, n] C_n + D_c x_c
    out = out_weight (y * silu(z))

head_scan ("mamba2" wiring): parameters width, heads, vdim, state, groups, norm_groups, taps, eps.
Tensors: in_weight [2*inner + 2*groups*state + heads, width] (z, x, B, C, dt; inner = heads*vdim),
conv_weight [inner + 2*groups*state, taps], conv_bias, dt_bias [heads], A_log [heads], D [heads],
norm_weight [inner], out_weight [width, inner].
    (x, B, C) <- silu(conv(x, B, C));  dt = softplus(dt + dt_bias), no clamp
    S_h <- exp(-exp(A_log_h) dt_h) S_h + dt_h B_g x_h^T  (S_h is [state, vdim], g = h / (heads / groups))
    y_h = S_h^T C_g + D_h x_h;   out = out_weight (rms_norm in norm_groups parts of (y * silu(z)) * norm_weight)

The convolution's last taps - 1 inputs and the state S are the sequence's state: one float32 row
per sequence in the cache's state area (``StateSpec``), zero for a new sequence, read and written
by the kernels through the step's table of slots.  Projections run as ordinary products with
32-bit results; everything behind them that enters the recurrence stays 32-bit.  A step may bring
any number of tokens of a sequence (a prompt, a chunk, one token): the kernels walk them in order
from the state the last step left.
"""

import torch

from ..cache.storage import StateSpec
from ..kernels import library as K
from .base import Mixer, operand_columns, packed_for_stream, pad_columns
from .registry import register


class _Recurrent(Mixer):
    only_launches_kernels = True

    def kernel_modules(self, dtype):
        return ("state_space",)

    def state_spec(self):
        return StateSpec((self.conv_state + self.scan_state,), "float32")

    def _state(self, memory):
        """(the convolution's inputs, the scan's state): column ranges of the entry's state rows."""
        rows = memory.state()
        return rows[:, :self.conv_state], rows[:, self.conv_state:]


@register("mixer", "selective_scan")
class SelectiveScan(_Recurrent):
    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        p = params
        self.width, self.inner, self.state, self.dt_rank = p["width"], p["inner"], p["state"], p["dt_rank"]
        self.taps = int(p["taps"])
        shapes = {"in_weight": (2 * self.inner, self.width), "conv_weight": (self.inner, self.taps),
                  "conv_bias": (self.inner,), "x_weight": (self.dt_rank + 2 * self.state, self.inner),
                  "dt_weight": (self.inner, self.dt_rank), "dt_bias": (self.inner,),
                  "A_log": (self.inner, self.state), "D": (self.inner,), "out_weight": (self.width, self.inner)}
        for role, shape in shapes.items():
            if tuple(tensors[role].shape) != shape:
                raise ValueError(f"selective_scan: {role} is {tuple(tensors[role].shape)}, expected {shape}")
        if not (1 <= self.state <= 256 and 1 <= self.dt_rank <= 1024):
            raise ValueError(f"selective_scan: state {self.state} (1..256) or dt_rank {self.dt_rank} (1..1024) outside what the kernels take")
        dtype = tensors["in_weight"].dtype
        self.in_weight = tensors["in_weight"].contiguous()
        self.inner_cols = operand_columns(self.inner, dtype)
        self.x_weight = pad_columns(tensors["x_weight"], self.inner_cols)
        self.out_weight = pad_columns(tensors["out_weight"], self.inner_cols)
        self.dt_weight = tensors["dt_weight"].contiguous()
        self.conv_weight, self.conv_bias = tensors["conv_weight"].contiguous(), tensors["conv_bias"]
        self.dt_bias, self.A_log, self.D = tensors["dt_bias"], tensors["A_log"].contiguous(), tensors["D"]
        self.conv_state, self.scan_state = (self.taps - 1) * self.inner, self.inner * self.state
        # second copies for decode steps, which read the weights and little else
        on_gpu = self.in_weight.is_cuda
        self.in_packed = K.PackedWeight(self.in_weight) if on_gpu else None
        self.x_packed = K.PackedWeight(self.x_weight) if on_gpu else None
        self.out_packed = packed_for_stream(self.out_weight) if on_gpu else None

    def forward(self, h, step, memory, stream):
        tokens, inner = h.shape[0], self.inner
        conv_state, scan_state = self._state(memory)
        xz = step.buffer("scan.in", tokens, 2 * inner, "float32")
        K.gemm(h, self.in_weight, K.epilogue_f32(xz), packed=self.in_packed)
        x = step.buffer("scan.x", tokens, inner, "float32")
        # the next product reads x in the products' type; in a float32 model that is x itself
        cast = step.buffer("scan.x_operand", tokens, self.inner_cols, step.dtype) if step.dtype_is_bf16 else None
        K.causal_conv(xz[:, :inner], self.conv_weight, self.conv_bias, x, conv_state, step, cast=cast)
        low = step.buffer("scan.low", tokens, self.dt_rank + 2 * self.state, "float32")
        K.gemm(cast if cast is not None else x, self.x_weight, K.epilogue_f32(low), packed=self.x_packed)
        dt = step.buffer("scan.dt", tokens, inner, "float32")
        K.dt_project(low[:, :self.dt_rank], self.dt_weight, self.dt_bias, dt)
        gated = step.buffer("scan.gated", tokens, self.inner_cols, step.dtype)
        K.selective_scan(x, xz[:, inner:], dt, low[:, self.dt_rank:self.dt_rank + self.state],
                         low[:, self.dt_rank + self.state:], self.A_log, self.D, gated, scan_state, step,
                         carry=K.scan_carry(step, self.scan_state, inner))
        stream.add_product(step, gated, self.out_weight, packed=self.out_packed)


@register("mixer", "head_scan")
class HeadScan(_Recurrent):
    def __init__(self, params, tensors):
        super().__init__(params, tensors)
        p = params
        self.width, self.heads, self.vdim, self.state = p["width"], p["heads"], p["vdim"], p["state"]
        self.groups, self.norm_groups, self.taps, self.eps = p["groups"], p["norm_groups"], int(p["taps"]), float(p["eps"])
        self.inner, self.bc = self.heads * self.vdim, self.groups * self.state
        self.channels = self.inner + 2 * self.bc
        if self.heads % self.groups != 0 or self.inner % self.norm_groups != 0:
            raise ValueError(f"head_scan: {self.heads} heads in {self.groups} groups, {self.inner} channels in "
                             f"{self.norm_groups} parts of the norm: both must divide")
        shapes = {"in_weight": (self.inner + self.channels + self.heads, self.width),
                  "conv_weight": (self.channels, self.taps), "conv_bias": (self.channels,),
                  "dt_bias": (self.heads,), "A_log": (self.heads,), "D": (self.heads,),
                  "norm_weight": (self.inner,), "out_weight": (self.width, self.inner)}
        for role, shape in shapes.items():
            if tuple(tensors[role].shape) != shape:
                raise ValueError(f"head_scan: {role} is {tuple(tensors[role].shape)}, expected {shape}")
        if not 1 <= self.state <= 256:
            raise ValueError(f"head_scan: state {self.state} outside 1..256, what the kernel takes")
        dtype = tensors["in_weight"].dtype
        self.in_weight = tensors["in_weight"].contiguous()
        self.inner_cols = operand_columns(self.inner, dtype)
        self.out_weight = pad_columns(tensors["out_weight"], self.inner_cols)
        self.conv_weight, self.conv_bias = tensors["conv_weight"].contiguous(), tensors["conv_bias"]
        self.dt_bias, self.A_log, self.D, self.norm_weight = tensors["dt_bias"], tensors["A_log"], tensors["D"], tensors["norm_weight"]
        # (the scan's kernel lays a head's state out in tiles of four channels)
        self.conv_state, self.scan_state = (self.taps - 1) * self.channels, self.heads * self.state * ((self.vdim + 3) // 4 * 4)
        on_gpu = self.in_weight.is_cuda
        self.in_packed = K.PackedWeight(self.in_weight) if on_gpu else None
        self.out_packed = packed_for_stream(self.out_weight) if on_gpu else None

    def forward(self, h, step, memory, stream):
        tokens, inner, bc = h.shape[0], self.inner, self.bc
        conv_state, scan_state = self._state(memory)
        fused = step.buffer("scan.in", tokens, inner + self.channels + self.heads, "float32")
        K.gemm(h, self.in_weight, K.epilogue_f32(fused), packed=self.in_packed)
        xbc = step.buffer("scan.x", tokens, self.channels, "float32")
        K.causal_conv(fused[:, inner:inner + self.channels], self.conv_weight, self.conv_bias, xbc, conv_state, step)
        y = step.buffer("scan.y", tokens, inner, "float32")
        K.head_scan(xbc[:, :inner], xbc[:, inner:inner + bc], xbc[:, inner + bc:], fused[:, inner + self.channels:],
                    self.dt_bias, self.A_log, self.D, y, scan_state, step, self.heads, self.vdim, self.state, self.groups,
                    carry=K.scan_carry(step, self.scan_state, self.heads))
        gated = step.buffer("scan.gated", tokens, self.inner_cols, step.dtype)
        K.gated_norm(y, fused[:, :inner], self.norm_weight, self.norm_groups, self.eps, gated)
        stream.add_product(step, gated, self.out_weight, packed=self.out_packed)
