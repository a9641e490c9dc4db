"""Host-side mirror of the reference's tensor seams for the quantized path (device-backed, no CPU fallback).

  Shape            reference core/src/commonMain/kotlin/sk/ai/net/Shape.kt (dimensions, volume, rank)
  DeviceTensor     fp32 activations on the device; the receiver of matmul, as Linear.forward needs
                   (core/.../nn/Linear.kt:48: input.matmul(weight.t()) + bias)
  QuantizedTensor  GGUF block bytes on the device with the logical [out, in] shape of Linear
                   (core/.../nn/Linear.kt:26-28); t() is a view flag, never a copy (the reference's t()
                   materialises a transpose on every forward, core/.../impl/DoublesTensor.kt:362-387)
  QuantizedLinear  Module.forward for y = x . W^T (+ bias)   (core/.../nn/Module.kt:12, nn/Linear.kt:43-49)
  ReLU, MLP        the activation module (core/.../nn/activations/relu.kt:7-12) and the sequential container
                   (core/.../nn/topology/MLP.kt:8-19: forward feeds each module's output to the next)

Error behaviour follows the reference: misaligned inner dimensions raise ValueError("Shapes do not align.")
(core/.../impl/DoublesTensor.kt:256,268); operand ranks the reference's matmul does not know raise
ValueError("Unsupported tensor shapes for multiplication: ...") (DoublesTensor.kt:359).
"""
from __future__ import annotations

import numpy as np

from . import runtime, synth


class Shape:
    def __init__(self, *dimensions):
        self.dimensions = tuple(int(d) for d in dimensions)

    @property
    def rank(self):
        return len(self.dimensions)

    @property
    def volume(self):
        v = 1
        for d in self.dimensions:
            v *= d
        return v

    def __eq__(self, other):
        return isinstance(other, Shape) and self.dimensions == other.dimensions

    def __repr__(self):
        return f"Shape{self.dimensions}"


class QuantizedTensor:
    def __init__(self, ctx, ggml_type, shape, buf, transposed=False):
        if shape.rank != 2:
            raise ValueError("quantized weights are rank-2 [out, in] tensors")
        runtime.row_bytes(ggml_type, shape.dimensions[1])  # the reference's block-multiple check (Quants.kt:10-20)
        self.ctx, self.ggml_type, self._shape, self.buf, self.transposed = ctx, ggml_type, shape, buf, transposed
        self.expanded = None  # device copy made by expand_for_gemm

    @classmethod
    def from_bytes(cls, ctx, ggml_type, n_out, n_in, raw):
        raw = np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
        if raw.size != n_out * runtime.row_bytes(ggml_type, n_in):
            raise ValueError("byte count does not match the shape")
        return cls(ctx, ggml_type, Shape(n_out, n_in), ctx.to_device(raw))

    @property
    def shape(self):
        d = self._shape.dimensions
        return Shape(d[1], d[0]) if self.transposed else self._shape

    @property
    def rank(self):
        return 2

    @property
    def size(self):
        return self._shape.volume

    def t(self):
        v = QuantizedTensor(self.ctx, self.ggml_type, self._shape, self.buf, not self.transposed)
        v.expanded = self.expanded
        return v

    def expand_for_gemm(self):
        """Keeps the fp16-pair copy of the weights that rank-2 products multiply with (4 bytes per weight of device
        memory), so that later products skip the per-call weight pass.  Q4_K has no such pass and is left as it is."""
        if self.expanded is None and self.ggml_type != synth.Q4_K:
            n_out, n_in = self._shape.dimensions
            self.expanded = self.ctx.gemm_expand(self.ggml_type, self.buf, n_out, n_in)
        return self

    def dequantize(self):
        """-> DeviceTensor [out, in] fp32 (bit-exact ggml dequantization)."""
        out = DeviceTensor.empty(self.ctx, self._shape)
        self.ctx.dequant(self.ggml_type, self.buf, self._shape.volume, out.buf)
        return out

    def matmul(self, other):
        raise ValueError(
            f"Unsupported tensor shapes for multiplication: {list(self.shape.dimensions)} and "
            f"{list(other.shape.dimensions)}"
        )


class DeviceTensor:
    def __init__(self, ctx, shape, buf):
        self.ctx, self.shape, self.buf = ctx, shape, buf

    @classmethod
    def empty(cls, ctx, shape):
        return cls(ctx, shape, ctx.alloc(max(4 * shape.volume, 16)))

    @classmethod
    def from_numpy(cls, ctx, array):
        a = np.ascontiguousarray(array, dtype=np.float32)
        return cls(ctx, Shape(*a.shape), ctx.to_device(a))

    @property
    def rank(self):
        return self.shape.rank

    @property
    def size(self):
        return self.shape.volume

    def numpy(self):
        return self.buf.download(np.float32, self.shape.volume).reshape(self.shape.dimensions)

    def matmul(self, other):
        """x.matmul(W.t()) for a transposed quantized weight: rank 1 -> matvec, rank 2 -> GEMM; ranks 3 and 4 multiply
        every [.., in] row, as the reference does for a 3-D or 4-D tensor times a matrix
        (core/.../impl/DoublesTensor.kt:281-357; TensorTest.kt:393-538): the leading dimensions are the GEMM's rows."""
        if isinstance(other, QuantizedTensor) and other.transposed and self.rank in (3, 4):
            lead = self.shape.dimensions[:-1]
            if self.shape.dimensions[-1] != other._shape.dimensions[1]:
                raise ValueError("Shapes do not align.")
            rows = DeviceTensor(self.ctx, Shape(self.shape.volume // self.shape.dimensions[-1], self.shape.dimensions[-1]), self.buf)
            out = rows.matmul(other)
            return DeviceTensor(self.ctx, Shape(*lead, other._shape.dimensions[0]), out.buf)
        if not isinstance(other, QuantizedTensor) or not other.transposed or self.rank not in (1, 2):
            raise ValueError(
                f"Unsupported tensor shapes for multiplication: {list(self.shape.dimensions)} and "
                f"{list(other.shape.dimensions)}"
            )
        n_out, n_in = other._shape.dimensions
        if self.shape.dimensions[-1] != n_in:
            raise ValueError("Shapes do not align.")
        if self.rank == 1:
            y = DeviceTensor.empty(self.ctx, Shape(n_out))
            self.ctx.matvec_q(other.ggml_type, other.buf, n_out, n_in, self.buf, y.buf)
            return y
        m = self.shape.dimensions[0]
        a16 = self.ctx.alloc(max(2 * m * n_in, 16))
        self.ctx.f32_to_bf16(self.buf, m * n_in, a16)
        c = DeviceTensor.empty(self.ctx, Shape(m, n_out))
        if other.expanded is not None:
            self.ctx.gemm_expanded(other.expanded, n_out, n_in, a16, m, c.buf)
        else:
            self.ctx.gemm_q(other.ggml_type, other.buf, n_out, n_in, a16, m, c.buf)
        return c

    def relu(self):
        """max(x, 0) elementwise (core/.../impl/DoublesTensor.kt:389-390)."""
        out = DeviceTensor.empty(self.ctx, self.shape)
        self.ctx.relu(self.buf, self.shape.volume, out.buf)
        return out

    def __add__(self, other):
        if not isinstance(other, DeviceTensor):
            raise TypeError("device tensors add device tensors")
        rows = self.shape.volume // other.shape.volume
        if other.shape.dimensions != self.shape.dimensions[-other.rank:] or rows * other.shape.volume != self.shape.volume:
            raise ValueError("Shapes do not align.")
        out = DeviceTensor.empty(self.ctx, self.shape)
        self.ctx.copy(out.buf, self.buf, 4 * self.shape.volume)
        for r in range(rows):  # the bias broadcast of Linear: one row at a time
            self.ctx.add_inplace(out.buf.ptr + 4 * r * other.shape.volume, other.buf, other.shape.volume)
        return out


class QuantizedLinear:
    """y = x . W^T + b with W [out, in] quantized on the device (bias optional, fp32)."""

    def __init__(self, weight: QuantizedTensor, bias: DeviceTensor | None = None, name="Linear"):
        self.name, self.weight, self.bias = name, weight, bias

    def forward(self, x: DeviceTensor) -> DeviceTensor:
        y = x.matmul(self.weight.t())
        return y + self.bias if self.bias is not None else y

    __call__ = forward


class ReLU:
    def __init__(self, name="ReLU"):
        self.name = name

    def forward(self, x: DeviceTensor) -> DeviceTensor:
        return x.relu()

    __call__ = forward


class MLP:
    """Sequential composition: forward(x) = m_n(... m_2(m_1(x)))."""

    def __init__(self, *modules, name="FeedForwardNetwork"):
        self.name, self.modules = name, list(modules)

    def forward(self, x: DeviceTensor) -> DeviceTensor:
        for m in self.modules:
            x = m.forward(x)
        return x

    __call__ = forward
