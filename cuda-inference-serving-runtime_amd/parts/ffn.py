"""Gated feed-forward (SwiGLU): x + (silu(h Wg^T) * (h Wu^T)) Wd^T
(reference: runtime/model.py:116-119).  Gate and up run as one product against
the concatenated weight [gate; up].  With `bias` every projection adds `<name>.*_proj.bias`:
the products run as they are and a small kernel adds the bias (no fused activation then)."""
import torch

from ..kernels import ops
from .base import FeedForward, TensorSpec, matrix_operand, register_part


class GatedMLP(FeedForward):
    def __init__(self, name, hidden, intermediate, activation="silu", bias=False):
        if activation != "silu":
            raise ValueError(f"activation {activation!r}: only silu has a kernel")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.bias = bool(bias)
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def tensor_specs(self):
        n, H, I = self.name, self.hidden, self.intermediate
        specs = [TensorSpec(f"{n}.gate_proj.weight", (I, H)), TensorSpec(f"{n}.up_proj.weight", (I, H)),
                 TensorSpec(f"{n}.down_proj.weight", (H, I))]
        if self.bias:
            specs += [TensorSpec(f"{n}.gate_proj.bias", (I,)), TensorSpec(f"{n}.up_proj.bias", (I,)), TensorSpec(f"{n}.down_proj.bias", (H,))]
        return specs

    def bind(self, tensors, dtype):
        gate = matrix_operand(tensors[f"{self.name}.gate_proj.weight"], dtype)
        up = matrix_operand(tensors[f"{self.name}.up_proj.weight"], dtype)
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = matrix_operand(tensors[f"{self.name}.down_proj.weight"], dtype)
        if self.bias:   # (a bias keeps the type it is stored in; it is added in float)
            self.b_gate_up = torch.cat([tensors[f"{self.name}.gate_proj.bias"], tensors[f"{self.name}.up_proj.bias"]], dim=0).contiguous()
            self.b_down = tensors[f"{self.name}.down_proj.bias"].contiguous()

    def fuses_norm(self, norm, residual, ctx):
        return not self.bias and getattr(norm, "fusable_as", None) == "rms" and ops.fused_norm_ok(residual, self.w_gate_up, residual.shape[0])

    def forward(self, h, residual, ctx, norm=None):
        T = residual.shape[0]
        act = ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype)
        if self.bias:
            gate_up = ops.gemm(h, self.w_gate_up, ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
            ops.swiglu(ops.bias_add(gate_up, self.b_gate_up), act)
            return ops.bias_add(ctx.add_product(act, self.w_down, residual), self.b_down)
        if norm is not None:
            ops.gemm_swiglu(residual, self.w_gate_up, act, norm=(norm.weight, norm.eps, None), scratch=ctx.scratch)
        elif ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.scratch)   # one kernel: product and activation
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, gate_up=ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype), scratch=ctx.scratch)
        return ctx.add_product(act, self.w_down, residual)


class ClampedGLU(FeedForward):
    """y = (g sigmoid(slope g) (u + shift)) Wd^T with g = min(h Wg^T, limit), u = clamp(h Wu^T, -limit, limit).
    Gate and up run as one product against [gate; up]; `names` = (gate, up, down), the tensors' names under `name`."""

    def __init__(self, name, hidden, intermediate, limit, slope=1.702, shift=1.0, names=("gate", "up", "down")):
        if not limit > 0:
            raise ValueError("the clamp's limit must be positive")
        self.name, self.hidden, self.intermediate = name, hidden, intermediate
        self.limit, self.slope, self.shift, self.names = float(limit), float(slope), float(shift), tuple(names)
        self.w_gate_up = self.w_down = None

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def tensor_specs(self):
        H, I = self.hidden, self.intermediate
        return [TensorSpec(self._tensor(0), (I, H)), TensorSpec(self._tensor(1), (I, H)), TensorSpec(self._tensor(2), (H, I))]

    def bind(self, tensors, dtype):
        gate, up = (matrix_operand(tensors[self._tensor(i)], dtype) for i in (0, 1))
        self.w_gate_up = torch.cat([gate, up], dim=0).contiguous()
        self.w_down = matrix_operand(tensors[self._tensor(2)], dtype)

    def output(self, h, ctx):
        """The feed-forward's result, float [T, hidden], without the residual sum."""
        T = h.shape[0]
        law = (self.limit, self.slope, self.shift)
        act = ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype)
        if ops.swiglu_fused_ok(h, self.w_gate_up):
            ops.gemm_swiglu(h, self.w_gate_up, act, scratch=ctx.scratch, law=law)      # the product and the activation are one kernel
        else:
            ops.gemm_swiglu(h, self.w_gate_up, act, gate_up=ctx.buffer("ffn.gate_up", (T, 2 * self.intermediate), ctx.dtype),
                            scratch=ctx.scratch, law=law)
        return ctx.product_for_norm(act, self.w_down, "ffn.out")

    def forward(self, h, residual, ctx, norm=None):
        from .block import add_sublayer
        return add_sublayer(residual, self.output(h, ctx), None, 1.0)


class DenseMLP(FeedForward):
    """y = act(h Wu^T) Wd^T, one matrix up and one down, no gate.  `activation`: "gelu" (the exact form, with the error
    function) or "gelu_tanh".  `names` = (up, down), the tensors' names under `name`."""

    def __init__(self, name, hidden, intermediate, activation="gelu", names=("up", "down")):
        if activation not in ops.GELU_KINDS:
            raise ValueError(f"activation {activation!r}: one of {sorted(ops.GELU_KINDS)}")
        self.name, self.hidden, self.intermediate, self.activation = name, hidden, intermediate, activation
        self.names = tuple(names)
        self.w_up = self.w_down = None

    def _tensor(self, which):
        return f"{self.name}.{self.names[which]}"

    def tensor_specs(self):
        return [TensorSpec(self._tensor(0), (self.intermediate, self.hidden)), TensorSpec(self._tensor(1), (self.hidden, self.intermediate))]

    def bind(self, tensors, dtype):
        self.w_up, self.w_down = (matrix_operand(tensors[self._tensor(i)], dtype) for i in (0, 1))

    def _activations(self, h, ctx):
        T = h.shape[0]
        # the activation is the epilogue of the product where a kernel of this repository runs it
        return ops.gemm_gelu(h, self.w_up, ctx.buffer("ffn.act", (T, self.intermediate), ctx.dtype), self.activation, scratch=ctx.scratch,
                             product=ctx.buffer("ffn.up", (T, self.intermediate), ctx.dtype))

    def output(self, h, ctx):
        """The feed-forward's result, float [T, hidden], without the residual sum."""
        return ctx.product_for_norm(self._activations(h, ctx), self.w_down, "ffn.out")

    def forward(self, h, residual, ctx, norm=None):
        return ctx.add_product(self._activations(h, ctx), self.w_down, residual)


register_part("ffn", "gated_mlp", GatedMLP)
register_part("ffn", "dense_mlp", DenseMLP)
register_part("ffn", "clamped_glu", ClampedGLU)
