"""RMSNorm: y = x * rsqrt(mean(x^2) + eps) * w in float
(reference: runtime/reference.py:5-6, kernels/ops.cu:3-19).
LayerNorm: y = (x - mean) * rsqrt(var + eps) * w (+ b), var the mean of the squared deviations, in float."""
import torch

from ..kernels import ops
from .base import Part, TensorSpec, register_part


class RMSNorm(Part):
    # What a kernel that takes over this norm must compute: "rms" = x * rsqrt(mean(x^2) + eps) * weight, with the
    # attributes `weight` (float [dim]) and `eps`.  A mixer, feed-forward or head fuses any norm that says so.
    fusable_as = "rms"
    adds_partials = True    # forward adds the partial sums of a product left unfinished before it (ctx.add_product)

    def __init__(self, name, dim, eps, tensor=None):
        """`tensor`: the weight's full name where it is not `<name>.weight`."""
        self.name, self.dim, self.eps = name, dim, float(eps)
        self.tensor = tensor if tensor is not None else name + ".weight"
        self.weight = None

    def tensor_specs(self):
        return [TensorSpec(self.tensor, (self.dim,), init="one_plus_normal")]

    def bind(self, tensors, dtype):
        self.weight = tensors[self.tensor].to(torch.float32).contiguous()  # exact widening

    def forward(self, x, ctx, rows=None, tag="norm"):
        n_out = x.shape[0] if rows is None else rows.shape[0]
        out = ctx.buffer(tag, (n_out, self.dim), ctx.dtype)
        partials = ctx.take_unfinished(x)
        if partials is not None:
            # the product before was left as partial sums: they, the residual and the norm are one kernel
            if rows is None and ops.partials_ok(x):
                return ops.rmsnorm_partials(x, partials, self.weight, out, self.eps)
            ops.add_partials(x, partials)
        return ops.rmsnorm(x, self.weight, out, self.eps, rows)


class LayerNorm(Part):
    """The centred norm with a weight and, with `bias`, a bias.  `gain`: a constant that multiplies the result (it rides
    in the weight and the bias): a model whose head scales its logits gives it to its last norm, since the head is linear.
    No product takes this norm over (it states no `fusable_as`) and it adds no partial sums."""

    def __init__(self, name, dim, eps, tensor=None, bias=False, bias_tensor=None, gain=1.0):
        self.name, self.dim, self.eps, self.gain = name, dim, float(eps), float(gain)
        self.tensor = tensor if tensor is not None else name + ".weight"
        self.bias_tensor = (bias_tensor if bias_tensor is not None else name + ".bias") if bias else None
        self.weight = self.bias = None

    def tensor_specs(self):
        specs = [TensorSpec(self.tensor, (self.dim,), init="one_plus_normal")]
        if self.bias_tensor is not None:
            specs.append(TensorSpec(self.bias_tensor, (self.dim,)))
        return specs

    def bind(self, tensors, dtype):
        self.weight = (tensors[self.tensor].to(torch.float32) * self.gain).contiguous()
        if self.bias_tensor is not None:
            self.bias = (tensors[self.bias_tensor].to(torch.float32) * self.gain).contiguous()

    def forward(self, x, ctx, rows=None, tag="norm"):
        n_out = x.shape[0] if rows is None else rows.shape[0]
        ctx.settle(x)
        return ops.layernorm(x, self.weight, ctx.buffer(tag, (n_out, self.dim), ctx.dtype), self.eps, rows, bias=self.bias)


register_part("norm", "rmsnorm", RMSNorm)
register_part("norm", "layernorm", LayerNorm)
