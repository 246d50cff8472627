"""Arrangement of parts in a layer.  PreNormBlock is the Llama arrangement
(reference: runtime/model.py:106-119): x = x + mixer(norm1(x)); x = x + ffn(norm2(x)),
the residual stream x kept in float.  SandwichBlock norms each sublayer's result as well
and scales it: x = x + m norm1b(mixer(norm1(x))); x = x + m norm2b(ffn(norm2(x)))."""
from ..kernels import ops
from .base import Part, register_part


class PreNormBlock(Part):
    def __init__(self, mixer_norm, mixer, ffn_norm=None, ffn=None):
        """`ffn` None (and no `ffn_norm`): a layer without a feed-forward."""
        if (ffn is None) != (ffn_norm is None):
            raise ValueError("a feed-forward comes with the norm before it, or not at all")
        self.mixer_norm, self.mixer, self.ffn_norm, self.ffn = mixer_norm, mixer, ffn_norm, ffn

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.ffn_norm, self.ffn) if p is not None]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype):
        for p in self.parts():
            p.bind(tensors, dtype)

    def prepare(self, device, dtype):
        for p in self.parts():
            p.prepare(device, dtype)

    # What the block keeps between steps, asked of the block (not of a part inside it): one mixer here, so one need
    # of each kind; an arrangement with more parts that keep something answers for all of them.
    def cache_need(self):
        return self.mixer.cache_need()

    def cache_read(self):
        return self.mixer.cache_read() if hasattr(self.mixer, "cache_read") else None

    def state_need(self):
        return self.mixer.state_need()

    def kernel_units(self, dtype):
        """Shared objects beside the core that the parts need (names of kernels.library.units())."""
        return [u for p in self.parts() if hasattr(p, "kernel_units") for u in p.kernel_units(dtype)]

    def step_arrays(self):
        """Step arrays that the parts want every step's metadata to carry from the start (engine.context.StepArray)."""
        return [a for p in self.parts() if hasattr(p, "step_arrays") for a in p.step_arrays()]

    def first_norm(self):
        """The norm that reads the residual stream first: the block before may leave its last product to it."""
        return self.mixer_norm

    def forward(self, residual, ctx, site):
        # ctx.next_norm names the norm that reads the residual stream after the part that runs: a part's last
        # product may be left to it (ctx.add_product); on entry it is the norm after this block
        after = ctx.next_norm
        ffn_fuses = self.ffn is not None and self.ffn.fuses_norm(self.ffn_norm, residual, ctx)
        ctx.next_norm = after if self.ffn is None else None if ffn_fuses else self.ffn_norm
        if self.mixer.fuses_norm(self.mixer_norm, residual, ctx):
            ctx.settle(residual)
            residual = self.mixer.forward(None, residual, ctx, site, norm=self.mixer_norm)
        else:
            residual = self.mixer.forward(self.mixer_norm.forward(residual, ctx), residual, ctx, site)
        if self.ffn is None:
            return residual
        if ffn_fuses:
            ctx.settle(residual)
            ctx.next_norm = after
            return self.ffn.forward(None, residual, ctx, norm=self.ffn_norm)
        h = self.ffn_norm.forward(residual, ctx)
        ctx.settle(residual)       # (a norm that adds no partial sums)
        ctx.next_norm = after
        return self.ffn.forward(h, residual, ctx)


class NormedMean:
    """What a mixer made of two mixers side by side hands to the arrangement around it: half the sum of two results,
    each RMS-normed over the width with a weight of its own (float [T, H] each, or the partial sums of a cut product).  The arrangement's kernel that adds
    a sublayer's result to the residual stream makes the mean on the way (ops.post_norm_add)."""

    def __init__(self, first, first_weight, second, second_weight, eps):
        self.first, self.first_weight, self.second, self.second_weight, self.eps = first, first_weight, second, second_weight, eps


def add_sublayer(residual, result, norm, mult, eps=None, following=None):
    """residual += mult * norm(result) (norm None: mult * result); `result` float rows or a NormedMean.
    `following` = (norm part, out): the RMS norm that reads the residual stream next is made by the same kernel."""
    weight = None if norm is None else norm.weight
    eps = norm.eps if norm is not None else eps
    then = None if following is None else (following[0].weight, following[0].eps, following[1])
    if isinstance(result, NormedMean):
        if eps is not None and eps != result.eps:
            raise ValueError("the norms inside a mean of two results and the norm around it must share their eps (one kernel)")
        return ops.post_norm_add(residual, result.first, weight, result.eps, mult,
                                 second=(result.second, result.first_weight, result.second_weight), following=then)
    return ops.post_norm_add(residual, result, weight, 0.0 if eps is None else eps, mult, following=then)


class SandwichBlock(Part):
    """A norm before and after each sublayer, the normed result times `mult` added to the float residual stream.
    Its mixer and feed-forward give their result without the residual sum (`output`); `ffn` None: a layer without
    a feed-forward.  The norms after the sublayers are RMS norms (`weight`, `eps`); the sum, the norm and the scale
    are one kernel."""

    def __init__(self, mixer_norm, mixer, mixer_post, ffn_norm=None, ffn=None, ffn_post=None, mult=1.0):
        if (ffn is None) != (ffn_norm is None) or (ffn is None) != (ffn_post is None):
            raise ValueError("a feed-forward comes with the norms before and after it, or not at all")
        for post in (mixer_post, ffn_post):
            if post is not None and getattr(post, "fusable_as", None) != "rms":
                raise ValueError("the norm after a sublayer must be an RMS norm (weight, eps)")
        if not hasattr(mixer, "output") or (ffn is not None and not hasattr(ffn, "output")):
            raise ValueError("the sublayers of this arrangement must give their result without the residual sum (output)")
        self.mixer_norm, self.mixer, self.mixer_post = mixer_norm, mixer, mixer_post
        self.ffn_norm, self.ffn, self.ffn_post = ffn_norm, ffn, ffn_post
        self.mult = float(mult)

    def parts(self):
        return [p for p in (self.mixer_norm, self.mixer, self.mixer_post, self.ffn_norm, self.ffn, self.ffn_post) if p is not None]

    def tensor_specs(self):
        return [s for p in self.parts() for s in p.tensor_specs()]

    def bind(self, tensors, dtype):
        for p in self.parts():
            p.bind(tensors, dtype)

    def prepare(self, device, dtype):
        for p in self.parts():
            p.prepare(device, dtype)

    def cache_need(self):
        return self.mixer.cache_need()

    def cache_read(self):
        return self.mixer.cache_read()

    def state_need(self):
        return self.mixer.state_need()

    def kernel_units(self, dtype):
        return [u for p in self.parts() if hasattr(p, "kernel_units") for u in p.kernel_units(dtype)]

    def step_arrays(self):
        return [a for p in self.parts() if hasattr(p, "step_arrays") for a in p.step_arrays()]

    def first_norm(self):
        return self.mixer_norm

    @staticmethod
    def _plain_rms(norm):
        return norm is not None and getattr(norm, "fusable_as", None) == "rms"

    def forward(self, residual, ctx, site):
        # the kernel that adds a sublayer's result also makes the norm that reads the residual stream next, where that
        # is an RMS norm over all rows: this block's second norm, or the following block's first (ctx.next_norm), which
        # finds its rows waiting in ctx.normed
        after = ctx.next_norm
        ctx.next_norm = None          # (no product of this block is left to a later norm)
        h = ctx.take_normed(self.mixer_norm, residual)
        if h is None:
            h = self.mixer_norm.forward(residual, ctx)
            ctx.settle(residual)
        T = residual.shape[0]
        last = self.ffn is None

        def following(norm, tag):
            return (norm, ctx.buffer(tag, (T, residual.shape[1]), ctx.dtype)) if self._plain_rms(norm) else None

        then = following(after if last else self.ffn_norm, "norm.ahead" if last else "norm.inside")
        add_sublayer(residual, self.mixer.output(h, ctx, site), self.mixer_post, self.mult, following=then)
        if last:
            if then is not None:
                ctx.leave_normed(after, residual, then[1])
            return residual
        h = then[1] if then is not None else self.ffn_norm.forward(residual, ctx)
        then = following(after, "norm.ahead")
        add_sublayer(residual, self.ffn.output(h, ctx), self.ffn_post, self.mult, following=then)
        if then is not None:
            ctx.leave_normed(after, residual, then[1])
        return residual


register_part("block", "prenorm", PreNormBlock)
register_part("block", "sandwich", SandwichBlock)
