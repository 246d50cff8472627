"""The Novosun decoder as a list of parts chosen by NovosunConfig, layer by layer: every layer norms before and
after its mixer and its feed-forward and adds the results scaled (the sandwich arrangement); a "gla" layer mixes
with gated linear attention, a "parallel" layer with softmax attention (queries and keys normed per head, no
positions, a gate a head) beside a state-space layer, half the sum of their normed results; feed-forwards are
clamped gated units.  Tensor names: `embed`, `l<i>.norm1|norm1b|norm2|norm2b`, `l<i>.mix.*`, `l<i>.mlp.gate|up|down`,
`final.norm`, `head`.
"""
from ..config.base import register_architecture
from ..config.novosun import NovosunConfig
from ..parts import make_part, TokenEmbedding, LMHead
from .model import Model


def build_novosun(config):
    c = config
    H, eps = c.width, c.norm_eps

    def norm(tensor):
        return make_part("norm", "rmsnorm", name=tensor, dim=H, eps=eps, tensor=tensor)

    layers = []
    for i, spec in enumerate(c.layers):
        p = f"l{i}"
        if spec.type == "gla":
            m = spec.gla
            mixer = make_part("mixer", "gated_linear_attention", name=p + ".mix", hidden=H, heads=m.heads, dim=m.dim,
                              vdim=m.vdim, tau=m.tau, eps=eps)
        else:
            a, s = spec.left, spec.right
            left = make_part("mixer", "normed_gated_attention", name=p + ".mix.left", hidden=H, heads=a.heads,
                             kv_heads=a.kv_heads, dim=a.dim, vdim=a.vdim, scale=a.scale, eps=eps)
            right = make_part("mixer", "state_space_duality", name=p + ".mix.right", hidden=H, heads=s.heads, vdim=s.vdim,
                              state=s.state, groups=s.groups, taps=s.conv, norm_groups=s.norm_groups, eps=eps)
            mixer = make_part("mixer", "side_by_side", name=p + ".mix", hidden=H, first=left, second=right, eps=eps)
        ffn = {}
        if spec.mlp is not None:
            ffn = dict(ffn_norm=norm(p + ".norm2"), ffn_post=norm(p + ".norm2b"),
                       ffn=make_part("ffn", "clamped_glu", name=p + ".mlp", hidden=H, intermediate=spec.mlp.ff, limit=spec.mlp.limit))
        layers.append(make_part("block", "sandwich", mixer_norm=norm(p + ".norm1"), mixer=mixer, mixer_post=norm(p + ".norm1b"),
                                mult=c.residual_mult, **ffn))
    embedding = TokenEmbedding("embed", c.vocab, H, tensor="embed")
    head = LMHead("head", c.vocab, H, tensor="head")
    return Model(c, embedding, layers, norm("final.norm"), head, max_positions=c.max_positions, vocab_size=c.vocab)


register_architecture(["Novosun", "novosun"], NovosunConfig, build_novosun)
