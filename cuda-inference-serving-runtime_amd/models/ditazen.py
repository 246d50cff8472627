"""The Ditazen decoder as a list of parts chosen by DitazenConfig, layer by layer: pre-norm layers with centred norms
(a weight, no bias), whose mixer is latent attention (two kinds: queries from one projection, split-half rotary pairs and
a sliding window; or queries through a normed latent, neighbouring pairs with scaled frequencies, and all keys
up to its own) or the gated delta rule, and whose feed-forward, if any, is one matrix up, gelu, one matrix down.  The logits are
the embedding table times the normed last rows, times `logit_scale` (which the last norm's weight carries).  A layer
that names another's weights is the same part run at a further place of the schedule, with a cache or state of its own.
Tensor names: `embed`, `l<i>.norm1|norm2`, `l<i>.mix.*`, `l<i>.mlp.up|down`, `final.norm`.
"""
from ..config.base import register_architecture
from ..config.ditazen import DitazenConfig
from ..parts import make_part, TokenEmbedding, LMHead
from .model import Model, ScheduleEntry


def build_ditazen(config):
    c = config
    H, eps = c.width, c.norm_eps

    def norm(tensor, gain=1.0):
        return make_part("norm", "layernorm", name=tensor, dim=H, eps=eps, tensor=tensor, gain=gain)

    positions = {}

    def position(m, interleaved):
        # one part (one pair of tables) for all layers that turn alike
        key = (m.rot_dim, m.rot, interleaved)
        if key not in positions:
            scaling = None if m.rot.scaling is None else dict(zip(("factor", "original", "fast", "slow"), m.rot.scaling))
            positions[key] = make_part("position", "rotary", head_dim=m.rot_dim, theta=m.rot.base, max_positions=c.max_positions,
                                       rotary_dim=m.rot.dims, pairing="interleaved" if interleaved else "split_half", scaling=scaling)
        return positions[key]

    layers, place = [], {}
    for i, spec in enumerate(c.layers):
        if spec.weights_of is not None:
            continue
        p = f"l{i}"
        if spec.type == "delta":
            m = spec.delta
            mixer = make_part("mixer", "gated_delta_rule", name=p + ".mix", hidden=H, heads=m.heads, kv_heads=m.kv_heads, dim=m.dim,
                              vdim=m.vdim, taps=m.conv, eps=eps)
        else:
            m, second = spec.latent, spec.type == "latent_attention_2"
            q_rank = None
            if second:
                from ..weights.loader import AnySize
                q_rank = m.q_rank if m.q_rank is not None else AnySize(max(8, H // 2))
            mixer = make_part("mixer", "latent_attention", name=p + ".mix", hidden=H, heads=m.heads, dim=m.dim, rot_dim=m.rot_dim,
                              vdim=m.vdim, kv_rank=m.kv_rank, scale=m.scale, eps=eps, position=position(m, second),
                              q_rank=q_rank, window=m.window)
        ffn = {}
        if spec.mlp is not None:
            ffn = dict(ffn_norm=norm(p + ".norm2"),
                       ffn=make_part("ffn", "dense_mlp", name=p + ".mlp", hidden=H, intermediate=spec.mlp.ff, activation=spec.mlp.act))
        place[i] = len(layers)
        layers.append(make_part("block", "prenorm", mixer_norm=norm(p + ".norm1"), mixer=mixer, **ffn))
    schedule = [ScheduleEntry(place[i if spec.weights_of is None else spec.weights_of]) for i, spec in enumerate(c.layers)]
    embedding = TokenEmbedding("embed", c.vocab, H, tensor="embed")
    head = LMHead("head", c.vocab, H, tied_to=embedding)
    return Model(c, embedding, layers, norm("final.norm", gain=c.logit_scale), head, schedule=schedule,
                 max_positions=c.max_positions, vocab_size=c.vocab)


register_architecture(["Ditazen", "ditazen"], DitazenConfig, build_ditazen)
