"""Tiny Novosun configurations with weights of the tests' own making, written with the `safetensors` library (not the
engine's writer), and the plain implementation's logits for them.

The configurations differ from each other in every size and constant, and inside each the sizes that could be
confused are unequal (one has no attention at all, so no pages): key and value sizes of a head, head counts of the two mixers of a layer, key/value heads,
groups and norm groups, taps.  One has a width that is no multiple of 8, a single head and a convolution of one
tap (no inputs to carry); one is drawn sharp: scores with a spread of several units, so that a query's result hangs
on one key, often far back, and decays close to one, so that the state remembers the first tokens.
"""
import json
from pathlib import Path

import numpy as np


def gla(heads, dim, vdim, tau, mlp=None):
    return {"type": "gla", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau}, "mlp": mlp}


def parallel(left, right, mlp=None):
    names_l, names_r = ("heads", "kv_heads", "dim", "vdim", "scale"), ("heads", "vdim", "state", "groups", "conv", "norm_groups")
    return {"type": "parallel", "mixer": {"left": dict(zip(names_l, left)), "right": dict(zip(names_r, right))}, "mlp": mlp}


def mlp(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def config(vocab, width, mult, eps, layers):
    return {"architecture": "Novosun", "vocab": vocab, "width": width, "residual_mult": mult, "norm": {"eps": eps}, "layers": layers}


CONFIGS = {
    # both kinds of layer twice, in an order of their own; layers with and without a feed-forward
    "p": config(131, 64, 0.5, 1e-5, [
        gla(3, 16, 24, 8.0, mlp(96, 1.5)),
        parallel((6, 2, 24, 16, 0.2), (4, 8, 12, 1, 4, 4)),
        parallel((2, 2, 16, 40, 0.25), (6, 16, 20, 3, 2, 1), mlp(72, 3.0)),
        gla(2, 40, 8, 4.0)]),
    # a width that is no multiple of 8, one head each, one tap, one group, values larger than keys
    "q": config(77, 100, 1.0, 1e-6, [
        parallel((1, 1, 8, 24, 0.4), (1, 12, 5, 1, 1, 1), mlp(52, 2.5)),
        gla(1, 12, 20, 2.0, mlp(36, 0.75))]),
    # sharp: one key carries a query, decays close to one (the weights' maker reads "sharp")
    "s": config(97, 48, 0.7, 1e-5, [
        parallel((4, 1, 16, 32, 1.0), (2, 24, 16, 2, 3, 2), mlp(64, 2.0)),
        gla(2, 24, 16, 16.0, mlp(64, 2.0)),
        parallel((2, 1, 32, 16, 0.8), (3, 16, 8, 1, 5, 3))]),
    # no layer keeps pages: the cache manager has state slots only
    "g": config(53, 40, 0.6, 1e-5, [gla(2, 8, 12, 6.0, mlp(48, 2.0)), gla(1, 20, 8, 3.0)]),
}
SEEDS = {"p": 11, "q": 12, "s": 13, "g": 14}


def tensor_shapes(c, rank=6):
    H, V = c["width"], c["vocab"]
    shapes = {"embed": (V, H), "head": (V, H), "final.norm": (H,)}
    for i, layer in enumerate(c["layers"]):
        p = f"l{i}."
        shapes[p + "norm1"] = shapes[p + "norm1b"] = (H,)
        m = layer["mixer"]
        if layer["type"] == "gla":
            K, W = m["heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (K, H), p + "mix.k": (K, H), p + "mix.v": (W, H), p + "mix.g": (W, H), p + "mix.o": (H, W),
                           p + "mix.norm": (m["vdim"],), p + "mix.a1": (rank + i, H), p + "mix.a2": (K, rank + i), p + "mix.a2.b": (K,)})
        else:
            a, s = m["left"], m["right"]
            inner, GN = s["heads"] * s["vdim"], s["groups"] * s["state"]
            shapes.update({p + "mix.left.q": (a["heads"] * a["dim"], H), p + "mix.left.k": (a["kv_heads"] * a["dim"], H),
                           p + "mix.left.v": (a["kv_heads"] * a["vdim"], H), p + "mix.left.q.norm": (a["dim"],),
                           p + "mix.left.k.norm": (a["dim"],), p + "mix.left.g": (a["heads"], H),
                           p + "mix.left.o": (H, a["heads"] * a["vdim"]),
                           p + "mix.right.in": (2 * inner + 2 * GN + s["heads"], H), p + "mix.right.conv": (inner + 2 * GN, s["conv"]),
                           p + "mix.right.conv.b": (inner + 2 * GN,), p + "mix.right.dt_bias": (s["heads"],),
                           p + "mix.right.A_log": (s["heads"],), p + "mix.right.D": (s["heads"],),
                           p + "mix.right.norm": (inner,), p + "mix.right.o": (H, inner),
                           p + "mix.left.out": (H,), p + "mix.right.out": (H,)})
        if layer["mlp"] is not None:
            F = layer["mlp"]["ff"]
            shapes.update({p + "norm2": (H,), p + "norm2b": (H,), p + "mlp.gate": (F, H), p + "mlp.up": (F, H), p + "mlp.down": (H, F)})
    return shapes


def make_weights(c, seed, sharp=False):
    """Matrices N(0, 1/in) (so that every projection's output has a spread of about one), norm weights 1 + N(0, 0.1),
    convolution taps N(0, 0.5), step-size biases N(0, 1), A_log U(-2, 0.5), D N(1, 0.3), decay biases N(1, 1).
    `sharp`: decay biases N(5, 1) and A_log U(-5, -3), so that the states forget slowly."""
    import torch
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(c).items()):
        last = name.rsplit(".", 1)[-1]
        if name.endswith("norm") or last in ("norm1", "norm1b", "norm2", "norm2b", "out"):
            w = 1.0 + 0.1 * rng.standard_normal(shape)
        elif name.endswith("conv"):
            w = 0.5 * rng.standard_normal(shape)
        elif name.endswith("conv.b"):
            w = 0.1 * rng.standard_normal(shape)
        elif last == "dt_bias":
            w = rng.standard_normal(shape)
        elif last == "A_log":
            w = rng.uniform(-5.0, -3.0, shape) if sharp else rng.uniform(-2.0, 0.5, shape)
        elif last == "D":
            w = 1.0 + 0.3 * rng.standard_normal(shape)
        elif name.endswith("a2.b"):
            w = (5.0 if sharp else 1.0) + rng.standard_normal(shape)
        elif name == "embed":
            w = rng.standard_normal(shape)
        else:
            w = rng.standard_normal(shape) / np.sqrt(shape[-1])
        out[name] = torch.from_numpy(np.asarray(w, np.float32)).to(torch.bfloat16)
    return out


def write_folder(folder, c, seed, sharp=False):
    from safetensors.torch import save_file
    folder = Path(folder)
    folder.mkdir(parents=True, exist_ok=True)
    (folder / "config.json").write_text(json.dumps(c))
    save_file(make_weights(c, seed, sharp), str(folder / "model.safetensors"))
    return folder


_PLAIN = {}


def plain_logits(folder, tokens):
    """float64 logits [T, V] of the plain implementation, cached per (folder, tokens)."""
    import plain_novosun
    key = (str(folder), tuple(tokens))
    if key not in _PLAIN:
        cfg, w = _PLAIN.setdefault(("folder", str(folder)), plain_novosun.read_folder(folder))
        _PLAIN[key] = plain_novosun.forward(cfg, w, list(tokens))
    return _PLAIN[key]
