"""Tiny Ditazen configurations with weights of the tests' own making, written with the `safetensors` library (not the
engine's writer), and the plain implementation's logits for them.

The configurations differ from each other in every size and constant, and inside each the sizes that could be
confused are unequal: plain and turning coordinates of a query, the latent's size and the heads' sizes, key and value
sizes of the delta rule, its two head counts.  One has a width that is no multiple of 8, one head everywhere, a
convolution of one tap (no inputs to carry), a window of one token, fewer turning pairs than the coordinates kept for
them, and leaves the size of the query latent to the file; one is drawn sharp: scores with a spread of several
units, so that a query's result hangs on one key, often the one at the window's edge, and decays close to one, so
that the state remembers the first tokens.
"""
import json
from pathlib import Path

import numpy as np


def rot(base, dims, scaling=None):
    out = {"base": base, "dims": dims}
    if scaling:
        out["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return out


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, rotary, window, mlp=None, **more):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rotary,
             "mask": {"size": window}}
    return {"type": "latent_attention", "mixer": mixer, "mlp": mlp, **more}


def latent2(heads, dim, rot_dim, vdim, kv_rank, q_rank, scale, rotary, mlp=None, **more):
    mixer = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rotary}
    if q_rank is not None:
        mixer["q_rank"] = q_rank
    return {"type": "latent_attention_2", "mixer": mixer, "mlp": mlp, **more}


def delta(heads, kv_heads, dim, vdim, conv, mlp=None, **more):
    return {"type": "delta", "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv}, "mlp": mlp, **more}


def mlp(ff, act=None):
    return {"kind": "dense", "ff": ff, **({"act": act} if act else {})}


def again(layer, owner):
    return {**json.loads(json.dumps(layer)), "weights_of": owner}


def config(vocab, width, logit_scale, eps, layers):
    return {"architecture": "Ditazen", "vocab": vocab, "width": width, "logit_scale": logit_scale, "norm": {"eps": eps}, "layers": layers}


_A = [latent(3, 16, 8, 24, 40, 0.2, rot(10000.0, 8), 21, mlp(96)),
      delta(4, 2, 16, 24, 3, mlp(80)),
      latent2(2, 24, 16, 8, 48, 40, 0.15, rot(50000.0, 16, (8.0, 64, 16.0, 2.0)))]
_S = [latent(4, 8, 16, 16, 24, 0.35, rot(1000.0, 16), 19, mlp(64)),
      delta(2, 2, 24, 16, 4),
      latent2(2, 16, 8, 24, 32, 16, 0.4, rot(20000.0, 8, (4.0, 32, 8.0, 1.0)), mlp(48))]
_F = latent2(3, 16, 8, 16, 24, 32, 0.45, rot(8000.0, 8, (4.0, 128, 16.0, 1.0)), mlp(56))
CONFIGS = {
    # every kind of layer, then two of them once more with the first ones' weights; a layer without a feed-forward
    "a": config(131, 64, 0.3, 1e-5, _A + [again(_A[1], 1), again(_A[0], 0)]),
    # a width that is no multiple of 8, one head each, one tap, a window of one token, 4 of 6 coordinates turn, the
    # query latent's size left to the file, the tanh form of the activation
    "b": config(77, 100, 1.7, 1e-6, [
        latent2(1, 10, 6, 12, 20, None, 0.4, rot(300.0, 4, (2.0, 16, 4.0, 1.0)), mlp(52, "gelu_tanh")),
        delta(1, 1, 12, 20, 1, mlp(36)),
        latent(1, 12, 6, 8, 18, 0.5, rot(100.0, 6), 1)]),
    # sharp: one key carries a query, decays close to one (the weights' maker reads "sharp"); the window and the full
    # layer run twice
    "s": config(97, 48, 0.6, 1e-5, _S + [again(_S[0], 0), again(_S[2], 2)]),
    # twenty heads over the one key head (more than the sixteen a wave's tile of the matrix-core kernels holds), and a
    # latent too large for those kernels (it runs the row-wise kernel); a state of 256 rows
    "w": config(61, 56, 0.8, 1e-5, [
        latent(20, 8, 8, 8, 16, 0.3, rot(500.0, 8), 33, mlp(40)),
        latent2(3, 8, 8, 16, 296, 16, 0.06, rot(3000.0, 8, (2.0, 64, 8.0, 2.0))),
        delta(2, 1, 256, 8, 2)]),
    # only attention over all keys (no window, no state): what the last rows know of the first ones they know through
    # far keys alone; drawn sharp
    "f": config(89, 40, 0.9, 1e-5, [_F, again(_F, 0)]),
    # no layer keeps pages: the cache manager has state slots only
    "d": config(53, 40, 1.0, 1e-5, [delta(4, 1, 8, 12, 2, mlp(48)), delta(3, 3, 20, 8, 5)]),
}
SEEDS = {"a": 21, "b": 22, "s": 23, "d": 24, "w": 25, "f": 26}
SHARP = ("s", "f")
FILE_Q_RANK = 28       # the query latent of configuration "b", which config.json does not give


def tensor_shapes(c):
    H, V = c["width"], c["vocab"]
    shapes = {"embed": (V, H), "final.norm": (H,)}
    for i, layer in enumerate(c["layers"]):
        if "weights_of" in layer:
            continue
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = (H,)
        if layer["type"] == "delta":
            K, W = m["kv_heads"] * m["dim"], m["heads"] * m["vdim"]
            shapes.update({p + "mix.q": (K, H), p + "mix.k": (K, H), p + "mix.v": (W, H), p + "mix.q.conv": (K, m["conv"]),
                           p + "mix.k.conv": (K, m["conv"]), p + "mix.v.conv": (W, m["conv"]), p + "mix.b": (m["heads"], H),
                           p + "mix.a": (m["heads"], H), p + "mix.A_log": (m["heads"],), p + "mix.dt_bias": (m["heads"],),
                           p + "mix.norm": (m["vdim"],), p + "mix.g": (W, H), p + "mix.o": (H, W)})
        else:
            nh, D, R, Vd, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            if layer["type"] == "latent_attention_2":
                q_rank = m.get("q_rank", FILE_Q_RANK)
                shapes.update({p + "mix.dq": (q_rank, H), p + "mix.dq.norm": (q_rank,), p + "mix.uq": (nh * (D + R), q_rank)})
            else:
                shapes[p + "mix.q"] = (nh * (D + R), H)
            shapes.update({p + "mix.dkv": (r + R, H), p + "mix.dkv.norm": (r,), p + "mix.uk": (nh * D, r), p + "mix.uv": (nh * Vd, r),
                           p + "mix.g": (nh, H), p + "mix.o": (H, nh * Vd)})
        if layer["mlp"] is not None:
            F = layer["mlp"]["ff"]
            shapes.update({p + "norm2": (H,), p + "mlp.up": (F, H), p + "mlp.down": (H, F)})
    return shapes


def make_weights(c, seed, sharp=False):
    """Matrices N(0, 1/in) (so that every projection's output has a spread of about one), norm weights 1 + N(0, 0.1),
    convolution taps N(0, 0.5), step-size biases N(0, 1), A_log U(-2, 0.5).  `sharp`: the query projections times 2
    (scores spread over several units), A_log U(-7, -5) (states that forget slowly)."""
    import torch
    rng = np.random.default_rng(seed)
    out = {}
    for name, shape in sorted(tensor_shapes(c).items()):
        last = name.rsplit(".", 1)[-1]
        if last in ("norm", "norm1", "norm2"):
            w = 1.0 + 0.1 * rng.standard_normal(shape)
        elif last == "conv":
            w = 0.5 * rng.standard_normal(shape)
        elif last == "dt_bias":
            w = rng.standard_normal(shape)
        elif last == "A_log":
            w = rng.uniform(-7.0, -5.0, shape) if sharp else rng.uniform(-2.0, 0.5, shape)
        elif name == "embed":
            w = rng.standard_normal(shape)
        else:
            w = rng.standard_normal(shape) / np.sqrt(shape[-1])
            if sharp and last in ("uq", "q") and ".mix." in name and not name.endswith("conv"):
                w = w * 2.0
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
    import plain_ditazen
    key = (str(folder), tuple(tokens))
    if key not in _PLAIN:
        cfg, w = _PLAIN.setdefault(("folder", str(folder)), plain_ditazen.read_folder(folder))
        _PLAIN[key] = plain_ditazen.forward(cfg, w, list(tokens))
    return _PLAIN[key]
