"""Plain, slow Ditazen forward pass: whole sequences, no cache, float64 NumPy.

One function per mechanism, written from the design's equations; nothing here is shared with the engine (it reads
a model folder with `json` and the `safetensors` library and never touches a GPU).  Every engine path of the design
is compared with `forward()`.

Notation: x is the residual stream [T, width]; a linear weight W is stored [out, in] and applied as x W^T;
positions count from 0; a mixer's tensors are `<layer>.mix.<name>`.

  layer           x += mixer(ln(x) w1); x += ff(ln(x) w2), ln the centred norm with a weight and no bias
  latent mixers   c = rms(Wdkv h)[:r] wc, kr = rot(Wdkv h [r:]); per head j: K_j = Wuk_j c, V_j = Wuv_j c,
                  score = (qn_j . K_j + rot(qr_j) . kr) scale, softmax over the visible keys, result times
                  sigmoid((Wg h)_j), then Wo.  Queries from Wq h, or through a normed latent Wuq (rms(Wdq h) wq).
  delta mixer     q, k, v through a causal convolution and silu, q and k made unit vectors per head,
                  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q, then rms over each head's result,
                  a weight, silu of a gate projection, Wo.
"""
import json
import math
from pathlib import Path

import numpy as np


def linear(x, w):
    return np.asarray(x, np.float64) @ np.asarray(w, np.float64).T


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_erf(z):
    z = np.asarray(z, np.float64)
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def gelu_tanh(z):
    z = np.asarray(z, np.float64)
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def rms(x, eps):
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * w, var the mean of the squared deviations; no bias."""
    x = np.asarray(x, np.float64)
    d = x - x.mean(axis=-1, keepdims=True)
    return d / np.sqrt(np.mean(d * d, axis=-1, keepdims=True) + eps) * np.asarray(weight, np.float64)


# -- rotary positions -------------------------------------------------------------------------------------------

def rotary_frequencies(rot):
    """(frequencies [dims / 2], factor on cos and sin) of a `rot` entry: base^(-2i/dims), with `scaling` the
    frequencies between the `fast` and `slow` turn counts go over to frequency / factor along a ramp."""
    dims, base = rot["dims"], float(rot["base"])
    f = base ** (-2.0 * np.arange(dims // 2, dtype=np.float64) / dims)
    s = rot.get("scaling")
    if not s:
        return f, 1.0

    def at(turns):
        return dims * math.log(s["original"] / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(at(s["fast"])), 0)
    hi = min(math.ceil(at(s["slow"])), dims - 1)
    ramp = np.clip((np.arange(dims // 2, dtype=np.float64) - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / s["factor"] * ramp + f * (1.0 - ramp), 0.1 * math.log(s["factor"]) + 1.0


def rotate(x, positions, rot, interleaved):
    """x [T, ..., n]: the first rot.dims coordinates turn by position * frequency; pair i is (i, i + dims/2), or
    with `interleaved` (2i, 2i + 1); the rest pass."""
    x = np.array(x, np.float64)
    dims = rot["dims"]
    f, mag = rotary_frequencies(rot)
    a = np.asarray(positions, np.float64)[:, None] * f[None, :]
    shape = (len(positions),) + (1,) * (x.ndim - 2) + (dims // 2,)
    cos, sin = (np.cos(a) * mag).reshape(shape), (np.sin(a) * mag).reshape(shape)
    if interleaved:
        u, v = x[..., 0:dims:2].copy(), x[..., 1:dims:2].copy()
        x[..., 0:dims:2], x[..., 1:dims:2] = u * cos - v * sin, v * cos + u * sin
    else:
        u, v = x[..., :dims // 2].copy(), x[..., dims // 2:dims].copy()
        x[..., :dims // 2], x[..., dims // 2:dims] = u * cos - v * sin, v * cos + u * sin
    return x


# -- latent attention -------------------------------------------------------------------------------------------

def visible(T, window):
    """mask[i, j]: query i sees key j (j <= i, and with a window i - j < window)."""
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    return (j <= i) & ((i - j < window) if window else True)


def latent_attention(h, w, p, m, eps, second):
    """`second` False: queries from one projection, pairs (i, i + dims/2), the last mask.size keys.
    True: queries through a normed latent, pairs (2i, 2i + 1) with scaled frequencies, all keys up to the query's own."""
    T = h.shape[0]
    H, D, R, V, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = np.arange(T)
    if second:
        q = linear(rms(linear(h, w[p + ".dq"]), eps) * np.asarray(w[p + ".dq.norm"], np.float64), w[p + ".uq"])
    else:
        q = linear(h, w[p + ".q"])
    q = q.reshape(T, H, D + R)
    q_plain, q_rot = q[..., :D], rotate(q[..., D:], pos, m["rot"], second)
    dkv = linear(h, w[p + ".dkv"])
    c = rms(dkv[:, :r], eps) * np.asarray(w[p + ".dkv.norm"], np.float64)
    k_rot = rotate(dkv[:, r:], pos, m["rot"], second)                       # [T, R], one for all heads
    k_plain = linear(c, w[p + ".uk"]).reshape(T, H, D)
    v = linear(c, w[p + ".uv"]).reshape(T, H, V)
    window = None if second else m["mask"]["size"]
    see = visible(T, window)
    gate = sigmoid(linear(h, w[p + ".g"]))                                   # [T, H]
    out = np.zeros((T, H, V))
    for j in range(H):
        s = (q_plain[:, j] @ k_plain[:, j].T + q_rot[:, j] @ k_rot.T) * m["scale"]
        s = np.where(see, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, j] = (e / e.sum(axis=1, keepdims=True)) @ v[:, j] * gate[:, j:j + 1]
    return linear(out.reshape(T, H * V), w[p + ".o"])


# -- gated delta rule -------------------------------------------------------------------------------------------

def causal_conv(x, taps):
    """y[t, c] = sum_j taps[c, j] x[t - (n - 1) + j, c]: tap n - 1 weighs x[t], and x is zero before row 0."""
    x, taps = np.asarray(x, np.float64), np.asarray(taps, np.float64)
    n = taps.shape[1]
    padded = np.concatenate([np.zeros((n - 1, x.shape[1])), x])
    return sum(padded[j:j + x.shape[0]] * taps[:, j][None, :] for j in range(n))


def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + 1e-6)


def delta_scan(q, k, v, beta, g):
    """One head.  q, k [T, D]; v [T, V]; beta, g [T].  S [D, V] is zero before the first row."""
    T, V = v.shape
    S = np.zeros((k.shape[1], V))
    out = np.zeros((T, V))
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        out[t] = S.T @ q[t]
    return out


def delta(h, w, p, m, eps):
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(linear(h, w[p + ".q"]), w[p + ".q.conv"])).reshape(T, G, D)
    k = silu(causal_conv(linear(h, w[p + ".k"]), w[p + ".k.conv"])).reshape(T, G, D)
    v = silu(causal_conv(linear(h, w[p + ".v"]), w[p + ".v.conv"])).reshape(T, H, V)
    q, k = unit(q) * D ** -0.5, unit(k)
    beta = sigmoid(linear(h, w[p + ".b"]))
    g = np.exp(-np.exp(np.asarray(w[p + ".A_log"], np.float64)) * softplus(linear(h, w[p + ".a"]) + np.asarray(w[p + ".dt_bias"], np.float64)))
    each = H // G
    o = np.stack([delta_scan(q[:, j // each], k[:, j // each], v[:, j], beta[:, j], g[:, j]) for j in range(H)], axis=1)
    o = rms(o, eps) * np.asarray(w[p + ".norm"], np.float64)
    return linear(o.reshape(T, H * V) * silu(linear(h, w[p + ".g"])), w[p + ".o"])


# -- the model --------------------------------------------------------------------------------------------------

ACTIVATIONS = {"gelu": gelu_erf, "gelu_erf": gelu_erf, "gelu_tanh": gelu_tanh}


def feed_forward(h, w, p, mlp):
    return linear(ACTIVATIONS[mlp.get("act", "gelu")](linear(h, w[p + ".up"])), w[p + ".down"])


def mixer(kind, h, w, p, m, eps):
    if kind == "latent_attention":
        return latent_attention(h, w, p, m, eps, False)
    if kind == "latent_attention_2":
        return latent_attention(h, w, p, m, eps, True)
    if kind == "delta":
        return delta(h, w, p, m, eps)
    raise ValueError(kind)


def forward(config, w, tokens, tap=None):
    """Logits [T, vocab] of one sequence; `tap(i, x)` sees the residual stream after every layer run."""
    eps = config["norm"]["eps"]
    x = np.asarray(w["embed"], np.float64)[np.asarray(tokens)]
    for i, layer in enumerate(config["layers"]):
        p = f"l{layer.get('weights_of', i)}"
        x = x + mixer(layer["type"], layer_norm(x, w[p + ".norm1"], eps), w, p + ".mix", layer["mixer"], eps)
        if layer.get("mlp") is not None:
            x = x + feed_forward(layer_norm(x, w[p + ".norm2"], eps), w, p + ".mlp", layer["mlp"])
        if tap is not None:
            tap(i, x)
    return linear(layer_norm(x, w["final.norm"], eps), w["embed"]) * config["logit_scale"]


def read_folder(folder):
    """(config dict, {name: float64 array}) of a model folder, read with the safetensors library."""
    import torch
    from safetensors.torch import load_file
    folder = Path(folder)
    config = json.loads((folder / "config.json").read_text())
    tensors = {k: v.to(torch.float64).numpy() for k, v in load_file(str(folder / "model.safetensors")).items()}
    return config, tensors


def greedy(config, w, prompt, n_new):
    """The tokens that picking the largest logit generates after `prompt` (the lowest index wins a tie)."""
    tokens, new = list(prompt), []
    for _ in range(n_new):
        new.append(int(np.argmax(forward(config, w, tokens)[-1])))
        tokens.append(new[-1])
    return new
