"""Plain, slow Novosun forward pass: whole sequences, no cache, float64 NumPy.

One function per mechanism, written from the design's equations; nothing here
is shared with the engine (it reads a model folder with `json` and the
`safetensors` library and never touches a GPU).  Every engine path of the design
is compared with `forward()`.

Notation: x is the residual stream [T, width]; a linear weight W is stored
[out, in] and applied as x W^T; positions count from 0.
"""
import json
from pathlib import Path

import numpy as np


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis (eps inside the root)."""
    x = np.asarray(x, np.float64)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def rmsnorm(x, weight, eps):
    return rms(x, eps) * np.asarray(weight, np.float64)


def linear(x, w):
    return np.asarray(x, np.float64) @ np.asarray(w, np.float64).T


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-np.asarray(z, np.float64)))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def clamped_glu(gate, up, limit):
    """y = g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit)."""
    g = np.minimum(gate, limit)
    u = np.clip(up, -limit, limit)
    return g * sigmoid(1.702 * g) * (u + 1.0)


def feed_forward(h, w, p, mlp):
    return linear(clamped_glu(linear(h, w[p + ".gate"]), linear(h, w[p + ".up"]), mlp["limit"]), w[p + ".down"])


def decayed_outer_scan(q, k, v, decay):
    """S_t = diag(decay_t) S_{t-1} + k_t v_t^T, o_t = S_t^T q_t for one head.
    q, k, decay [T, R]; v [T, C]; the state S [R, C] starts at zero."""
    T, R = k.shape
    S = np.zeros((R, v.shape[1]))
    out = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = decay[t][:, None] * S + np.outer(k[t], v[t])
        out[t] = S.T @ q[t]
    return out


def gla(h, w, p, m, eps):
    """Gated linear attention: a decay per key channel, alpha = sigmoid(z)^(1/tau), z from a low-rank projection."""
    T = h.shape[0]
    H, D, V, tau = m["heads"], m["dim"], m["vdim"], m["tau"]
    q = (linear(h, w[p + ".q"]) * D ** -0.5).reshape(T, H, D)
    k = linear(h, w[p + ".k"]).reshape(T, H, D)
    v = linear(h, w[p + ".v"]).reshape(T, H, V)
    z = linear(linear(h, w[p + ".a1"]), w[p + ".a2"]) + w[p + ".a2.b"]
    alpha = (sigmoid(z) ** (1.0 / tau)).reshape(T, H, D)
    o = np.stack([decayed_outer_scan(q[:, i], k[:, i], v[:, i], alpha[:, i]) for i in range(H)], axis=1)
    o = rmsnorm(o, w[p + ".norm"], eps).reshape(T, H * V)
    return linear(o * silu(linear(h, w[p + ".g"])), w[p + ".o"])


def softmax_attention(h, w, p, m, eps):
    """Grouped-query attention without positions: RMS norm of queries and keys per head, a given score scale,
    a sigmoid gate per head on the output."""
    T = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = rmsnorm(linear(h, w[p + ".q"]).reshape(T, H, D), w[p + ".q.norm"], eps)
    k = rmsnorm(linear(h, w[p + ".k"]).reshape(T, G, D), w[p + ".k.norm"], eps)
    v = linear(h, w[p + ".v"]).reshape(T, G, V)
    gate = sigmoid(linear(h, w[p + ".g"]))                      # [T, H]
    out = np.zeros((T, H, V))
    for i in range(H):
        j = i // (H // G)
        s = (q[:, i] @ k[:, j].T) * m["scale"]
        s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
        s = np.exp(s - s.max(axis=-1, keepdims=True))
        out[:, i] = (s / s.sum(axis=-1, keepdims=True)) @ v[:, j]
    return linear((out * gate[:, :, None]).reshape(T, H * V), w[p + ".o"])


def causal_conv(x, taps, bias):
    """y_t[c] = bias[c] + sum_j taps[c, j] x_{t - (K-1) + j}[c], zeros before the start (the last tap is the current token's)."""
    T, K = x.shape[0], taps.shape[1]
    padded = np.concatenate([np.zeros((K - 1, x.shape[1])), x])
    return bias + sum(padded[j:j + T] * taps[:, j] for j in range(K))


def mamba2(h, w, p, m, eps):
    """State-space duality layer: a scalar decay per head and step, exp(-exp(A_log) dt)."""
    T = h.shape[0]
    H, V, N, G, parts = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = H * V
    zxbcdt = linear(h, w[p + ".in"])
    z, xbc, dt = zxbcdt[:, :inner], zxbcdt[:, inner:2 * inner + 2 * G * N], zxbcdt[:, 2 * inner + 2 * G * N:]
    xbc = silu(causal_conv(xbc, np.asarray(w[p + ".conv"], np.float64), np.asarray(w[p + ".conv.b"], np.float64)))
    x = xbc[:, :inner].reshape(T, H, V)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + w[p + ".dt_bias"])                        # [T, H]
    decay = np.exp(-np.exp(np.asarray(w[p + ".A_log"], np.float64)) * dt)
    y = np.zeros((T, H, V))
    for i in range(H):
        g = i // (H // G)
        y[:, i] = decayed_outer_scan(C[:, g], B[:, g], dt[:, i:i + 1] * x[:, i], np.repeat(decay[:, i:i + 1], N, axis=1))
        y[:, i] += w[p + ".D"][i] * x[:, i]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.reshape(T, parts, inner // parts), eps).reshape(T, inner) * w[p + ".norm"]
    return linear(y, w[p + ".o"])


def parallel(h, w, p, m, eps):
    """Half the sum of the two mixers' outputs, each RMS-normed over the model width first."""
    left = rmsnorm(softmax_attention(h, w, p + ".left", m["left"], eps), w[p + ".left.out"], eps)
    right = rmsnorm(mamba2(h, w, p + ".right", m["right"], eps), w[p + ".right.out"], eps)
    return 0.5 * (left + right)


MIXERS = {"gla": gla, "parallel": parallel}


def forward(cfg, w, tokens, layers_out=None):
    """Logits [T, vocab] of the whole sequence; `layers_out` (a list) receives the residual stream after every layer."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = np.asarray(w["embed"], np.float64)[np.asarray(tokens)]
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        y = MIXERS[layer["type"]](rmsnorm(x, w[p + ".norm1"], eps), w, p + ".mix", layer["mixer"], eps)
        x = x + mult * rmsnorm(y, w[p + ".norm1b"], eps)
        if layer.get("mlp") is not None:
            y = feed_forward(rmsnorm(x, w[p + ".norm2"], eps), w, p + ".mlp", layer["mlp"])
            x = x + mult * rmsnorm(y, w[p + ".norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.copy())
    return linear(rmsnorm(x, w["final.norm"], eps), w["head"])


def read_folder(folder):
    """(config.json as a dict, {name: float64 array}) of a model folder."""
    from safetensors import safe_open
    folder = Path(folder)
    cfg = json.loads((folder / "config.json").read_text())
    weights = {}
    with safe_open(str(folder / "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).double().numpy()
    return cfg, weights


def greedy(cfg, w, prompt, n):
    tokens, out = list(prompt), []
    for _ in range(n):
        out.append(int(np.argmax(forward(cfg, w, tokens)[-1])))
        tokens.append(out[-1])
    return out
