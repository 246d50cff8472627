"""The plain Ditazen implementation pinned by what fixes it beside its own text (closed forms, brute force, causality),
and the configuration, registry, declared tensors, schedule, rotary tables and random-weights mode of the design in the
framework.  No GPU."""
import json
import math

import numpy as np
import pytest

import plain_ditazen as P
from ditazen_models import CONFIGS, SEEDS, SHARP, FILE_Q_RANK, tensor_shapes, write_folder


def test_delta_rule_writes_what_it_is_asked_to_remember():
    """With beta = 1, g = 1 and orthonormal keys the state returns each value at its key, and a second write at a key
    replaces the first; with g < 1 what was written fades by g a token."""
    D, V = 4, 3
    keys = np.eye(D)
    v = np.arange(1.0, 1.0 + 5 * V).reshape(5, V)
    k = np.stack([keys[0], keys[1], keys[2], keys[0], keys[3]])
    q = np.stack([keys[0], keys[0], keys[1], keys[0], keys[1]])
    out = P.delta_scan(q, k, v, np.ones(5), np.ones(5))
    np.testing.assert_allclose(out, [v[0], v[0], v[1], v[3], v[1]])
    out = P.delta_scan(q, k, v, np.ones(5), np.full(5, 0.5))
    np.testing.assert_allclose(out[1], 0.5 * v[0])
    np.testing.assert_allclose(out[4], 0.125 * v[1])
    half = P.delta_scan(q, k, v, np.full(5, 0.5), np.ones(5))        # a write strength of one half moves half the way
    np.testing.assert_allclose(half[3], 0.5 * v[0] + 0.5 * (v[3] - 0.5 * v[0]))


def test_delta_rule_reads_after_its_own_write():
    rng = np.random.default_rng(0)
    q, k, v = rng.standard_normal((1, 5)), rng.standard_normal((1, 5)), rng.standard_normal((1, 2))
    out = P.delta_scan(q, k, v, np.array([0.7]), np.array([0.3]))
    np.testing.assert_allclose(out[0], (q[0] @ k[0]) * 0.7 * v[0])


def test_causal_conv_sees_zeros_before_the_start_and_the_last_tap_is_the_current_token():
    x = np.arange(1.0, 6.0)[:, None]
    np.testing.assert_allclose(P.causal_conv(x, np.array([[100.0, 10.0, 1.0]]))[:, 0], [1, 12, 123, 234, 345])


def test_norms():
    x = np.array([[1.0, 2.0, 6.0]])
    np.testing.assert_allclose(P.layer_norm(x, np.array([1.0, 2.0, 1.0]), 0.5), (x - 3.0) / math.sqrt(14.0 / 3 + 0.5) * [1, 2, 1])
    np.testing.assert_allclose(P.rms(np.array([[3.0, 4.0]]), 0.5), np.array([[3.0, 4.0]]) / math.sqrt(12.5 + 0.5))
    np.testing.assert_allclose(P.unit(np.array([[3.0, 4.0]])), np.array([[3.0, 4.0]]) / math.sqrt(25.0 + 1e-6))


def test_gelu_forms():
    z = np.array([-3.0, -0.5, 0.0, 0.7, 2.5])
    from scipy.stats import norm
    np.testing.assert_allclose(P.gelu_erf(z), z * norm.cdf(z), rtol=1e-12)        # z times the normal distribution function
    assert np.abs(P.gelu_tanh(z) - P.gelu_erf(z)).max() < 5e-3 and np.abs(P.gelu_tanh(z) - P.gelu_erf(z)).max() > 1e-5


def test_rotation_is_a_complex_turn_and_scores_depend_on_distances():
    rng = np.random.default_rng(1)
    rot = {"base": 100.0, "dims": 6}
    x, y = rng.standard_normal((1, 8)), rng.standard_normal((1, 8))
    for interleaved in (False, True):
        a = P.rotate(x, [5], rot, interleaved)[0]
        pairs = [(2 * i, 2 * i + 1) if interleaved else (i, i + 3) for i in range(3)]
        for i, (u, v) in enumerate(pairs):
            z = complex(x[0, u], x[0, v]) * np.exp(1j * 5 * 100.0 ** (-2 * i / 6))
            np.testing.assert_allclose([a[u], a[v]], [z.real, z.imag])
        np.testing.assert_allclose(a[6:], x[0, 6:])                  # coordinates past rot.dims pass
        near = P.rotate(x, [9], rot, interleaved)[0, :6] @ P.rotate(y, [4], rot, interleaved)[0, :6]
        far = P.rotate(x, [105], rot, interleaved)[0, :6] @ P.rotate(y, [100], rot, interleaved)[0, :6]
        np.testing.assert_allclose(near, far)


def test_scaled_frequencies():
    """Pairs that turn often keep their frequency, pairs that turn less than `slow` times over the original length turn
    `factor` times slower, and cosines and sines grow by 0.1 ln(factor) + 1."""
    rot = {"base": 10000.0, "dims": 32, "scaling": {"factor": 4.0, "original": 512, "fast": 32.0, "slow": 1.0}}
    f, mag = P.rotary_frequencies(rot)
    plain = 10000.0 ** (-2.0 * np.arange(16) / 32)
    turns = 512 * plain / (2 * math.pi)
    assert mag == pytest.approx(0.1 * math.log(4.0) + 1.0)
    np.testing.assert_allclose(f[turns > 40], plain[turns > 40])
    np.testing.assert_allclose(f[turns < 0.8], plain[turns < 0.8] / 4.0)
    between = (turns < 30) & (turns > 1.1)
    assert between.any() and ((f[between] < plain[between]) & (f[between] > plain[between] / 4.0)).all()
    assert (np.diff(f) < 0).all()


def test_window_and_latent_attention_by_hand():
    """One head worked by hand: keys and values from the normed latent, the turning part shared by the heads, the last
    `window` keys, the gate."""
    rng = np.random.default_rng(2)
    W, T, H, D, R, V, r = 10, 9, 2, 3, 4, 5, 6
    m = {"heads": H, "dim": D, "rot_dim": R, "vdim": V, "kv_rank": r, "scale": 0.8, "rot": {"base": 50.0, "dims": 4}, "mask": {"size": 4}}
    w = {"a.q": rng.standard_normal((H * (D + R), W)), "a.dkv": rng.standard_normal((r + R, W)), "a.dkv.norm": rng.uniform(0.5, 1.5, r),
         "a.uk": rng.standard_normal((H * D, r)), "a.uv": rng.standard_normal((H * V, r)), "a.g": rng.standard_normal((H, W)),
         "a.o": np.eye(H * V)}
    h = rng.standard_normal((T, W))
    out = P.latent_attention(h, w, "a", m, 1e-5, False).reshape(T, H, V)
    t, head = 7, 1
    low = h @ w["a.dkv"].T
    c = P.rms(low[:, :r], 1e-5) * w["a.dkv.norm"]
    kr = P.rotate(low[:, r:], np.arange(T), m["rot"], False)
    q = (h[t] @ w["a.q"].T).reshape(H, D + R)[head]
    qr = P.rotate(q[None, D:], [t], m["rot"], False)[0]
    seen = range(t - 3, t + 1)
    s = np.array([0.8 * (q[:D] @ (w["a.uk"][head * D:(head + 1) * D] @ c[j]) + qr @ kr[j]) for j in seen])
    p = np.exp(s - s.max()); p /= p.sum()
    want = sum(pj * (w["a.uv"][head * V:(head + 1) * V] @ c[j]) for pj, j in zip(p, seen)) * P.sigmoid(h[t] @ w["a.g"][head])
    np.testing.assert_allclose(out[t, head], want, rtol=1e-10)
    assert P.visible(6, 2).tolist()[4] == [False, False, False, True, True, False]


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_logits_depend_on_earlier_tokens_only(tmp_path, name):
    cfg, w = P.read_folder(write_folder(tmp_path, CONFIGS[name], SEEDS[name], sharp=name in SHARP))
    tokens = np.random.default_rng(1).integers(0, cfg["vocab"], 40).tolist()
    full = P.forward(cfg, w, tokens)
    np.testing.assert_allclose(P.forward(cfg, w, tokens[:23]), full[:23], rtol=1e-9, atol=1e-9)
    other = list(tokens)
    other[0] = (other[0] + 1) % cfg["vocab"]
    changed = np.abs(P.forward(cfg, w, other) - full).max(axis=-1)
    assert changed[0] > 1e-6 and (changed[1:6] > 1e-9).all()


# -- the design in the framework (no GPU) --------------------------------------------------------------------------------

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_config_is_read_and_the_model_declares_the_designs_tensors(name):
    from runtime.engine.loading import build_from_config_dict
    from runtime.config import DitazenConfig
    raw = CONFIGS[name]
    arch, cfg, model = build_from_config_dict(raw)
    assert isinstance(cfg, DitazenConfig) and arch.name == "Ditazen"
    assert DitazenConfig.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    declared = {s.name: s for s in model.tensor_specs()}
    want = tensor_shapes(raw)
    assert set(declared) == set(want)
    assert all(declared[n].fits(tuple(want[n])) for n in want)
    # a layer that names another's weights is that layer's part at a further place, with a cache or state of its own
    owners = [layer.get("weights_of", i) for i, layer in enumerate(raw["layers"])]
    own = sorted(set(owners))
    assert [entry.layer for entry in model.schedule] == [own.index(o) for o in owners]
    kinds = [layer["type"] for layer in raw["layers"]]
    assert sorted(model.cache_needs()) == [i for i, k in enumerate(kinds) if k != "delta"]
    assert sorted(model.state_needs()) == [i for i, k in enumerate(kinds) if k == "delta"]
    for i, layer in enumerate(raw["layers"]):
        m = layer["mixer"]
        if layer["type"] == "delta":
            channels = 2 * m["kv_heads"] * m["dim"] + m["heads"] * m["vdim"]
            assert model.state_needs()[i].shape == (m["heads"] * m["dim"] * m["vdim"] + (m["conv"] - 1) * channels,)
        else:
            need = model.cache_needs()[i]
            assert (need.kv_heads, need.head_dim) == (1, -(-(m["kv_rank"] + m["rot_dim"]) // 8) * 8)
            assert need.window == (m["mask"]["size"] if layer["type"] == "latent_attention" else None)


def test_config_errors_name_the_place():
    from runtime.config import DitazenConfig, ConfigError
    good = json.loads(json.dumps(CONFIGS["a"]))
    for change, text in [(lambda c: c["layers"][0].update(type="rnn"), "layers[0]"),
                         (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "layers[1].mixer"),
                         (lambda c: c["layers"][1]["mixer"].pop("conv"), "layers[1].mixer"),
                         (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "layers[0].mlp"),
                         (lambda c: c["layers"][0]["mixer"].pop("mask"), "layers[0].mixer"),
                         (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=10), "layers[0].mixer"),
                         (lambda c: c["layers"][2]["mixer"]["rot"]["scaling"].pop("slow"), "layers[2].mixer.rot.scaling"),
                         (lambda c: c["layers"][3].update(weights_of=3), "layers[3]"),
                         (lambda c: c["layers"][4].update(weights_of=3), "layers[4]"),
                         (lambda c: c["layers"][4]["mixer"].update(heads=5), "layers[4]"),
                         (lambda c: c.pop("vocab"), "vocab")]:
        raw = json.loads(json.dumps(good))
        change(raw)
        with pytest.raises(ConfigError, match=text.replace("[", r"\[").replace("]", r"\]")):
            DitazenConfig.from_dict(raw)


def test_a_layer_may_name_a_layer_that_names_the_one_with_the_tensors():
    from runtime.config import DitazenConfig, ConfigError
    from runtime.engine.loading import build_from_config_dict
    raw = json.loads(json.dumps(CONFIGS["a"]))
    raw["layers"].append({**json.loads(json.dumps(raw["layers"][3])), "weights_of": 3})      # layer 3 runs with layer 1's
    cfg = DitazenConfig.from_dict(raw)
    assert [layer.weights_of for layer in cfg.layers] == [None, None, None, 1, 0, 1]
    _, _, model = build_from_config_dict(raw)
    assert [entry.layer for entry in model.schedule] == [0, 1, 2, 1, 0, 1] and sorted(model.state_needs()) == [1, 3, 5]
    raw["layers"][1]["weights_of"] = 5                                                        # a ring has no tensors at all
    with pytest.raises(ConfigError, match=r"layers\[1\]"):
        DitazenConfig.from_dict(raw)


def test_rotary_tables_of_the_framework_follow_the_scaling():
    from runtime.parts import RotaryEmbedding
    rot = {"base": 50000.0, "dims": 16, "scaling": {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}}
    part = RotaryEmbedding(24, rot["base"], 300, rotary_dim=16, pairing="interleaved", scaling=rot["scaling"])
    f, mag = P.rotary_frequencies(rot)
    np.testing.assert_allclose(part.frequencies(), f, rtol=1e-14)
    assert part.magnitude() == pytest.approx(mag) and part.angles().shape == (300, 8)
    assert RotaryEmbedding(24, 100.0, 10).magnitude() == 1.0
    with pytest.raises(ValueError, match="slow"):
        RotaryEmbedding(24, 100.0, 10, scaling={"factor": 2.0, "original": 8, "fast": 4})


def test_a_file_decides_the_size_of_the_query_latent(tmp_path):
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import open_folder, check_against, WeightError
    folder = write_folder(tmp_path / "m", CONFIGS["b"], 1)
    _, _, model = build_from_config_dict(CONFIGS["b"])
    assert check_against(model.tensor_specs(), open_folder(folder)) == []
    from safetensors.torch import load_file, save_file
    tensors = load_file(str(folder / "model.safetensors"))
    assert tensors["l0.mix.dq"].shape[0] == FILE_Q_RANK
    tensors["l0.mix.dkv"] = tensors["l0.mix.dkv"][:-1]
    bad = tmp_path / "bad"
    bad.mkdir()
    (bad / "config.json").write_text(json.dumps(CONFIGS["b"]))
    save_file(tensors, str(bad / "model.safetensors"))
    with pytest.raises(WeightError, match="l0.mix.dkv"):
        check_against(model.tensor_specs(), open_folder(bad))


def test_random_weights_mode_writes_a_folder_the_plain_implementation_reads(tmp_path):
    from runtime.engine import write_random_model
    write_random_model(tmp_path, CONFIGS["b"], seed=5, std=0.1)
    cfg, w = P.read_folder(tmp_path)
    assert cfg["layers"] == CONFIGS["b"]["layers"] and w["l0.mix.dq"].shape[0] == w["l0.mix.uq"].shape[1]
    logits = P.forward(cfg, w, [1, 2, 3, 4])
    assert logits.shape == (4, 77) and np.isfinite(logits).all()


def test_a_named_configuration_of_the_design():
    from runtime.config import preset, DitazenConfig
    cfg = DitazenConfig.from_dict(preset("ditazen-tiny"))
    assert {layer.type for layer in cfg.layers} == {"latent_attention", "latent_attention_2", "delta"}
    assert any(layer.weights_of is not None for layer in cfg.layers)
