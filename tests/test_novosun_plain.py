"""The plain Novosun implementation pinned by what fixes it beside its own text (closed forms, brute force, causality),
and the configuration, registry, declared tensors and random-weights mode of the design in the framework.  No GPU."""
import json

import numpy as np
import pytest

import plain_novosun as P
from novosun_models import CONFIGS, SEEDS, tensor_shapes, write_folder


def test_scan_equals_the_closed_form_sum():
    """o_t = sum_{s<=t} (q_t . (prod_{s<u<=t} a_u) * k_s) v_s"""
    rng = np.random.default_rng(0)
    T, R, C = 9, 5, 3
    q, k, v = rng.standard_normal((T, R)), rng.standard_normal((T, R)), rng.standard_normal((T, C))
    a = rng.uniform(0.3, 1.0, (T, R))
    want = np.zeros((T, C))
    for t in range(T):
        for s in range(t + 1):
            want[t] += ((q[t] * np.prod(a[s + 1:t + 1], axis=0)) @ k[s]) * v[s]
    np.testing.assert_allclose(P.decayed_outer_scan(q, k, v, a), want, rtol=1e-12)


def test_causal_conv_sees_zeros_before_the_start_and_the_last_tap_is_the_current_token():
    x = np.arange(1.0, 6.0)[:, None]                     # one channel: 1 2 3 4 5
    taps = np.array([[100.0, 10.0, 1.0]])
    np.testing.assert_allclose(P.causal_conv(x, taps, np.array([0.5]))[:, 0], [1.5, 12.5, 123.5, 234.5, 345.5])


def test_clamped_gate():
    g, u = np.array([-1.0, 0.5, 9.0, 9.0]), np.array([0.25, -7.0, 7.0, 0.0])
    lim = 2.0
    want = [-1.0 / (1 + np.exp(1.702)) * 1.25, 0.5 / (1 + np.exp(-0.851)) * (-2.0 + 1), 2.0 / (1 + np.exp(-3.404)) * 3.0,
            2.0 / (1 + np.exp(-3.404)) * 1.0]
    np.testing.assert_allclose(P.clamped_glu(g, u, lim), want, rtol=1e-12)


def test_rms_has_eps_inside_the_root():
    x = np.array([[3.0, 4.0]])
    np.testing.assert_allclose(P.rms(x, 0.5), x / np.sqrt(12.5 + 0.5))


@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_logits_depend_on_earlier_tokens_only_and_on_all_of_them(tmp_path, name):
    cfg, w = P.read_folder(write_folder(tmp_path, CONFIGS[name], SEEDS[name], sharp=name == "s"))
    rng = np.random.default_rng(1)
    tokens = rng.integers(0, cfg["vocab"], 40).tolist()
    full = P.forward(cfg, w, tokens)
    np.testing.assert_allclose(P.forward(cfg, w, tokens[:23]), full[:23], rtol=1e-9, atol=1e-9)
    other = list(tokens)
    other[0] = (other[0] + 1) % cfg["vocab"]
    changed = np.abs(P.forward(cfg, w, other) - full).max(axis=-1)
    assert (changed[1:] > 1e-6).all(), "the first token must reach every later position"


def test_attention_head_groups_and_gate(tmp_path):
    """Query head h reads key/value head h // (H / G); a gate of minus infinity silences its head."""
    rng = np.random.default_rng(2)
    H, G, D, V, W, T = 4, 2, 6, 10, 8, 7
    m = {"heads": H, "kv_heads": G, "dim": D, "vdim": V, "scale": 0.7}
    w = {"a.q": rng.standard_normal((H * D, W)), "a.k": rng.standard_normal((G * D, W)), "a.v": rng.standard_normal((G * V, W)),
         "a.q.norm": np.ones(D), "a.k.norm": np.ones(D), "a.g": np.zeros((H, W)), "a.o": np.eye(H * V)}
    h = rng.standard_normal((T, W))
    out = P.softmax_attention(h, w, "a", m, 1e-6).reshape(T, H, V) * 2.0      # gates of zero halve
    q = P.rms((h @ w["a.q"].T).reshape(T, H, D), 1e-6)
    k = P.rms((h @ w["a.k"].T).reshape(T, G, D), 1e-6)
    v = (h @ w["a.v"].T).reshape(T, G, V)
    t, head = 5, 3
    s = np.exp(0.7 * (k[:t + 1, 1] @ q[t, head]))
    np.testing.assert_allclose(out[t, head], (s / s.sum()) @ v[:t + 1, 1], rtol=1e-10)


# -- the design in the framework (no GPU) --------------------------------------------------------------------------------

@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_config_is_read_and_the_model_declares_the_designs_tensors(name):
    from runtime.engine.loading import build_from_config_dict
    from runtime.config import NovosunConfig
    raw = CONFIGS[name]
    arch, cfg, model = build_from_config_dict(raw)
    assert isinstance(cfg, NovosunConfig) and arch.name == "Novosun"
    assert NovosunConfig.from_dict(json.loads(json.dumps(cfg.to_dict()))) == cfg
    declared = {s.name: s for s in model.tensor_specs()}
    want = tensor_shapes(raw)
    assert set(declared) == set(want)
    assert all(declared[n].fits(tuple(want[n])) for n in want)
    kinds = [layer["type"] for layer in raw["layers"]]
    assert sorted(model.cache_needs()) == [i for i, k in enumerate(kinds) if k == "parallel"]
    assert sorted(model.state_needs()) == list(range(len(kinds)))          # every mixer carries a state
    for i, layer in enumerate(raw["layers"]):
        if layer["type"] == "parallel":
            a, s = layer["mixer"]["left"], layer["mixer"]["right"]
            assert model.cache_needs()[i].head_dim == -(-max(a["dim"], a["vdim"]) // 8) * 8
            channels = s["heads"] * s["vdim"] + 2 * s["groups"] * s["state"]
            assert model.state_needs()[i].shape == (s["heads"] * s["state"] * s["vdim"] + (s["conv"] - 1) * channels,)


def test_config_errors_name_the_place():
    from runtime.config import NovosunConfig, ConfigError
    good = json.loads(json.dumps(CONFIGS["p"]))
    for change, text in [(lambda c: c["layers"][0].update(type="rnn"), "layers[0]"),
                         (lambda c: c["layers"][1]["mixer"]["left"].update(kv_heads=4), "layers[1].mixer.left"),
                         (lambda c: c["layers"][1]["mixer"]["right"].pop("conv"), "layers[1].mixer.right"),
                         (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "layers[0].mlp"),
                         (lambda c: c.pop("residual_mult"), "residual_mult"),
                         (lambda c: c["layers"][3]["mixer"].update(tau=0), "layers[3].mixer")]:
        raw = json.loads(json.dumps(good))
        change(raw)
        with pytest.raises(ConfigError, match=text.replace("[", r"\[").replace("]", r"\]")):
            NovosunConfig.from_dict(raw)


def test_a_file_decides_the_rank_of_the_decay_projection_and_both_sides_must_agree(tmp_path):
    from runtime.engine.loading import build_from_config_dict
    from runtime.weights import open_folder, check_against, WeightError
    folder = write_folder(tmp_path / "m", CONFIGS["p"], 1)
    _, _, model = build_from_config_dict(CONFIGS["p"])
    assert check_against(model.tensor_specs(), open_folder(folder)) == []       # ranks 6 and 9: neither is the default
    from safetensors.torch import load_file, save_file
    tensors = load_file(str(folder / "model.safetensors"))
    tensors["l0.mix.q"] = tensors["l0.mix.q"][:-1]
    bad = tmp_path / "bad"
    bad.mkdir()
    (bad / "config.json").write_text(json.dumps(CONFIGS["p"]))
    save_file(tensors, str(bad / "model.safetensors"))
    with pytest.raises(WeightError, match="l0.mix.q"):
        check_against(model.tensor_specs(), open_folder(bad))


def test_random_weights_mode_writes_a_folder_the_plain_implementation_reads(tmp_path):
    from runtime.engine import write_random_model
    write_random_model(tmp_path, CONFIGS["q"], seed=5, std=0.1)
    cfg, w = P.read_folder(tmp_path)
    assert cfg["layers"] == CONFIGS["q"]["layers"] and w["l1.mix.a1"].shape[0] == w["l1.mix.a2"].shape[1]
    logits = P.forward(cfg, w, [1, 2, 3, 4])
    assert logits.shape == (4, 77) and np.isfinite(logits).all()
