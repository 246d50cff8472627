"""The Novosun design in the engine against the plain implementation (tests/plain_novosun.py): every mechanism's
kernels alone, then whole models of the tests' own sizes: prompts, token-by-token decoding, portions down to two
tokens, mixed batches with pages and state slots used again, keys far back and at page borders in a model drawn
sharp, the first tokens, long decoding, captured programs, and greedy generation through the scheduler."""
import numpy as np
import pytest
import torch

import plain_novosun as P
from conftest import assert_close, random_tokens
from novosun_models import CONFIGS, SEEDS, plain_logits, write_folder
from trace_tools import Trace

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DTYPES = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    base = tmp_path_factory.mktemp("novosun")
    return {name: write_folder(base / name, CONFIGS[name], SEEDS[name], sharp=name == "s") for name in CONFIGS}


def dev(a, dtype=torch.float32):
    return torch.from_numpy(np.ascontiguousarray(a)).to(dtype).to(DEV)


def ints(a):
    return torch.tensor(list(a), dtype=torch.int32, device=DEV)


def close(got, want, tol=2e-5):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape
    err = np.abs(got - want).max() / max(np.abs(want).max(), 1e-30)
    assert err < tol, f"differs by {err:.3e}"


# -- mechanisms alone -----------------------------------------------------------------------------------------------------

@pytest.mark.parametrize("heads, share, R, C, vector, columns", [
    (3, 1, 16, 24, True, None), (2, 1, 40, 8, True, 4), (6, 3, 20, 16, False, 8), (4, 4, 12, 8, False, 16),
    (1, 1, 5, 12, False, None), (2, 2, 130, 70, True, 16), (5, 1, 1, 3, True, None)])
def test_linear_scan_over_segments_with_states_carried_and_slots_used_again(heads, share, R, C, vector, columns):
    """Three segments of unequal length in one launch, then their continuations (one of them a single token) in another
    order and on slots that other requests held before; a decay per state row or per head, q and k shared by groups."""
    from runtime.kernels import ops
    rng = np.random.default_rng(R * 100 + C)
    lengths = {"a": 19, "b": 1, "c": 37}
    groups = heads // share
    data = {}
    for key, n in lengths.items():
        n2 = n + 6
        data[key] = dict(q=rng.standard_normal((n2, groups, R)), k=rng.standard_normal((n2, groups, R)), v=rng.standard_normal((n2, heads, C)),
                         a=rng.uniform(0.5, 1.0, (n2, heads, R if vector else 1)), s=rng.uniform(0.1, 2.0, (n2, heads)))
    want = {}
    for key, d in data.items():
        want[key] = np.stack([P.decayed_outer_scan(d["q"][:, h // share], d["k"][:, h // share], d["v"][:, h] * d["s"][:, h:h + 1],
                                                   np.broadcast_to(d["a"][:, h], (len(d["q"]), R))) for h in range(heads)], axis=1) * 0.37
    state = torch.full((4, heads * R * C + 5), 7.0, device=DEV)          # slots hold rubbish until a request takes them

    def launch(order, slots, spans):
        rows = {name: np.concatenate([data[k][name][lo:hi].reshape(hi - lo, -1) for k, (lo, hi) in zip(order, spans)]) for name in "qkvas"}
        starts = np.concatenate(([0], np.cumsum([hi - lo for lo, hi in spans])))
        out = torch.zeros(rows["v"].shape, device=DEV)
        ops.linear_scan(dev(rows["q"]), dev(rows["k"]), dev(rows["v"]), dev(rows["a"]), out, state, ints(starts), ints(slots), heads, R, C,
                        share=share, step=dev(rows["s"]), q_scale=0.37, columns=columns)
        return np.split(out.cpu().numpy().reshape(-1, heads, C), starts[1:-1])

    for slot in (0, 2, 3):
        state[slot, :heads * R * C].zero_()
    first = launch("abc", [2, 0, 3], [(0, lengths[k]) for k in "abc"])
    for key, got in zip("abc", first):
        close(got, want[key][:lengths[key]])
    # continuations: c goes on with one token, a with six, b moves nowhere; a fourth request takes slot 1 from zero
    second = launch("ca", [3, 2], [(37, 38), (19, 25)])
    close(second[0], want["c"][37:38])
    close(second[1], want["a"][19:25])
    assert float(state[1, 0]) == 7.0 and float(state[0, -1]) == 7.0, "a slot or a tail that no segment named was written"


@pytest.mark.parametrize("heads, share, R, C, vector, piece", [(2, 1, 24, 20, True, 64), (4, 2, 16, 8, False, 64), (1, 1, 130, 33, True, 128)])
def test_linear_scan_in_pieces_side_by_side_equals_the_scan_in_order(heads, share, R, C, vector, piece):
    """Long segments are cut into pieces that waves of their own walk (end states from zero, the states at the pieces'
    starts in order, then the results): segments of several pieces, of exactly one and two pieces, of one row and of
    one row more than a piece, starting from states that an earlier launch left, beside each other in one launch."""
    from runtime.kernels import ops
    rng = np.random.default_rng(R + C)
    lengths = {"a": 4 * piece + 37, "b": 1, "c": 2 * piece, "d": piece + 1, "e": piece}
    groups = heads // share
    data, want = {}, {}
    for key, n in lengths.items():
        n2 = n + 12
        d = data[key] = dict(q=rng.standard_normal((n2, groups, R)), k=rng.standard_normal((n2, groups, R)), v=rng.standard_normal((n2, heads, C)),
                             a=rng.uniform(0.8, 1.0, (n2, heads, R if vector else 1)))
        want[key] = np.stack([P.decayed_outer_scan(d["q"][:, h // share], d["k"][:, h // share], d["v"][:, h],
                                                   np.broadcast_to(d["a"][:, h], (n2, R))) for h in range(heads)], axis=1)
    state = torch.zeros((5, heads * R * C), device=DEV)
    slots = {"a": 3, "b": 0, "c": 4, "d": 1, "e": 2}

    def launch(spans, piece):
        keys = list(spans)
        rows = {name: np.concatenate([data[k][name][lo:hi].reshape(hi - lo, -1) for k, (lo, hi) in spans.items()]) for name in "qkva"}
        starts = np.concatenate(([0], np.cumsum([hi - lo for lo, hi in spans.values()])))
        T = len(rows["v"])
        out = torch.zeros(rows["v"].shape, device=DEV)
        carry = None
        if piece:
            n, n_decay = ops.scan_carry(T, piece, heads, R, C, vector)
            carry = (torch.full((n,), 5.0, device=DEV), torch.full((n_decay,), 5.0, device=DEV))
        ops.linear_scan(dev(rows["q"]), dev(rows["k"]), dev(rows["v"]), dev(rows["a"]), out, state, ints(starts), ints([slots[k] for k in keys]),
                        heads, R, C, share=share, piece=piece, carry=carry)
        return dict(zip(keys, np.split(out.cpu().numpy().reshape(-1, heads, C), starts[1:-1])))

    first = launch({"a": (0, 9), "c": (0, 3), "e": (0, 2)}, 0)                       # some start from a state that is not zero
    got = launch({k: ({"a": 9, "c": 3, "e": 2}.get(k, 0), n + {"a": 9, "c": 3, "e": 2}.get(k, 0)) for k, n in lengths.items()}, piece)
    for k, n in lengths.items():
        lo = {"a": 9, "c": 3, "e": 2}.get(k, 0)
        close(got[k], want[k][lo:lo + n], 5e-5)
    after = launch({k: (n + {"a": 9, "c": 3, "e": 2}.get(k, 0), n + {"a": 9, "c": 3, "e": 2}.get(k, 0) + 1) for k, n in lengths.items() if k != "b"}, 0)
    for k in after:                                                                      # the states the pieces left
        at = lengths[k] + {"a": 9, "c": 3, "e": 2}.get(k, 0)
        close(after[k], want[k][at:at + 1], 5e-5)


@pytest.mark.parametrize("channels, taps, heads", [(10, 4, 3), (7, 2, 1), (300, 3, 2), (5, 1, 2), (6, 16, 0)])
def test_short_convolution_carries_its_last_inputs_across_portions_of_any_size(channels, taps, heads):
    from runtime.kernels import ops
    rng = np.random.default_rng(channels)
    n = {"a": 23, "b": 10}
    width = 4 + channels + heads
    x = {k: rng.standard_normal((v, width)) for k, v in n.items()}
    w, b = rng.standard_normal((channels, taps)), rng.standard_normal(channels)
    dt_bias, a_log = rng.standard_normal(max(heads, 1)), rng.uniform(-2, 0.5, max(heads, 1))
    want = {k: P.silu(P.causal_conv(x[k][:, 4:4 + channels], w, b)) for k in n}
    state = torch.full((3, 11 + (taps - 1) * channels), 3.0, device=DEV)
    conv_state = state[:, 11:]
    state[0, 11:].zero_()
    state[2, 11:].zero_()
    fed = {"a": 0, "b": 0}
    got = {"a": [], "b": []}
    for portion in [{"a": 1, "b": 2}, {"a": 2}, {"b": 1, "a": 1}, {"a": 7, "b": 6}, {"a": 1}, {"a": 1, "b": 1}, {"a": 10}]:       # shorter than the taps, and longer
        keys = list(portion)
        single = all(count == 1 for count in portion.values())        # steps of single tokens move the state on in the same launch
        rows = np.concatenate([x[k][fed[k]:fed[k] + portion[k]] for k in keys])
        starts = np.concatenate(([0], np.cumsum([portion[k] for k in keys])))
        seg_of_row = np.repeat(np.arange(len(keys)), [portion[k] for k in keys])
        full = dev(rows)
        out = torch.zeros((len(rows), channels), device=DEV)
        gates = None
        if heads:
            step, decay = torch.zeros((len(rows), heads), device=DEV), torch.zeros((len(rows), heads), device=DEV)
            gates = (full[:, 4 + channels:], dev(dt_bias), dev(a_log), step, decay)
        ops.conv_silu(full[:, 4:4 + channels], dev(w), dev(b), conv_state, out, ints(seg_of_row), ints(starts),
                      ints([{"a": 2, "b": 0}[k] for k in keys]), gates=gates, single_rows=single)
        if heads:
            dt = P.softplus(rows[:, 4 + channels:] + dt_bias)
            close(step.cpu().numpy(), dt)
            close(decay.cpu().numpy(), np.exp(-np.exp(a_log) * dt))
        for k, piece in zip(keys, np.split(out.cpu().numpy(), starts[1:-1])):
            got[k].append(piece)
            fed[k] += portion[k]
    for k in n:
        close(np.concatenate(got[k]), want[k][:fed[k]])
    assert float(state[1, -1]) == 3.0 and float(state[0, 0]) == 3.0


def test_decay_gate_group_norm_gate_post_norm_and_clamped_gate():
    from runtime.kernels import ops
    rng = np.random.default_rng(3)
    T = 5
    z, bias = rng.standard_normal((T, 13 + 4)) * 4, rng.standard_normal(13)
    full = dev(z)
    out = torch.zeros((T, 13), device=DEV)
    ops.decay_gate(full[:, 4:], dev(bias), out, 7.0)
    close(out.cpu().numpy(), P.sigmoid(z[:, 4:] + bias) ** (1 / 7.0))
    up = rng.standard_normal((9, 13))                     # the same with the second half of a low-rank projection on the way
    out = torch.zeros((T, 9), device=DEV)
    ops.decay_gate_low_rank(full[:, 4:], dev(up.T), dev(bias[:9]), out, 3.0)
    close(out.cpu().numpy(), P.sigmoid(z[:, 4:] @ up.T + bias[:9]) ** (1 / 3.0))
    # the norm of a mixer's result: gate after the norm with a weight shared by the heads; gate before it with a skip term
    heads, V = 3, 10
    y, g, w = rng.standard_normal((T, heads * V)), rng.standard_normal((T, heads * V)), rng.standard_normal(V)
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 8e-3)):
        out = torch.zeros((T, heads * V), device=DEV, dtype=dtype)
        ops.group_norm_gate(dev(y), dev(g), dev(w), out, heads, 1e-3, gate_first=False, shared_weight=True)
        close(out.float().cpu().numpy(), (P.rmsnorm(y.reshape(T, heads, V), w, 1e-3).reshape(T, -1)) * P.silu(g), tol)
        w2, d, x = rng.standard_normal(heads * V), rng.standard_normal(6), rng.standard_normal((T, heads * V))
        ops.group_norm_gate(dev(y), dev(g), dev(w2), out, 2, 1e-3, gate_first=True, skip=(dev(d), dev(x)))
        u = (y + np.repeat(d, 5) * x) * P.silu(g)
        close(out.float().cpu().numpy(), P.rms(u.reshape(T, 2, 15), 1e-3).reshape(T, -1) * w2, tol)
    # a sublayer's result into the residual stream, alone and as the mean of two normed results, with the norm that reads
    # the stream next made on the way: rows in registers (up to 4,096 floats), waiting in LDS (up to 16,384), read again
    for H in (300, 2048, 5000, 17000):
        x0, a, b = rng.standard_normal((T, H)), rng.standard_normal((T, H)), 3 * rng.standard_normal((T, H))
        wa, wb, wn = (1 + 0.1 * rng.standard_normal(H) for _ in range(3))
        x = dev(x0)
        ops.post_norm_add(x, dev(a), dev(wn), 1e-2, 0.3)
        close(x.cpu().numpy(), x0 + 0.3 * P.rmsnorm(a, wn, 1e-2))
        x = dev(x0)
        ahead = torch.zeros((T, H), device=DEV)
        ops.post_norm_add(x, dev(a), dev(wn), 1e-2, 0.6, second=(dev(b), dev(wa), dev(wb)), following=(dev(wb), 1e-4, ahead))
        mean = 0.5 * (P.rmsnorm(a, wa, 1e-2) + P.rmsnorm(b, wb, 1e-2))
        close(x.cpu().numpy(), x0 + 0.6 * P.rmsnorm(mean, wn, 1e-2))
        close(ahead.cpu().numpy(), P.rmsnorm(x0 + 0.6 * P.rmsnorm(mean, wn, 1e-2), wb, 1e-4))
        x = dev(x0)
        ops.post_norm_add(x, dev(a), None, 0.0, 1.0, second=(dev(b), dev(wa), dev(wb)))
        close(x.cpu().numpy(), x0 + 0.5 * (P.rmsnorm(a, wa, 0.0) + P.rmsnorm(b, wb, 0.0)))
        x = dev(x0)
        ahead = torch.zeros((T, H), device=DEV, dtype=torch.bfloat16)
        ops.post_norm_add(x, dev(a), dev(wn), 1e-2, 0.3, following=(dev(wa), 1e-3, ahead))
        close(x.cpu().numpy(), x0 + 0.3 * P.rmsnorm(a, wn, 1e-2))
        close(ahead.float().cpu().numpy(), P.rmsnorm(x0 + 0.3 * P.rmsnorm(a, wn, 1e-2), wa, 1e-3), 8e-3)
    for inter in (21, 24):                                 # (rows of a multiple of eight: 16-byte accesses)
        gu = rng.standard_normal((T, 2 * inter)) * 3
        for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 8e-3)):
            operand = dev(gu, dtype)
            out = ops.glu_clamped(operand, torch.zeros((T, inter), device=DEV, dtype=dtype), 1.25)
            ref = operand.float().cpu().numpy()
            close(out.float().cpu().numpy(), P.clamped_glu(ref[:, :inter], ref[:, inter:], 1.25), tol)
@pytest.mark.parametrize("rows", [1, 8, 24, 64])
def test_a_cut_product_is_left_to_the_sum_that_reads_it(rows):
    """Against large weights the wide kernel cuts a product along its inner size; the kernel that adds a sublayer's
    result to the residual stream takes the slices' partial sums instead of a finished product (alone, and as both
    halves of a mean of two results)."""
    from runtime.kernels import ops
    rng = np.random.default_rng(rows)
    K, N = 8192, 2048
    a1, a2 = (dev(rng.standard_normal((rows, K)), torch.bfloat16) for _ in range(2))
    w1, w2 = (dev(rng.standard_normal((N, K)) / np.sqrt(K), torch.bfloat16) for _ in range(2))
    made = []

    def product(a, w):
        kept = {}
        got = ops.gemm_for_norm(a, w, torch.zeros((rows, N), device=DEV), lambda n: kept.setdefault("parts", torch.zeros(n, device=DEV)))
        made.append(isinstance(got, ops.Partials))
        return got

    y1, y2 = product(a1, w1), product(a2, w2)
    if rows > 4:
        assert all(made) and y1.slices >= 2, "this shape was meant to be cut"
    r1, r2 = (a.float() @ w.float().T for a, w in ((a1, w1), (a2, w2)))
    x0 = rng.standard_normal((rows, N))
    wn, wa, wb = (1 + 0.1 * rng.standard_normal(N) for _ in range(3))
    x = dev(x0)
    ahead = torch.zeros((rows, N), device=DEV)
    ops.post_norm_add(x, y1, dev(wn), 1e-5, 0.3, following=(dev(wa), 1e-5, ahead))
    want = x0 + 0.3 * P.rmsnorm(r1.cpu().numpy(), wn, 1e-5)
    close(x.cpu().numpy(), want, 1e-4)
    close(ahead.cpu().numpy(), P.rmsnorm(want, wa, 1e-5), 1e-4)
    x = dev(x0)
    ops.post_norm_add(x, y1, dev(wn), 1e-5, 0.5, second=(y2, dev(wa), dev(wb)))
    mean = 0.5 * (P.rmsnorm(r1.cpu().numpy(), wa, 1e-5) + P.rmsnorm(r2.cpu().numpy(), wb, 1e-5))
    close(x.cpu().numpy(), x0 + 0.5 * P.rmsnorm(mean, wn, 1e-5), 1e-4)


@pytest.mark.parametrize("rows", [1, 3, 16, 40, 100])
@pytest.mark.parametrize("inner, width", [(64, 48), (1024, 4096)])
def test_clamped_gate_as_the_epilogue_of_the_product_over_gate_and_up(rows, inner, width):
    """Every kernel that takes the product over [gate; up] (matrix-vector, narrow, skinny, wide, tiled) with the clamped
    law, against the float product of the same operands (gate and up rounded to bfloat16 before the activation)."""
    from runtime.kernels import ops
    rng = np.random.default_rng(rows + inner)
    a = dev(rng.standard_normal((rows, inner)), torch.bfloat16)
    w = dev(rng.standard_normal((2 * width, inner)) * 2.0 / np.sqrt(inner), torch.bfloat16)
    out = ops.gemm_swiglu(a, w, torch.zeros((rows, width), device=DEV, dtype=torch.bfloat16), law=(1.25, 1.702, 1.0))
    gu = (a.float() @ w.float().T).to(torch.bfloat16).float().cpu().numpy()
    want = P.clamped_glu(gu[:, :width], gu[:, width:], 1.25)
    got = out.float().cpu().numpy()
    assert np.abs(got - want).max() < 2e-2 * np.abs(want).max()       # (a bfloat16 step of gate or up moves the result this far)
    assert np.sqrt(((got - want) ** 2).mean()) < 4e-3 * np.abs(want).max()


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads, kv_heads, dim, vdim", [(4, 2, 24, 16), (2, 2, 16, 40), (3, 1, 8, 8), (1, 1, 70, 130)])
def test_normed_queries_and_keys_land_in_padded_heads_and_pages(dtype, heads, kv_heads, dim, vdim):
    from runtime.kernels import ops
    rng = np.random.default_rng(dim)
    tdtype = {"float32": torch.float32, "bfloat16": torch.bfloat16}[dtype]
    T, P_, pad, pages = 6, 8, -(-max(dim, vdim) // 8) * 8, 5
    width = (heads + kv_heads) * dim + kv_heads * vdim + heads
    qkv = dev(rng.standard_normal((T, width)), tdtype)
    wq, wk = 1 + 0.2 * rng.standard_normal(dim), 1 + 0.2 * rng.standard_normal(dim)
    kcache = torch.full((pages, kv_heads, P_, pad), 9.0, device=DEV, dtype=tdtype)
    vcache = torch.full((pages, kv_heads, pad, P_), 9.0, device=DEV, dtype=tdtype)
    slots = [17, 3, -1, 39, 8, 15]                        # page borders, a row without a slot
    q = ops.qk_norm_scatter(qkv, dev(wq), dev(wk), torch.zeros((T, heads * pad), device=DEV, dtype=tdtype), kcache, vcache,
                            ints(slots), heads, kv_heads, dim, vdim, pad, P_, 1e-4)
    ref = qkv.float().cpu().numpy()
    tol = 2e-5 if dtype == "float32" else 8e-3
    got_q = q.float().cpu().numpy().reshape(T, heads, pad)
    close(got_q[:, :, :dim], P.rmsnorm(ref[:, :heads * dim].reshape(T, heads, dim), wq, 1e-4), tol)
    assert (got_q[:, :, dim:] == 0).all()
    keys = P.rmsnorm(ref[:, heads * dim:(heads + kv_heads) * dim].reshape(T, kv_heads, dim), wk, 1e-4)
    values = ref[:, (heads + kv_heads) * dim:(heads + kv_heads) * dim + kv_heads * vdim].reshape(T, kv_heads, vdim)
    kc, vc = kcache.float().cpu().numpy(), vcache.float().cpu().numpy()
    written = np.zeros((pages, P_), bool)
    for t, slot in enumerate(slots):
        if slot < 0:
            continue
        page, at = divmod(slot, P_)
        written[page, at] = True
        close(kc[page, :, at, :dim], keys[t], tol)
        close(vc[page, :, :vdim, at], values[t], tol)
        assert (kc[page, :, at, dim:] == 0).all() and (vc[page, :, vdim:, at] == 0).all()
    assert (kc.transpose(0, 2, 1, 3)[~written] == 9.0).all() and (vc.transpose(0, 3, 1, 2)[~written] == 9.0).all(), "a place that no row named was written"
    gates = rng.standard_normal((T, heads + 3))
    attn = dev(rng.standard_normal((T, heads * pad)), tdtype)
    gbuf = dev(gates, tdtype)
    out = ops.head_gate(attn, gbuf[:, 3:], torch.zeros((T, heads * vdim), device=DEV, dtype=tdtype), heads, vdim, pad)
    want = attn.float().cpu().numpy().reshape(T, heads, pad)[:, :, :vdim] * P.sigmoid(gbuf.float().cpu().numpy()[:, 3:, None])
    close(out.float().cpu().numpy().reshape(T, heads, vdim), want, tol)


# -- whole models ---------------------------------------------------------------------------------------------------------

def make_runner(folder, dtype, pages=40, page_size=16, max_requests=4, execution="eager"):
    from runtime.engine import load_model, ModelRunner
    return ModelRunner(load_model(folder, dtype=dtype), n_pages=pages, page_size=page_size, max_requests=max_requests, execution=execution)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_layers_one_by_one_and_a_whole_prompt(folders, name, dtype):
    from runtime.engine import StepEntry
    cfg, w = P.read_folder(folders[name])
    tokens = random_tokens(3, 45, cfg["vocab"])
    layers = []
    want = P.forward(cfg, w, tokens, layers)
    runner = make_runner(folders[name], dtype)
    seen = {}
    runner.layer_tap = lambda i, x: seen.__setitem__(i, x.float().cpu().numpy().copy())
    runner.create("r")
    got = runner.step([StepEntry("r", tokens, list(range(len(tokens))))]).cpu().numpy()
    for i, x in enumerate(layers):
        close(seen[i], x, 2e-5 if dtype == "float32" else 3e-2)
    assert_close(got, want, dtype, "whole prompt")


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_prompt_then_tokens_one_by_one_and_portions_down_to_two_tokens(folders, name, dtype, execution):
    from runtime.engine import StepEntry
    V = CONFIGS[name]["vocab"]
    tokens = random_tokens(4, 150, V)
    want = plain_logits(folders[name], tokens)
    runner = make_runner(folders[name], dtype, execution=execution)
    runner.create("d")
    got = [runner.step([StepEntry("d", tokens[:97], list(range(97)))]).cpu().numpy()]
    got += [runner.step([StepEntry("d", [t], [0])]).cpu().numpy() for t in tokens[97:]]      # a long run of single tokens
    assert_close(np.concatenate(got), want, dtype, "prompt, then decoded")
    runner.release("d")
    runner.create("c")                                     # the same slot and pages once more, now in portions
    at, got = 0, []
    for n in [2, 3, 1, 2, 17, 2, 16, 31, 1, 5, 2, 33, 2, 100]:
        n = min(n, len(tokens) - at)
        got.append(runner.step([StepEntry("c", tokens[at:at + n], list(range(n)))]).cpu().numpy())
        at += n
    assert at == len(tokens)
    assert_close(np.concatenate(got), want, dtype, "portions")
    runner.cache.check()


@pytest.mark.parametrize("name, dtype, execution", [("q", "float32", "graph"), ("p", "bfloat16", "graph"), ("s", "float32", "eager")])
def test_long_decoding_from_the_first_token(folders, name, dtype, execution):
    """A request decoded one token at a time from its very first token, over a dozen pages, beside a second request that
    joins late and leaves early (its slot and pages go back while the first goes on)."""
    from runtime.engine import StepEntry
    V = CONFIGS[name]["vocab"]
    long, short = random_tokens(21, 210, V), random_tokens(22, 40, V)
    want = {"l": plain_logits(folders[name], long), "s": plain_logits(folders[name], short)}
    runner = make_runner(folders[name], dtype, pages=17, execution=execution)
    runner.create("l")
    got = {"l": [], "s": []}
    for t, token in enumerate(long):
        entries = [StepEntry("l", [token], [0])]
        if 60 <= t < 100:
            if t == 60:
                runner.create("s")
            entries.append(StepEntry("s", [short[t - 60]], [0]))
        out = runner.step(entries).cpu().numpy()
        got["l"].append(out[0])
        if len(entries) == 2:
            got["s"].append(out[1])
        if t == 99:
            runner.release("s")
    assert_close(np.stack(got["l"]), want["l"], dtype, "long decoding")
    assert_close(np.stack(got["s"]), want["s"], dtype, "the request that joined late")
    runner.cache.check()


def mixed(V, seed, lengths=(70, 33, 120, 9, 64, 97, 40, 130), live_at_once=4):
    """Up to `live_at_once` live requests: portions of some beside single tokens of others; requests end and new ones
    start on the pages and state slots they gave back; one request sits out some steps."""
    rng = np.random.default_rng(seed)
    seqs = {f"m{i}": random_tokens(seed * 100 + i, n, V) for i, n in enumerate(lengths)}
    waiting, live, fed, trace, step = list(seqs), [], {}, Trace(), 0
    while waiting or live:
        while waiting and len(live) < live_at_once:
            rid = waiting.pop(0); live.append(rid); fed[rid] = 0
        entries, ending = [], []
        for rid in list(live):
            remaining = len(seqs[rid]) - fed[rid]
            if rid == live[0] and step % 5 == 3 and len(live) > 1:
                continue
            if remaining > 12:
                n = max(1, min(int(rng.choice([2, 3, 7, 16, 21, 40])), remaining - 8))
                want = [n - 1] if rng.random() < 0.5 else list(range(n))
            else:
                n, want = 1, [0]
            entries.append((rid, seqs[rid][fed[rid]:fed[rid] + n], want))
            fed[rid] += n
            if fed[rid] == len(seqs[rid]):
                ending.append(rid); live.remove(rid)
        if entries:
            trace.add(entries, end=ending)
        step += 1
    return trace, seqs


@pytest.mark.parametrize("execution", ["eager", "graph"])
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", sorted(CONFIGS))
def test_mixed_batches_through_the_replay_program_with_pages_and_slots_used_again(folders, tmp_path, name, dtype, execution):
    from runtime.engine.replay import replay, MAX_LIVE
    V = CONFIGS[name]["vocab"]
    trace, seqs = mixed(V, seed=5)
    assert any(len(s["entries"]) == 4 for s in trace.steps)
    done = []
    runner = replay(folders[name], dtype, tmp_path, trace.peak, trace.lines(), echo=done.append, execution=execution)
    assert done == [f"done {i}" for i in range(len(trace.steps))]
    assert runner.cache.slots.n_slots == MAX_LIVE < len(seqs), "state slots must be used again"
    assert all(sum(-(-len(s) // 16) for s in seqs.values()) > g.pool.n_pages for g in runner.cache.groups), "pages must be used again"
    runner.cache.check()
    trace.check(folders[name], tmp_path, dtype, V, seqs, plain=plain_logits)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_gives_what_each_gives_alone(folders, dtype):
    from runtime.engine import StepEntry
    name = "p"
    V = CONFIGS[name]["vocab"]
    seqs = {k: random_tokens(50 + i, n, V) for i, (k, n) in enumerate({"a": 61, "b": 5, "c": 1, "d": 30}.items())}
    alone = {}
    for k, toks in seqs.items():
        runner = make_runner(folders[name], dtype)
        runner.create(k)
        alone[k] = runner.step([StepEntry(k, toks, list(range(len(toks))))]).cpu().numpy()
    runner = make_runner(folders[name], dtype, max_requests=4)
    for k in seqs:
        runner.create(k)
    got = runner.step([StepEntry(k, toks, list(range(len(toks)))) for k, toks in seqs.items()]).cpu().numpy()
    at = 0
    for k, toks in seqs.items():
        piece = got[at:at + len(toks)]
        at += len(toks)
        err = np.abs(piece - alone[k]).max() / np.abs(alone[k]).max()
        assert err < (1e-5 if dtype == "float32" else 2e-2), f"request {k} differs from itself alone by {err:.2e}"


@pytest.mark.parametrize("dtype", DTYPES)
def test_far_keys_page_borders_and_old_state_in_a_model_drawn_sharp(folders, dtype):
    """In the sharp model a query's result hangs on one key (scores spread over several units) and the states forget
    slowly: a wrong page, a lost key or a state that started late shows in the logits.  A prompt of 23 pages and a
    half, cut in the middle of a page, then tokens one by one over two page borders."""
    from runtime.engine import StepEntry
    name = "s"
    cfg, w = P.read_folder(folders[name])
    tokens = random_tokens(9, 410, cfg["vocab"])
    want = plain_logits(folders[name], tokens)
    # the test means something only if far keys carry weight: the plain model without its first 200 tokens differs
    late = P.forward(cfg, w, tokens[200:])
    assert np.abs(late[-40:] - want[-40:]).max() > 0.05 * np.abs(want).max(), "the first 200 tokens do not reach the last 40"
    runner = make_runner(folders[name], dtype, pages=26)
    runner.create("f")
    got = [runner.step([StepEntry("f", tokens[:201], list(range(201)))]).cpu().numpy(),
           runner.step([StepEntry("f", tokens[201:376], list(range(175)))]).cpu().numpy()]
    got += [runner.step([StepEntry("f", [t], [0])]).cpu().numpy() for t in tokens[376:]]
    got = np.concatenate(got)
    assert_close(got, want, dtype, "far keys")
    assert_close(got[:3], want[:3], dtype, "the first tokens")


@pytest.mark.parametrize("name, dtype, execution, overlap", [("p", "float32", "graph", True), ("p", "float32", "eager", False),
                                                             ("p", "bfloat16", "graph", True), ("g", "float32", "graph", True)])
def test_greedy_generation_through_the_scheduler(folders, name, dtype, execution, overlap):
    from runtime.engine.scheduler import Engine
    cfg, w = P.read_folder(folders[name])
    prompts = [random_tokens(70 + i, n, cfg["vocab"]) for i, n in enumerate([11, 3, 26, 1, 40])]
    engine = Engine.from_folder(folders[name], dtype=dtype, pages=24, page_size=16, execution=execution,
                                max_active=3, token_budget=24, prefill_chunk=9, overlap=overlap)
    got = engine.generate(prompts, max_new_tokens=10)
    for prompt, new in zip(prompts, got):
        assert len(new) == 10
        if dtype == "float32":
            assert new == P.greedy(cfg, w, prompt, 10)
        else:       # bfloat16: every picked token is the plain model's best or within rounding of it, given the same past
            logits = P.forward(cfg, w, prompt + new)[len(prompt) - 1:-1]
            for row, token in zip(logits, new):
                assert row.max() - row[token] < 0.05 * (row.max() - row.min())
    engine.runner.cache.check()
    assert not engine.runner.cache.lengths, "every request gave back what it held"


def test_command_line_serves_the_design(folders, tmp_path):
    """`python -m runtime` chooses the design by config.json: requests of a file against a folder, in float32, give the
    plain model's greedy tokens; the named configuration with random weights generates and reports its state slots."""
    import json, os, subprocess, sys
    from conftest import ROOT
    cfg, w = P.read_folder(folders["p"])
    requests = [{"key": "x", "prompt": [1, 2, 3, 4, 5, 6, 7], "max_new_tokens": 5}, {"key": "y", "prompt": [9], "max_new_tokens": 4}]
    (tmp_path / "requests.json").write_text(json.dumps(requests))
    env = dict(os.environ, PYTHONPATH=str(ROOT))
    proc = subprocess.run([sys.executable, "-m", "runtime", "--checkpoint", str(folders["p"]), "--dtype", "float32",
                           "--requests", str(tmp_path / "requests.json"), "--policy", "chunked", "--pages", "16",
                           "--token-budget", "6", "--prefill-chunk", "3"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    by_key = {r["key"]: r for r in json.loads(proc.stdout)["requests"]}
    assert by_key["x"]["generated"] == P.greedy(cfg, w, [1, 2, 3, 4, 5, 6, 7], 5)
    assert by_key["y"]["generated"] == P.greedy(cfg, w, [9], 4)
    proc = subprocess.run([sys.executable, "-m", "runtime", "--model", "novosun-tiny", "--tokens", "5,6,7", "--max-new-tokens", "3",
                           "--overlap", "--report"], capture_output=True, text=True, timeout=300, env=env, cwd=str(tmp_path))
    assert proc.returncode == 0, proc.stderr[-2000:]
    out = json.loads(proc.stdout)
    assert out["weights"] == "random-novosun-tiny" and len(out["requests"][0]["generated"]) == 3
    assert out["runner"]["replays"] >= 1 and out["runner"]["cache"][0]["resident_pages"] == 0
