"""Malilorn on the CPU: the plain model's mechanisms pinned by their own invariants, the
configuration and the checkpoint, and the engine (cache, state slots, step function, scheduler,
trace replay) with substitute kernels against the plain model."""
import math
import os

import pytest
import torch

from litellmengine_amd.cache import CacheManager
from litellmengine_amd.config import ConfigError, MalilornConfig, load_config
from litellmengine_amd.config.registry import architecture_of
from litellmengine_amd.engine import LLMEngine, ModelRunner, StepEntry
from litellmengine_amd.models import load_model
from litellmengine_amd.weights.loader import WeightError
from tests.malilorn_util import (CONFIGS, PAGE_SIZES, make_model_dir, plain_logits, read, residual_streams, rewrite,
                                 run_tool, sharpen)
from tests.plain import malilorn_plain as plain
from tests.tiny import random_tokens
from tests.torch_ops import TorchOps
from tests.trace_util import TraceBuilder, changing_portions, check_dumps, mixed, tail_one_by_one, whole


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


# -- the plain model's mechanisms, each alone ------------------------------------------------
def test_plain_convolution_written_out():
    """The last tap meets the token itself, the first one the token J - 1 places back; zeros before the start."""
    u, taps = rnd((6, 3), 1), rnd((3, 4), 2)
    y = plain.short_conv(u, taps)
    for t in range(6):
        for c in range(3):
            want = sum(float(taps[c, j]) * float(u[t - 3 + j, c]) for j in range(4) if t - 3 + j >= 0)
            assert abs(float(y[t, c]) - want) < 1e-12
    # one tap is a factor per channel; a unit last tap hands the input on
    assert torch.allclose(plain.short_conv(u, taps[:, :1]), u * taps[:, 0])
    unit = torch.zeros((3, 5), dtype=torch.float64)
    unit[:, -1] = 1.0
    assert torch.equal(plain.short_conv(u, unit), u)
    unit = torch.zeros((3, 5), dtype=torch.float64)
    unit[:, 0] = 1.0  # the first tap alone: the input four tokens late
    assert torch.equal(plain.short_conv(u, unit)[4:], u[:2]) and float(plain.short_conv(u, unit)[:4].abs().max()) == 0.0


def test_plain_rotation_pairs_halves_and_leaves_the_rest():
    x = rnd((5, 2, 12), 3)
    f = plain.rotary_frequencies(100.0, 8, None)
    assert torch.allclose(f, torch.tensor([100.0 ** (-2 * i / 8) for i in range(4)], dtype=torch.float64))
    y = plain.rotate_half_split(x, torch.arange(5), f)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 8:], x[..., 8:])
    for i in range(4):  # element i turns with element i + 4, and a turn keeps the pair's length
        assert torch.allclose(y[..., i] ** 2 + y[..., i + 4] ** 2, x[..., i] ** 2 + x[..., i + 4] ** 2)
    a = float(3 * f[1])
    assert abs(float(y[3, 1, 1]) - (float(x[3, 1, 1]) * math.cos(a) - float(x[3, 1, 5]) * math.sin(a))) < 1e-12
    assert abs(float(y[3, 1, 5]) - (float(x[3, 1, 5]) * math.cos(a) + float(x[3, 1, 1]) * math.sin(a))) < 1e-12
    # scores depend on the distance only
    q, k = rnd((1, 1, 8), 4), rnd((1, 1, 8), 5)
    at = lambda p, t: plain.rotate_half_split(t, torch.tensor([p]), f)[0, 0]
    assert abs(float(at(9, q) @ at(4, k)) - float(at(25, q) @ at(20, k))) < 1e-9


def test_stretched_frequencies_in_three_bands():
    s = {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 64}
    plainf, f = plain.rotary_frequencies(10000.0, 32, None), plain.rotary_frequencies(10000.0, 32, s)
    kept = stretched = between = 0
    for a, b in zip(plainf.tolist(), f.tolist()):
        l = 2 * math.pi / a
        if l < 64 / 4.0:
            assert b == a
            kept += 1
        elif l > 64 / 1.0:
            assert abs(b - a / 8.0) < 1e-15
            stretched += 1
        else:
            assert a / 8.0 < b < a
            between += 1
    assert kept and stretched and between
    from litellmengine_amd.parts.position import scaled_frequencies
    from litellmengine_amd.config.kezasun_config import FrequencyScaling

    assert torch.allclose(scaled_frequencies(plainf, FrequencyScaling(8.0, 1.0, 4.0, 64.0)), f, rtol=1e-12)


def test_plain_attention_by_hand_with_grouped_heads_and_wider_values():
    T, H, G, d, dv = 5, 4, 2, 6, 9
    q, k, v = rnd((T, H, d), 6), rnd((T, G, d), 7), rnd((T, G, dv), 8)
    out = plain.causal_attention(q, k, v, 0.3)
    assert out.shape == (T, H, dv)
    assert torch.allclose(out[0], v[0].repeat_interleave(2, dim=0))  # the first token sees itself only
    t, h = 3, 2
    s = torch.tensor([float(q[t, h] @ k[j, 1]) * 0.3 for j in range(t + 1)], dtype=torch.float64)
    p = torch.exp(s - s.max())
    assert torch.allclose(out[t, h], (p / p.sum()) @ v[: t + 1, 1])


def test_plain_recurrence_written_out():
    T, d = 6, 4
    r, k, v = rnd((T, d), 9), rnd((T, d), 10), rnd((T, d), 11)
    decay, u = torch.rand((T, d), generator=torch.Generator().manual_seed(1), dtype=torch.float64), rnd((d,), 12)
    o = plain.matrix_state_walk(r, k, v, decay, u)
    for t in range(T):  # every earlier token through the decays of the tokens between, the current one with the bonus
        want = (r[t] * u * k[t]).sum() * v[t]
        for s in range(t):
            want = want + (r[t] * decay[s + 1 : t].prod(dim=0) * k[s]).sum() * v[s]
        assert torch.allclose(o[t], want)


def test_plain_router_scores_weights_and_shared_gate():
    h = rnd((7, 10), 13)
    w = {"m.router": rnd((6, 10), 14)}
    ids, weights = plain.routed_choice(h, w, "m.", 2)
    s = plain.sigmoid(h @ w["m.router"].T)
    for t in range(7):
        order = sorted(range(6), key=lambda e: -float(s[t, e]))
        assert ids[t].tolist() == order[:2]
        assert torch.allclose(weights[t], s[t, order[:2]])  # as they are: they do not add up to one
    assert float((weights.sum(-1) - 1).abs().min()) > 1e-3
    # the weight meets the expert's input: behind a squared activation it counts twice
    for e in range(6):
        w[f"m.e{e}.up"], w[f"m.e{e}.down"] = rnd((5, 10), 20 + e), rnd((10, 5), 30 + e)
    out = plain.moe_ff(h, w, "m.", {"router": {"experts": 6, "top": 2}})
    t = 4
    want = sum(float(g) ** 2 * plain.small_expert(h[t], w, f"m.e{int(e)}.") for e, g in zip(ids[t], weights[t]))
    assert torch.allclose(out[t], want)
    w["m.shared.up"], w["m.shared.down"], w["m.shared.sg"] = rnd((3, 10), 40), rnd((10, 3), 41), rnd((1, 10), 42)
    both = plain.moe_ff(h, w, "m.", {"router": {"experts": 6, "top": 2}, "shared": {"ff": 3}})
    gate = plain.sigmoid(h @ w["m.shared.sg"].T)
    assert torch.allclose(both - out, plain.small_expert(h, w, "m.shared.") * gate)


def test_plain_cap_on_the_logits():
    cfg, w = {"vocab": 5, "width": 4, "norm": {"eps": 1e-5}, "layers": [], "logit_softcap": 2.0}, {
        "embed": rnd((5, 4), 50, 3.0), "final.norm": torch.ones(4, dtype=torch.float64)}
    capped = plain.forward(cfg, w, [1, 2])
    free = plain.forward({**cfg, "logit_softcap": None}, w, [1, 2])
    assert float(capped.abs().max()) < 2.0 < float(free.abs().max())
    assert torch.allclose(capped, 2.0 * torch.tanh(free / 2.0))


# -- configuration and checkpoint -------------------------------------------------------------
@pytest.mark.parametrize("which", list(CONFIGS))
def test_config_round_trip_and_registry(tmp_path, which):
    cfg = MalilornConfig.from_dict(CONFIGS[which])
    assert MalilornConfig.from_dict(cfg.to_dict()) == cfg
    assert architecture_of(CONFIGS[which]).name == "Malilorn"
    d = make_model_dir(tmp_path, which)
    assert load_config(d) == cfg
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    assert "head" not in read(d)[1] and model.head.weight is model.embedding.weight  # the head is the embedding table


def test_sizes_left_to_the_checkpoint_and_defaults(tmp_path):
    import copy
    import json

    c = copy.deepcopy(CONFIGS["C"])
    d = make_model_dir(tmp_path, "C")
    for layer in c["layers"]:
        del layer["mixer"]["right"]["decay_rank"]  # the checkpoint's shapes say it
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(c, f)
    assert [l.mixer.right.decay_rank for l in load_config(d).layers] == [3, 2, 6]
    assert MalilornConfig.from_dict(c).layers[0].mixer.right.decay_rank is None
    load_model(d, "float32", device="cpu", ops=TorchOps())
    m = MalilornConfig.from_dict({"vocab": 9, "width": 8, "norm": {"eps": 1e-5}, "layers": [
        {"type": "parallel", "mlp": None, "mixer": {"left": {"heads": 2, "dim": 4}, "right": {"heads": 1, "dim": 8}}}]})
    a = m.layers[0].mixer
    assert (a.left.kv_heads, a.left.vdim, a.left.conv, a.left.rot_dims, a.left.scale) == (2, 4, 0, 0, 0.5)
    assert (a.left_scale, a.right_scale, m.logit_softcap) == (1.0, 1.0, None)


def test_config_faults_are_named():
    import copy

    def broken(change):
        c = copy.deepcopy(CONFIGS["A"])
        change(c)
        with pytest.raises(ConfigError) as e:
            MalilornConfig.from_dict(c)
        return str(e.value)

    assert "layers[1].type" in broken(lambda c: c["layers"][1].update(type="serial"))
    assert "kv_heads" in broken(lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4))
    assert "rot.dims" in broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=26))
    assert "kind" in broken(lambda c: c["layers"][1]["mlp"].update(kind="wide"))
    assert "top" in broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=6))
    assert "right" in broken(lambda c: c["layers"][2]["mixer"].pop("right"))
    assert "eps" in broken(lambda c: c["norm"].pop("eps"))


def test_checkpoint_faults_are_listed_together(tmp_path):
    from safetensors.torch import load_file, save_file

    d = make_model_dir(tmp_path, "A")
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["l0.mlp.e3.up"]
    t["l2.mlp.gate"] = torch.zeros((4, 72))  # layer 2 has no feed-forward
    t["l1.mix.left.q.conv"] = torch.zeros((48, 4))  # five taps are configured
    save_file(t, path)
    with pytest.raises(WeightError) as e:
        load_model(d, "float32", device="cpu", ops=TorchOps())
    assert all(n in str(e.value) for n in ("l0.mlp.e3.up", "l2.mlp.gate", "l1.mix.left.q.conv"))


# -- the engine with substitute kernels -------------------------------------------------------
def cpu_runner(d, page_size, num_pages, max_requests=4):
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         dtype=torch.float32, device="cpu")
    return model, cache, ModelRunner(model, cache)


def watch_layers(model, seen):
    """After every block: the residual stream (a block of this arrangement leaves nothing to add)."""
    for b in model.blocks:
        def wrapped(hidden, delta, step, layer_cache, next_norm=None, inner=b.forward):
            out = inner(hidden, delta, step, layer_cache, next_norm=next_norm)
            seen.append(hidden.double().cpu().clone())
            return out
        b.forward = wrapped


@pytest.mark.parametrize("which", list(CONFIGS))
def test_one_layer_at_a_time_follows_the_plain_model(tmp_path, which):
    d = make_model_dir(tmp_path, which)
    sharpen(d, 8.0)
    tokens = random_tokens(45, CONFIGS[which]["vocab"], 3)
    want = residual_streams(d, tokens)
    model, cache, runner = cpu_runner(d, PAGE_SIZES[which], 16)
    seen = []
    watch_layers(model, seen)
    runner.step([StepEntry(runner.admit(), tokens, [])])
    assert len(seen) == len(want)
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert (got - ref).abs().max() < 1e-4 * max(1.0, float(ref.abs().max())), f"layer {i}"
    for b in model.blocks:
        del b.forward  # (the wrappers hold the model in a cycle)


def all_ways_trace(requests):
    tb = TraceBuilder()
    names = list(requests)
    whole(tb, names[0] + "#whole", requests[names[0]])
    tail_one_by_one(tb, names[1] + "#tail", requests[names[1]], tail=20)
    changing_portions(tb, names[2] + "#cut", requests[names[2]], seed=1)
    mixed(tb, {rid + "#mix": t for rid, t in requests.items()}, seed=5)
    return tb


@pytest.mark.parametrize("which", list(CONFIGS))
def test_trace_cpu(tmp_path, which):
    """Whole, with a decoded tail, in portions down to two tokens, and mixed in a pool of the live peak
    with four slots (pages, slots and state rows are used again)."""
    d = make_model_dir(tmp_path, which)
    sharpen(d, 8.0)
    vocab = CONFIGS[which]["vocab"]
    requests = {rid: random_tokens(n, vocab, 20 + i) for i, (rid, n) in enumerate(
        {"a": 70, "b": 45, "c": 100, "d": 33, "e": 64, "f": 1}.items())}
    tb = all_ways_trace(requests)
    out = str(tmp_path / "out")
    run_tool(d, "float32", out, tb, page_size=PAGE_SIZES[which], in_process_ops=TorchOps())
    # (the plain model itself, run in float32, moves by up to 7e-4 on these weights: 3e-4 is about five times
    # the worst error seen here, where products and sums are float64 and only what is stored is float32)
    check_dumps(out, tb, plain_logits(d, requests), 3e-4)


def test_both_mixers_states_share_a_row_and_are_zeroed_when_a_slot_is_used_again(tmp_path):
    d = make_model_dir(tmp_path, "A")
    sharpen(d, 8.0)
    cfg, w = read(d)
    model, cache, runner = cpu_runner(d, 4, 12, max_requests=1)
    left, right = model.blocks[0].mixer.left, model.blocks[0].mixer.right
    assert cache.states[0].shape[1] == left.state_spec().shape[0] + right.state_spec().shape[0]
    assert left.state_spec().shape[0] == 2 * (6 * 24 + 2 * 24 + 2 * 40)  # two rows of q, k and v behind three taps
    first, second = random_tokens(9, 131, 1), random_tokens(6, 131, 2)
    s = runner.admit()
    runner.step([StepEntry(s, first, [])])
    assert all(float(st[s].abs().max()) > 0 for st in cache.states.values()) and len(cache.states) == 4
    runner.release(s)
    s2 = runner.admit()
    assert s2 == s and all(float(st[s].abs().max()) == 0 for st in cache.states.values())
    got = runner.step([StepEntry(s2, second, [5])])
    assert (got[0].double() - plain.forward(cfg, w, second)[5]).abs().max() < 1e-5


@pytest.mark.parametrize("which", ["A", "C"])
def test_greedy_generation_through_the_scheduler(tmp_path, which):
    """Requests of unequal lengths batched, prompts in portions, then a pool so small that requests
    are preempted and recomputed (their state rows start from zero again): the same tokens."""
    d = make_model_dir(tmp_path, which)
    sharpen(d, 8.0)
    cfg, w = read(d)
    prompts = [random_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate((1, 7, 23, 40))]
    want = [plain.greedy(cfg, w, p, 6) for p in prompts]
    for run_ahead in (False, True):
        model = load_model(d, "float32", device="cpu", ops=TorchOps())
        eng = LLMEngine(model, page_size=8, num_pages=16, max_requests=4, prefill_chunk=16, max_tokens_per_step=24,
                        run_ahead=run_ahead)
        assert eng.generate(prompts, 6) == want
    small = LLMEngine(load_model(d, "float32", device="cpu", ops=TorchOps()), page_size=8, num_pages=8, max_requests=4,
                      prefill_chunk=16, max_tokens_per_step=24, run_ahead=False)
    assert small.generate(prompts, 6) == want
    assert all(g.pool.num_held == 0 for g in small.cache.groups)


def test_a_lost_key_a_lost_tap_or_a_lost_state_would_show(tmp_path):
    """The measure of the GPU traces with sharpened weights: in the plain model of such weights, hiding the
    first key from every query, dropping the convolution's farthest tap, or what the recurrences knew before the
    last 60 tokens, moves the logits by far more than the 32-bit tolerance."""
    d = make_model_dir(tmp_path, "A", seed=5, dtype=torch.bfloat16)
    sharpen(d, 9.0, memory=1.6)
    cfg, w = read(d)
    tokens = random_tokens(140, cfg["vocab"], 42)
    base = plain.forward(cfg, w, tokens)
    moved = lambda other: (other - base).abs().max(dim=1).values / base.abs().max()
    seen = plain.causal_attention
    try:  # every query from the second token on loses the sequence's first key
        def blind(q, k, v, scale):
            out = seen(q, k, v, scale)
            out[2:] = seen(q[1:], k[1:], v[1:], scale)[1:]
            return out
        plain.causal_attention = blind
        m = moved(plain.forward(cfg, w, tokens))
    finally:
        plain.causal_attention = seen
    assert float(m[2:].max()) > 5e-3 and float((m[2:] > 1e-4).float().mean()) > 0.2
    w2 = dict(w)
    for name in w:
        if name.endswith(".conv"):
            w2[name] = w[name].clone()
            w2[name][:, 0] = 0.0
    assert float((moved(plain.forward(cfg, w2, tokens))[3:] > 1e-3).float().mean()) > 0.9
    fresh = plain.forward(cfg, w, tokens[-60:])[-1]
    only_right = {**cfg, "layers": [dict(l, mixer=dict(l["mixer"], left_scale=0.0)) for l in cfg["layers"]]}
    whole_run, fresh = plain.forward(only_right, w, tokens)[-1], plain.forward(only_right, w, tokens[-60:])[-1]
    assert float((whole_run - fresh).abs().max() / whole_run.abs().max()) > 1e-3
