"""Birelix on the CPU: the plain implementation's mechanisms pinned one by one, configuration and checkpoint
handling, and the engine (step function, cache and state manager, scheduler) with substitute kernels
against the plain implementation."""
import math
import os

import pytest
import torch

from litellmengine_amd.cache import CacheManager
from litellmengine_amd.config import BirelixConfig, ConfigError, load_config
from litellmengine_amd.config.registry import architecture_of
from litellmengine_amd.engine import LLMEngine, ModelRunner, StepEntry
from litellmengine_amd.models import load_model
from litellmengine_amd.weights.loader import WeightError
from tests.birelix_util import (CONFIGS, PAGE_SIZES, delta, dense, latent, layer, make_model_dir, moe, plain_logits, read,
                                residual_streams, rewrite, run_tool, sharpen, window)
from tests.plain import birelix_plain as plain
from tests.tiny import random_tokens
from tests.torch_ops import TorchOps
from tests.trace_util import TraceBuilder, changing_portions, check_dumps, mixed, tail_one_by_one, whole


def rnd(shape, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(shape, generator=g, dtype=torch.float64) * scale


# -- the plain mechanisms, each against what it is defined by ---------------------------------------
def test_plain_delta_rule_written_out():
    """Without decay and with whole corrections the state stores values under their keys: orthonormal keys are
    read back exactly, and writing a key again replaces what it held."""
    d, e = 6, 4
    keys = torch.linalg.qr(rnd((d, d), 1)).Q  # rows: orthonormal keys
    v = rnd((5, e), 2)
    k = torch.stack([keys[0], keys[1], keys[2], keys[0], keys[3]])
    ones = torch.ones(5, dtype=torch.float64)
    o, S = plain.delta_walk(k, k, v, ones, ones)
    assert torch.allclose(o, v, atol=1e-12)  # every token reads its own write
    assert torch.allclose(S.T @ keys[0], v[3], atol=1e-12)  # the second write under the first key replaced the first
    assert torch.allclose(S.T @ keys[1], v[1], atol=1e-12)
    # a step by hand, with decay and a partial correction
    q, k, v = rnd((3, d), 3), rnd((3, d), 4), rnd((3, e), 5)
    beta, g = torch.tensor([0.3, 0.9, 0.5], dtype=torch.float64), torch.tensor([0.8, 0.2, 1.0], dtype=torch.float64)
    S = torch.zeros((d, e), dtype=torch.float64)
    outs = []
    for t in range(3):
        S = g[t] * S
        S = S + torch.outer(k[t], beta[t] * (v[t] - k[t] @ S))
        outs.append(q[t] @ S)
    o, last = plain.delta_walk(q, k, v, beta, g)
    assert torch.allclose(o, torch.stack(outs), atol=1e-12) and torch.allclose(last, S, atol=1e-12)
    # the state carries over: a walk cut in two equals the walk in one go
    o1, S1 = plain.delta_walk(q[:2], k[:2], v[:2], beta[:2], g[:2])
    o2, S2 = plain.delta_walk(q[2:], k[2:], v[2:], beta[2:], g[2:], state=S1)
    assert torch.allclose(torch.cat([o1, o2]), o, atol=1e-12) and torch.allclose(S2, last, atol=1e-12)


def test_plain_convolution_unit_vectors_and_decay():
    u, taps = rnd((7, 3), 1), rnd((3, 4), 2)
    y = plain.short_conv(u, taps)
    for t in range(7):
        for c in range(3):
            want = sum(float(taps[c, j]) * float(u[t - 3 + j, c]) for j in range(4) if t - 3 + j >= 0)
            assert abs(float(y[t, c]) - want) < 1e-12
    assert torch.allclose(plain.short_conv(u, torch.ones((3, 1), dtype=torch.float64)), u)  # one tap of one: the input itself
    x = rnd((5, 8), 3)
    n = plain.unit_vector(x)
    assert torch.allclose((n * n).sum(-1), (x * x).sum(-1) / ((x * x).sum(-1) + 1e-6), atol=1e-12)
    assert float(plain.unit_vector(torch.zeros((1, 4), dtype=torch.float64)).abs().max()) == 0.0  # no division by zero
    z = torch.tensor([-30.0, -1.0, 0.0, 2.0, 40.0], dtype=torch.float64)
    assert torch.allclose(plain.softplus(z), torch.log1p(torch.exp(z.clamp(max=30))).where(z < 30, z), atol=1e-12)
    assert torch.allclose(plain.gelu_tanh(torch.tensor([0.0, 1.0, -1.0], dtype=torch.float64)),
                          torch.tensor([0.0, 0.8411919906082768, -0.15880800939172324], dtype=torch.float64), atol=1e-12)


def test_plain_rotation_pairs_neighbours_and_keeps_relative_positions():
    x = rnd((6, 2, 10), 1)
    pos = torch.arange(6)
    y = plain.rotate_neighbours(x, pos, 6, 100.0)
    assert torch.equal(y[..., 6:], x[..., 6:]) and torch.allclose(y[0], x[0])  # the rest passes; position 0 is the identity
    for i in range(3):  # pairs keep their length and turn by pos * base^(-2i/dims)
        assert torch.allclose(y[..., 2 * i] ** 2 + y[..., 2 * i + 1] ** 2, x[..., 2 * i] ** 2 + x[..., 2 * i + 1] ** 2, atol=1e-12)
        a = 4 * 100.0 ** (-2.0 * i / 6)
        u, v = x[4, 0, 2 * i], x[4, 0, 2 * i + 1]
        assert abs(float(y[4, 0, 2 * i]) - float(u * math.cos(a) - v * math.sin(a))) < 1e-12
        assert abs(float(y[4, 0, 2 * i + 1]) - float(v * math.cos(a) + u * math.sin(a))) < 1e-12
    q, k = rnd((1, 6), 2), rnd((1, 6), 3)
    dots = [float((plain.rotate_neighbours(q, torch.tensor([p + 5]), 6, 50.0) * plain.rotate_neighbours(k, torch.tensor([p]), 6, 50.0)).sum())
            for p in (0, 7, 300)]
    assert max(dots) - min(dots) < 1e-9  # scores depend on the distance alone


def test_plain_softmax_with_one_more_place_and_the_window():
    s = rnd((4, 4), 1)
    seen = torch.tril(torch.ones(4, 4, dtype=torch.bool))
    p = plain.sink_softmax(s, seen)
    for i in range(4):
        e = [math.exp(float(s[i, j])) for j in range(i + 1)]
        for j in range(4):
            assert abs(float(p[i, j]) - (e[j] / (1.0 + sum(e)) if j <= i else 0.0)) < 1e-12
    far_below = plain.sink_softmax(torch.full((1, 3), -50.0, dtype=torch.float64), torch.ones(1, 3, dtype=torch.bool))
    assert float(far_below.sum()) < 1e-20  # the extra place takes the weight: the heads' result is next to nothing
    # a window of 3 sees the token itself and the two before it
    m = window(2, 1, 4, 4, 0.5, size=3)
    w = {"p.q": rnd((8, 6), 2), "p.k": rnd((4, 6), 3), "p.v": rnd((4, 6), 4), "p.o": torch.eye(8, dtype=torch.float64),
         "p.q.b": rnd((8,), 5), "p.k.b": rnd((4,), 6), "p.v.b": rnd((4,), 7)}
    h = rnd((9, 6), 8)
    full = plain.window_mixer(h, w, "p.", m, 1e-5)
    assert torch.allclose(plain.window_mixer(h[4:], w, "p.", m, 1e-5)[2:], full[6:], atol=1e-12)  # nothing before i - 2 counts
    assert not torch.allclose(plain.window_mixer(h[5:], w, "p.", m, 1e-5)[1], full[6], atol=1e-6)  # i - 2 itself does
    # q and k are divided by their heads' root mean square: scaling a head's projection changes nothing
    w2 = dict(w)
    w2["p.q"], w2["p.q.b"] = w["p.q"].clone(), w["p.q.b"].clone()
    w2["p.q"][:4] *= 7.0
    w2["p.q.b"][:4] *= 7.0
    assert torch.allclose(plain.window_mixer(h, w2, "p.", m, 1e-12), plain.window_mixer(h, w, "p.", m, 1e-12), atol=1e-6)


def test_plain_latent_attention_written_out():
    m = latent(2, 4, 2, 3, 5, 4, 0.3, 100.0)
    w = {"p.dq": rnd((4, 6), 1), "p.dq.norm": rnd((4,), 2), "p.uq": rnd((12, 4), 3), "p.dkv": rnd((7, 6), 4),
         "p.dkv.norm": rnd((5,), 5), "p.uk": rnd((8, 5), 6), "p.uv": rnd((6, 5), 7), "p.g": rnd((2, 6), 8), "p.o": rnd((6, 6), 9)}
    h = rnd((5, 6), 10)
    got = plain.latent_mixer(h, w, "p.", m, 1e-5)
    t = 3  # one token by hand
    cq = plain.rms_norm(h[t] @ w["p.dq"].T, w["p.dq.norm"], 1e-5)
    q = (cq @ w["p.uq"].T).view(2, 6)
    heads = []
    for a in range(2):
        scores, values = [], []
        for j in range(t + 1):
            down = h[j] @ w["p.dkv"].T
            c = plain.rms_norm(down[:5], w["p.dkv.norm"], 1e-5)
            k_plain = (c @ w["p.uk"].T).view(2, 4)[a]
            k_rot = plain.rotate_neighbours(down[5:].view(1, 2), torch.tensor([j]), 2, 100.0)[0]
            q_rot = plain.rotate_neighbours(q[a, 4:].view(1, 2), torch.tensor([t]), 2, 100.0)[0]
            scores.append(float((q[a, :4] @ k_plain + q_rot @ k_rot) * 0.3))
            values.append((c @ w["p.uv"].T).view(2, 3)[a])
        p = torch.softmax(torch.tensor(scores, dtype=torch.float64), 0)
        gate = plain.sigmoid(h[t] @ w["p.g"].T)[a]
        heads.append(sum(pj * vj for pj, vj in zip(p, values)) * gate)
    assert torch.allclose(got[t], torch.cat(heads) @ w["p.o"].T, atol=1e-12)


def test_plain_router_groups_and_clamped_experts():
    z = torch.tensor([2.0, -1.0, 0.5, 0.3, 1.9, 1.0], dtype=torch.float64)
    s = plain.sigmoid(z)
    # two groups of three, one kept: group 0 is worth s0 + s2, group 1 s4 + s5: group 1 wins although expert 0 is the best
    ids, weights = plain.router_choice(z, 2, 2, 1)
    assert ids.tolist() == [4, 5] and torch.allclose(weights, s[[4, 5]] / s[[4, 5]].sum())
    ids, _ = plain.router_choice(z, 3, 2, 2)  # both kept: the three best of all
    assert ids.tolist() == [0, 4, 5]
    ids, weights = plain.router_choice(z, 1, 6, 3)  # groups of one expert: a group is worth its expert
    assert ids.tolist() == [0] and abs(float(weights[0]) - 1.0) < 1e-12
    w = {"e.gate": rnd((3, 4), 1, 3.0), "e.up": rnd((3, 4), 2, 3.0), "e.down": rnd((4, 3), 3)}
    x = rnd((1, 4), 4)
    w["e.gate"][0] = x[0] * 2.0  # one gate value far above the limit
    g, u = x @ w["e.gate"].T, x @ w["e.up"].T
    assert float(g.max()) > 1.0 and float(u.abs().max()) > 1.0  # the limits bite
    g, u = g.clamp(max=1.0), u.clamp(-1.0, 1.0)
    want = (g / (1.0 + torch.exp(-1.702 * g)) * (u + 1.0)) @ w["e.down"].T
    assert torch.allclose(plain.clamped_expert(x, w, "e.", 1.0), want, atol=1e-12)
    assert not torch.allclose(plain.clamped_expert(x, w, "e.", 50.0), want, atol=1e-3)


# -- configuration and checkpoints -------------------------------------------------------------------
def test_config_round_trip_defaults_and_faults(tmp_path):
    for which, spec in CONFIGS.items():
        cfg = BirelixConfig.from_dict(spec)
        assert BirelixConfig.from_dict(cfg.to_dict()) == cfg
        assert architecture_of(spec).name == "Birelix"
    base = CONFIGS["A"]
    cfg = BirelixConfig.from_dict(base)
    assert cfg.embedding_scale == 3.0 and cfg.layers[2].mixer.window == 19 and cfg.layers[2].mlp is None
    assert cfg.layers[0].mlp.groups == 3 and cfg.layers[0].mlp.groups_kept == 2 and cfg.layers[0].mlp.limit == 1.5

    def changed(path, value):
        import copy

        d = copy.deepcopy(base)
        at = d
        for key in path[:-1]:
            at = at[key]
        if value is None:
            del at[path[-1]]
        else:
            at[path[-1]] = value
        return d

    assert BirelixConfig.from_dict(changed(["layers", 2, "mixer", "mask"], None)).layers[2].mixer.window is None
    assert BirelixConfig.from_dict(changed(["layers", 2, "mixer", "vdim"], None)).layers[2].mixer.vdim == 24
    assert BirelixConfig.from_dict(changed(["embedding"], None)).embedding_scale == 1.0
    for path, value in ((["layers", 0, "type"], "conv"), (["layers", 2, "mixer", "kv_heads"], 4), (["layers", 0, "mlp", "router", "top"], 5),
                        (["layers", 0, "mlp", "router", "groups", "count"], 4), (["layers", 0, "mlp", "expert", "limit"], None),
                        (["layers", 1, "mixer", "rot", "dims"], 14), (["layers", 1, "mlp", "kind"], "sparse"), (["norm"], None),
                        (["layers", 3, "mixer", "conv"], 0), (["width"], 0)):
        with pytest.raises(ConfigError):
            BirelixConfig.from_dict(changed(path, value))


def test_sizes_left_to_the_checkpoint_are_read_from_its_shapes(tmp_path):
    d = make_model_dir(tmp_path, "A")
    import json

    with open(os.path.join(d, "config.json")) as f:
        spec = json.load(f)
    del spec["layers"][1]["mixer"]["kv_rank"], spec["layers"][1]["mixer"]["q_rank"], spec["layers"][0]["mixer"]["conv"]
    with open(os.path.join(d, "config.json"), "w") as f:
        json.dump(spec, f)
    cfg = load_config(d)
    assert cfg.layers[1].mixer.kv_rank == 40 and cfg.layers[1].mixer.q_rank == 24 and cfg.layers[0].mixer.conv == 3
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    tokens = random_tokens(12, 131, 1)
    cache = CacheManager(model, page_size=4, num_pages=8, max_requests=1, dtype=torch.float32, device="cpu")
    runner = ModelRunner(model, cache)
    got = runner.step([StepEntry(runner.admit(), tokens, [11])])
    assert (got[0].double() - plain_logits(d, {"a": tokens})["a"][11]).abs().max() < 1e-5
    with pytest.raises(ConfigError):  # without a checkpoint's shapes the sizes have to be said
        BirelixConfig.from_dict(spec).with_tensor_shapes({})


def test_checkpoint_faults_are_reported_together(tmp_path):
    d = make_model_dir(tmp_path, "A")
    from safetensors.torch import load_file, save_file

    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["l0.mix.A_log"]
    t["l1.mix.dq.norm"] = torch.ones(5)
    t["l2.mix.q.b"] = torch.ones(7, 2)
    t["l4.mix.norm"] = torch.ones(3)  # a window attention has no norm weights
    save_file(t, path, metadata={"format": "pt"})
    with pytest.raises(WeightError) as e:
        load_model(d, "float32", device="cpu", ops=TorchOps())
    assert all(n in str(e.value) for n in ("l0.mix.A_log", "l1.mix.dq.norm", "l2.mix.q.b", "l4.mix.norm"))


# -- the engine with substitute kernels -------------------------------------------------------------
def cpu_runner(d, page_size, num_pages, max_requests=4):
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         dtype=torch.float32, device="cpu")
    return model, cache, ModelRunner(model, cache)


def watch_layers(model, seen):
    """After every block: the residual stream with what the block leaves to be added."""
    for b in model.blocks:
        def wrapped(hidden, delta, step, layer_cache, next_norm=None, inner=b.forward):
            out = inner(hidden, delta, step, layer_cache, next_norm=next_norm)
            h = hidden.double().cpu().clone()
            if out is not None:
                h = h + (out.total() if hasattr(out, "total") else out).double().cpu()
            seen.append(h)
            return out
        b.forward = wrapped


@pytest.mark.parametrize("which", list(CONFIGS))
def test_one_layer_at_a_time_follows_the_plain_model(tmp_path, which):
    d = make_model_dir(tmp_path, which)
    sharpen(d, 3.0)
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
    sharpen(d, 3.0)
    vocab = CONFIGS[which]["vocab"]
    requests = {rid: random_tokens(n, vocab, 20 + i) for i, (rid, n) in enumerate(
        {"a": 70, "b": 45, "c": 100, "d": 33, "e": 64, "f": 1}.items())}
    tb = all_ways_trace(requests)
    out = str(tmp_path / "out")
    run_tool(d, "float32", out, tb, page_size=PAGE_SIZES[which], in_process_ops=TorchOps())
    check_dumps(out, tb, plain_logits(d, requests), 1e-4)


def test_the_states_and_the_kept_rows_share_a_row_and_are_zeroed_when_a_slot_is_used_again(tmp_path):
    d = make_model_dir(tmp_path, "A")
    sharpen(d, 3.0)
    cfg, w = read(d)
    model, cache, runner = cpu_runner(d, 4, 12, max_requests=1)
    mixer = model.blocks[0].mixer
    cols = 2 * 2 * 24 + 6 * 20
    assert mixer.state_spec().shape[0] == 6 * 20 * 24 + 2 * cols  # six matrices, then two rows of q, k and v behind three taps
    assert set(cache.states) == {0, 3}  # the two delta layers; attention keeps pages, not rows
    first, second = random_tokens(9, 131, 1), random_tokens(6, 131, 2)
    s = runner.admit()
    runner.step([StepEntry(s, first, [])])
    assert all(float(st[s].abs().max()) > 0 for st in cache.states.values())
    assert float(cache.states[0][s, 6 * 20 * 24:].abs().max()) > 0  # the kept rows behind the matrices
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
    sharpen(d, 2.0)
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


def test_a_lost_key_a_lost_place_a_lost_tap_or_a_lost_state_would_show(tmp_path):
    """The measure of the GPU traces with sharpened weights: in the plain model of such weights, a window that is
    one token short, a softmax without its extra place, a convolution without its farthest tap, or a delta state
    that forgot what came before the last 60 tokens moves the logits by far more than the 32-bit tolerance."""
    d = make_model_dir(tmp_path, "B", seed=5, dtype=torch.bfloat16)
    sharpen(d, 3.0, memory=1.6)
    cfg, w = read(d)
    tokens = random_tokens(140, cfg["vocab"], 42)
    base = plain.forward(cfg, w, tokens)
    moved = lambda other: (other - base).abs().max(dim=1).values / base.abs().max()
    import copy

    short = copy.deepcopy(cfg)
    short["layers"][2]["mixer"]["mask"]["size"] -= 1
    m = moved(plain.forward(short, w, tokens))
    assert float(m[:47].max()) == 0.0 and float(m[47:].max()) > 1e-3 and float((m[47:] > 1e-4).float().mean()) > 0.3
    kept = plain.sink_softmax
    try:
        plain.sink_softmax = lambda s, seen: torch.softmax(s.masked_fill(~seen, -math.inf), dim=-1)
        assert float((moved(plain.forward(cfg, w, tokens)) > 1e-3).float().mean()) > 0.9
    finally:
        plain.sink_softmax = kept
    w2 = dict(w)
    for name in w:
        if name.endswith(".conv"):
            w2[name] = w[name].clone()
            w2[name][:, 0] = 0.0
    assert float((moved(plain.forward(cfg, w2, tokens))[3:] > 1e-3).float().mean()) > 0.9
    only_delta = {**cfg, "layers": [l for l in cfg["layers"] if l["type"] == "delta"]}
    wd = dict(w)
    for new, old in enumerate(i for i, l in enumerate(cfg["layers"]) if l["type"] == "delta"):
        for name in w:
            if name.startswith(f"l{old}."):
                wd[f"l{new}." + name[len(f"l{old}."):]] = w[name]
    whole_run, fresh = plain.forward(only_delta, wd, tokens)[-1], plain.forward(only_delta, wd, tokens[-60:])[-1]
    assert float((whole_run - fresh).abs().max() / whole_run.abs().max()) > 1e-3
