#!/usr/bin/env python3
"""Decode and prefill throughput of the engine at Qwen3-8B layer sizes, one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--layers L] [--batch B] [--context C]

    python bench.py --dtype float32                               # the same in true 32-bit
    python bench.py --sizes 32b | --sizes 0p6b                    # the decode workload at other layer sizes
    python bench.py --workload reference-0p6b [--dtype float32]   # the reference's own benchmark shape
    python bench.py --workload mixed-32b [--layers L]             # a prompt chunk beside 63 decoded tokens
    python bench.py --workload serving                            # requests of many lengths arriving over time
    python bench.py --workload visadra [--sizes small|mid|wide]   # Visadra beside Qwen3 at equal layer sizes, kernel by kernel
    python bench.py --workload kezasun [--sizes small|mid|wide]   # Kezasun beside Visadra, kernel by kernel
    python bench.py --workload malilorn [--sizes small|mid|wide]  # Malilorn beside Kezasun, kernel by kernel
    python bench.py --workload birelix [--sizes small|mid|wide]   # Birelix beside Kezasun, kernel by kernel

A "step" is one decode step of the whole engine (scheduler, model step over the
paged cache, sampling) with `batch` live requests whose context ends at
`context` tokens.  Seeded random weights (bfloat16), uniform random token ids.
One JSON line is printed: `value` = decoded tokens per second, `prefill` = a
2048-token prompt in one step, `more` = the same measurements, shorter, of the true 32-bit
path, of the Qwen3-32B sizes and of the reference's own benchmark shape (default line only;
--no-more skips them), `roofline` = bytes the decode step has to read
(every weight it uses once + the cache of the live requests) / its time against
8 TB/s, `points` = decode at batch 1 and 64.  Both rooflines are also given against
what this machine reaches on kernels that do nothing else (`measured_peak`: a
read-only kernel over 4 GiB, a kernel of matrix instructions on registers).  The reference publishes nothing
for this configuration (its only table is Qwen3-0.6B in float32 on an unnamed
GPU, readme.md:62-66), so `vs_baseline` is null.
"""
import argparse
import json
import sys
import time

# Qwen3-8B layer sizes
SIZES = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=36, hidden_size=4096,
    num_attention_heads=32, num_key_value_heads=8, head_dim=128, intermediate_size=12288, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
)
# Qwen3-0.6B layer sizes: the model of the reference's published table (readme.md:62-66)
SIZES_0P6B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=28, hidden_size=1024,
    num_attention_heads=16, num_key_value_heads=8, head_dim=128, intermediate_size=3072, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=True,
)
# Qwen3-32B layer sizes
SIZES_32B = dict(
    architectures=["Qwen3ForCausalLM"], model_type="qwen3", num_hidden_layers=64, hidden_size=5120,
    num_attention_heads=64, num_key_value_heads=8, head_dim=128, intermediate_size=25600, vocab_size=151936,
    rope_theta=1000000.0, rms_norm_eps=1e-6, tie_word_embeddings=False,
)
REFERENCE_TOK_S = 189.06  # readme.md:66: 32 requests x 64 new tokens, paged batch kernel, FP32, an unnamed CUDA GPU
HBM_PEAK = 8.0e12  # bytes/s
MFMA_PEAK = {"bf16": 2.5e15, "fp32": 157.3e12}
PAGE_SIZE = 16
PREFILL_TOKENS = 2048


def weight_bytes_per_step(cfg, elem=2):
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h  # qkv
    per_layer += h * cfg.num_attention_heads * d  # o
    per_layer += 3 * h * cfg.intermediate_size  # gate, up, down
    per_layer += 2 * h + 2 * d  # norms
    return (per_layer * cfg.num_hidden_layers + h + cfg.vocab_size * h) * elem


def kv_bytes_per_token(cfg, elem=2):
    return 2 * cfg.num_key_value_heads * cfg.head_dim * cfg.num_hidden_layers * elem


def prefill_flops(cfg, tokens):
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h + h * cfg.num_attention_heads * d
    per_layer += 3 * h * cfg.intermediate_size
    linear = 2.0 * tokens * per_layer * cfg.num_hidden_layers + 2.0 * cfg.vocab_size * h  # head: one row
    attention = 4.0 * cfg.num_attention_heads * d * (tokens * (tokens + 1) / 2) * cfg.num_hidden_layers
    return linear + attention


def make_engine(model, batch, context, max_tokens_per_step=8192):
    from litellmengine_amd.engine import LLMEngine

    pages_each = (context + PAGE_SIZE - 1) // PAGE_SIZE + 1
    return LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_each * batch, max_requests=batch,
                     max_tokens_per_step=max_tokens_per_step, prefill_chunk=2048, max_pages_per_request=pages_each)


def vocab_of(cfg):
    return cfg.vocab_size if hasattr(cfg, "vocab_size") else cfg.vocab


def random_prompts(n, length, vocab, seed):
    import torch

    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n, length), generator=g).tolist()


def time_decode(model, cfg, batch, context, steps, warmup):
    """`steps` timed decode steps of `batch` requests; the last one runs at a
    attends to `context` keys.  Returns seconds per step."""
    import torch

    engine = make_engine(model, batch, context)
    prompt_len = context - (steps + warmup)
    for p in random_prompts(batch, prompt_len, vocab_of(cfg), 100 + batch):
        engine.prefill(engine.add_request(p, steps + warmup + 1))  # each prompt alone, in portions
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    lens = [r.cached_len for r in engine.scheduler.requests.values()]
    assert all(n == context for n in lens), lens
    return dt


def time_prefill(model, cfg, tokens, repeats=3):
    import torch

    engine = make_engine(model, 1, tokens + 16, max_tokens_per_step=tokens)
    best = None
    for i in range(repeats + 1):
        req = engine.add_request(random_prompts(1, tokens, vocab_of(cfg), 7 + i)[0], 1)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        engine.step()  # the whole prompt in one step, one token drawn
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert req.finished and engine.num_steps == i + 1
        if i > 0:  # the first run warms up
            best = dt if best is None else min(best, dt)
    return best


def measure_peaks(dtype):
    """What this machine reaches on kernels that do nothing else: (bytes/s of a kernel that only
    reads 4 GiB from HBM, flops/s of a kernel that only issues matrix instructions of `dtype`
    on registers).  The rooflines are given against the published peaks and against these."""
    import torch

    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()

    def timed(launch, repeats=8):
        # by the wall clock around a run of launches (no timing events: recording one makes the runtime
        # keep time stamps of every later launch of the process, which costs the short kernels of a
        # decode step about a microsecond each)
        launch()
        torch.cuda.synchronize()
        best = None
        for _ in range(3):
            t0 = time.perf_counter()
            for _ in range(repeats):
                launch()
            torch.cuda.synchronize()
            dt = (time.perf_counter() - t0) / repeats
            best = dt if best is None else min(best, dt)
        return best

    data = torch.empty(1 << 30, dtype=torch.int32, device="cuda")  # 4 GiB: far more than the caches hold
    data.fill_(1)
    nbytes = data.numel() * 4
    read = max(nbytes / timed(lambda b=b: ops.probe_read_stream(data, b)) for b in (256, 16384, 65536))
    del data
    torch.cuda.empty_cache()
    tdtype = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    units = torch.cuda.get_device_properties(0).multi_processor_count
    flops = [0.0]

    def mfma():
        flops[0] = ops.probe_mfma(tdtype, 8 * units, 4000)

    seconds = timed(mfma, repeats=2)
    return read, flops[0] / seconds


def flat_config(cfg, full_layers, **more):
    d = {"layers": cfg.num_hidden_layers, "layers_of_full_model": full_layers, "hidden": cfg.hidden_size,
         "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
         "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "page_size": PAGE_SIZE,
         "parallelism": "none (1 GPU)"}
    d.update(more)
    return d


def time_reference_workload(dtype, runs, warmup):
    """The shape of the reference's benchmark (src/benchmark/generation_benchmark.cpp:259-315,
    :430-526): 32 requests, 64-token prompts, 64 new tokens each, greedy; warm-up runs, then
    the whole run is timed, prompts included.  Returns (config, requests, prompt length, new
    tokens, seconds a run)."""
    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.engine import LLMEngine
    from litellmengine_amd.models import random_model

    cfg = Qwen3Config.from_dict(SIZES_0P6B)
    model = random_model(cfg, seed=0, dtype=dtype)
    requests, prompt_len, new_tokens = 32, 64, 64
    pages_each = (prompt_len + new_tokens + PAGE_SIZE - 1) // PAGE_SIZE + 1
    engine = LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_each * requests, max_requests=requests,
                       max_tokens_per_step=requests * prompt_len, max_pages_per_request=pages_each)
    times = []
    for run in range(warmup + runs):
        prompts = random_prompts(requests, prompt_len, cfg.vocab_size, 1000 + run)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        out = engine.generate(prompts, new_tokens)
        torch.cuda.synchronize()
        dt = time.perf_counter() - t0
        assert all(len(o) == new_tokens for o in out)
        if run >= warmup:
            times.append(dt)
    return cfg, requests, prompt_len, new_tokens, sum(times) / len(times)


def reference_workload(args):
    cfg, requests, prompt_len, new_tokens, dt = time_reference_workload(args.dtype, args.steps, args.warmup)
    value = requests * new_tokens / dt
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": "new tok/s of 32 requests x 64-token prompts x 64 new tokens, prompts included, Qwen3-0.6B sizes",
        "value": round(value, 2), "unit": "tok/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": round(value / REFERENCE_TOK_S, 2), "dtype": short,
        "data": "synthetic: seeded random weights, uniform random token ids; the reference's 189.06 tok/s is FP32 "
                "on an unnamed CUDA GPU with a real checkpoint and one text prompt",
        "config": flat_config(cfg, SIZES_0P6B["num_hidden_layers"], model="Qwen3-0.6B sizes (random weights)",
                              global_batch=requests, seq_len=prompt_len + new_tokens, new_tokens=new_tokens),
    }))
    return 0


def mixed_workload(args):
    """One 2048-token portion of a long prompt beside 63 decoded tokens at context 4096,
    Qwen3-32B layer sizes: the step a serving loop runs while a prompt comes in."""
    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.models import random_model

    layers = args.layers if args.layers != SIZES["num_hidden_layers"] else SIZES_32B["num_hidden_layers"]
    cfg = Qwen3Config.from_dict(dict(SIZES_32B, num_hidden_layers=layers))
    model = random_model(cfg, seed=0, dtype=args.dtype)
    decoders, context, chunk = 63, 4096, PREFILL_TOKENS
    steps, warmup = args.steps, args.warmup
    long_prompt = chunk * (steps + warmup)
    pages_dec = (context + PAGE_SIZE - 1) // PAGE_SIZE + 1
    pages_long = (long_prompt + PAGE_SIZE - 1) // PAGE_SIZE + 2
    from litellmengine_amd.engine import LLMEngine

    engine = LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_dec * decoders + pages_long,
                       max_requests=decoders + 1, max_tokens_per_step=chunk + decoders, prefill_chunk=chunk,
                       max_pages_per_request=max(pages_dec, pages_long))
    prompt_len = context - (steps + warmup)
    for p in random_prompts(decoders, prompt_len, cfg.vocab_size, 300):
        engine.prefill(engine.add_request(p, steps + warmup + 1))
    long_req = engine.add_request(random_prompts(1, long_prompt, cfg.vocab_size, 301)[0], 1)
    for _ in range(warmup):
        engine.step()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        engine.step()
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / steps
    assert long_req.finished and long_req.cached_len == long_prompt, (long_req.cached_len, long_prompt)
    lens = [r.cached_len for r in engine.scheduler.requests.values() if r is not long_req]
    assert all(n == context for n in lens), lens
    tokens = chunk + decoders
    h, d = cfg.hidden_size, cfg.head_dim
    per_layer = (cfg.num_attention_heads + 2 * cfg.num_key_value_heads) * d * h + h * cfg.num_attention_heads * d
    per_layer += 3 * h * cfg.intermediate_size
    past_mean = chunk * (warmup + (steps - 1) / 2.0)  # keys before the timed portions, on average
    attn = 4.0 * cfg.num_attention_heads * d * (chunk * past_mean + chunk * (chunk + 1) / 2 + decoders * context)
    flops = (2.0 * tokens * per_layer + attn) * cfg.num_hidden_layers + 2.0 * (decoders + 1) * cfg.vocab_size * h
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": "tokens/s of a mixed step: a 2048-token prompt portion beside 63 decoded tokens at context 4096, "
                  "Qwen3-32B sizes",
        "value": round(tokens / dt, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": round(dt * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: seeded random weights, uniform random token ids",
        "config": flat_config(cfg, SIZES_32B["num_hidden_layers"], model="Qwen3-32B sizes (random weights)",
                              global_batch=decoders + 1, seq_len=context, prompt_portion=chunk),
        "roofline": {"bound": "mfma", "achieved": round(flops / dt / 1e12, 1), "peak": MFMA_PEAK[short] / 1e12,
                     "unit": "TFLOP/s", "frac": round(flops / dt / MFMA_PEAK[short], 4)},
    }))
    return 0


def serving_workload(args):
    """Requests of many lengths arriving over time, through the engine's own scheduler, at the
    Qwen3-8B layer sizes: 200 requests, prompts of 30 to 3050 tokens, 16 to 256 new tokens each,
    one arriving every second step, at most 64 live, a budget of 2048 tokens a step.  The whole run
    is timed (prompt portions beside decoded tokens, graph captures included); all tokens / time."""
    import collections
    import random

    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.engine import LLMEngine
    from litellmengine_amd.models import random_model

    cfg = Qwen3Config.from_dict(dict(SIZES, num_hidden_layers=args.layers))
    model = random_model(cfg, seed=0, dtype=args.dtype)
    rng = random.Random(5)
    requests, live, every = 200, 64, 2
    sizes = [(rng.choice([30, 100, 300, 700, 1500, 3000]) + rng.randint(0, 50), rng.choice([16, 64, 128, 256]))
             for _ in range(requests)]
    longest = max(p + g for p, g in sizes)
    pages_each = (longest + PAGE_SIZE - 1) // PAGE_SIZE + 1
    engine = LLMEngine(model, page_size=PAGE_SIZE, num_pages=pages_each * live, max_requests=live,
                       max_tokens_per_step=PREFILL_TOKENS, max_pages_per_request=pages_each)
    todo = [(random_prompts(1, p, cfg.vocab_size, 100 + i)[0], g) for i, (p, g) in enumerate(sizes)]
    kinds = collections.defaultdict(lambda: [0, 0.0])  # kind -> steps, seconds, then the tokens of every such step
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    steps = 0
    while todo or engine.has_work():
        if todo and steps % every == 0:
            prompt, new = todo.pop(0)
            engine.add_request(prompt, new)
        before = sum(r.cached_len for r in engine.scheduler.requests.values())
        captures, graph_steps = engine.runner.num_captures, engine.runner.num_graph_steps
        ts = time.perf_counter()
        engine.step()
        torch.cuda.synchronize()
        dt = time.perf_counter() - ts
        ran = sum(r.cached_len for r in engine.scheduler.requests.values()) - before
        kind = ("capture" if engine.runner.num_captures > captures else
                "decode_only_graph" if engine.runner.num_graph_steps > graph_steps else
                "le64" if ran <= 64 else "le256" if ran <= 256 else "le1024" if ran <= 1024 else "gt1024")
        kinds[kind][0] += 1
        kinds[kind][1] += dt
        kinds[kind].append(ran)
        steps += 1
    total = time.perf_counter() - t0
    new_tokens = sum(g for _, g in sizes)
    all_tokens = sum(p + g for p, g in sizes)
    short = "bf16" if args.dtype == "bfloat16" else "fp32"
    print(json.dumps({
        "metric": "tokens/s, prompts included, of 200 requests (prompts of 30-3050 tokens, 16-256 new tokens) "
                  "arriving one every second step, at most 64 live, Qwen3-8B sizes",
        "value": round(all_tokens / total, 1), "unit": "tok/s", "n_gpus": 1, "steps": steps, "warmup": 0,
        "ms_per_step": round(total / steps * 1e3, 3), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": short, "data": "synthetic: seeded random weights, uniform random token ids, seeded lengths",
        "config": flat_config(cfg, SIZES["num_hidden_layers"], model="Qwen3-8B sizes (random weights)",
                              global_batch=live, requests=requests, token_budget=PREFILL_TOKENS),
        "new_tokens_per_s": round(new_tokens / total, 1), "seconds": round(total, 3),
        "graph_captures": engine.runner.num_captures,
        "steps_by_tokens": {k: {"steps": v[0], "ms_each": round(v[1] / v[0] * 1e3, 2), "share": round(v[1] / total, 3),
                                "tokens_each": round(sum(v[2:]) / v[0], 1)}
                            for k, v in sorted(kinds.items())},
    }))
    return 0


def more_workloads(steps, warmup):
    """What else the default line carries, each measured like the headline but shorter: the true
    32-bit path at the Qwen3-8B sizes (decode at batch 8, a 2048-token prompt), decode at batch 8
    at the Qwen3-32B sizes, and the reference's own benchmark shape at the Qwen3-0.6B sizes.
    Flat: numbers, and for each workload one string that names its sizes."""
    import gc

    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.models import random_model

    def sizes_of(cfg, what):
        return (f"{what}: {cfg.num_hidden_layers} layers, hidden {cfg.hidden_size}, {cfg.num_attention_heads}/"
                f"{cfg.num_key_value_heads} heads of {cfg.head_dim}, intermediate {cfg.intermediate_size}, vocab "
                f"{cfg.vocab_size}, page {PAGE_SIZE}, random weights")

    def free():
        gc.collect()
        torch.cuda.empty_cache()

    more = {}
    steps, warmup = max(4, min(steps, 10)), max(1, min(warmup, 2))
    cfg = Qwen3Config.from_dict(SIZES)
    model = random_model(cfg, seed=0, dtype="float32")
    dt = time_decode(model, cfg, 8, 4096, steps, warmup)
    step_bytes = weight_bytes_per_step(cfg, 4) + 8 * (4096 - (steps - 1) / 2.0) * kv_bytes_per_token(cfg, 4)
    pt = time_prefill(model, cfg, PREFILL_TOKENS, repeats=1)
    more.update({
        "fp32_8b": sizes_of(cfg, "true 32-bit path, Qwen3-8B sizes, decode batch 8 at context 4096 and a 2048-token prompt"),
        "fp32_8b_decode_b8_tok_s": round(8 / dt, 2), "fp32_8b_decode_b8_ms": round(dt * 1e3, 3),
        "fp32_8b_decode_b8_hbm_frac": round(step_bytes / dt / HBM_PEAK, 4),
        "fp32_8b_prefill_tok_s": round(PREFILL_TOKENS / pt, 1), "fp32_8b_prefill_ms": round(pt * 1e3, 2),
        "fp32_8b_prefill_frac": round(prefill_flops(cfg, PREFILL_TOKENS) / pt / MFMA_PEAK["fp32"], 4),
    })
    del model
    free()
    cfg = Qwen3Config.from_dict(SIZES_32B)
    model = random_model(cfg, seed=0, dtype="bfloat16")
    dt = time_decode(model, cfg, 8, 4096, steps, warmup)
    step_bytes = weight_bytes_per_step(cfg, 2) + 8 * (4096 - (steps - 1) / 2.0) * kv_bytes_per_token(cfg, 2)
    more.update({
        "bf16_32b": sizes_of(cfg, "Qwen3-32B sizes, bf16, decode batch 8 at context 4096"),
        "bf16_32b_decode_b8_tok_s": round(8 / dt, 2), "bf16_32b_decode_b8_ms": round(dt * 1e3, 3),
        "bf16_32b_decode_b8_hbm_frac": round(step_bytes / dt / HBM_PEAK, 4),
    })
    del model
    free()
    cfg, requests, prompt_len, new_tokens, dt = time_reference_workload("bfloat16", 3, 1)
    more.update({
        "bf16_0p6b_reference_shape": sizes_of(cfg, f"Qwen3-0.6B sizes, bf16, {requests} requests x {prompt_len}-token prompts x "
                                              f"{new_tokens} new tokens, prompts included (the shape of the reference's "
                                              f"{REFERENCE_TOK_S} tok/s, which is FP32 on an unnamed CUDA GPU)"),
        "bf16_0p6b_reference_shape_tok_s": round(requests * new_tokens / dt, 1),
        "bf16_0p6b_reference_shape_ms": round(dt * 1e3, 2),
    })
    free()
    return more


# ---------------------------------------------------------------------------------------------
# Visadra (minGRU and latent-attention mixers, dense and routed feed-forwards) beside Qwen3 at
# equal layer sizes: whole-model prefill and decode, and every kernel of its own beside the like
# kernel of Qwen3, each against its roofline (bytes it must move at 8 TB/s, or flops at 2.5 PFLOP/s,
# whichever takes longer).
# ---------------------------------------------------------------------------------------------
VISADRA_SIZES = {
    # width, heads, dim, rot, vdim, rank, minGRU width, dense ff, experts, top, expert ff, shared ff
    "small": (1024, 8, 64, 32, 64, 256, 1536, 4096, 16, 2, 512, 1024),
    "mid": (2048, 16, 128, 64, 128, 512, 3072, 8192, 64, 6, 1408, 2816),
    "wide": (4096, 32, 128, 64, 128, 512, 6144, 12288, 64, 6, 2048, 4096),
}


def visadra_configs(which, groups):
    """(Visadra config, Qwen3 config of equal width, depth, head count and dense feed-forward)."""
    from litellmengine_amd.config import Qwen3Config, VisadraConfig

    W, H, dim, rot, vdim, rank, gw, ff, E, top, eff, sff = VISADRA_SIZES[which]
    att = {"heads": H, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": (dim + rot) ** -0.5,
           "rot": {"base": 10000.0, "dims": rot}}
    moe = {"kind": "moe", "router": {"experts": E, "top": top}, "expert": {"ff": eff}, "shared": {"ff": sff}}
    dense = {"kind": "dense", "ff": ff}
    four = [{"type": "latent_attention", "mixer": att, "mlp": dense}, {"type": "mingru", "mixer": {"width": gw}, "mlp": moe},
            {"type": "mingru_2", "mixer": {"width": gw}, "mlp": dense}, {"type": "latent_attention", "mixer": att, "mlp": moe}]
    v = VisadraConfig.from_dict({"architecture": "Visadra", "vocab": 32768, "width": W, "embedding": {"scale": 1.0},
                                 "logit_scale": 1.0, "norm": {"eps": 1e-6}, "layers": four * groups})
    q = Qwen3Config.from_dict(dict(SIZES, num_hidden_layers=4 * groups, hidden_size=W, num_attention_heads=H,
                                   num_key_value_heads=max(1, H // 4), head_dim=128, intermediate_size=ff, vocab_size=32768))
    return v, q


def timed_launches(launch, repeats=20):
    import torch

    launch()
    torch.cuda.synchronize()
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        for _ in range(repeats):
            launch()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / repeats
        best = dt if best is None else min(best, dt)
    return best


def visadra_kernels(which):
    """Each kernel of Visadra's own at two shapes (a 2048-token prompt; 8 decoded tokens after 4096) beside
    the like kernel of Qwen3 at equal sizes: microseconds and the share of its roofline."""
    import torch

    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()
    W, H, dim, rot, vdim, rank, gw, ff, E, top, eff, sff = VISADRA_SIZES[which]
    dev, bf = "cuda", torch.bfloat16
    P = PAGE_SIZE
    rnd = lambda *shape, dtype=bf, scale=1.0: (torch.randn(shape, device=dev) * scale).to(dtype)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=dev)
    out = {}

    def entry(name, seconds, flops, nbytes, like=None):
        floor = max(flops / MFMA_PEAK["bf16"], nbytes / HBM_PEAK)
        e = {"us": round(seconds * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "frac": round(floor / seconds, 4),
             "bound": "mfma" if flops / MFMA_PEAK["bf16"] > nbytes / HBM_PEAK else "hbm"}
        if like is not None:
            e["like"] = like
            e["times_farther_from_roofline"] = round(like["frac"] / e["frac"], 2) if e["frac"] > 0 else None
        out[name] = e
        return e

    for shape, S, q_len, past in (("prefill_2048", 1, 2048, 0), ("decode_b8_ctx4096", 8, 1, 4095)):
        N, kv = S * q_len, past + q_len
        pages_each = -(-kv // P)
        table = torch.arange(S * pages_each, dtype=torch.int32, device=dev).view(S, pages_each).contiguous()
        seq_slots, cu = ints(list(range(S))), ints([i * q_len for i in range(S + 1)])
        kv_lens = ints([kv] * S)
        token_seq = ints([i // q_len for i in range(N)])
        visible = S * (q_len * past + q_len * (q_len + 1) / 2)  # (query, key) pairs
        # latent attention beside grouped-query attention
        lat_pages = rnd(S * pages_each + 1, P * (2 * rank + rot))
        q_lat, q_rot = rnd(H, N, rank, scale=0.1).transpose(0, 1), rnd(N, H, rot, dtype=torch.float32, scale=0.1)
        sink = torch.zeros(H, device=dev)
        t = timed_launches(lambda: ops.latent_attention(q_lat, q_rot, lat_pages, P, rank, rot, table, seq_slots, cu, kv_lens,
                                                        token_seq, sink, None, 0.1, q_len, kv, bf))
        nkv, d = max(1, H // 4), 128
        kv_layer = rnd(S * pages_each + 1, 2, nkv, P, d)
        q = rnd(N, H, d, scale=0.1)
        tq = timed_launches(lambda: ops.paged_attention(q, kv_layer, table, seq_slots, cu, kv_lens, token_seq, None, 0.1,
                                                        q_len, q_len, kv))
        like = entry(f"{shape}/paged_attention (Qwen3)", tq, 4.0 * H * d * visible, 2.0 * (S * kv * 2 * nkv * d + 2 * N * H * d))
        entry(f"{shape}/latent_attention", t, 2.0 * H * (2 * rank + rot) * visible,
              2.0 * (S * kv * (2 * rank + rot) + 2 * N * H * rank), dict(like, name="paged_attention"))
        # the latents' and keys' way into the pages
        dkv, nw = rnd(N, rank + rot), torch.ones(rank, device=dev, dtype=bf)
        cos_sin = ops.rope_table(ints([past + i % q_len for i in range(N)]), torch.ones(rot // 2, device=dev))
        slots = ints([int(table[i // q_len, (past + i % q_len) // P]) * P + (past + i % q_len) % P for i in range(N)]) if N <= 64 else \
            (table.long()[:, : pages_each].repeat_interleave(P, 1)[:, past:kv] * P + torch.arange(past, kv, device=dev) % P).reshape(-1).int()
        t = timed_launches(lambda: ops.latent_kv_write(dkv, nw, 1e-6, cos_sin, rot, slots, lat_pages, P, rank, rot))
        qkv = rnd(N, (H + 2 * nkv) * d)
        cs2 = ops.rope_table(ints([past + i % q_len for i in range(N)]), torch.ones(d // 2, device=dev))
        one = torch.ones(d, device=dev, dtype=bf)
        tq = timed_launches(lambda: ops.qk_norm_rope_write(qkv, slots, one, one, cs2, d, 1e-6, kv_layer, H, nkv, d))
        like = entry(f"{shape}/qk_norm_rope_write (Qwen3)", tq, 0, 2.0 * N * (2 * H + 4 * nkv) * d)
        entry(f"{shape}/latent_kv_write", t, 0, 2.0 * N * (3 * rank + 2 * rot), dict(like, name="qk_norm_rope_write"))
        # the recurrence: nothing like it in Qwen3; beside the residual add + norm, which moves rows as it does
        zxg, bias = rnd(N, 3 * gw, dtype=torch.float32), torch.zeros(gw, device=dev)
        state = torch.zeros(S + 1, gw, device=dev)
        t = timed_launches(lambda: ops.mingru_scan(zxg, bias, bias, state, seq_slots, cu, bf, q_len))
        hidden, delta, w = rnd(N, W, dtype=torch.float32), rnd(N, W), torch.ones(W, device=dev, dtype=bf)
        tq = timed_launches(lambda: ops.add_rmsnorm(hidden, delta, w, 1e-6, bf))
        like = entry(f"{shape}/add_rmsnorm (Qwen3)", tq, 0, N * W * (4 + 4 + 2 + 2.0))
        entry(f"{shape}/mingru_scan", t, 0, N * gw * (12 + 2.0), dict(like, name="add_rmsnorm"))
        t = timed_launches(lambda: ops.rmsnorm_add(hidden, delta, w, 1e-6, bf))
        entry(f"{shape}/rmsnorm_add", t, 0, N * W * (4 + 4 + 2 + 2.0), dict(like, name="add_rmsnorm"))
        # the routed experts beside the dense gated feed-forward (its two products and the activation)
        x = rnd(N, W, scale=0.1)
        gate_up, down = rnd(E, 2 * eff, W, scale=0.02), rnd(E, W, eff, scale=0.02)
        ids, gains = ops.moe_route(rnd(N, E, dtype=torch.float32), torch.zeros(E, device=dev), top)
        t = timed_launches(lambda: ops.moe_experts(x, ids, gains, gate_up, down), repeats=5)
        used = min(E, N * top)
        wgu, wd = rnd(2 * ff, W, scale=0.02), rnd(W, ff, scale=0.02)
        tq = timed_launches(lambda: ops.linear(ops.gate_up_silu(x, wgu), wd), repeats=5)
        like = entry(f"{shape}/gated feed-forward (Qwen3)", tq, 6.0 * N * W * ff, 2.0 * (3 * W * ff + 2 * N * W))
        entry(f"{shape}/moe_experts", t, 6.0 * N * top * W * eff, 2.0 * (3 * used * W * eff + 2 * N * W),
              dict(like, name="gated feed-forward"))
        del lat_pages, kv_layer
    return out


def visadra_workload(args):
    import torch

    from litellmengine_amd.models import random_model

    which = args.sizes if args.sizes in VISADRA_SIZES else "mid"
    groups = max(1, args.layers // 4) if args.layers != SIZES["num_hidden_layers"] else 2
    vcfg, qcfg = visadra_configs(which, groups)
    line = {"metric": f"Visadra beside Qwen3 at equal layer sizes ({which}): prefill tok/s @ 2048 and decode tok/s @ batch "
                      f"{args.batch}, context {args.context}", "unit": "tok/s", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic: seeded random weights, uniform random token ids", "higher_is_better": True,
            "config": {"sizes": dict(zip(("width", "heads", "dim", "rot_dim", "vdim", "kv_rank", "mingru_width", "dense_ff",
                                          "experts", "top", "expert_ff", "shared_ff"), VISADRA_SIZES[which])),
                       "layers": 4 * groups, "pattern": "latent+dense, mingru+moe, mingru+dense, latent+moe"}}
    steps, warmup = min(args.steps, 16), min(args.warmup, 4)
    for name, cfg in (("visadra", vcfg), ("qwen3", qcfg)):
        model = random_model(cfg, seed=0, dtype="bfloat16")
        dt = time_decode(model, cfg, args.batch, args.context, steps, warmup)
        pt = time_prefill(model, cfg, PREFILL_TOKENS)
        line[name] = {"decode_tok_s": round(args.batch / dt, 1), "decode_ms_per_step": round(dt * 1e3, 3),
                      "prefill_tok_s": round(PREFILL_TOKENS / pt, 1), "prefill_ms": round(pt * 1e3, 3)}
        del model
        torch.cuda.empty_cache()
    line["value"] = line["visadra"]["decode_tok_s"]
    line["steps"], line["warmup"] = steps, warmup
    line["kernels"] = visadra_kernels(which)
    print(json.dumps(line))
    return 0


KEZASUN_SIZES = {
    # width, wkv heads, wkv dim, decay rank, q heads, kv heads, dim, vdim, rotated, window, experts, identity, top, expert ff, groups, kept
    "small": (1024, 16, 64, 32, 8, 2, 128, 128, 64, 1024, 16, 4, 4, 512, 4, 2),
    "mid": (2048, 32, 64, 64, 16, 4, 128, 128, 64, 2048, 64, 8, 6, 1408, 8, 4),
    "wide": (4096, 64, 64, 64, 32, 8, 128, 128, 64, 4096, 64, 8, 6, 2048, 8, 4),
}


def kezasun_config(which, groups):
    from litellmengine_amd.config import KezasunConfig

    W, wh, wd, rank, H, G, dim, vdim, rot, window, E, I, top, eff, ng, keep = KEZASUN_SIZES[which]
    att = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "mask": {"size": window},
           "rot": {"base": 250000.0, "dims": rot, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}}
    moe = {"kind": "moe", "expert": {"ff": eff},
           "router": {"experts": E, "identity": I, "top": top, "groups": {"count": ng, "keep": keep}}}
    rec = {"heads": wh, "dim": wd, "decay_rank": rank}
    layers = []
    for g in range(groups):
        layers += [{"type": "wkv", "mixer": rec, "mlp": moe}, {"type": "attention", "mixer": att, "mlp": moe},
                   {"type": "wkv", "mixer": rec, "mlp": moe},
                   {"type": "attention", "mixer": dict(att, kv_from=4 * g + 1), "mlp": moe}]
    return KezasunConfig.from_dict({"architecture": "Kezasun", "vocab": 32768, "width": W, "residual_mult": 0.3,
                                    "norm": {"eps": 1e-6}, "layers": layers})


def kezasun_kernels(which):
    """Each kernel of Kezasun's own at two shapes (a 2048-token prompt; 8 decoded tokens after 4096) beside the
    like kernel of Visadra (the closest model: a recurrence, attention with a sink, routed experts) at its
    sizes of the same name: microseconds and the share of its roofline."""
    import torch

    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()
    W, wh, wd, rank, H, G, dim, vdim, rot, window, E, I, top, eff, ng, keep = KEZASUN_SIZES[which]
    VW, VH, vdim_k, vrot, vvdim, vrank, gw, vff, VE, vtop, veff, vsff = VISADRA_SIZES[which]
    dev, bf = "cuda", torch.bfloat16
    P = PAGE_SIZE
    rnd = lambda *shape, dtype=bf, scale=1.0: (torch.randn(shape, device=dev) * scale).to(dtype)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=dev)
    out = {}

    def entry(name, seconds, flops, nbytes, like=None):
        floor = max(flops / MFMA_PEAK["bf16"], nbytes / HBM_PEAK)
        e = {"us": round(seconds * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "frac": round(floor / seconds, 4),
             "bound": "mfma" if flops / MFMA_PEAK["bf16"] > nbytes / HBM_PEAK else "hbm"}
        if like is not None:
            e["like"] = like
            e["times_farther_from_roofline"] = round(like["frac"] / e["frac"], 2) if e["frac"] > 0 else None
        out[name] = e
        return e

    for shape, S, q_len, past in (("prefill_2048", 1, 2048, 0), ("decode_b8_ctx4096", 8, 1, 4095)):
        N, kv = S * q_len, past + q_len
        pages_each = -(-kv // P)
        table = torch.arange(S * pages_each, dtype=torch.int32, device=dev).view(S, pages_each).contiguous()
        seq_slots, cu = ints(list(range(S))), ints([i * q_len for i in range(S + 1)])
        kv_lens = ints([kv] * S)
        token_seq = ints([i // q_len for i in range(N)])
        positions = ints([past + i % q_len for i in range(N)])
        slots = (table.long().repeat_interleave(P, 1)[:, past:kv] * P + torch.arange(past, kv, device=dev) % P).reshape(-1).int()
        # attention over a window with a sink beside latent attention with a sink
        seen = sum(min(window, past + i + 1) for i in range(q_len)) * S  # (query, key) pairs inside the window
        D = -(-max(dim, vdim) // 32) * 32
        kv_layer = rnd(S * pages_each + 1, 2, G, P, D)
        q = rnd(N, H, D, scale=0.1)
        sinks = torch.zeros(H, device=dev)
        t = timed_launches(lambda: ops.paged_attention(q, kv_layer, table, seq_slots, cu, kv_lens, token_seq, window, 0.1,
                                                       q_len, q_len, kv, sinks=sinks))
        lat_pages = rnd(S * pages_each + 1, P * (2 * vrank + vrot))
        q_lat, q_rot = rnd(VH, N, vrank, scale=0.1).transpose(0, 1), rnd(N, VH, vrot, dtype=torch.float32, scale=0.1)
        vsink = torch.zeros(VH, device=dev)
        tv = timed_launches(lambda: ops.latent_attention(q_lat, q_rot, lat_pages, P, vrank, vrot, table, seq_slots, cu, kv_lens,
                                                         token_seq, vsink, None, 0.1, q_len, kv, bf))
        visible = S * (q_len * past + q_len * (q_len + 1) / 2)
        like = entry(f"{shape}/latent_attention (Visadra)", tv, 2.0 * VH * (2 * vrank + vrot) * visible,
                     2.0 * (S * kv * (2 * vrank + vrot) + 2 * N * VH * vrank))
        keys_read = S * min(kv, window + q_len - 1)
        entry(f"{shape}/paged_attention, window and sink", t, 4.0 * H * D * seen, 2.0 * (keys_read * 2 * G * D + 2 * N * H * D),
              dict(like, name="latent_attention"))
        # norm over the whole projection, rotation and the cache write beside the latents' way into the pages
        cols = H * dim + G * (dim + vdim) + H
        qkv, bias = rnd(N, cols), rnd(cols)
        qw, kw = torch.ones(H * dim, device=dev), torch.ones(G * dim, device=dev)
        cos_sin = ops.rope_table(positions, torch.ones(rot // 2, device=dev))
        t = timed_launches(lambda: ops.proj_norm_rope_write(qkv, bias, slots, qw, kw, cos_sin, rot, 1e-6, kv_layer, H, G, dim, vdim))
        dkv, nw = rnd(N, vrank + vrot), torch.ones(vrank, device=dev, dtype=bf)
        cs2 = ops.rope_table(positions, torch.ones(vrot // 2, device=dev))
        tv = timed_launches(lambda: ops.latent_kv_write(dkv, nw, 1e-6, cs2, vrot, slots, lat_pages, P, vrank, vrot))
        like = entry(f"{shape}/latent_kv_write (Visadra)", tv, 0, 2.0 * N * (3 * vrank + 2 * vrot))
        entry(f"{shape}/proj_norm_rope_write", t, 0, 2.0 * N * (cols + H * D + 2 * G * D), dict(like, name="latent_kv_write"))
        a = rnd(N, H * D)
        t = timed_launches(lambda: ops.head_gate(a, qkv, cols - H, H, vdim))
        entry(f"{shape}/head_gate", t, 0, 2.0 * N * (H * D + H * vdim), dict(like, name="latent_kv_write"))
        # the recurrence with a matrix state beside the gated recurrence
        HD = wh * wd
        r, k, v, wraw = (rnd(N, HD, dtype=torch.float32, scale=0.5) for _ in range(4))
        w0 = u = torch.zeros(HD, device=dev)
        g, x = rnd(N, HD), rnd(N, W)
        state = torch.zeros(S + 1, HD * wd + W, device=dev)
        t = timed_launches(lambda: ops.wkv_scan(r, k, v, wraw, w0, u, g, torch.ones(HD, device=dev), 1e-6, x, state, wh, wd,
                                                seq_slots, cu, bf, q_len))
        zxg, zb = rnd(N, 3 * gw, dtype=torch.float32), torch.zeros(gw, device=dev)
        vstate = torch.zeros(S + 1, gw, device=dev)
        tv = timed_launches(lambda: ops.mingru_scan(zxg, zb, zb, vstate, seq_slots, cu, bf, q_len))
        like = entry(f"{shape}/mingru_scan (Visadra)", tv, 0, N * gw * (12 + 2.0))
        # 4 flops per state element and token (decay and outer product, read-out with the bonus); the state itself is
        # read and written once per request
        entry(f"{shape}/wkv_scan", t, 0, N * HD * (16 + 2 + 2.0) + 2.0 * S * HD * wd * 4, dict(like, name="mingru_scan"))
        out[f"{shape}/wkv_scan"]["fp32_flops_T"] = round(6.0 * N * HD * wd / t / 1e12, 2)
        mu = rnd(5, W, dtype=torch.float32)
        t = timed_launches(lambda: ops.shift_mix(x, state, HD * wd, mu, token_seq, cu, seq_slots))
        entry(f"{shape}/shift_mix", t, 0, 2.0 * N * W * 6, dict(like, name="mingru_scan"))
        # the scaled add with its norm beside the output-norm add
        hidden, da, db = rnd(N, W, dtype=torch.float32), rnd(N, W), rnd(N, W, dtype=torch.float32)
        w = torch.ones(W, device=dev)
        t = timed_launches(lambda: ops.scaled_add_rmsnorm(hidden, da, db, 0.3, w, 1e-6, bf))
        wb = torch.ones(VW, device=dev, dtype=bf)
        hv, dv = rnd(N, VW, dtype=torch.float32), rnd(N, VW)
        tv = timed_launches(lambda: ops.rmsnorm_add(hv, dv, wb, 1e-6, bf))
        like = entry(f"{shape}/rmsnorm_add (Visadra)", tv, 0, N * VW * (4 + 4 + 2 + 2.0))
        entry(f"{shape}/scaled_add_rmsnorm", t, 0, N * W * (4 + 4 + 2 + 4 + 2.0), dict(like, name="rmsnorm_add"))
        # the routers and the experts
        logits = rnd(N, E + I, dtype=torch.float32)
        t = timed_launches(lambda: ops.moe_route_grouped(logits, torch.zeros(E + I, device=dev), top, ng, keep))
        vlogits = rnd(N, VE, dtype=torch.float32)
        tv = timed_launches(lambda: ops.moe_route(vlogits, torch.zeros(VE, device=dev), vtop))
        like = entry(f"{shape}/moe_route (Visadra)", tv, 0, N * (4.0 * VE + 8 * vtop))
        entry(f"{shape}/moe_route_grouped", t, 0, N * (4.0 * (E + I) + 8 * top), dict(like, name="moe_route"))
        xx = rnd(N, W, scale=0.1)
        gate_up, down = rnd(E, 2 * eff, W, scale=0.02), rnd(E, W, eff, scale=0.02)
        ids, gains = ops.moe_route_grouped(logits, torch.zeros(E + I, device=dev), top, ng, keep)
        t = timed_launches(lambda: ops.moe_experts(xx, ids, gains, gate_up, down), repeats=5)
        real = int((ids < E).sum())
        vx = rnd(N, VW, scale=0.1)
        vgu, vdown = rnd(VE, 2 * veff, VW, scale=0.02), rnd(VE, VW, veff, scale=0.02)
        vids, vgains = ops.moe_route(vlogits, torch.zeros(VE, device=dev), vtop)
        tv = timed_launches(lambda: ops.moe_experts(vx, vids, vgains, vgu, vdown), repeats=5)
        like = entry(f"{shape}/moe_experts (Visadra)", tv, 6.0 * N * vtop * VW * veff,
                     2.0 * (3 * min(VE, N * vtop) * VW * veff + 2 * N * VW))
        entry(f"{shape}/moe_experts with identity experts", t, 6.0 * real * W * eff,
              2.0 * (3 * min(E, real) * W * eff + 2 * N * W), dict(like, name="moe_experts"))
        del lat_pages, kv_layer
    return out


def kezasun_workload(args):
    import torch

    from litellmengine_amd.models import random_model

    which = args.sizes if args.sizes in KEZASUN_SIZES else "mid"
    groups = max(1, args.layers // 4) if args.layers != SIZES["num_hidden_layers"] else 2
    kcfg = kezasun_config(which, groups)
    vcfg, _ = visadra_configs(which, groups)
    line = {"metric": f"Kezasun beside Visadra at layer sizes of the same name ({which}): prefill tok/s @ 2048 and decode tok/s "
                      f"@ batch {args.batch}, context {args.context}", "unit": "tok/s", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic: seeded random weights, uniform random token ids", "higher_is_better": True,
            "config": {"sizes": dict(zip(("width", "wkv_heads", "wkv_dim", "decay_rank", "heads", "kv_heads", "dim", "vdim",
                                          "rotated", "window", "experts", "identity", "top", "expert_ff", "groups", "kept"),
                                         KEZASUN_SIZES[which])),
                       "layers": 4 * groups, "pattern": "wkv+moe, attention+moe, wkv+moe, attention (keys of the second)+moe"}}
    steps, warmup = min(args.steps, 16), min(args.warmup, 4)
    for name, cfg in (("kezasun", kcfg), ("visadra", vcfg)):
        model = random_model(cfg, seed=0, dtype="bfloat16")
        dt = time_decode(model, cfg, args.batch, args.context, steps, warmup)
        pt = time_prefill(model, cfg, PREFILL_TOKENS)
        line[name] = {"decode_tok_s": round(args.batch / dt, 1), "decode_ms_per_step": round(dt * 1e3, 3),
                      "prefill_tok_s": round(PREFILL_TOKENS / pt, 1), "prefill_ms": round(pt * 1e3, 3)}
        del model
        torch.cuda.empty_cache()
    line["value"] = line["kezasun"]["decode_tok_s"]
    line["steps"], line["warmup"] = steps, warmup
    line["kernels"] = kezasun_kernels(which)
    print(json.dumps(line))
    return 0

MALILORN_SIZES = {
    # width, q heads, kv heads, dim, vdim, rotated, taps, wkv heads, wkv dim, decay rank, experts, top, expert ff, shared ff, dense ff
    "small": (1024, 8, 2, 128, 128, 64, 4, 16, 64, 32, 16, 4, 512, 1024, 4096),
    "mid": (2048, 16, 4, 128, 128, 64, 4, 32, 64, 64, 64, 6, 1408, 2816, 8192),
    "wide": (4096, 32, 8, 128, 128, 64, 4, 64, 64, 64, 64, 6, 2048, 4096, 12288),
}


def malilorn_config(which, groups):
    from litellmengine_amd.config import MalilornConfig

    W, H, G, dim, vdim, rot, taps, wh, wd, rank, E, top, eff, sff, ff = MALILORN_SIZES[which]
    mixer = {"left": {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "conv": taps,
                      "rot": {"base": 250000.0, "dims": rot, "scaling": {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}}},
             "right": {"heads": wh, "dim": wd, "decay_rank": rank}, "left_scale": 1.0, "right_scale": 0.5}
    moe = {"kind": "moe", "expert": {"ff": eff}, "router": {"experts": E, "top": top}, "shared": {"ff": sff}}
    layers = []
    for g in range(groups):
        layers += [{"type": "parallel", "mixer": mixer, "mlp": {"kind": "dense", "ff": ff}}] + \
                  [{"type": "parallel", "mixer": mixer, "mlp": moe}] * 3
    return MalilornConfig.from_dict({"architecture": "Malilorn", "vocab": 32768, "width": W, "norm": {"eps": 1e-6},
                                     "logit_softcap": 30.0, "layers": layers})


def malilorn_kernels(which):
    """Each kernel of Malilorn's own at two shapes (a 2048-token prompt; 8 decoded tokens after 4096) beside the
    like kernel of Kezasun (the closest model: the same recurrence, grouped-query attention with keys and values
    of their own width, routed experts) at its sizes of the same name: microseconds and the share of its
    roofline.  The recurrence's walk, its mixes and the attention itself are Kezasun's kernels and are measured
    there (`--workload kezasun`); the attention is measured again here because it runs without a window."""
    import torch

    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()
    W, H, G, dim, vdim, rot, taps, wh, wd, rank, E, top, eff, sff, ff = MALILORN_SIZES[which]
    KW, kwh, kwd, krank, KH, KG, kdim, kvdim, krot, kwindow, KE, KI, ktop, keff, kng, kkeep = KEZASUN_SIZES[which]
    dev, bf = "cuda", torch.bfloat16
    P = PAGE_SIZE
    rnd = lambda *shape, dtype=bf, scale=1.0: (torch.randn(shape, device=dev) * scale).to(dtype)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=dev)
    out = {}

    def entry(name, seconds, flops, nbytes, like=None):
        floor = max(flops / MFMA_PEAK["bf16"], nbytes / HBM_PEAK)
        e = {"us": round(seconds * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "frac": round(floor / seconds, 4),
             "bound": "mfma" if flops / MFMA_PEAK["bf16"] > nbytes / HBM_PEAK else "hbm"}
        if like is not None:
            e["like"] = like
            e["times_farther_from_roofline"] = round(like["frac"] / e["frac"], 2) if e["frac"] > 0 else None
        out[name] = e
        return e

    for shape, S, q_len, past in (("prefill_2048", 1, 2048, 0), ("decode_b8_ctx4096", 8, 1, 4095)):
        N, kv = S * q_len, past + q_len
        pages_each = -(-kv // P)
        table = torch.arange(S * pages_each, dtype=torch.int32, device=dev).view(S, pages_each).contiguous()
        seq_slots, cu = ints(list(range(S))), ints([i * q_len for i in range(S + 1)])
        kv_lens = ints([kv] * S)
        token_seq = ints([i // q_len for i in range(N)])
        positions = ints([past + i % q_len for i in range(N)])
        slots = (table.long().repeat_interleave(P, 1)[:, past:kv] * P + torch.arange(past, kv, device=dev) % P).reshape(-1).int()
        # attention over every earlier key beside Kezasun's over a window with a sink (the same kernels)
        D = -(-max(dim, vdim) // 32) * 32
        kv_layer = rnd(S * pages_each + 1, 2, G, P, D)
        q = rnd(N, H, D, scale=0.1)
        t = timed_launches(lambda: ops.paged_attention(q, kv_layer, table, seq_slots, cu, kv_lens, token_seq, None, 0.1,
                                                       q_len, q_len, kv))
        KD = -(-max(kdim, kvdim) // 32) * 32
        kq, sinks = rnd(N, KH, KD, scale=0.1), torch.zeros(KH, device=dev)
        kkv = rnd(S * pages_each + 1, 2, KG, P, KD)
        tk = timed_launches(lambda: ops.paged_attention(kq, kkv, table, seq_slots, cu, kv_lens, token_seq, kwindow, 0.1,
                                                        q_len, q_len, kv, sinks=sinks))
        seen = sum(min(kwindow, past + i + 1) for i in range(q_len)) * S
        like = entry(f"{shape}/paged_attention, window and sink (Kezasun)", tk, 4.0 * KH * KD * seen,
                     2.0 * (S * min(kv, kwindow + q_len - 1) * 2 * KG * KD + 2 * N * KH * KD))
        visible = S * (q_len * past + q_len * (q_len + 1) / 2)
        entry(f"{shape}/paged_attention, every earlier key", t, 4.0 * H * D * visible,
              2.0 * (S * kv * 2 * G * D + 2 * N * H * D), dict(like, name="paged_attention"))
        # convolution, heads' norm, rotation and the cache write (with the state rows' update) beside the projection norm's kernel
        cols = (H + G) * dim + G * vdim
        u = rnd(N, cols)
        conv_w = rnd(cols, taps, dtype=torch.float32)
        state = torch.zeros(S + 1, (taps - 1) * cols, device=dev)
        qw = kw = torch.ones(dim, device=dev)
        cos_sin = ops.rope_table(positions, torch.ones(rot // 2, device=dev))

        def conv():
            ops.conv_norm_rope_write(u, conv_w, state, token_seq, cu, seq_slots, slots, qw, kw, cos_sin, rot, 1e-6, kv_layer,
                                     H, G, dim, vdim)
            ops.conv_state_update(u, state, taps - 1, cu, seq_slots)

        t = timed_launches(conv)
        kcols = KH * kdim + KG * (kdim + kvdim) + KH
        kqkv, kbias = rnd(N, kcols), rnd(kcols)
        kqw, kkw = torch.ones(KH * kdim, device=dev), torch.ones(KG * kdim, device=dev)
        kcs = ops.rope_table(positions, torch.ones(krot // 2, device=dev))
        tk = timed_launches(lambda: ops.proj_norm_rope_write(kqkv, kbias, slots, kqw, kkw, kcs, krot, 1e-6, kkv, KH, KG, kdim, kvdim))
        like = entry(f"{shape}/proj_norm_rope_write (Kezasun)", tk, 0, 2.0 * N * (kcols + KH * KD + 2 * KG * KD))
        entry(f"{shape}/conv_norm_rope_write + conv_state_update", t, 0,
              2.0 * N * (cols + H * D + 2 * G * D) + 8.0 * S * (taps - 1) * cols, dict(like, name="proj_norm_rope_write"))
        # the two norms around one add beside the scaled add with its norm
        hidden, ya, yb = rnd(N, W, dtype=torch.float32), rnd(N, W), rnd(N, W, dtype=torch.float32)
        w = torch.ones(W, device=dev)
        t = timed_launches(lambda: ops.rmsnorm_add_rmsnorm(hidden, ya, w, 1e-6, w, 1e-6, bf, yb))
        kh, ka, kb = rnd(N, KW, dtype=torch.float32), rnd(N, KW), rnd(N, KW, dtype=torch.float32)
        kwn = torch.ones(KW, device=dev)
        tk = timed_launches(lambda: ops.scaled_add_rmsnorm(kh, ka, kb, 0.3, kwn, 1e-6, bf))
        like = entry(f"{shape}/scaled_add_rmsnorm (Kezasun)", tk, 0, N * KW * (4 + 4 + 2 + 4 + 2.0))
        entry(f"{shape}/rmsnorm_add_rmsnorm", t, 0, N * W * (4 + 4 + 2 + 4 + 2.0), dict(like, name="scaled_add_rmsnorm"))
        # activations: gated relu with biases (dense), squared relu with a row gate (shared expert) beside silu_mul
        z2, b2 = rnd(N, 2 * ff), rnd(2 * ff)
        t = timed_launches(lambda: ops.bias_act(z2, "relu", True, bias=b2))
        ts = timed_launches(lambda: ops.silu_mul(z2))
        like = entry(f"{shape}/silu_mul (Qwen3)", ts, 0, 2.0 * N * 3 * ff)
        entry(f"{shape}/bias_act, gated relu with biases", t, 0, 2.0 * N * 3 * ff, dict(like, name="silu_mul"))
        # the routers and the experts
        logits = rnd(N, E + 1, dtype=torch.float32)
        t = timed_launches(lambda: ops.moe_route(logits, None, top, score="sigmoid", experts=E))
        klogits, kcorr = rnd(N, KE + KI, dtype=torch.float32), torch.zeros(KE + KI, device=dev)
        tk = timed_launches(lambda: ops.moe_route_grouped(klogits, kcorr, ktop, kng, kkeep))
        like = entry(f"{shape}/moe_route_grouped (Kezasun)", tk, 0, N * (4.0 * (KE + KI) + 8 * ktop))
        entry(f"{shape}/moe_route, sigmoid scores", t, 0, N * (4.0 * (E + 1) + 8 * top), dict(like, name="moe_route_grouped"))
        xx = rnd(N, W, scale=0.1)
        up, down = rnd(E, eff, W, scale=0.02), rnd(E, W, eff, scale=0.02)
        ids, gains = ops.moe_route(logits, None, top, score="sigmoid", experts=E)
        t = timed_launches(lambda: ops.moe_experts(xx, ids, gains, up, down, form="relu2", gain_on_input=True), repeats=5)
        kx = rnd(N, KW, scale=0.1)
        kgu, kdown = rnd(KE, 2 * keff, KW, scale=0.02), rnd(KE, KW, keff, scale=0.02)
        kids, kgains = ops.moe_route_grouped(klogits, kcorr, ktop, kng, kkeep)
        tk = timed_launches(lambda: ops.moe_experts(kx, kids, kgains, kgu, kdown), repeats=5)
        real = int((kids < KE).sum())
        like = entry(f"{shape}/moe_experts with identity experts (Kezasun)", tk, 6.0 * real * KW * keff,
                     2.0 * (3 * min(KE, real) * KW * keff + 2 * N * KW))
        entry(f"{shape}/moe_experts, no gate, weighted at the input", t, 4.0 * N * top * W * eff,
              2.0 * (2 * min(E, N * top) * W * eff + 2 * N * W), dict(like, name="moe_experts"))
        # the cap on the logits beside the scaling of the logits (the wanted rows: one a request)
        lg = rnd(S, 32768, dtype=torch.float32)
        t = timed_launches(lambda: ops.softcap_(lg, 30.0))
        tk = timed_launches(lambda: ops.scale_(lg, 1.0))
        like = entry(f"{shape}/scale_ (Visadra)", tk, 0, 8.0 * S * 32768)
        entry(f"{shape}/softcap_", t, 0, 8.0 * S * 32768, dict(like, name="scale_"))
        del kv_layer, kkv
    return out


def malilorn_workload(args):
    import torch

    from litellmengine_amd.models import random_model

    which = args.sizes if args.sizes in MALILORN_SIZES else "mid"
    groups = max(1, args.layers // 4) if args.layers != SIZES["num_hidden_layers"] else 1
    mcfg = malilorn_config(which, groups)
    kcfg = kezasun_config(which, 2 * groups)
    line = {"metric": f"Malilorn beside Kezasun at layer sizes of the same name ({which}): prefill tok/s @ 2048 and decode tok/s "
                      f"@ batch {args.batch}, context {args.context}", "unit": "tok/s", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic: seeded random weights, uniform random token ids", "higher_is_better": True,
            "config": {"sizes": dict(zip(("width", "heads", "kv_heads", "dim", "vdim", "rotated", "taps", "wkv_heads", "wkv_dim",
                                          "decay_rank", "experts", "top", "expert_ff", "shared_ff", "dense_ff"),
                                         MALILORN_SIZES[which])),
                       "layers": 4 * groups,
                       "pattern": "every layer attention behind a convolution beside a recurrence; dense, moe, moe, moe",
                       "beside": f"Kezasun with {8 * groups} layers: as many attentions and as many recurrences, twice the feed-forwards"}}
    steps, warmup = min(args.steps, 16), min(args.warmup, 4)
    for name, cfg in (("malilorn", mcfg), ("kezasun", kcfg)):
        model = random_model(cfg, seed=0, dtype="bfloat16")
        dt = time_decode(model, cfg, args.batch, args.context, steps, warmup)
        pt = time_prefill(model, cfg, PREFILL_TOKENS)
        line[name] = {"decode_tok_s": round(args.batch / dt, 1), "decode_ms_per_step": round(dt * 1e3, 3),
                      "prefill_tok_s": round(PREFILL_TOKENS / pt, 1), "prefill_ms": round(pt * 1e3, 3)}
        del model
        torch.cuda.empty_cache()
    line["value"] = line["malilorn"]["decode_tok_s"]
    line["steps"], line["warmup"] = steps, warmup
    line["kernels"] = malilorn_kernels(which)
    print(json.dumps(line))
    return 0


BIRELIX_SIZES = {
    # width; latent: heads, dim, rotated, vdim, kv rank, q rank; window attention: q heads, kv heads, dim, vdim, window;
    # delta: value heads, query/key heads, dim, vdim, taps; experts, top, expert ff, groups, kept, limit; dense ff
    "small": (1024, 8, 128, 64, 128, 512, 768, 8, 2, 128, 128, 1024, 16, 8, 64, 64, 4, 16, 4, 512, 4, 2, 7.0, 4096),
    "mid": (2048, 16, 128, 64, 128, 512, 1536, 16, 4, 128, 128, 2048, 32, 16, 64, 64, 4, 64, 6, 1408, 8, 4, 7.0, 8192),
    "wide": (4096, 32, 128, 64, 128, 512, 1536, 32, 8, 128, 128, 4096, 64, 32, 64, 64, 4, 64, 6, 2048, 8, 4, 7.0, 12288),
}


def birelix_config(which, groups):
    from litellmengine_amd.config import BirelixConfig

    (W, LH, ldim, lrot, lvdim, rank, qrank, H, G, dim, vdim, window, DH, DG, ddim, dvdim, taps, E, top, eff, ng, keep, limit,
     ff) = BIRELIX_SIZES[which]
    lat = {"heads": LH, "dim": ldim, "rot_dim": lrot, "vdim": lvdim, "kv_rank": rank, "q_rank": qrank,
           "scale": (ldim + lrot) ** -0.5, "rot": {"base": 10000.0, "dims": lrot}}
    att = {"heads": H, "kv_heads": G, "dim": dim, "vdim": vdim, "scale": dim ** -0.5, "mask": {"size": window}}
    dlt = {"heads": DH, "kv_heads": DG, "dim": ddim, "vdim": dvdim, "conv": taps}
    moe = {"kind": "moe", "expert": {"ff": eff, "limit": limit}, "router": {"experts": E, "top": top, "groups": {"count": ng, "keep": keep}}}
    four = [{"type": "latent_attention", "mixer": lat, "mlp": {"kind": "dense", "ff": ff}}, {"type": "delta", "mixer": dlt, "mlp": moe},
            {"type": "latent_attention", "mixer": lat, "mlp": moe}, {"type": "attention", "mixer": att, "mlp": moe}]
    return BirelixConfig.from_dict({"architecture": "Birelix", "vocab": 32768, "width": W, "embedding": {"scale": W ** 0.5},
                                    "norm": {"eps": 1e-6}, "layers": four * groups})


def birelix_kernels(which):
    """Each kernel of Birelix's own at two shapes (a 2048-token prompt; 8 decoded tokens after 4096) beside the
    like kernel of Kezasun (the closest model: a recurrence with a matrix state per head, grouped-query attention
    over a window with a sink, experts chosen among the best groups) at its sizes of the same name, or of Visadra
    for the latent attention: microseconds and the share of its roofline."""
    import torch

    from litellmengine_amd.csrc.ops import default_ops

    ops = default_ops()
    (W, LH, ldim, lrot, lvdim, rank, qrank, H, G, dim, vdim, window, DH, DG, ddim, dvdim, taps, E, top, eff, ng, keep, limit,
     ff) = BIRELIX_SIZES[which]
    KW, kwh, kwd, krank, KH, KG, kdim, kvdim, krot, kwindow, KE, KI, ktop, keff, kng, kkeep = KEZASUN_SIZES[which]
    dev, bf = "cuda", torch.bfloat16
    P = PAGE_SIZE
    rnd = lambda *shape, dtype=bf, scale=1.0: (torch.randn(shape, device=dev) * scale).to(dtype)
    ints = lambda values: torch.tensor(values, dtype=torch.int32, device=dev)
    out = {}

    def entry(name, seconds, flops, nbytes, like=None):
        floor = max(flops / MFMA_PEAK["bf16"], nbytes / HBM_PEAK)
        e = {"us": round(seconds * 1e6, 1), "roofline_us": round(floor * 1e6, 2), "frac": round(floor / seconds, 4),
             "bound": "mfma" if flops / MFMA_PEAK["bf16"] > nbytes / HBM_PEAK else "hbm"}
        if like is not None:
            e["like"] = like
            e["times_farther_from_roofline"] = round(like["frac"] / e["frac"], 2) if e["frac"] > 0 else None
        out[name] = e
        return e

    for shape, S, q_len, past in (("prefill_2048", 1, 2048, 0), ("decode_b8_ctx4096", 8, 1, 4095)):
        N, kv = S * q_len, past + q_len
        pages_each = -(-kv // P)
        table = torch.arange(S * pages_each, dtype=torch.int32, device=dev).view(S, pages_each).contiguous()
        seq_slots, cu = ints(list(range(S))), ints([i * q_len for i in range(S + 1)])
        kv_lens = ints([kv] * S)
        token_seq = ints([i // q_len for i in range(N)])
        slots = (table.long().repeat_interleave(P, 1)[:, past:kv] * P + torch.arange(past, kv, device=dev) % P).reshape(-1).int()
        # the delta rule's walk beside the walk of the recurrence with a decayed matrix state
        q, k = rnd(N, DG * ddim, dtype=torch.float32, scale=ddim ** -0.5), rnd(N, DG * ddim, dtype=torch.float32, scale=ddim ** -0.5)
        v, ba = rnd(N, DH * dvdim, dtype=torch.float32), rnd(N, 2 * DH, dtype=torch.float32)
        a_log = dt_bias = torch.zeros(DH, device=dev)
        dstate = torch.zeros(S + 1, DH * dvdim * ddim, device=dev)
        t = timed_launches(lambda: ops.delta_scan(q, k, v, ba, a_log, dt_bias, dstate, DH, DG, ddim, dvdim, seq_slots, cu))
        HD = kwh * kwd
        r, kk, vv, wraw = (rnd(N, HD, dtype=torch.float32, scale=0.5) for _ in range(4))
        w0 = u0 = torch.zeros(HD, device=dev)
        g, x = rnd(N, HD), rnd(N, KW)
        kstate = torch.zeros(S + 1, HD * kwd + KW, device=dev)
        tk = timed_launches(lambda: ops.wkv_scan(r, kk, vv, wraw, w0, u0, g, torch.ones(HD, device=dev), 1e-6, x, kstate, kwh, kwd,
                                                 seq_slots, cu, bf, q_len))
        like = entry(f"{shape}/wkv_scan (Kezasun)", tk, 0, N * HD * (16 + 2 + 2.0) + 2.0 * S * HD * kwd * 4)
        e = entry(f"{shape}/delta_scan", t, 0, N * (2 * DG * ddim + 2 * DH * dvdim + 2 * DH) * 4.0 + 2.0 * S * DH * dvdim * ddim * 4,
                  dict(like, name="wkv_scan"))
        e["fp32_flops_T"] = round(8.0 * N * DH * dvdim * ddim / t / 1e12, 2)
        # the output norm with its gate (the recurrence beside it does this in its walk's epilogue) beside the gates per head
        o, gate, nw = rnd(N, DH * dvdim, dtype=torch.float32), rnd(N, DH * dvdim), torch.ones(dvdim, device=dev)
        t = timed_launches(lambda: ops.delta_out_norm(o, gate, nw, 1e-6, DH, dvdim))
        KD = -(-max(kdim, kvdim) // 32) * 32
        a, gates = rnd(N, KH * KD), rnd(N, KH)
        tk = timed_launches(lambda: ops.head_gate(a, gates, 0, KH, kvdim))
        like = entry(f"{shape}/head_gate (Kezasun)", tk, 0, 2.0 * N * (KH * KD + KH * kvdim))
        entry(f"{shape}/delta_out_norm", t, 0, N * DH * dvdim * (4 + 2 + 2.0), dict(like, name="head_gate"))
        # the convolution with silu and unit vectors (and the kept rows' update) beside the mixes of neighbouring tokens
        cols = 2 * DG * ddim + DH * dvdim
        uu, conv_w = rnd(N, cols), rnd(cols, taps, dtype=torch.float32)
        cstate = torch.zeros(S + 1, (taps - 1) * cols, device=dev)

        def conv():
            ops.delta_conv(uu, conv_w, cstate, token_seq, cu, seq_slots, DG, ddim, DH, dvdim, 1e-6, ddim ** -0.5)
            ops.conv_state_update(uu, cstate, taps - 1, cu, seq_slots)

        t = timed_launches(conv)
        mu = rnd(5, KW, dtype=torch.float32)
        tk = timed_launches(lambda: ops.shift_mix(x, kstate, HD * kwd, mu, token_seq, cu, seq_slots))
        like = entry(f"{shape}/shift_mix (Kezasun)", tk, 0, 2.0 * N * KW * 6)
        entry(f"{shape}/delta_conv + conv_state_update", t, 0, N * cols * (2 + 4.0) + 8.0 * S * (taps - 1) * cols,
              dict(like, name="shift_mix"))
        # q and k normed head by head (biases, no weights, no rotation) with the cache write beside the norm over whole projections
        D = -(-max(dim, vdim) // 32) * 32
        kv_layer = rnd(S * pages_each + 1, 2, G, P, D)
        pcols = H * dim + G * (dim + vdim)
        qkv, bias = rnd(N, pcols), rnd(pcols)
        t = timed_launches(lambda: ops.proj_norm_rope_write(qkv, bias, slots, None, None, None, 0, 1e-6, kv_layer, H, G, dim, vdim,
                                                            per_head=True))
        kkv = rnd(S * pages_each + 1, 2, KG, P, KD)
        kcols = KH * kdim + KG * (kdim + kvdim) + KH
        kqkv, kbias = rnd(N, kcols), rnd(kcols)
        kqw, kkw = torch.ones(KH * kdim, device=dev), torch.ones(KG * kdim, device=dev)
        positions = ints([past + i % q_len for i in range(N)])
        kcs = ops.rope_table(positions, torch.ones(krot // 2, device=dev))
        tk = timed_launches(lambda: ops.proj_norm_rope_write(kqkv, kbias, slots, kqw, kkw, kcs, krot, 1e-6, kkv, KH, KG, kdim, kvdim))
        like = entry(f"{shape}/proj_norm_rope_write (Kezasun)", tk, 0, 2.0 * N * (kcols + KH * KD + 2 * KG * KD))
        entry(f"{shape}/proj_norm_rope_write, head by head", t, 0, 2.0 * N * (pcols + H * D + 2 * G * D),
              dict(like, name="proj_norm_rope_write"))
        # latent attention with an ordinary softmax beside the same kernel with sinks
        lat_pages = rnd(S * pages_each + 1, P * (2 * rank + lrot))
        q_lat, q_rot = rnd(LH, N, rank, scale=0.1).transpose(0, 1), rnd(N, LH, lrot, dtype=torch.float32, scale=0.1)
        args = (q_lat, q_rot, lat_pages, P, rank, lrot, table, seq_slots, cu, kv_lens, token_seq)
        t = timed_launches(lambda: ops.latent_attention(*args, None, None, 0.1, q_len, kv, bf))
        vsink = torch.zeros(LH, device=dev)
        tv = timed_launches(lambda: ops.latent_attention(*args, vsink, None, 0.1, q_len, kv, bf))
        visible = S * (q_len * past + q_len * (q_len + 1) / 2)
        fl, by = 2.0 * LH * (2 * rank + lrot) * visible, 2.0 * (S * kv * (2 * rank + lrot) + 2 * N * LH * rank)
        like = entry(f"{shape}/latent_attention with sinks (Visadra)", tv, fl, by)
        entry(f"{shape}/latent_attention, ordinary softmax", t, fl, by, dict(like, name="latent_attention"))
        # the routers and the experts
        logits = rnd(N, E, dtype=torch.float32)
        t = timed_launches(lambda: ops.moe_route_grouped(logits, None, top, ng, keep, score="sigmoid", group_top=2))
        klogits, kcorr = rnd(N, KE + KI, dtype=torch.float32), torch.zeros(KE + KI, device=dev)
        tk = timed_launches(lambda: ops.moe_route_grouped(klogits, kcorr, ktop, kng, kkeep))
        like = entry(f"{shape}/moe_route_grouped (Kezasun)", tk, 0, N * (4.0 * (KE + KI) + 8 * ktop))
        entry(f"{shape}/moe_route_grouped, sigmoid scores, groups by their two largest", t, 0, N * (4.0 * E + 8 * top),
              dict(like, name="moe_route_grouped"))
        xx = rnd(N, W, scale=0.1)
        gu, down = rnd(E, 2 * eff, W, scale=0.02), rnd(E, W, eff, scale=0.02)
        ids, gains = ops.moe_route_grouped(logits, None, top, ng, keep, score="sigmoid", group_top=2)
        t = timed_launches(lambda: ops.moe_experts(xx, ids, gains, gu, down, form="gated_clamp", limit=limit), repeats=5)
        kx = rnd(N, KW, scale=0.1)
        kgu, kdown = rnd(KE, 2 * keff, KW, scale=0.02), rnd(KE, KW, keff, scale=0.02)
        kids, kgains = ops.moe_route_grouped(klogits, kcorr, ktop, kng, kkeep)
        tk = timed_launches(lambda: ops.moe_experts(kx, kids, kgains, kgu, kdown), repeats=5)
        real = int((kids < KE).sum())
        like = entry(f"{shape}/moe_experts with identity experts (Kezasun)", tk, 6.0 * real * KW * keff,
                     2.0 * (3 * min(KE, real) * KW * keff + 2 * N * KW))
        entry(f"{shape}/moe_experts, clamped", t, 6.0 * N * top * W * eff, 2.0 * (3 * min(E, N * top) * W * eff + 2 * N * W),
              dict(like, name="moe_experts"))
        # the dense feed-forward's activation beside silu_mul
        z2 = rnd(N, 2 * ff)
        t = timed_launches(lambda: ops.bias_act(z2, "gelu_tanh", True))
        ts = timed_launches(lambda: ops.silu_mul(z2))
        like = entry(f"{shape}/silu_mul (Qwen3)", ts, 0, 2.0 * N * 3 * ff)
        entry(f"{shape}/bias_act, gated tanh-gelu", t, 0, 2.0 * N * 3 * ff, dict(like, name="silu_mul"))
        del kv_layer, kkv, lat_pages
    return out


def birelix_workload(args):
    import torch

    from litellmengine_amd.models import random_model

    which = args.sizes if args.sizes in BIRELIX_SIZES else "mid"
    groups = max(1, args.layers // 4) if args.layers != SIZES["num_hidden_layers"] else 2
    bcfg = birelix_config(which, groups)
    kcfg = kezasun_config(which, groups)
    names = ("width", "latent_heads", "latent_dim", "latent_rotated", "latent_vdim", "kv_rank", "q_rank", "heads", "kv_heads", "dim",
             "vdim", "window", "delta_heads", "delta_kv_heads", "delta_dim", "delta_vdim", "taps", "experts", "top", "expert_ff",
             "groups", "kept", "limit", "dense_ff")
    line = {"metric": f"Birelix beside Kezasun at layer sizes of the same name ({which}): prefill tok/s @ 2048 and decode tok/s "
                      f"@ batch {args.batch}, context {args.context}", "unit": "tok/s", "n_gpus": 1, "dtype": "bf16",
            "data": "synthetic: seeded random weights, uniform random token ids", "higher_is_better": True,
            "config": {"sizes": dict(zip(names, BIRELIX_SIZES[which])), "layers": 4 * groups,
                       "pattern": "latent+dense, delta+moe, latent+moe, attention+moe",
                       "beside": f"Kezasun with {4 * groups} layers: wkv+moe, attention+moe, wkv+moe, attention+moe"}}
    steps, warmup = min(args.steps, 16), min(args.warmup, 4)
    for name, cfg in (("birelix", bcfg), ("kezasun", kcfg)):
        model = random_model(cfg, seed=0, dtype="bfloat16")
        dt = time_decode(model, cfg, args.batch, args.context, steps, warmup)
        pt = time_prefill(model, cfg, PREFILL_TOKENS)
        line[name] = {"decode_tok_s": round(args.batch / dt, 1), "decode_ms_per_step": round(dt * 1e3, 3),
                      "prefill_tok_s": round(PREFILL_TOKENS / pt, 1), "prefill_ms": round(pt * 1e3, 3)}
        del model
        torch.cuda.empty_cache()
    line["value"] = line["birelix"]["decode_tok_s"]
    line["steps"], line["warmup"] = steps, warmup
    line["kernels"] = birelix_kernels(which)
    print(json.dumps(line))
    return 0


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=64)
    ap.add_argument("--warmup", type=int, default=8)
    ap.add_argument("--layers", type=int, default=SIZES["num_hidden_layers"])
    ap.add_argument("--batch", type=int, default=8)
    ap.add_argument("--context", type=int, default=4096)
    ap.add_argument("--dtype", default="bfloat16", choices=["bfloat16", "float32"])
    ap.add_argument("--no-points", action="store_true", help="skip the batch 1 / 64 points and the prefill")
    ap.add_argument("--no-more", action="store_true", help="skip the other workloads that the default line carries")
    ap.add_argument("--sizes", default="8b", choices=["8b", "0p6b", "32b", "small", "mid", "wide"],
                    help="layer sizes of the decode workload: Qwen3-8B (default, the headline), Qwen3-0.6B or Qwen3-32B; "
                         "small, mid or wide: the layer sizes of --workload visadra, kezasun, malilorn and birelix")
    ap.add_argument("--workload", default="decode", choices=["decode", "reference-0p6b", "mixed-32b", "serving", "visadra", "kezasun", "malilorn", "birelix"],
                    help="decode (default: the headline line), the reference's own benchmark shape at Qwen3-0.6B "
                         "sizes, a mixed prompt-portion + decode step at Qwen3-32B sizes, requests arriving over time, "
                         "Visadra beside Qwen3 at equal layer sizes with every kernel against its roofline, Kezasun "
                         "beside Visadra the same way, or Malilorn or Birelix beside Kezasun the same way")
    args = ap.parse_args()
    if args.gpus != 1:
        print(f"bench.py measures one GPU only: --gpus {args.gpus} is not supported")
        return 2
    if args.workload != "decode":
        import torch

        torch.cuda.set_device(0)
        if args.workload == "reference-0p6b":
            args.steps, args.warmup = min(args.steps, 5), min(args.warmup, 1)
            return reference_workload(args)
        if args.workload == "serving":
            return serving_workload(args)
        if args.workload == "visadra":
            return visadra_workload(args)
        if args.workload == "kezasun":
            return kezasun_workload(args)
        if args.workload == "malilorn":
            return malilorn_workload(args)
        if args.workload == "birelix":
            return birelix_workload(args)
        args.steps, args.warmup = min(args.steps, 3), min(args.warmup, 1)
        return mixed_workload(args)

    import torch

    from litellmengine_amd.config import Qwen3Config
    from litellmengine_amd.models import random_model

    table = {"8b": SIZES, "0p6b": SIZES_0P6B, "32b": SIZES_32B}[args.sizes]
    layers = args.layers if args.layers != SIZES["num_hidden_layers"] or args.sizes == "8b" else table["num_hidden_layers"]
    sizes = dict(table, num_hidden_layers=layers)
    cfg = Qwen3Config.from_dict(sizes)
    name = {"8b": "Qwen3-8B", "0p6b": "Qwen3-0.6B", "32b": "Qwen3-32B"}[args.sizes]
    torch.cuda.set_device(0)
    model = random_model(cfg, seed=0, dtype=args.dtype)
    elem = 2 if args.dtype == "bfloat16" else 4
    short = "bf16" if args.dtype == "bfloat16" else "fp32"

    dt = time_decode(model, cfg, args.batch, args.context, args.steps, args.warmup)
    value = args.batch / dt
    avg_ctx = args.context - (args.steps - 1) / 2.0
    step_bytes = weight_bytes_per_step(cfg, elem) + args.batch * avg_ctx * kv_bytes_per_token(cfg, elem)
    achieved = step_bytes / dt
    line = {
        "metric": f"decode tok/s @ batch {args.batch}, {name} sizes, context {args.context} (+ prefill tok/s @ 2048, % roofline)",
        "value": round(value, 2),
        "unit": "tok/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(dt * 1e3, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": short,
        "data": "synthetic: seeded random weights, uniform random token ids",
        "config": {
            "model": f"{name} sizes (random weights)", "layers": cfg.num_hidden_layers,
            "layers_of_full_model": table["num_hidden_layers"], "hidden": cfg.hidden_size,
            "q_heads": cfg.num_attention_heads, "kv_heads": cfg.num_key_value_heads, "head_dim": cfg.head_dim,
            "intermediate": cfg.intermediate_size, "vocab": cfg.vocab_size, "global_batch": args.batch,
            "seq_len": args.context, "page_size": PAGE_SIZE, "prefill_tokens": PREFILL_TOKENS, "parallelism": "none (1 GPU)",
        },
        "roofline": {"bound": "hbm", "achieved": round(achieved / 1e9, 1), "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK, 4)},
    }
    if not args.no_points:
        # The decode points come before the probes of the peaks (measured so, batch 1 came out 2 %
        # faster in three runs out of three; three seconds of matrix instructions or of reading
        # before a decode run, in one process, changed nothing: the cause is not known).
        points = {}
        s = max(8, args.steps // 2)
        points["decode_b1"] = round(1 / time_decode(model, cfg, 1, args.context, s, 4), 2)
        pt = time_prefill(model, cfg, PREFILL_TOKENS)
        line["prefill"] = {"value": round(PREFILL_TOKENS / pt, 1), "tokens": PREFILL_TOKENS, "ms": round(pt * 1e3, 3),
                           "frac": round(prefill_flops(cfg, PREFILL_TOKENS) / pt / MFMA_PEAK[short], 4)}
        points["decode_b64"] = round(64 / time_decode(model, cfg, 64, args.context, s, 4), 2)
        read_peak, mfma_peak = measure_peaks(args.dtype)
        line["roofline"]["measured_peak"] = round(read_peak / 1e9, 1)
        line["roofline"]["frac_of_measured"] = round(achieved / read_peak, 4)
        line["prefill"]["measured_peak_tflops"] = round(mfma_peak / 1e12, 1)
        line["prefill"]["frac_of_measured"] = round(prefill_flops(cfg, PREFILL_TOKENS) / pt / mfma_peak, 4)
        line["points"] = points
        headline = (args.sizes == "8b" and args.dtype == "bfloat16" and layers == SIZES["num_hidden_layers"]
                    and args.batch == 8 and args.context == 4096)
        if headline and not args.no_more:
            del model
            line["more"] = more_workloads(args.steps, args.warmup)
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
