"""Birelix configurations drawn at random, every size within what config.json allows: two to six layers of the
three mixers in any order; latent attention with 1 to 16 heads, plain parts of 8 to 128 elements, rotated parts of
2 to 64, values of 8 to 128, latents of 8 to 160 and query latents of 6 to 96; window attention with heads of 16
to 256 elements and values of another width, one to four kv heads, groups of 1 to 8, windows of 1 to 200 tokens or
none; delta layers with heads of 8 to 256 key channels and 8 to 160 value channels, one to four query/key heads
with one to four value heads each, one to six taps; dense and routed feed-forwards in any order, one to all
experts chosen, one to six groups of which one to all are kept, limits of 0.5 to 7, layers without a
feed-forward; embedding scales, widths that are multiples of 8 or of 2 only, odd vocabularies, pages of 4 to 64
tokens.  Each goes through the replay loop of bin/trace_run (in this process) in all four ways of cutting, with a
pool so small that pages are used again and four request slots, and every row is compared with the plain
implementation: float32 always, bfloat16 with every layer's routed experts made equal so that rounding cannot move
anything through a choice."""
import io
import os
import random

import pytest
import torch

import numpy as np

from tests.birelix_util import delta, dense, latent, layer, moe, plain_logits, read, sharpen, window
from tests.plain import birelix_plain as plain
from tests.tiny import random_tokens
from tests.trace_util import TraceBuilder, changing_portions, mixed, tail_one_by_one, whole

pytestmark = pytest.mark.gpu

# (LLE_RANDOM_DRAWS=100 runs more of them by hand.)
TOL = {"float32": 2e-4, "bfloat16": 1.5e-1}


def draw_layer(rng):
    kind = rng.choice(["latent_attention", "attention", "delta"])
    if kind == "latent_attention":
        dim, rot = rng.choice([8, 16, 32, 64, 128]), rng.choice([2, 6, 8, 16, 32, 64])
        mixer = latent(rng.choice([1, 2, 3, 8, 16]), dim, rot, rng.choice([8, 24, 32, 64, 128]), rng.choice([8, 16, 40, 64, 128, 160]),
                       rng.choice([6, 16, 48, 96]), round(rng.choice([0.7, 1.0, 1.4]) / (dim + rot) ** 0.5, 4),
                       rng.choice([50.0, 1e4, 1e5]), dims=rng.choice([rot, rot, 2, rot // 4 * 2 or 2]))
    elif kind == "attention":
        dim = rng.choice([16, 32, 48, 64, 64, 96, 128, 256])
        nkv = rng.choice([1, 1, 2, 3, 4])
        mixer = window(nkv * rng.choice([1, 2, 3, 4, 8]), nkv, dim, rng.choice([dim, dim, 16, 32, 64, 80, 256]),
                       round(rng.choice([0.7, 1.0, 1.4]) / dim ** 0.5, 4), rng.choice([None, 1, 2, 7, 16, 33, 64, 70, 200]))
    else:
        nkv = rng.choice([1, 1, 2, 3, 4])
        mixer = delta(nkv * rng.choice([1, 1, 2, 3, 4]), nkv, rng.choice([8, 16, 24, 32, 64, 64, 100, 128, 256]),
                      rng.choice([8, 16, 20, 32, 64, 128, 160]), rng.choice([1, 2, 3, 4, 4, 6]))
    kind_ff = rng.choice(["none", "dense", "moe", "moe"])
    if kind_ff == "none":
        mlp = None
    elif kind_ff == "dense":
        mlp = dense(rng.choice([8, 20, 64, 200, 320]))
    else:
        count = rng.choice([1, 2, 3, 4, 6])
        per = rng.choice([1, 2, 3, 4])
        keep = rng.randint(1, count)
        mlp = moe(count * per, rng.randint(1, min(keep * per, 4)), rng.choice([8, 20, 64, 72, 96]),
                  rng.choice([0.5, 1.0, 2.0, 7.0]), count, keep)
    return layer(kind, mixer, mlp)


def draw(seed: int):
    rng = random.Random(seed)
    spec = {"architecture": "Birelix", "vocab": rng.choice([50, 97, 256, 311, 576]),
            "width": rng.choice([64, 72, 96, 128, 136, 200, 256, 320, 52, 90]),
            "embedding": {"scale": rng.choice([1.0, 4.0, 8.0, 13.5])},
            "norm": {"eps": rng.choice([1e-6, 1e-5, 3e-6])}, "layers": [draw_layer(rng) for _ in range(rng.randint(2, 6))]}
    page = rng.choice([4, 8, 16, 16, 16, 32, 64])
    lengths = {r: rng.randint(20, 260) for r in "abcdef"}
    return spec, page, rng.choice([1.0, 2.0, 3.0]), lengths


def check_rows(out_dir, trace, expected, tol, compared):
    """Every dumped row of a position below `compared[request]` against the plain model's logits."""
    worst = 0.0
    for n, rows in trace.rows.items():
        vocab = next(iter(expected.values())).shape[1]
        got = torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{n}.f32"), dtype="<f4").reshape(len(rows), vocab))
        for i, (rid, pos) in enumerate(rows):
            rid0 = rid.split("#")[0]
            if pos >= compared[rid0]:
                continue
            want = expected[rid0][pos]
            err = (got[i].double() - want).abs().max().item() / max(1.0, want.abs().max().item())
            assert err < tol, f"step {n}, request {rid}, position {pos}: error {err:.3g} (first wrong row of the step: {i})"
            worst = max(worst, err)
    return worst


@pytest.mark.parametrize("seed", range(7000, 7000 + int(os.environ.get("LLE_RANDOM_DRAWS", "12"))))
def test_a_configuration_drawn_at_random(tmp_path, seed):
    from litellmengine_amd.config import BirelixConfig
    from litellmengine_amd.entrypoints.trace_run import replay
    from litellmengine_amd.models import load_model
    from litellmengine_amd.weights import write_model_dir

    spec, page, factor, lengths = draw(seed)
    cfg = BirelixConfig.from_dict(spec)
    said = f"seed {seed}: {spec}, pages of {page}, sharpened {factor}:"
    requests = {r: random_tokens(n, cfg.vocab, seed * 10 + i) for i, (r, n) in enumerate(lengths.items())}
    tb = TraceBuilder()
    whole(tb, "a#whole", requests["a"])
    tail_one_by_one(tb, "b#tail", requests["b"], tail=min(32, lengths["b"] - 2))
    changing_portions(tb, "c#cut", requests["c"], seed=seed)
    mixed(tb, {r + "#mix": t for r, t in requests.items()}, seed=seed)
    # the pool: what the live requests hold at most, each rounded up to whole pages
    pool = -(-tb.max_tokens // page) * page + 4 * page
    for dtype in ("float32", "bfloat16"):
        model_dir = str(tmp_path / f"model_{dtype}")
        write_model_dir(cfg, model_dir, seed, torch.bfloat16)
        # (bfloat16: the scores as they are; rounded queries and keys under sharpened scores alone move the logits by tenths)
        # and the gates, routers and the delta rule's beta and decay projections as they are: grown, they turn the rounding
        # of their inputs into tenths as well, which the same arithmetic on the CPU with bfloat16 storage shows too)
        sharpen(model_dir, factor if dtype == "float32" else 1.0, same_experts=dtype == "bfloat16",
                memory=1.4 if dtype == "float32" else 1.0, skip=() if dtype == "float32" else (".mix.g", ".mlp.router", ".mix.b", ".mix.a"))
        want = plain_logits(model_dir, requests)
        out = str(tmp_path / dtype)
        model = load_model(model_dir, dtype, device="cuda:0")
        replay(model, out, pool, page, 4, io.StringIO(tb.text()), io.StringIO())
        compared = {r: len(t) for r, t in requests.items()}
        if dtype == "float32":
            # where a router's last choice leads the best one left out by next to nothing, float32 rounding may choose
            # otherwise than the float64 model: a request is compared up to its first such token (a gap below 1e-3)
            cfg_d, w = read(model_dir)
            for r, t in requests.items():
                close = (plain.router_margins(cfg_d, w, t) < 1e-3).nonzero()
                if len(close):
                    compared[r] = int(close[0])
        worst = check_rows(out, tb, want, TOL[dtype], compared)
        said += f" {dtype} {worst:.2e}"
    print(said)
