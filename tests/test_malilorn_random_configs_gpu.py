"""Malilorn configurations drawn at random, every size within what config.json allows: two to five layers,
attention heads of 16 to 256 elements with values of another width (wider and narrower), one to four kv heads,
groups of 1 to 8, convolutions of 1 to 6 taps or none, rotations over a pair, a part or the whole head or none,
with and without stretched frequencies, recurrence heads of 8 to 128 channels, decay ranks of 1 to 40, dense
and routed feed-forwards in any order with one to all experts chosen, with and without a shared expert, layers
without a feed-forward, mixer constants of one and others, a cap on the logits or none, widths that are
multiples of 8 or of 2 only, odd vocabularies, pages of 4 to 64 tokens.  Each goes through the replay loop of
bin/trace_run (in this process) in all four ways of cutting, with a pool so small that pages are used again
and four request slots, and every row is compared with the plain implementation: float32 always, bfloat16 with
every layer's routed experts made equal so that rounding cannot move anything through a choice."""
import io
import os
import random

import pytest
import torch

import numpy as np

from tests.malilorn_util import dense, left, moe, par, plain_logits, read, sharpen
from tests.plain import malilorn_plain as plain
from tests.tiny import random_tokens
from tests.trace_util import TraceBuilder, changing_portions, mixed, tail_one_by_one, whole

pytestmark = pytest.mark.gpu

# Some draws are badly conditioned: at a sharpening of 7 the plain model itself, run in float32 instead of
# float64, moved by a quarter of the largest logit on one of 120 draws, where the engine was off by 5e-3; the
# sharpening therefore stops at 5.  (LLE_RANDOM_DRAWS=120 runs more of them by hand.)
TOL = {"float32": 5e-3, "bfloat16": 1.5e-1}


def draw(seed: int):
    rng = random.Random(seed)
    width = rng.choice([64, 72, 96, 128, 136, 200, 256, 320])
    layers = []
    for i in range(rng.randint(2, 5)):
        dim = rng.choice([16, 32, 48, 64, 64, 96, 128, 256])
        vdim = rng.choice([dim, dim, 16, 32, 64, 80, 256])
        nkv = rng.choice([1, 1, 2, 3, 4])
        group = rng.choice([1, 2, 3, 4, 8])
        dims = min(dim, rng.choice([0, 2, dim // 4 * 2, dim, 16]))
        scaling = rng.choice([None, (8.0, 1.0, 4.0, 1024), (4.0, 1.0, 8.0, 64), (32.0, 2.0, 3.0, 300)])
        a = left(nkv * group, nkv, dim, vdim, round(rng.choice([0.7, 1.0, 1.0, 1.4]) / dim ** 0.5, 4), rng.choice([0, 1, 2, 3, 4, 4, 6]),
                 rng.choice([50.0, 1e4, 5e5]), dims, scaling)
        mixer = par(a, rng.choice([1, 2, 3, 4, 6]), rng.choice([8, 16, 24, 32, 48, 64, 64, 96, 128]),
                    rng.choice([1, 4, 7, 16, 32, 40]), rng.choice([1.0, 0.5, 1.2, 2.0]), rng.choice([1.0, 0.5, 0.3, 1.5]))
        kind = rng.choice(["none", "dense", "moe", "moe"])
        if kind == "none":
            mlp = None
        elif kind == "dense":
            mlp = dense(rng.choice([8, 20, 64, 200, 320]))
        else:
            experts = rng.choice([1, 2, 3, 8, 12, 16])
            mlp = moe(experts, rng.randint(1, min(experts, 4)), rng.choice([8, 20, 64, 72, 96]),
                      shared=rng.choice([None, 8, 40, 128]))
        layers.append({"type": "parallel", "mixer": mixer, "mlp": mlp})
    spec = {"architecture": "Malilorn", "vocab": rng.choice([50, 97, 256, 311, 576]), "width": width,
            "norm": {"eps": rng.choice([1e-6, 1e-5, 3e-6])}, "layers": layers}
    cap = rng.choice([None, 15.0, 30.0, 50.0])
    if cap:
        spec["logit_softcap"] = cap
    page = rng.choice([4, 8, 16, 16, 16, 32, 64])
    lengths = {r: rng.randint(20, 180) for r in "abcdef"}
    return spec, page, rng.choice([2.0, 3.0, 5.0]), lengths


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


@pytest.mark.parametrize("seed", range(5000, 5000 + int(os.environ.get("LLE_RANDOM_DRAWS", "12"))))
def test_a_configuration_drawn_at_random(tmp_path, seed):
    from litellmengine_amd.config import MalilornConfig
    from litellmengine_amd.entrypoints.trace_run import replay
    from litellmengine_amd.models import load_model
    from litellmengine_amd.weights import write_model_dir

    spec, page, factor, lengths = draw(seed)
    cfg = MalilornConfig.from_dict(spec)
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
        sharpen(model_dir, factor if dtype == "float32" else 1.0, same_experts=dtype == "bfloat16",
                memory=1.4 if dtype == "float32" else 1.0)
        want = plain_logits(model_dir, requests)
        out = str(tmp_path / dtype)
        model = load_model(model_dir, dtype, device="cuda:0")
        replay(model, out, pool, page, 4, io.StringIO(tb.text()), io.StringIO())
        compared = {r: len(t) for r, t in requests.items()}
        if dtype == "float32":
            # Two of 120 draws had a token whose last chosen expert led the best one left out by 1e-4 and 3e-6 of a
            # logit: float32 rounding chose otherwise than the float64 model there, in one of them only beside other
            # requests in a batch.  A request is compared up to its first such token (a gap below 1e-3).
            cfg_d, w = read(model_dir)
            for r, t in requests.items():
                close = (plain.router_margins(cfg_d, w, t) < 1e-3).nonzero()
                if len(close):
                    compared[r] = int(close[0])
        worst = check_rows(out, tb, want, TOL[dtype], compared)
        said += f" {dtype} {worst:.2e}"
    print(said)
