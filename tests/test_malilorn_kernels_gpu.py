"""The kernels that Malilorn added (the short convolution with the heads' norm, rotation and cache write, its
state rows; activations with biases and row gates; the router by sigmoid scores; experts without a gate that
are weighted at their input; two norms around one add; the cap on the logits; state rows that are columns of a
wider row), each alone against its plain torch form (tests/torch_ops.py), in float32 and bfloat16, at sizes
that are no powers of two."""
import pytest
import torch

from tests.torch_ops import TorchOps, v_pages

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
REF = TorchOps(torch.float64)


def ops():
    from litellmengine_amd.csrc.ops import default_ops

    return default_ops()


def tol(dtype, scale=1.0):
    return (2e-5 if dtype == torch.float32 else 2e-2) * scale


def rnd(shape, dtype, seed, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


def ints(values):
    return torch.tensor(values, dtype=torch.int32).cuda()


def batch(q_lens):
    """Device arrays of a step whose requests bring `q_lens` tokens, on slots 2, 0, 3, ..."""
    slots = [2, 0, 3, 1, 4, 5, 6, 7][: len(q_lens)]
    cu = [0]
    for n in q_lens:
        cu.append(cu[-1] + n)
    token_seq = [s for s, n in enumerate(q_lens) for _ in range(n)]
    return ints(slots), ints(cu), ints(token_seq), cu[-1]


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("sizes", [  # nq, nkv, dim, vdim, D, rot, taps, page size
    (6, 2, 24, 40, 64, 8, 3, 4), (8, 1, 128, 96, 128, 64, 4, 16), (1, 1, 48, 10, 64, 2, 1, 8), (5, 5, 8, 12, 32, 0, 5, 16),
    (4, 2, 64, 64, 64, 64, 2, 16), (2, 1, 16, 24, 32, 4, 9, 8), (3, 1, 256, 200, 256, 100, 8, 16)])
@pytest.mark.parametrize("q_lens", [[1, 1, 1], [7, 1, 2, 30], [70]])
def test_conv_norm_rope_write_and_its_state(dtype, sizes, q_lens):
    """Single tokens, portions shorter and longer than the taps reach, from state rows that are not zero and are
    columns of a wider row; a padding row (page slot -1) writes nothing; the state is advanced afterwards.  Up to
    eight taps take the kernel that walks runs of tokens with the window in registers, nine the plain one."""
    o = ops()
    nq, nkv, dim, vdim, D, rot, J, P = sizes
    seq_slots, cu, token_seq, N = batch(q_lens)
    cols = (nq + nkv) * dim + nkv * vdim
    u = rnd((N, cols), dtype, 1)
    taps = rnd((cols, J), torch.float32, 2, 0.5)
    wide = rnd((9, 13 + (J - 1) * cols + 5), torch.float32, 3)
    state = wide[:, 13 : 13 + (J - 1) * cols] if J > 1 else None
    qw, kw = 1.0 + rnd((dim,), torch.float32, 4, 0.2), 1.0 + rnd((dim,), torch.float32, 5, 0.2)
    angles = rnd((N, rot // 2), torch.float32, 6, 3.0)
    cos_sin = torch.stack([torch.cos(angles), torch.sin(angles)], dim=-1).contiguous()
    pages = -(-N // P) + 2
    perm = torch.randperm(pages * P, generator=torch.Generator().manual_seed(7))[:N].to(torch.int32)
    perm[N // 2] = -1  # a row that stands for nobody
    slots = perm.cuda()
    kv = rnd((pages, 2, nkv, P, D), dtype, 8)
    want_kv, want_wide = kv.clone(), wide.clone()
    want_state = want_wide[:, 13 : 13 + (J - 1) * cols] if J > 1 else None
    want = REF.conv_norm_rope_write(u, taps, want_state, token_seq, cu, seq_slots, slots, qw, kw, cos_sin, rot, 1e-5, want_kv,
                                    nq, nkv, dim, vdim)
    got = o.conv_norm_rope_write(u, taps, state, token_seq, cu, seq_slots, slots, qw, kw, cos_sin, rot, 1e-5, kv, nq, nkv,
                                 dim, vdim)
    assert got.shape == (N, nq, D) and (got.double() - want.double()).abs().max() < tol(dtype, 8)
    assert D == dim or float(got[:, :, dim:].abs().max()) == 0.0
    assert (kv.double() - want_kv.double()).abs().max() < tol(dtype, 8)
    assert torch.equal(wide, want_wide)  # the state is left as it was
    if J > 1:
        REF.conv_state_update(u, want_state, J - 1, cu, seq_slots)
        o.conv_state_update(u, state, J - 1, cu, seq_slots)
        assert torch.equal(wide, want_wide)  # the new rows exactly, the neighbouring columns untouched
        for s, n in enumerate(q_lens):
            last = u[int(cu[s + 1]) - 1].float()
            assert torch.equal(state[int(seq_slots[s]), (J - 2) * cols :], last)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("q_lens,heads", [([1, 300, 2, 700, 1, 1, 45], (8, 2)), ([3, 1500, 1, 2, 1400, 5, 90, 1], (12, 4)),
                                          ([5000], (4, 4))])
def test_conv_runs_of_tokens_across_requests(dtype, q_lens, heads):
    """Steps long enough that a wavefront walks runs of 4, 8 and 16 tokens with its window in registers: requests
    begin and end inside the runs, single tokens sit between long portions, the states are not zero."""
    o = ops()
    (nq, nkv), dim, vdim, D, rot, J, P = heads, 32, 48, 64, 16, 4, 16
    seq_slots, cu, token_seq, N = batch(q_lens)
    cols = (nq + nkv) * dim + nkv * vdim
    u = rnd((N, cols), dtype, 1)
    taps = rnd((cols, J), torch.float32, 2, 0.5)
    state = rnd((9, (J - 1) * cols), torch.float32, 3)
    qw, kw = 1.0 + rnd((dim,), torch.float32, 4, 0.2), 1.0 + rnd((dim,), torch.float32, 5, 0.2)
    angles = rnd((N, rot // 2), torch.float32, 6, 3.0)
    cos_sin = torch.stack([torch.cos(angles), torch.sin(angles)], dim=-1).contiguous()
    pages = -(-N // P) + 1
    slots = torch.randperm(pages * P, generator=torch.Generator().manual_seed(7))[:N].to(torch.int32).cuda()
    kv = torch.zeros((pages, 2, nkv, P, D), dtype=dtype).cuda()
    want_kv, want_state = kv.clone(), state.clone()
    want = REF.conv_norm_rope_write(u, taps, want_state, token_seq, cu, seq_slots, slots, qw, kw, cos_sin, rot, 1e-5, want_kv,
                                    nq, nkv, dim, vdim)
    got = o.conv_norm_rope_write(u, taps, state, token_seq, cu, seq_slots, slots, qw, kw, cos_sin, rot, 1e-5, kv, nq, nkv, dim,
                                 vdim)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 8)
    assert (kv.double() - want_kv.double()).abs().max() < tol(dtype, 8)
    REF.conv_state_update(u, want_state, J - 1, cu, seq_slots)
    o.conv_state_update(u, state, J - 1, cu, seq_slots)
    assert torch.equal(state, want_state)


def test_conv_portions_equal_one_go():
    """A request's tokens in one step, and the same tokens in steps of 1, 2, 3, 1, ... through the state rows."""
    o = ops()
    nq, nkv, dim, vdim, D, J, P, T = 2, 1, 16, 24, 32, 4, 8, 23
    cols = (nq + nkv) * dim + nkv * vdim
    u, taps = rnd((T, cols), torch.float32, 1), rnd((cols, J), torch.float32, 2)
    qw = kw = torch.ones(dim).cuda()
    slots_all = torch.arange(T, dtype=torch.int32).cuda()
    kv1, kv2 = torch.zeros((4, 2, nkv, P, D)).cuda(), torch.zeros((4, 2, nkv, P, D)).cuda()
    st1, st2 = torch.zeros((2, (J - 1) * cols)).cuda(), torch.zeros((2, (J - 1) * cols)).cuda()
    one = o.conv_norm_rope_write(u, taps, st1, ints([0] * T), ints([0, T]), ints([1]), slots_all, qw, kw, None, 0, 1e-5,
                                 kv1, nq, nkv, dim, vdim)
    o.conv_state_update(u, st1, J - 1, ints([0, T]), ints([1]))
    at, parts = 0, []
    for n in [1, 2, 3, 1, 1, 5, 2, 8]:
        parts.append(o.conv_norm_rope_write(u[at : at + n].contiguous(), taps, st2, ints([0] * n), ints([0, n]), ints([1]),
                                            slots_all[at : at + n].contiguous(), qw, kw, None, 0, 1e-5, kv2, nq, nkv, dim, vdim))
        o.conv_state_update(u[at : at + n].contiguous(), st2, J - 1, ints([0, n]), ints([1]))
        at += n
    assert at == T
    assert (torch.cat(parts) - one).abs().max() < 1e-6 and (kv1 - kv2).abs().max() < 1e-6 and torch.equal(st1, st2)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["silu", "relu", "relu2"])
@pytest.mark.parametrize("gated", [False, True])
@pytest.mark.parametrize("F", [52, 72])
def test_bias_act(dtype, kind, gated, F):
    """Rows of a multiple of 8 take 16-byte pieces in bfloat16, others one element a thread."""
    o = ops()
    N = 37
    z = rnd((N, 2 * F if gated else F), dtype, 1, 2.0)
    bias = rnd((z.shape[1],), dtype, 2)
    gate = rnd((N, 7), torch.float32, 3, 2.0)
    for b, rg in ((None, None), (bias, None), (None, (gate, 5)), (bias, (gate, 0))):
        got, want = o.bias_act(z, kind, gated, bias=b, row_gate=rg), REF.bias_act(z, kind, gated, bias=b, row_gate=rg)
        assert got.shape == (N, F) and (got.double() - want.double()).abs().max() < tol(dtype, 8)


def test_softcap():
    o = ops()
    x = rnd((13, 77), torch.float32, 1, 20.0)
    want = 15.0 * torch.tanh(x.double() / 15.0)
    got = o.softcap_(x, 15.0)
    assert got is x and (x.double() - want).abs().max() < 1e-5 and float(x.abs().max()) <= 15.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [40, 1000, 2500, 9000])
@pytest.mark.parametrize("pair", [False, True])
def test_two_norms_around_one_add(dtype, H, pair):
    o = ops()
    hidden = rnd((7, H), torch.float32, 2, 3.0)
    y = rnd((7, H), dtype, 3)
    extra = rnd((7, H), torch.float32, 4) if pair else None
    w, w2 = 1.0 + rnd((H,), torch.float32, 5, 0.1), 1.0 + rnd((H,), torch.float32, 6, 0.1)
    want_h = hidden.clone()
    want = REF.rmsnorm_add_rmsnorm(want_h, y, w, 1e-5, w2, 1e-6, dtype, extra)
    got = o.rmsnorm_add_rmsnorm(hidden, y, w, 1e-5, w2, 1e-6, dtype, extra)
    assert (hidden.double() - want_h.double()).abs().max() < 2e-6
    assert got.dtype == dtype and (got.double() - want.double()).abs().max() < tol(dtype, 4)
    # the same as the two launches it replaces
    h2 = rnd((7, H), torch.float32, 2, 3.0)
    o.rmsnorm_add(h2, y, w, 1e-5, dtype, extra)
    assert (h2 - hidden).abs().max() < 2e-6
    assert (o.add_rmsnorm(h2, None, w2, 1e-6, dtype).double() - got.double()).abs().max() < tol(dtype, 2)


def test_router_by_sigmoid_scores_with_ties_and_a_wider_row():
    o = ops()
    N, E = 33, 12
    logits = rnd((N, E + 1), torch.float32, 1, 2.0)
    logits[3, 2] = logits[3, 7] = logits[3].max() + 1.0  # a tie: the lower index comes first
    logits[5, :E] = 0.0  # all equal: the first ones
    logits[:, E] = 100.0  # not an expert: never chosen
    for top in (1, 2, 12):
        ids, gains = o.moe_route(logits, None, top, score="sigmoid", experts=E)
        want_ids, want_gains = REF.moe_route(logits, None, top, score="sigmoid", experts=E)
        assert torch.equal(ids, want_ids) and (gains - want_gains).abs().max() < 1e-6
        assert ids[3, 0] == 2 and ids[5].tolist() == list(range(top)) and int(ids.max()) < E
    # the router of the softmax over the chosen is as it was, with and without a bias
    bias = rnd((E + 1,), torch.float32, 2)
    ids, gains = o.moe_route(logits, bias, 3)
    want_ids, want_gains = REF.moe_route(logits, bias, 3)
    assert torch.equal(ids, want_ids) and (gains - want_gains).abs().max() < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [5, 300])
@pytest.mark.parametrize("top", [1, 3])
def test_experts_without_a_gate_weighted_at_their_input(dtype, N, top):
    """Few pairs (every pair streams its expert) and many (sorted tiles on the matrix cores in bfloat16); an
    expert that nobody chose; F that is no multiple of a wavefront's 64 columns."""
    o = ops()
    E, F, K = 7, 88, 72
    x = rnd((N, K), dtype, 1)
    up, down = rnd((E, F, K), dtype, 2, 0.2), rnd((E, K, F), dtype, 3, 0.2)
    logits = rnd((N, E), torch.float32, 4, 2.0)
    logits[:, 4] = -50.0  # nobody chooses expert 4
    ids, gains = o.moe_route(logits, None, top, score="sigmoid")
    want = REF.moe_experts(x, ids, gains, up, down, form="relu2", gain_on_input=True)
    got = o.moe_experts(x, ids, gains, up, down, form="relu2", gain_on_input=True)
    assert got.dtype == torch.float32 and (got.double() - want.double()).abs().max() < tol(dtype, 4) * float(want.abs().max() + 1)
    # the weight at the input of a squared activation counts twice at the output
    at_output = o.moe_experts(x, ids, gains * gains, up, down, form="relu2", gain_on_input=False)
    assert (at_output - got).abs().max() < tol(dtype, 4) * float(want.abs().max() + 1)
    # the gated form is as it was
    gu = rnd((E, 2 * F, K), dtype, 5, 0.2)
    want = REF.moe_experts(x, ids, gains, gu, down)
    assert (o.moe_experts(x, ids, gains, gu, down).double() - want.double()).abs().max() < tol(dtype, 4) * float(want.abs().max() + 1)


@pytest.mark.parametrize("dtype", DTYPES)
def test_recurrence_on_state_rows_that_are_columns_of_a_wider_row(dtype):
    o = ops()
    H, dim, W = 2, 24, 56
    q_lens = [3, 1, 150]
    seq_slots, cu, token_seq, N = batch(q_lens)
    HD = H * dim
    r, k, v = (rnd((N, HD), torch.float32, s, 0.5) for s in (1, 2, 3))
    wraw = rnd((N, HD), torch.float32, 4) - 1.0
    w0, u = rnd((HD,), torch.float32, 5, 0.5), rnd((HD,), torch.float32, 6, 0.5)
    g, x = rnd((N, HD), dtype, 7), rnd((N, W), dtype, 8)
    norm_w = rnd((HD,), torch.float32, 9) + 1.0
    mu = torch.rand((5, W), generator=torch.Generator().manual_seed(3)).cuda()
    wide = rnd((9, 31 + HD * dim + W + 9), torch.float32, 10, 0.3)
    want_wide = wide.clone()
    state, want_state = wide[:, 31 : 31 + HD * dim + W], want_wide[:, 31 : 31 + HD * dim + W]
    got_mix = o.shift_mix(x, state, HD * dim, mu, token_seq, cu, seq_slots)
    want_mix = REF.shift_mix(x, want_state, HD * dim, mu, token_seq, cu, seq_slots)
    assert (got_mix.double() - want_mix.double()).abs().max() < tol(dtype)
    want = REF.wkv_scan(r, k, v, wraw, w0, u, g, norm_w, 1e-5, x, want_state, H, dim, seq_slots, cu, dtype)
    got = o.wkv_scan(r, k, v, wraw, w0, u, g, norm_w, 1e-5, x, state, H, dim, seq_slots, cu, dtype, max(q_lens))
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    assert (wide.double() - want_wide.double()).abs().max() < 2e-4
    assert torch.equal(wide[:, :31], want_wide[:, :31]) and torch.equal(wide[:, -9:], want_wide[:, -9:])
