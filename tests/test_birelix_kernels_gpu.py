"""The kernels that Birelix added (the delta rule's convolution, walk and output norm, q and k normed head by head
without weights, latent attention without a sink, the sigmoid router with groups worth their two largest scores,
clamped experts, the tanh form of gelu), each alone against its plain torch form (tests/torch_ops.py), in float32
and bfloat16, at sizes that are no powers of two."""
import pytest
import torch

from tests.test_kezasun_kernels_gpu import batch, ints, ops, rnd, tol
from tests.test_visadra_kernels_gpu import latent_case
from tests.torch_ops import TorchOps

pytestmark = pytest.mark.gpu

DTYPES = [torch.float32, torch.bfloat16]
REF = TorchOps(torch.float64)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("G,H,dim,vdim,J,q_lens", [(2, 6, 24, 20, 3, [5, 1, 1, 2]), (1, 1, 100, 12, 1, [7, 1]), (3, 3, 64, 256, 4, [1, 1, 1]),
                                                   (2, 4, 256, 72, 6, [40, 3]), (1, 4, 8, 100, 2, [1, 9, 2]), (1, 2, 16, 8, 9, [12, 1]),
                                                   (16, 32, 8, 8, 4, [300, 1, 37, 2, 260])])
def test_delta_convolution(dtype, G, H, dim, vdim, J, q_lens):
    """Single tokens, portions shorter and longer than the taps reach, state rows that are not zero and are
    columns of a wider row, more taps than the kernel for runs of tokens takes, and so many tokens that a
    wavefront walks runs of them across the requests' borders; then the same tokens in smaller portions through
    the state give the same rows."""
    o = ops()
    cols = 2 * G * dim + H * vdim
    seq_slots, cu, token_seq, N = batch(q_lens)
    u = rnd((N, cols), dtype, 1)
    taps = rnd((cols, J), torch.float32, 2, 0.5)
    wide = rnd((9, 13 + max(1, J - 1) * cols), torch.float32, 3)
    state = wide[:, 13:] if J > 1 else None
    want = REF.delta_conv(u, taps, state, token_seq, cu, seq_slots, G, dim, H, vdim, 1e-6, dim ** -0.5)
    got = o.delta_conv(u, taps, state, token_seq, cu, seq_slots, G, dim, H, vdim, 1e-6, dim ** -0.5)
    for g, w, name in zip(got, want, "qkv"):
        assert g.dtype == torch.float32 and g.shape == w.shape
        assert (g.double() - w.double()).abs().max() < 2e-5, name
    assert ((got[1].view(N, G, dim) ** 2).sum(-1) - 1).abs().max() < 1e-3  # keys are unit vectors
    if J == 1:
        return
    # the first request's tokens one at a time, the state advanced in between, against the portion in one go
    n0 = q_lens[0]
    st = wide.clone()
    rows = []
    for t in range(n0):
        one = u[t : t + 1].contiguous()
        args = (ints([0]), ints([0, 1]), ints([int(seq_slots[0])]))
        rows.append(o.delta_conv(one, taps, st[:, 13:], args[0], args[1], args[2], G, dim, H, vdim, 1e-6, dim ** -0.5))
        o.conv_state_update(one, st[:, 13:], J - 1, args[1], args[2])
    for i in range(3):
        assert (torch.cat([r[i] for r in rows]) - got[i][:n0]).abs().max() < 1e-6
    assert torch.equal(st[:, :13], wide[:, :13])  # the columns in front belong to somebody else


@pytest.mark.parametrize("H,G,dim,vdim,q_lens", [(6, 2, 24, 20, [5, 1, 1, 30]), (1, 1, 100, 12, [17, 1]), (4, 4, 64, 64, [1, 1, 1]),
                                                 (2, 1, 256, 40, [70]), (4, 1, 8, 100, [3, 9]), (3, 3, 128, 16, [1, 26]),
                                                 (2, 2, 16, 33, [12, 1]), (4, 2, 32, 24, [40, 1, 33, 2])])
def test_delta_walk(H, G, dim, vdim, q_lens):
    """From states that are not zero, portions beside single tokens (steps of many tokens make decays and betas in
    a launch ahead of the walk, short ones in the walk); then a portion cut in pieces gives the same rows and the
    same state as in one go."""
    o = ops()
    seq_slots, cu, token_seq, N = batch(q_lens)
    unit = lambda t, heads: torch.nn.functional.normalize(t.view(N, heads, dim), dim=-1).reshape(N, heads * dim).contiguous()
    q, k = unit(rnd((N, G * dim), torch.float32, 1), G) * dim ** -0.5, unit(rnd((N, G * dim), torch.float32, 2), G)
    v = rnd((N, H * vdim), torch.float32, 3)
    ba = rnd((N, 2 * H), torch.float32, 4, 2.0)
    a_log, dt_bias = rnd((H,), torch.float32, 5), rnd((H,), torch.float32, 6)
    wide = rnd((9, H * vdim * dim + 11), torch.float32, 7, 0.3)
    got_state, want_state = wide.clone(), wide.clone()
    want = REF.delta_scan(q, k, v, ba, a_log, dt_bias, want_state, H, G, dim, vdim, seq_slots, cu)
    got = o.delta_scan(q, k, v, ba, a_log, dt_bias, got_state, H, G, dim, vdim, seq_slots, cu)
    assert (got.double() - want.double()).abs().max() < 2e-5
    assert (got_state.double() - want_state.double()).abs().max() < 2e-5
    assert torch.equal(got_state[:, H * vdim * dim:], wide[:, H * vdim * dim:])  # what lies behind the matrices stays
    # the last request in pieces of 1, 2, 3, ... tokens
    s = len(q_lens) - 1
    lo, hi = int(cu[s]), int(cu[s + 1])
    st = wide.clone()
    rows, at, n = [], lo, 1
    while at < hi:
        n = min(n, hi - at)
        sl = slice(at, at + n)
        rows.append(o.delta_scan(q[sl].contiguous(), k[sl].contiguous(), v[sl].contiguous(), ba[sl].contiguous(), a_log, dt_bias,
                                 st, H, G, dim, vdim, ints([int(seq_slots[s])]), ints([0, n])))
        at += n
        n += 1
    assert (torch.cat(rows) - got[lo:hi]).abs().max() < 1e-6
    assert (st[int(seq_slots[s])] - got_state[int(seq_slots[s])]).abs().max() < 1e-6


def test_delta_walk_a_state_that_forgets_at_once_one_that_never_does_and_a_key_written_twice():
    o = ops()
    H, G, dim, vdim, N = 2, 1, 32, 16, 6
    keys = torch.linalg.qr(torch.randn((dim, dim), generator=torch.Generator().manual_seed(1))).Q[:N].contiguous().cuda()
    keys[4] = keys[0]  # the fifth token writes under the first token's key
    v = rnd((N, H * vdim), torch.float32, 2)
    ba = torch.zeros((N, 2 * H)).cuda()
    ba[:, :H] = 40.0  # beta = 1: whole corrections
    ba[:, H] = -40.0  # head 0: softplus = 0, the decay is one
    ba[:, H + 1] = 40.0  # head 1: the decay is exp(-40 e^0): nothing stays
    state = torch.zeros((3, H * vdim * dim)).cuda()
    a_log, dt_bias = torch.zeros(H).cuda(), torch.zeros(H).cuda()
    # every token asks for the first token's key
    q = keys[0].repeat(N, 1).contiguous()
    got = o.delta_scan(q, keys, v, ba, a_log, dt_bias, state, H, G, dim, vdim, ints([1]), ints([0, N])).view(N, H, vdim)
    vv = v.view(N, H, vdim)
    for t in range(N):  # head 0 remembers: the first value until the fifth token replaces it
        assert (got[t, 0] - (vv[0, 0] if t < 4 else vv[4, 0])).abs().max() < 1e-5
    assert (got[0, 1] - vv[0, 1]).abs().max() < 1e-5 and (got[4, 1] - vv[4, 1]).abs().max() < 1e-5  # the token's own write
    assert got[[1, 2, 3, 5], 1].abs().max() < 1e-6  # head 1 has forgotten by the next token


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,vdim", [(6, 20), (1, 256), (5, 100)])
def test_delta_output_norm(dtype, H, vdim):
    o = ops()
    x = rnd((9, H * vdim), torch.float32, 1, 3.0)
    gate = rnd((9, H * vdim), dtype, 2)
    w = 1.0 + rnd((vdim,), torch.float32, 3, 0.1)
    got = o.delta_out_norm(x, gate, w, 1e-5, H, vdim)
    want = REF.delta_out_norm(x, gate, w, 1e-5, H, vdim)
    assert got.dtype == dtype and (got.double() - want.double()).abs().max() < tol(dtype, 4)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,dim,vdim,D", [(6, 2, 24, 40, 64), (4, 4, 64, 64, 64), (1, 1, 48, 10, 64), (40, 8, 16, 32, 32)])
def test_q_and_k_normed_head_by_head_without_weights(dtype, nq, nkv, dim, vdim, D):
    o = ops()
    N, P, pages = 11, 16, 5
    cols = nq * dim + nkv * (dim + vdim)
    qkv = rnd((N, cols), dtype, 1)
    qkv[:, :dim] *= 30.0  # one head far larger than the others: a norm over the whole projection would crush the rest
    bias = rnd((cols,), dtype, 2, 0.5)
    slots = ints([3, 17, 18, 79, -1, 0, 33, 34, 35, 64, 5])
    kv_got = torch.full((pages + 1, 2, nkv, P, D), 7.0, dtype=dtype).cuda()
    kv_want = kv_got.clone()
    want = REF.proj_norm_rope_write(qkv, bias, slots, None, None, None, 0, 1e-5, kv_want, nq, nkv, dim, vdim, True, True, per_head=True)
    got = o.proj_norm_rope_write(qkv, bias, slots, None, None, None, 0, 1e-5, kv_got, nq, nkv, dim, vdim, True, True, per_head=True)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    assert (kv_got.double() - kv_want.double()).abs().max() < tol(dtype, 4)
    rms = (got[:, :, :dim].float() ** 2).mean(-1).sqrt()
    assert (rms - 1).abs().max() < (1e-3 if dtype == torch.float32 else 2e-2)  # every head has a root mean square of one
    whole_projection = REF.proj_norm_rope_write(qkv, bias, slots, None, None, None, 0, 1e-5, kv_want.clone(), nq, nkv, dim, vdim, True, False)
    if nq > 1:
        assert (whole_projection.double() - want.double()).abs().max() > 0.5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P,rank,rot,H,lens,pasts", [(16, 96, 8, 5, [7, 1, 1], [0, 40, 300]), (4, 40, 12, 3, [33, 2, 1], [5, 0, 17]),
                                                     (16, 64, 32, 8, [1, 1, 1, 1], [0, 31, 32, 700]), (32, 512, 64, 16, [40, 1, 1], [100, 1900, 333])])
def test_latent_attention_without_a_sink(dtype, P, rank, rot, H, lens, pasts):
    """An ordinary softmax: nothing but the keys in the sum, in both kernels, with and without key ranges; with a
    sink far below every score the result is the same."""
    o = ops()
    c = latent_case(dtype, P, rank, rot, H, lens, pasts, 21, pages_total=160)
    N = c["N"]
    q_rot = rnd((N, H, rot), torch.float32, 23)
    for q_dtype in {torch.float32, dtype}:
        q_lat = rnd((H, N, rank), q_dtype, 24, 0.3).transpose(0, 1)
        args = [q_lat, q_rot, c["pages"], P, rank, rot, c["table"], c["seq_slots"], c["cu"], c["kv_lens"], c["token_seq"],
                None, None, 0.11, max(lens), max(c["kv_lens"].tolist()), dtype]
        want = REF.latent_attention(*args)
        got = o.latent_attention(*args)
        assert (got.double() - want.double()).abs().max() < tol(dtype, 2)
        args[11] = torch.full((H,), -80.0).cuda()
        assert (o.latent_attention(*args).double() - got.double()).abs().max() < tol(dtype, 0.5)
    # a single key: the softmax gives it all the weight, whatever its score
    one = latent_case(dtype, P, rank, rot, H, [1], [0], 5)
    q_lat = rnd((1, H, rank), dtype, 6, 0.01)
    got = o.latent_attention(q_lat, rnd((1, H, rot), torch.float32, 7, 0.01), one["pages"], P, rank, rot, one["table"], one["seq_slots"],
                             one["cu"], one["kv_lens"], one["token_seq"], None, None, 1.0, 1, 1, dtype)
    page = int(one["table"][int(one["seq_slots"][0]), 0])
    assert (got[0].float() - one["pages"][page, :rank].float()).abs().max() < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES + ["bfloat16 queries"])
@pytest.mark.parametrize("far", [3, 15, 16, 597])
def test_latent_attention_without_a_sink_one_key_among_hundreds(dtype, far):
    """One key (near the start, on both sides of a page's border, near the end) is made to carry the softmax of a
    decoded token after 600 others: the result is that key's latent row."""
    o = ops()
    P, rank, rot, H = 16, 64, 8, 2
    q_dtype = torch.float32 if dtype != "bfloat16 queries" else torch.bfloat16  # (the latter: the matrix-core kernel)
    dtype = torch.bfloat16 if dtype == "bfloat16 queries" else dtype
    c = latent_case(dtype, P, rank, rot, H, [1], [600], 31)
    page = int(c["table"][int(c["seq_slots"][0]), far // P])
    row = c["pages"][page, (far % P) * rank : (far % P + 1) * rank].float()
    q_lat = (row * 40.0 / (row * row).sum()).view(1, 1, rank).repeat(1, H, 1).contiguous().to(q_dtype)
    q_rot = torch.zeros((1, H, rot), dtype=torch.float32).cuda()
    args = [q_lat, q_rot, c["pages"], P, rank, rot, c["table"], c["seq_slots"], c["cu"], c["kv_lens"], c["token_seq"], None,
            None, 1.0, 1, 601, dtype]
    got = o.latent_attention(*args)
    assert (got.double() - REF.latent_attention(*args).double()).abs().max() < tol(dtype)
    assert (got[0, 0].float() - row).abs().max() < 0.05 and (got[0, 1].float() - row).abs().max() < 0.05


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("E,top,groups,keep,group_top", [(12, 4, 4, 3, 2), (10, 3, 2, 1, 2), (70, 5, 7, 2, 3), (6, 1, 6, 1, 2), (64, 6, 8, 8, 2),
                                                         (9, 3, 3, 2, 1)])
def test_sigmoid_router_with_groups_worth_their_largest_scores(E, top, groups, keep, group_top):
    o = ops()
    logits = rnd((37, E), torch.float32, 1, 2.0)
    ids, gains = o.moe_route_grouped(logits, None, top, groups, keep, score="sigmoid", group_top=group_top)
    wi, wg = REF.moe_route_grouped(logits, None, top, groups, keep, score="sigmoid", group_top=group_top)
    assert torch.equal(ids, wi)
    assert (gains.double() - wg.double()).abs().max() < 1e-6
    assert (gains.sum(-1) - 1).abs().max() < 1e-5


def test_sigmoid_router_a_group_of_two_good_experts_beats_the_group_of_the_best_and_ties():
    o = ops()
    z = torch.tensor([[2.0, -1.0, 0.5, 0.3, 1.9, 1.0]]).cuda()
    ids, gains = o.moe_route_grouped(z, None, 2, 2, 1, score="sigmoid", group_top=2)
    assert ids.tolist() == [[4, 5]]
    s = torch.sigmoid(z[0, [4, 5]])
    assert (gains[0] - s / s.sum()).abs().max() < 1e-6
    ids, _ = o.moe_route_grouped(z, None, 2, 2, 1, score="sigmoid", group_top=1)  # by their best expert alone: group 0
    assert ids.tolist() == [[0, 2]]
    same = torch.zeros((2, 8)).cuda()  # every score one half: the lower index wins, among groups and among experts
    ids, gains = o.moe_route_grouped(same, None, 3, 4, 2, score="sigmoid", group_top=2)
    assert ids.tolist() == [[0, 1, 2]] * 2 and torch.allclose(gains, torch.full((2, 3), 1 / 3).cuda())


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,K,F,H,E,top,limit", [(3, 72, 24, 72, 5, 2, 1.0), (200, 72, 24, 72, 5, 4, 0.5), (150, 64, 100, 40, 3, 1, 7.0),
                                                 (7, 50, 9, 33, 4, 4, 1.5)])
def test_clamped_experts(dtype, N, K, F, H, E, top, limit):
    """Few pairs take the per-pair kernels, many bfloat16 pairs the tiles; the products are large enough for the
    limits to bite on the gate from above and on the other branch from both sides."""
    o = ops()
    x = rnd((N, K), dtype, 1)
    gate_up, down = rnd((E, 2 * F, K), dtype, 2, 0.4), rnd((E, H, F), dtype, 3, 0.2)
    g = torch.Generator().manual_seed(4)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(N)]).to(torch.int32).cuda()
    gains = torch.rand((N, top), generator=g).cuda()
    want = REF.moe_experts(x, ids, gains, gate_up, down, form="gated_clamp", limit=limit)
    got = o.moe_experts(x, ids, gains, gate_up, down, form="gated_clamp", limit=limit)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    unclamped = REF.moe_experts(x, ids, gains, gate_up, down, form="gated_clamp", limit=1e9)
    assert (unclamped.double() - want.double()).abs().max() > 0.05


@pytest.mark.parametrize("H", [6, 80, 1536])
def test_norm_of_32_bit_rows_handed_on_in_bfloat16(H):
    o = ops()
    x = rnd((9, H), torch.float32, 1, 3.0)
    w = (1.0 + rnd((H,), torch.float32, 2, 0.1)).to(torch.bfloat16)
    got = o.rmsnorm(x, w, 1e-5, out_dtype=torch.bfloat16)
    want = REF.rmsnorm(x, w, 1e-5, out_dtype=torch.bfloat16)
    assert got.dtype == torch.bfloat16 and (got.double() - want.double()).abs().max() < tol(torch.bfloat16, 4)
    same = o.rmsnorm(x, w, 1e-5, out_dtype=torch.float32)
    assert same.dtype == torch.float32 and (same.double() - REF.rmsnorm(x, w, 1e-5).double()).abs().max() < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("F", [24, 37])
def test_gelu_in_its_tanh_form(dtype, F):
    o = ops()
    z = rnd((13, 2 * F), dtype, 1, 2.0)
    got = o.bias_act(z, "gelu_tanh", gated=True)
    want = REF.bias_act(z, "gelu_tanh", gated=True)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    zz = z.double()
    by_hand = 0.5 * zz[:, :F] * (1 + torch.tanh(0.7978845608028654 * (zz[:, :F] + 0.044715 * zz[:, :F] ** 3))) * zz[:, F:]
    assert (want.double() - by_hand).abs().max() < tol(dtype, 4)
