"""The kernels that Kezasun added (the recurrence with a matrix state, projections normed as a whole,
sinks in the attention kernels, gates per head, the group-limited router, identity experts, the
scaled add with its norm), each alone against its plain torch form (tests/torch_ops.py), in float32
and bfloat16, at sizes that are no powers of two."""
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
@pytest.mark.parametrize("H", [40, 1000, 9000])
@pytest.mark.parametrize("pair", [False, True])
def test_scaled_add_rmsnorm(dtype, H, pair):
    o = ops()
    hidden = rnd((7, H), torch.float32, 2, 3.0)
    a = rnd((7, H), dtype, 3)
    b = rnd((7, H), torch.float32, 4) if pair else None
    w = (1.0 + rnd((H,), torch.float32, 5, 0.1))
    want_h = hidden.clone()
    want = REF.scaled_add_rmsnorm(want_h, a, b, 0.3, w, 1e-5, dtype)
    got = o.scaled_add_rmsnorm(hidden, a, b, 0.3, w, 1e-5, dtype)
    assert (hidden.double() - want_h.double()).abs().max() < 2e-6
    assert got.dtype == dtype and (got.double() - want.double()).abs().max() < tol(dtype, 4)
    # chosen rows only: the stream is left alone
    rows = ints([5, 0, 5])
    before = hidden.clone()
    want = REF.scaled_add_rmsnorm(hidden.clone(), a, b, -1.5, w, 1e-5, dtype, rows)
    got = o.scaled_add_rmsnorm(hidden, a, b, -1.5, w, 1e-5, dtype, rows)
    assert torch.equal(hidden, before) and got.shape == (3, H)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)


@pytest.mark.parametrize("dtype", DTYPES)
def test_head_gate_and_tanh(dtype):
    o = ops()
    a = rnd((9, 5 * 32), dtype, 1)
    gates = rnd((9, 23), dtype, 2, 2.0)
    got = o.head_gate(a, gates, 18, 5, 20)
    want = REF.head_gate(a, gates, 18, 5, 20)
    assert got.shape == (9, 100) and (got.double() - want.double()).abs().max() < tol(dtype)
    x = rnd((6, 17), dtype, 3, 2.0)
    want = REF.tanh_(x.clone())
    assert o.tanh_(x) is x and (x.double() - want.double()).abs().max() < tol(dtype)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("nq,nkv,dim,vdim,rot,D,own", [(6, 2, 24, 40, 8, 64, True), (4, 4, 64, 64, 64, 64, True),
                                                       (3, 1, 48, 16, 0, 64, True), (8, 2, 32, 32, 16, 32, False)])
def test_projection_norm_rotation_and_cache_write(dtype, nq, nkv, dim, vdim, rot, D, own):
    o = ops()
    N, P, pages = 11, 16, 5
    cols = nq * dim + (nkv * (dim + vdim) if own else 0) + nq
    qkv = rnd((N, cols), dtype, 1)
    bias = rnd((cols,), dtype, 2, 0.5)
    qw, kw = rnd((nq * dim,), torch.float32, 3) + 1.0, rnd((nkv * dim,), torch.float32, 4) + 1.0
    pos = ints([0, 1, 2, 700, 5, 6, 7, 8, 9, 100000, 11])
    inv = torch.pow(torch.tensor(1e4, dtype=torch.float64), -torch.arange(rot // 2, dtype=torch.float64) * 2 / max(rot, 1))
    cs = o.rope_table(pos, inv.float().cuda()) if rot else None
    slots = ints([3, 17, 18, 79, -1, 0, 33, 34, 35, 64, 5])
    kv_got = torch.full((pages + 1, 2, nkv, P, D), 7.0, dtype=dtype).cuda()
    kv_want = kv_got.clone()
    want = REF.proj_norm_rope_write(qkv, bias, slots, qw, kw, cs, rot, 1e-5, kv_want, nq, nkv, dim, vdim, own, own)
    got = o.proj_norm_rope_write(qkv, bias, slots, qw, kw if own else None, cs, rot, 1e-5, kv_got, nq, nkv, dim, vdim, own, own)
    assert got.shape == (N, nq, D)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    assert (kv_got.double() - kv_want.double()).abs().max() < tol(dtype, 4)
    if dim < D:
        assert float(got[:, :, dim:].abs().max()) == 0.0


def paged_setup(dtype, q_lens, pasts, nq, nkv, D, P, seed, sharp=None):
    """A cache with scrambled pages holding `past + q_len` keys per request, and the step's queries."""
    S = len(q_lens)
    seq_slots, cu, token_seq, N = batch(q_lens)
    kv_lens = [p + n for p, n in zip(pasts, q_lens)]
    max_pages = max(-(-l // P) for l in kv_lens) + 1
    total = sum(-(-l // P) for l in kv_lens)
    perm = torch.randperm(total + 3, generator=torch.Generator().manual_seed(seed)).tolist()
    table = torch.full((9, max_pages), -1, dtype=torch.int32)
    for s in range(S):
        for lp in range(-(-kv_lens[s] // P)):
            table[int(seq_slots[s]), lp] = perm.pop()
    kv = rnd((total + 4, 2, nkv, P, D), dtype, seed + 1)
    q = rnd((N, nq, D), dtype, seed + 2)
    if sharp is not None:  # one key of one request stands out for one head
        s, key, head = sharp
        page, off = int(table[int(seq_slots[s]), key // P]), key % P
        row = int(cu[s + 1]) - 1
        kv[page, 0, head // (nq // nkv), off] = (q[row, head].float() * 6.0).to(dtype)
    return q, kv, table.cuda(), seq_slots, cu, ints(kv_lens), token_seq, max(q_lens), max(kv_lens)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("D,P,nq,nkv", [(64, 16, 8, 2), (32, 16, 3, 3), (96, 32, 4, 1), (48, 8, 4, 2)])
@pytest.mark.parametrize("window", [None, 33])
def test_attention_with_sinks(dtype, D, P, nq, nkv, window):
    """Prompt portions, decoded tokens and long pasts (key splits) in one batch; every kernel that the sizes
    reach adds the sink's share once."""
    o = ops()
    q_lens, pasts = [1, 40, 1, 7, 130], [700, 0, 5, 90, 300]
    q, kv, table, seq_slots, cu, kv_lens, token_seq, mq, mk = paged_setup(dtype, q_lens, pasts, nq, nkv, D, P, 5)
    sinks = torch.tensor([0.0, 1.5, -2.0, 0.3, 0.0, 4.0, -0.7, 0.0][:nq]).cuda()
    scale = 0.35
    for sk in (sinks, torch.zeros(nq).cuda(), None):
        want = REF.paged_attention(q, kv, table, seq_slots, cu, kv_lens, token_seq, window, scale, sinks=sk)
        got = o.paged_attention(q, kv, table, seq_slots, cu, kv_lens, token_seq, window, scale, 1, mq, mk, sinks=sk)
        assert (got.double() - want.double()).abs().max() < tol(dtype, 2)
    # a sink that outweighs every key leaves next to nothing
    got = o.paged_attention(q, kv, table, seq_slots, cu, kv_lens, token_seq, window, scale, 1, mq, mk,
                            sinks=torch.full((nq,), 60.0).cuda())
    assert float(got.float().abs().max()) < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_far_key_and_the_windows_edge_with_a_sink(dtype):
    """One key made to carry the softmax: hundreds back without a window, just inside and just outside one."""
    o = ops()
    nq, nkv, D, P = 4, 2, 64, 16
    zeros = torch.zeros(nq).cuda()
    for window, key, seen in ((None, 3, True), (200, 1000 - 200, True), (200, 1000 - 201, False)):
        q, kv, table, seq_slots, cu, kv_lens, token_seq, mq, mk = paged_setup(dtype, [1, 1], [999, 50], nq, nkv, D, P, 9,
                                                                              sharp=(0, key, 2))
        want = REF.paged_attention(q, kv, table, seq_slots, cu, kv_lens, token_seq, window, 0.125, sinks=zeros)
        got = o.paged_attention(q, kv, table, seq_slots, cu, kv_lens, token_seq, window, 0.125, 1, mq, mk, sinks=zeros)
        assert (got.double() - want.double()).abs().max() < tol(dtype, 2)
        page, off = int(table[int(seq_slots[0]), key // P]), key % P
        value = v_pages(kv)[page, 1, :, off].double()
        carried = (got[0].view(nq, D)[2].double() - value).abs().max() < 0.05
        assert bool(carried) == seen


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("E,top,groups,keep", [(12, 4, 4, 3), (8, 8, 1, 1), (70, 5, 7, 2), (6, 1, 6, 1), (64, 6, 8, 8)])
def test_group_limited_router(E, top, groups, keep):
    o = ops()
    logits = rnd((37, E), torch.float32, 1, 2.0)
    correction = rnd((E,), torch.float32, 2, 0.3)
    ids, gains = o.moe_route_grouped(logits, correction, top, groups, keep)
    wi, wg = REF.moe_route_grouped(logits, correction, top, groups, keep)
    assert torch.equal(ids, wi)
    assert (gains.double() - wg.double()).abs().max() < 1e-6
    assert (gains.sum(-1) - 1).abs().max() < 1e-5


def test_router_ties_and_negative_choice_scores():
    """Equal scores: the lower index wins, among groups and among experts; a group that is left out stays out
    although every choice score in the kept groups is negative."""
    o = ops()
    logits = torch.zeros((3, 8)).cuda()  # every score 1/8
    ids, gains = o.moe_route_grouped(logits, torch.zeros(8).cuda(), 3, 4, 2)
    assert ids.tolist() == [[0, 1, 2]] * 3 and torch.allclose(gains, torch.full((3, 3), 1 / 3).cuda())
    correction = torch.tensor([-5.0, -6.0, -7.0, -5.5, -9.0, -9.0, -9.5, -9.0]).cuda()
    ids, _ = o.moe_route_grouped(logits, correction, 3, 4, 2)
    assert ids.tolist() == [[0, 3, 1]] * 3  # groups 0 and 1; never an expert of groups 2 and 3


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N", [3, 200])
def test_experts_with_identity_experts(dtype, N):
    """Ids from E on hand the input on; few pairs take the per-pair kernels, many bfloat16 pairs the tiles."""
    o = ops()
    E, I, top, K, F = 5, 3, 4, 72, 24
    x = rnd((N, K), dtype, 1)
    gate_up, down = rnd((E, 2 * F, K), dtype, 2, 0.2), rnd((E, K, F), dtype, 3, 0.2)
    g = torch.Generator().manual_seed(4)
    ids = torch.stack([torch.randperm(E + I, generator=g)[:top] for _ in range(N)]).to(torch.int32).cuda()
    ids[0] = torch.tensor([E, E + 1, E + 2, 0])
    gains = torch.rand((N, top), generator=g).cuda()
    want = REF.moe_experts(x, ids, gains, gate_up, down)
    got = o.moe_experts(x, ids, gains, gate_up, down)
    assert (got.double() - want.double()).abs().max() < tol(dtype, 2)


# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", DTYPES)
def test_shift_mix(dtype):
    o = ops()
    seq_slots, cu, token_seq, N = batch([1, 5, 2])
    W, off = 40, 24
    x = rnd((N, W), dtype, 1)
    state = rnd((9, off + W), torch.float32, 2)
    mu = rnd((5, W), torch.float32, 3)
    want = REF.shift_mix(x, state, off, mu, token_seq, cu, seq_slots)
    got = o.shift_mix(x, state, off, mu, token_seq, cu, seq_slots)
    assert got.shape == (5, N, W) and (got.double() - want.double()).abs().max() < tol(dtype)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,dim", [(3, 24), (2, 64), (1, 100), (5, 16), (1, 160), (2, 256)])
@pytest.mark.parametrize("q_lens", [[1, 1, 1], [9, 1, 30], [200, 3, 139]])
def test_wkv_scan(dtype, H, dim, q_lens):
    """Single tokens, short portions and portions long enough to be cut into pieces, from a state that is not
    zero; the state and the saved input row are advanced."""
    o = ops()
    seq_slots, cu, token_seq, N = batch(q_lens)
    HD, W = H * dim, 56
    r, k, v = (rnd((N, HD), torch.float32, s, 0.5) for s in (1, 2, 3))
    wraw = rnd((N, HD), torch.float32, 4) - 1.0
    w0, u = rnd((HD,), torch.float32, 5, 0.5), rnd((HD,), torch.float32, 6, 0.5)
    g, x = rnd((N, HD), dtype, 7), rnd((N, W), dtype, 8)
    norm_w = rnd((HD,), torch.float32, 9) + 1.0
    state = rnd((9, HD * dim + W), torch.float32, 10, 0.3)
    want_state = state.clone()
    want = REF.wkv_scan(r, k, v, wraw, w0, u, g, norm_w, 1e-5, x, want_state, H, dim, seq_slots, cu, dtype)
    got = o.wkv_scan(r, k, v, wraw, w0, u, g, norm_w, 1e-5, x, state, H, dim, seq_slots, cu, dtype, max(q_lens))
    assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
    assert (state.double() - want_state.double()).abs().max() < 2e-4
    # a walk in one go and a walk in pieces agree
    state2 = want_state.clone()
    state3 = want_state.clone()
    a = o.wkv_scan(r, k, v, wraw, w0, u, g, norm_w, 1e-5, x, state2, H, dim, seq_slots, cu, dtype, 0)
    b = o.wkv_scan(r, k, v, wraw, w0, u, g, norm_w, 1e-5, x, state3, H, dim, seq_slots, cu, dtype, 10 * o.WKV_PIECE)
    assert (a.double() - b.double()).abs().max() < tol(dtype, 4) and (state2 - state3).abs().max() < 2e-4


def test_wkv_decay_that_forgets_at_once_and_one_that_never_does():
    """A decay of about zero leaves only the last token's k v^T; a decay of one adds them all up."""
    o = ops()
    H, dim, T, W = 1, 16, 70, 8
    seq_slots, cu, token_seq, N = batch([T])
    r, k, v = (rnd((N, dim), torch.float32, s) for s in (1, 2, 3))
    zeros = torch.zeros(dim).cuda()
    g, x = rnd((N, dim), torch.float32, 7), rnd((N, W), torch.float32, 8)
    for raw, expect in ((5.0, lambda: torch.outer(k[-1], v[-1])), (-40.0, lambda: k.T @ v)):
        state = torch.zeros((9, dim * dim + W)).cuda()
        o.wkv_scan(r, k, v, torch.full((N, dim), raw).cuda(), zeros, zeros, g, zeros + 1, 1e-5, x, state, H, dim, seq_slots,
                   cu, torch.float32, T)
        S = state[int(seq_slots[0]), : dim * dim].view(dim, dim)
        assert (S - expect()).abs().max() < 1e-4
        assert torch.equal(state[int(seq_slots[0]), dim * dim :], x[-1])
