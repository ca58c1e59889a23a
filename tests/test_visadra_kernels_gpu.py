"""The kernels of the gated recurrence, of latent attention, of the routed feed-forward and of
the output-norm arrangement, each alone against its plain torch form (tests/torch_ops.py), in
float32 and bfloat16, at sizes that are no powers of two."""
import pytest
import torch

from tests.torch_ops import TorchOps

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


@pytest.mark.parametrize("dtype", DTYPES)
def test_embedding_scale_cast_and_logit_scale(dtype):
    o = ops()
    table = rnd((97, 72), dtype, 1)
    ids = ints([0, 96, 5, 5])
    got = o.embedding(ids, table, scale=0.37)
    assert torch.allclose(got, table[ids.long()].float() * 0.37, rtol=1e-7, atol=0)
    assert torch.equal(o.cast(got, dtype), got.to(dtype))
    x = got.clone()
    assert o.scale_(x, 1.75) is x and torch.allclose(x, got * 1.75, rtol=1e-7, atol=0)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [40, 1000, 4100])
@pytest.mark.parametrize("with_extra", [False, True])
def test_rmsnorm_add(dtype, H, with_extra):
    o = ops()
    hidden = rnd((7, H), torch.float32, 2, 3.0)
    y = rnd((7, H), torch.float32 if with_extra else dtype, 3)
    extra = rnd((7, H), dtype, 4) if with_extra else None
    w = torch.full((H,), 1.3, dtype=dtype).cuda()
    want_h = hidden.clone()
    want = REF.rmsnorm_add(want_h, y, w, 1e-4, dtype, extra)
    got = o.rmsnorm_add(hidden, y, w, 1e-4, dtype, extra)
    assert (hidden.double() - want_h.double()).abs().max() < 2e-5
    assert got.dtype == dtype and (got.double() - want.double()).abs().max() < tol(dtype, 8)


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("lens,W", [([1, 1, 1], 40), ([5, 1, 70, 2], 300), ([300, 3], 264), ([1000], 72), ([5, 1, 70, 2], 43)])
def test_mingru_scan(dtype, lens, W):
    """Requests of unequal lengths in one launch, single tokens beside portions long enough to be cut
    into pieces; the state rows of other slots stay as they are, and a second step goes on from the first."""
    o = ops()
    N = sum(lens)
    slots = [3, 0, 5, 1][: len(lens)]
    cu = [0]
    for n in lens:
        cu.append(cu[-1] + n)
    state = rnd((7, W), torch.float32, 5)
    for step in range(2):
        zxg = rnd((N, 3 * W), torch.float32 if step == 0 else dtype, 6 + step, 2.0)
        bz, bx = rnd((W,), torch.float32, 8), rnd((W,), torch.float32, 9)
        want_state = state.clone()
        want = REF.mingru_scan(zxg, bz, bx, want_state, ints(slots), ints(cu), dtype)
        got = o.mingru_scan(zxg, bz, bx, state, ints(slots), ints(cu), dtype, max(lens))
        assert (got.double() - want.double()).abs().max() < tol(dtype, 4)
        assert (state - want_state).abs().max() < 2e-5
        untouched = [r for r in range(7) if r not in slots]
        assert torch.equal(state[untouched], want_state[untouched])


def latent_case(dtype, P, rank, rot, H, lens, pasts, seed, pages_total=64):
    """Pages in a scrambled order, requests with a past in the cache; returns what the kernels take."""
    g = torch.Generator().manual_seed(seed)
    S = len(lens)
    order = torch.randperm(pages_total, generator=g).tolist()
    max_pages = max((p + n + P - 1) // P for p, n in zip(pasts, lens))
    table = torch.full((S + 2, max_pages), -1, dtype=torch.int32)
    slots_of = [4 % (S + 2), 0, 2, 1][:S]
    slot_map, token_seq, cu = [], [], [0]
    for s, (n, past) in enumerate(zip(lens, pasts)):
        for lp in range((past + n + P - 1) // P):
            table[slots_of[s], lp] = order.pop()
        for t in range(past, past + n):
            slot_map.append(int(table[slots_of[s], t // P]) * P + t % P)
            token_seq.append(s)
        cu.append(cu[-1] + n)
    pages = rnd((pages_total + 1, P * (2 * rank + rot) + 8), dtype, seed + 1)[:, : P * (2 * rank + rot)]  # rows with a stride of their own
    latents = pages[:, : P * rank].unflatten(1, (P, rank))  # the transposed part holds the same latents
    pages[:, P * rank : 2 * P * rank] = latents.transpose(1, 2).reshape(pages_total + 1, P * rank)
    kv_lens = [p + n for p, n in zip(pasts, lens)]
    positions = [t for n, past in zip(lens, pasts) for t in range(past, past + n)]
    return dict(table=table.cuda(), slots=ints(slot_map), token_seq=ints(token_seq), cu=ints(cu), seq_slots=ints(slots_of),
                kv_lens=ints(kv_lens), pages=pages, positions=ints(positions), N=sum(lens))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P,rank,rot,rot_dims", [(16, 96, 8, 8), (4, 40, 12, 6), (32, 520, 64, 64), (8, 24, 4, 0)])
def test_latent_kv_write_and_q_rope(dtype, P, rank, rot, rot_dims):
    o = ops()
    c = latent_case(dtype, P, rank, rot, 3, [5, 1, 9], [0, 17, 30], 11)
    N = c["N"]
    c["slots"][2] = -1  # a row that stands for nobody writes nothing
    dkv = rnd((N, rank + rot), dtype, 12)
    w = (1 + 0.1 * rnd((rank,), torch.float32, 13)).to(dtype)
    inv = torch.pow(torch.tensor(777.0, dtype=torch.float64), -2.0 * torch.arange(rot_dims // 2, dtype=torch.float64) / max(1, rot_dims))
    cos_sin = o.rope_table(c["positions"], inv.float().cuda()) if rot_dims else None
    want = c["pages"].clone()
    REF.latent_kv_write(dkv, w, 1e-5, cos_sin, rot_dims, c["slots"], want, P, rank, rot)
    o.latent_kv_write(dkv, w, 1e-5, cos_sin, rot_dims, c["slots"], c["pages"], P, rank, rot)
    assert (c["pages"].double() - want.double()).abs().max() < tol(dtype, 4)
    H, dim = 3, 20
    q = rnd((N, H * (dim + rot)), dtype, 14)
    got = o.latent_q_rope(q, cos_sin, rot_dims, H, dim, rot)
    ref = REF.latent_q_rope(q, cos_sin, rot_dims, H, dim, rot)
    assert got.dtype == torch.float32 and (got.double() - ref.double()).abs().max() < 1e-5


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("P,rank,rot,H,lens,pasts,window", [
    (16, 96, 8, 5, [7, 1, 1], [0, 40, 300], None),
    (4, 40, 12, 3, [33, 2, 1], [5, 0, 17], None),
    (16, 136, 16, 6, [20, 1], [290, 511], 37),
    (32, 520, 64, 2, [3, 1], [250, 100], None),
    (16, 128, 16, 6, [50, 1, 3], [200, 499, 0], 70),
    (32, 512, 64, 16, [40, 1, 1], [100, 1900, 333], None),
    (16, 64, 32, 3, [1, 1, 1, 1], [0, 31, 32, 700], None),
    (48, 256, 40, 20, [9, 2], [470, 15], 100),
])
def test_latent_attention(dtype, P, rank, rot, H, lens, pasts, window):
    """Mixed steps over scrambled pages against the plain form; the sinks are large enough to count.
    Queries come in 32-bit and in the cache's type, with the strides that the batched product leaves
    (bfloat16 queries take the matrix-core kernel where it takes the sizes: the last four cases and the
    first; long pasts are cut into key ranges that are merged)."""
    o = ops()
    c = latent_case(dtype, P, rank, rot, H, lens, pasts, 21, pages_total=160)
    N = c["N"]
    sink = rnd((H,), torch.float32, 22, 2.0)
    q_rot = rnd((N, H, rot), torch.float32, 23)
    for q_dtype in {torch.float32, dtype}:
        q_lat = rnd((H, N, rank), q_dtype, 24, 0.3).transpose(0, 1)
        args = (q_lat, q_rot, c["pages"], P, rank, rot, c["table"], c["seq_slots"], c["cu"], c["kv_lens"], c["token_seq"],
                sink, window, 0.11, max(lens), max(c["kv_lens"].tolist()), dtype)
        want = REF.latent_attention(*args)
        on_cores = q_dtype == torch.bfloat16 and rank % 16 == 0 and rank <= 512 and rot % 8 == 0 and P % 16 == 0
        for row_tiles in ((0, 1, 2) if on_cores else (0,)):  # as the sizes choose; one and two 16-row tiles a workgroup
            o.force_latent_row_tiles = row_tiles
            try:
                got = o.latent_attention(*args)
            finally:
                o.force_latent_row_tiles = 0
            assert o.last_latent_kernel[0] == ("matrix cores" if on_cores else "generic")
            if on_cores and max(pasts) > 1000:
                assert o.last_latent_kernel[1] > 1  # key ranges, merged
            assert got.shape == (N, H, rank) and (got.double() - want.double()).abs().max() < tol(dtype, 2)


@pytest.mark.parametrize("dtype", DTYPES + ["bfloat16 queries"])
def test_latent_attention_one_far_key_and_the_sink(dtype):
    """One key far back is made to carry the softmax, then the sink is: the result is that key's
    latent row, then (almost) nothing."""
    o = ops()
    P, rank, rot, H = 16, 64, 8, 2
    q_dtype = torch.float32 if dtype != "bfloat16 queries" else torch.bfloat16  # (the latter: the matrix-core kernel)
    dtype = torch.bfloat16 if dtype == "bfloat16 queries" else dtype
    c = latent_case(dtype, P, rank, rot, H, [1], [600], 31)
    far = 3  # position of the key that stands out
    page = int(c["table"][int(c["seq_slots"][0]), far // P])
    row = c["pages"][page, (far % P) * rank : (far % P + 1) * rank].float()
    q_lat = (row * 40.0 / (row * row).sum()).view(1, 1, rank).repeat(1, H, 1).contiguous().to(q_dtype)
    q_rot = torch.zeros((1, H, rot), dtype=torch.float32).cuda()
    sink = torch.tensor([-30.0, -30.0]).cuda()
    args = [q_lat, q_rot, c["pages"], P, rank, rot, c["table"], c["seq_slots"], c["cu"], c["kv_lens"], c["token_seq"], sink,
            None, 1.0, 1, 601, dtype]
    got = o.latent_attention(*args)
    want = REF.latent_attention(*args)
    assert (got.double() - want.double()).abs().max() < tol(dtype)
    assert (got[0, 0].float() - row).abs().max() < 0.05  # the far key alone
    args[11] = torch.tensor([200.0, -30.0]).cuda()
    got = o.latent_attention(*args)
    assert got[0, 0].float().abs().max() < 1e-3 and (got[0, 1].float() - row).abs().max() < 0.05


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,xw,col0,K,O", [(3, 28, 0, 20, 40), (5, 36, 4, 32, 24), (2, 130, 0, 130, 7)])
def test_heads_linear(dtype, heads, xw, col0, K, O):
    o = ops()
    x = rnd((9, heads * xw), dtype, 41)
    w = rnd((heads, O, K), dtype, 42)
    for out_dtype in {torch.float32, dtype}:
        got = o.heads_linear(x, heads, col0, K, w, out_dtype)
        want = REF.heads_linear(x, heads, col0, K, w, out_dtype)
        assert got.shape == (9, heads, O) and got.dtype == out_dtype
        assert (got.double() - want.double()).abs().max() < tol(out_dtype, 4)


def test_moe_route_picks_the_largest_and_the_lower_index_among_equals():
    o = ops()
    logits = rnd((50, 11), torch.float32, 51)
    bias = rnd((11,), torch.float32, 52)
    logits[7] = 0.0
    logits[7, 4] = logits[7, 9] = 5.0 - bias[4]
    logits[7, 9] = 5.0 - bias[9]  # experts 4 and 9 tie at 5
    for top in (1, 2, 3, 11):
        ids, gains = o.moe_route(logits, bias, top)
        want_ids, want_gains = REF.moe_route(logits, bias, top)
        rows = [r for r in range(50) if r != 7]
        assert torch.equal(ids[rows], want_ids[rows])
        assert (gains.double() - want_gains.double())[rows].abs().max() < 1e-6
        assert int(ids[7, 0]) == 4 and (top == 1 or int(ids[7, 1]) == 9)
        assert (gains.sum(1) - 1).abs().max() < 1e-6


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("N,K,F,H,E,top", [(1, 72, 40, 72, 5, 2), (37, 200, 24, 200, 9, 3), (4, 64, 130, 64, 3, 3),
                                           (300, 128, 64, 128, 8, 2), (70, 200, 24, 204, 9, 3), (513, 96, 136, 100, 40, 6),
                                           (200, 64, 8, 64, 2, 1)])
def test_moe_experts(dtype, N, K, F, H, E, top):
    """Few pairs stream their experts' rows; from 129 bfloat16 pairs on they are sorted by expert and go through
    the matrix cores in tiles (the last four cases; experts with no pair, with one, with more than a tile)."""
    o = ops()
    x = rnd((N, K), dtype, 61)
    gate_up = rnd((E, 2 * F, K), dtype, 62, 0.2)
    down = rnd((E, H, F), dtype, 63, 0.2)
    ids, gains = o.moe_route(rnd((N, E), torch.float32, 64), torch.zeros(E).cuda(), top)
    got = o.moe_experts(x, ids, gains, gate_up, down)
    want = REF.moe_experts(x, ids, gains, gate_up, down)
    assert got.dtype == torch.float32 and (got.double() - want.double()).abs().max() < tol(dtype, 4)
