"""Visadra on the CPU: the plain model's mechanisms pinned by their own invariants, the
configuration and the checkpoint, and the engine (cache, state slots, step function, scheduler,
trace replay) with substitute kernels against the plain model."""
import json
import math
import os

import pytest
import torch

from litellmengine_amd.config import ConfigError, VisadraConfig, load_config
from litellmengine_amd.config.registry import architecture_of
from litellmengine_amd.engine import LLMEngine, ModelRunner, StepEntry
from litellmengine_amd.cache import CacheManager
from litellmengine_amd.models import load_model
from litellmengine_amd.weights.loader import WeightError
from tests.plain import visadra_plain as plain
from tests.tiny import random_tokens
from tests.torch_ops import TorchOps
from tests.trace_util import TraceBuilder, changing_portions, check_dumps, mixed, tail_one_by_one, whole
from tests.visadra_util import CONFIGS, PAGE_SIZES, make_model_dir, plain_logits, rewrite, run_tool, sharpen


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed), dtype=torch.float64) * scale


# -- the plain model's mechanisms, each alone ------------------------------------------------
def test_plain_candidate_is_continuous_and_positive():
    u = torch.tensor([-30.0, -1.0, -1e-9, 0.0, 1e-9, 2.0], dtype=torch.float64)
    c = plain.mingru_candidate(u)
    assert (c > 0).all() and abs(float(c[2]) - 0.5) < 1e-8 and float(c[3]) == 0.5 and float(c[5]) == 2.5
    assert abs(float(c[1]) - 1 / (1 + math.e)) < 1e-12


def test_plain_mingru_state_is_a_running_mix_and_carries_over():
    w = {"m.z": rnd((6, 5), 1), "m.z.b": rnd((6,), 2), "m.x": rnd((6, 5), 3), "m.x.b": rnd((6,), 4),
         "m.g": rnd((6, 5), 5), "m.o": torch.eye(6, dtype=torch.float64)}
    h = rnd((9, 5), 6)
    y = plain.mingru(h, w, "m.")
    # written out for the last token: S_8 = sum_t z_t c_t prod_{s > t} (1 - z_s)
    z = torch.sigmoid(h @ w["m.z"].T + w["m.z.b"])
    c = plain.mingru_candidate(h @ w["m.x"].T + w["m.x.b"])
    S = sum(z[t] * c[t] * torch.prod(1 - z[t + 1 :], dim=0) for t in range(9))
    assert torch.allclose(y[8], S * plain.silu(h[8] @ w["m.g"].T), atol=1e-12)
    # a gate of one forgets everything before, a gate of zero keeps the state
    w2 = dict(w)
    w2["m.z.b"] = torch.full((6,), 60.0, dtype=torch.float64)
    assert torch.allclose(plain.mingru(h, w2, "m.")[5], (c[5] * plain.silu(h[5] @ w["m.g"].T)), atol=1e-9)
    # the second half from the state after the first equals the whole
    s = torch.zeros(6, dtype=torch.float64)
    for t in range(4):
        s = (1 - z[t]) * s + z[t] * c[t]
    assert torch.allclose(plain.mingru(h[4:], w, "m.", state=s), y[4:], atol=1e-12)


def test_plain_rotation_pairs_neighbours_and_leaves_the_rest():
    x = rnd((5, 3, 10), 7)
    y = plain.rotate_interleaved(x, [0, 1, 2, 3, 40], 100.0, 6)
    assert torch.equal(y[0], x[0]) and torch.equal(y[..., 6:], x[..., 6:])
    for i in range(3):  # a rotation keeps every pair's length
        assert torch.allclose(y[..., 2 * i] ** 2 + y[..., 2 * i + 1] ** 2, x[..., 2 * i] ** 2 + x[..., 2 * i + 1] ** 2)
    a = 40 * 100.0 ** (-2.0 / 6)
    assert abs(float(y[4, 1, 2]) - float(x[4, 1, 2] * math.cos(a) - x[4, 1, 3] * math.sin(a))) < 1e-12
    # scores depend on the distance only
    q, k = rnd((1, 6), 8), rnd((1, 6), 9)
    d1 = plain.rotate_interleaved(q, [9], 100.0, 6) @ plain.rotate_interleaved(k, [4], 100.0, 6).T
    d2 = plain.rotate_interleaved(q, [105], 100.0, 6) @ plain.rotate_interleaved(k, [100], 100.0, 6).T
    assert torch.allclose(d1, d2, atol=1e-10)


def test_plain_sink_takes_weight_and_gives_nothing():
    scores, values = rnd((4, 4), 10), rnd((4, 3), 11)
    no_sink = plain.sink_softmax_attention(scores, values, torch.tensor(-1e9, dtype=torch.float64))
    for i in range(4):
        p = torch.softmax(scores[i, : i + 1], 0)
        assert torch.allclose(no_sink[i], p @ values[: i + 1], atol=1e-12)
    s = torch.tensor(0.3, dtype=torch.float64)
    with_sink = plain.sink_softmax_attention(scores, values, s)
    e = torch.exp(scores[2, :3])
    assert torch.allclose(with_sink[2], (e @ values[:3]) / (e.sum() + torch.exp(s)), atol=1e-12)
    assert torch.allclose(with_sink[0], values[0] * torch.exp(scores[0, 0]) / (torch.exp(scores[0, 0]) + torch.exp(s)))
    windowed = plain.sink_softmax_attention(scores, values, s, window=2)
    e = torch.exp(scores[3, 2:4])
    assert torch.allclose(windowed[3], (e @ values[2:4]) / (e.sum() + torch.exp(s)), atol=1e-12)


def test_plain_latent_attention_equals_per_head_attention_written_out():
    m = {"heads": 2, "dim": 4, "rot_dim": 6, "vdim": 3, "kv_rank": 5, "scale": 0.4, "rot": {"base": 30.0, "dims": 4}}
    w = {"a.q": rnd((20, 7), 12), "a.dkv": rnd((11, 7), 13), "a.dkv.norm": 1 + 0.1 * rnd((5,), 14), "a.uk": rnd((8, 5), 15),
         "a.uv": rnd((6, 5), 16), "a.sink": rnd((2,), 17), "a.o": torch.eye(6, dtype=torch.float64)}
    h = rnd((3, 7), 18)
    got = plain.latent_attention(h, w, "a.", m, 1e-5)
    # the last token, head 1, by hand
    dkv = h @ w["a.dkv"].T
    c = dkv[:, :5] / torch.sqrt((dkv[:, :5] ** 2).mean(-1, keepdim=True) + 1e-5) * w["a.dkv.norm"]
    kr = plain.rotate_interleaved(dkv[:, 5:], [0, 1, 2], 30.0, 4)
    q = (h[2] @ w["a.q"].T)[10:]
    qr = plain.rotate_interleaved(q[4:].view(1, 6), [2], 30.0, 4)[0]
    k = c @ w["a.uk"][4:].T
    v = c @ w["a.uv"][3:].T
    sc = (k @ q[:4] + kr @ qr) * 0.4
    e = torch.exp(sc)
    assert torch.allclose(got[2, 3:], (e @ v) / (e.sum() + torch.exp(w["a.sink"][1])), atol=1e-12)


def test_plain_router_weights_are_a_softmax_over_the_chosen_only():
    h, wr, b = rnd((6, 4), 19), rnd((5, 4), 20), rnd((5,), 21)
    idx, wt = plain.route(h, wr, b, 2)
    logits = h @ wr.T + b
    for t in range(6):
        order = torch.argsort(logits[t], descending=True)[:2]
        assert idx[t].tolist() == order.tolist()
        e = torch.exp(logits[t, order])
        assert torch.allclose(wt[t], e / e.sum())
    assert torch.allclose(plain.route(h, wr, b, 1)[1], torch.ones(6, 1, dtype=torch.float64))


# -- configuration and checkpoint ---------------------------------------------------------------
@pytest.mark.parametrize("which", list(CONFIGS))
def test_config_round_trip_and_registry(tmp_path, which):
    cfg = VisadraConfig.from_dict(CONFIGS[which])
    assert cfg.to_dict() == CONFIGS[which]
    assert architecture_of(CONFIGS[which]).name == "Visadra"
    d = make_model_dir(tmp_path, which)
    assert load_config(d) == cfg
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    assert len(model.blocks) == len(CONFIGS[which]["layers"]) and model.vocab_size == cfg.vocab


def test_config_defaults():
    """Without `scale` a head's scores are scaled by 1 / sqrt(dim + rot_dim); without `rot` the base is 10000 and
    every rotated element turns; without `embedding` and `logit_scale` nothing is scaled."""
    d = json.loads(json.dumps(CONFIGS["A"]))
    m = d["layers"][0]["mixer"]
    del m["scale"], m["rot"], d["embedding"], d["logit_scale"]
    cfg = VisadraConfig.from_dict(d)
    a = cfg.layers[0].mixer
    assert a.scale == (a.dim + a.rot_dim) ** -0.5 and a.rot_base == 10000.0 and a.rot_dims == a.rot_dim
    assert cfg.embedding_scale == 1.0 and cfg.logit_scale == 1.0


def test_config_faults_are_named():
    bad = json.loads(json.dumps(CONFIGS["A"]))
    bad["layers"][1]["type"] = "lstm"
    with pytest.raises(ConfigError, match="layers\\[1\\].type"):
        VisadraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["A"]))
    bad["layers"][0]["mlp"]["router"]["top"] = 9
    with pytest.raises(ConfigError, match="top"):
        VisadraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["A"]))
    bad["layers"][0]["mixer"]["rot"]["dims"] = 14
    with pytest.raises(ConfigError, match="rot.dims"):
        VisadraConfig.from_dict(bad)
    bad = json.loads(json.dumps(CONFIGS["A"]))
    del bad["norm"]
    with pytest.raises(ConfigError, match="norm"):
        VisadraConfig.from_dict(bad)


def test_checkpoint_faults_are_listed_together(tmp_path):
    from safetensors.torch import load_file, save_file

    d = make_model_dir(tmp_path, "C")
    path = os.path.join(d, "model.safetensors")
    t = load_file(path)
    del t["l2.mlp.e3.up"]
    t["l0.mix.sink"] = torch.zeros(4)
    t["l1.norm9"] = torch.zeros(())
    save_file(t, path)
    with pytest.raises(WeightError) as e:
        load_model(d, "float32", device="cpu", ops=TorchOps())
    assert "l2.mlp.e3.up" in str(e.value) and "l1.norm9" in str(e.value) and "l0.mix.sink" in str(e.value)


# -- the engine with substitute kernels -------------------------------------------------------
def cpu_runner(d, page_size, num_pages, max_requests=4):
    model = load_model(d, "float32", device="cpu", ops=TorchOps())
    cache = CacheManager(model, page_size=page_size, num_pages=num_pages, max_requests=max_requests,
                         dtype=torch.float32, device="cpu")
    return model, cache, ModelRunner(model, cache)


@pytest.mark.parametrize("which", list(CONFIGS))
def test_one_layer_at_a_time_follows_the_plain_model(tmp_path, which):
    """The residual stream after every block of a whole prompt."""
    d = make_model_dir(tmp_path, which)
    cfg, w = plain.read_model_dir(d)
    tokens = random_tokens(37, cfg["vocab"], 3)
    want = plain.residual_streams(tokens, w, cfg)
    model, cache, runner = cpu_runner(d, PAGE_SIZES[which], 16)
    seen = []
    for b in model.blocks:
        def wrapped(hidden, delta, step, layer_cache, next_norm=None, inner=b.forward):
            out = inner(hidden, delta, step, layer_cache, next_norm=next_norm)
            seen.append(hidden.double().clone())
            return out
        b.forward = wrapped
    runner.step([StepEntry(runner.admit(), tokens, [])])
    for i, (got, ref) in enumerate(zip(seen, want)):
        assert (got - ref).abs().max() < 1e-5, f"layer {i} ({cfg['layers'][i]['type']})"
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
    sharpen(d, 15.0, gates=15.0)
    vocab = CONFIGS[which]["vocab"]
    requests = {rid: random_tokens(n, vocab, 20 + i) for i, (rid, n) in enumerate(
        {"a": 70, "b": 45, "c": 100, "d": 33, "e": 64, "f": 1}.items())}
    tb = all_ways_trace(requests)
    out = str(tmp_path / "out")
    run_tool(d, "float32", out, tb, page_size=PAGE_SIZES[which], in_process_ops=TorchOps())
    check_dumps(out, tb, plain_logits(d, requests), 2e-5)


def test_state_rows_are_zeroed_when_a_slot_is_used_again(tmp_path):
    d = make_model_dir(tmp_path, "A")
    cfg, w = plain.read_model_dir(d)
    model, cache, runner = cpu_runner(d, 4, 12, max_requests=1)
    first, second = random_tokens(9, 131, 1), random_tokens(6, 131, 2)
    s = runner.admit()
    runner.step([StepEntry(s, first, [])])
    assert any(float(st[s].abs().max()) > 0 for st in cache.states.values())
    runner.release(s)
    s2 = runner.admit()
    assert s2 == s and all(float(st[s].abs().max()) == 0 for st in cache.states.values())
    got = runner.step([StepEntry(s2, second, [5])])
    assert (got[0].double() - plain.model_logits(second, w, cfg)[5]).abs().max() < 1e-5


@pytest.mark.parametrize("which", ["A", "C"])
def test_greedy_generation_through_the_scheduler(tmp_path, which):
    """Requests of unequal lengths batched, prompts in portions, then a pool so small that requests
    are preempted and recomputed (their state rows start from zero again): the same tokens."""
    d = make_model_dir(tmp_path, which)
    cfg, w = plain.read_model_dir(d)
    prompts = [random_tokens(n, cfg["vocab"], 40 + i) for i, n in enumerate((1, 7, 23, 40))]
    want = [plain.generate_greedy(p, w, cfg, 6) for p in prompts]
    for run_ahead in (False, True):
        model = load_model(d, "float32", device="cpu", ops=TorchOps())
        eng = LLMEngine(model, page_size=8, num_pages=16, max_requests=4, prefill_chunk=16, max_tokens_per_step=24,
                        run_ahead=run_ahead)
        assert eng.generate(prompts, 6) == want
    small = LLMEngine(load_model(d, "float32", device="cpu", ops=TorchOps()), page_size=8, num_pages=8, max_requests=4,
                      prefill_chunk=16, max_tokens_per_step=24, run_ahead=False)
    assert small.generate(prompts, 6) == want
    assert all(g.pool.num_held == 0 for g in small.cache.groups)
