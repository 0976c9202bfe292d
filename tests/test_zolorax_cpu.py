"""Zolorax on the CPU: configuration, the model as data, the plain implementation's own
pins (each mechanism against a closed form or a crafted case), and the engine's cache
manager, state slots, batch builder and step function (with the plain torch kernel
references in place of the HIP kernels) against the plain whole-sequence implementation,
float32."""

import copy
import math

import pytest
import torch

import drives
from helpers import (ZOLO, ZOLO_A, ZOLO_B, random_prompt, write_zolorax_model, zolorax_attention,
                     zolorax_config, zolorax_dense, zolorax_moe, zolorax_rglru)
from kernel_refs import TorchOps
from plain import zolorax_plain as plain
from tokensprint_amd.config import ConfigError, ZoloraxConfig
from tokensprint_amd.config.registry import architecture_names, get_architecture
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import build_model, load_model
from tokensprint_amd.parts.base import PagedKVNeed, SlotStateNeed, flat_needs


@pytest.fixture(scope="module", params=sorted(ZOLO))
def setup(request, tmp_path_factory):
    cfg, seed, page = ZOLO[request.param]
    d = write_zolorax_model(tmp_path_factory.mktemp(f"zolo{request.param}"), cfg, seed,
                            torch.float32)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    lengths = [5, 11, 17, 40, 64, 1, 23]
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    return model, page, requests, ref


def runner_for(model, page, num_pages):
    return ModelRunner(model, page_size=page, num_pages=num_pages, num_slots=4)


TOL = (2e-4, 5e-5)


def test_whole(setup):
    model, page, requests, ref = setup
    drives.compare(drives.drive_whole(runner_for(model, page, 64 // page + 1), requests),
                   ref, *TOL)


def test_prefill_then_decode(setup):
    model, page, requests, ref = setup
    drives.compare(drives.drive_prefill_then_decode(runner_for(model, page, 64 // page + 1),
                                                    requests), ref, *TOL)


def test_portions(setup):
    model, page, requests, ref = setup
    drives.compare(drives.drive_portions(runner_for(model, page, 64 // page + 1), requests),
                   ref, *TOL)


def test_mixed_with_pages_and_slots_used_again(setup):
    model, page, requests, ref = setup
    runner = runner_for(model, page, 160 // page)
    drives.compare(drives.drive_mixed(runner, requests), ref, *TOL)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)
    assert runner.manager.slots.num_free == 4


def test_preempted_and_recomputed(setup):
    model, page, requests, ref = setup
    runner = runner_for(model, page, 160 // page)
    drives.compare(drives.drive_preempted(runner, requests), ref, *TOL)


# ------------------------------------------------------------------ configuration, spec


def test_config_reads_every_size():
    cfg = ZoloraxConfig.from_dict(ZOLO_A)
    assert (cfg.width, cfg.vocab_size, cfg.eps, len(cfg.layers)) == (40, 97, 1e-5, 5)
    a = cfg.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.window) == (4, 2, 12, 20, 0.4, 7)
    assert (a.rot_base, a.rot_dims) == (10000.0, 8)
    s = a.rot_scaling
    assert (s.factor, s.original, s.fast, s.slow) == (4.0, 64, 8.0, 1.0)
    assert a.kv_from is None and cfg.layers[2].mixer.kv_from == 0
    r = cfg.layers[1].mixer
    assert (r.width, r.blocks, r.conv) == (48, 4, 4)
    assert cfg.layers[1].mlp.ff == 56 and cfg.layers[2].mlp is None
    m = cfg.layers[0].mlp
    assert (m.ff, m.experts, m.top) == (12, 6, 2)
    b = ZoloraxConfig.from_dict(ZOLO_B)
    assert b.layers[2].mixer.window is None and b.layers[1].mixer.rot_scaling is None


def test_a_reader_runs_on_its_owners_cache_which_keeps_the_widest_window():
    arch = get_architecture("Zolorax")
    spec = arch.build_spec(arch.parse_config(ZOLO_A))
    assert [run.cache_of for run in spec.order] == [None, None, 0, None, 0]
    assert [run.layer for run in spec.order] == [0, 1, 2, 3, 4]
    _, model = build_model(ZOLO_A, "float32", "cpu", ops=TorchOps())
    needs = model.cache_needs()
    assert needs[2] is None and needs[4] is None
    # the owner sees 7 keys, its readers 19 and 3: the cache keeps 19
    assert needs[0] == PagedKVNeed(2, 32, 19)
    lru = flat_needs(needs[1])
    assert [type(n) for n in lru] == [SlotStateNeed, SlotStateNeed]
    assert {n.name: n.shape for n in lru} == {"lru.conv": (3, 48), "lru": (48,)}
    # the readers have no key/value tensors
    names = set(model.tensor_decls())
    assert {"l0.mix.k", "l0.mix.v", "l0.mix.k.norm"} <= names
    assert not {"l2.mix.k", "l2.mix.v", "l2.mix.k.norm", "l2.norm2"} & names
    assert {"l2.mix.q", "l2.mix.q.norm", "l2.mix.sink", "l2.mix.g", "l2.mix.o"} <= names
    # an owner that sees every key, beside one with a window: two groups of pages
    runner = ModelRunner(build_model(ZOLO_B, "float32", "cpu", ops=TorchOps())[1], page_size=8,
                         num_pages=4, num_slots=2)
    assert [(g.window, g.runs) for g in runner.storage.groups] == [(40, (1,)), (None, (2,))]


def _changed(path, value):
    cfg = copy.deepcopy(ZOLO_A)
    at = cfg
    for key in path[:-1]:
        at = at[key]
    if value is None:
        del at[path[-1]]
    else:
        at[path[-1]] = value
    return cfg


@pytest.mark.parametrize("path, value, message", [
    (("width",), None, "lacks 'width'"),
    (("norm", "eps"), 0, "positive"),
    (("layers", 0, "type"), "conv", "Zolorax has"),
    (("layers", 0, "mixer", "heads"), 3, "multiple of kv_heads"),
    (("layers", 0, "mixer", "rot", "dims"), 14, "even and at most dim"),
    (("layers", 1, "mixer", "blocks"), 5, "multiple of blocks"),
    (("layers", 2, "mixer", "kv_from"), 1, "earlier attention layer"),
    (("layers", 2, "mixer", "kv_from"), 4, "earlier attention layer"),
    (("layers", 2, "mixer", "dim"), 16, "differ"),
    (("layers", 0, "mlp", "router", "top"), 7, "cannot give"),
    (("layers", 1, "mlp", "kind"), "glu", "dense and moe"),
])
def test_config_errors(path, value, message):
    with pytest.raises(ConfigError, match=message):
        ZoloraxConfig.from_dict(_changed(path, value))


def test_a_reader_of_a_reader_is_refused():
    cfg = copy.deepcopy(ZOLO_A)
    cfg["layers"][4]["mixer"]["kv_from"] = 2
    with pytest.raises(ConfigError, match="keys and values of its own"):
        ZoloraxConfig.from_dict(cfg)


def test_random_weights_fit_the_declarations(tmp_path):
    d = write_zolorax_model(tmp_path, ZOLO_B, 3, torch.bfloat16)
    _, model = load_model(d, "bfloat16", "cpu", ops=TorchOps())
    # the norms' weights are stored around zero and held with the one added
    norm = model.blocks[0].mixer_norm
    assert norm.weight.dtype == torch.float32 and 0.6 < float(norm.weight.min()) \
        and float(norm.weight.max()) < 1.4


def test_the_architecture_is_registered_beside_the_others():
    assert {"Zolorax", "Palelix", "Zonopel", "Qwen3ForCausalLM"} <= set(architecture_names())


# ------------------------------------------------------------------ the plain mechanisms


def test_plain_norms():
    x = torch.tensor([[3.0, -4.0]], dtype=torch.float64)
    w = torch.tensor([0.5, -0.25], dtype=torch.float64)
    rms = math.sqrt(12.5 + 0.1)
    assert torch.allclose(plain.norm_one_plus(x, w, 0.1), x / rms * torch.tensor([1.5, 0.75]))
    assert torch.allclose(plain.norm_plain(x, w, 0.1), x / rms * w)


def test_plain_rotation_pairs_halves_and_leaves_the_rest():
    rot = {"base": 100.0, "dims": 4}
    x = torch.arange(1.0, 13.0, dtype=torch.float64).view(2, 1, 6)
    y = plain.rotate(x, rot)
    assert torch.equal(y[0], x[0])                     # position 0: nothing turns
    assert torch.equal(y[1, 0, 4:], x[1, 0, 4:])       # beyond the rotated dimensions
    for i, f in enumerate((1.0, 0.1)):                 # pair (i, i + 2), angle 1 * f
        u, v = x[1, 0, i], x[1, 0, i + 2]
        assert math.isclose(float(y[1, 0, i]), u * math.cos(f) - v * math.sin(f))
        assert math.isclose(float(y[1, 0, i + 2]), v * math.cos(f) + u * math.sin(f))


def test_plain_stretched_frequencies():
    rot = {"base": 10000.0, "dims": 8, "scaling": {"factor": 4.0, "original": 64, "fast": 8.0,
                                                    "slow": 1.0}}
    f, mult = plain.yarn_frequencies(rot)
    plain_f = 10000.0 ** (-2.0 * torch.arange(4, dtype=torch.float64) / 8)
    # d(8 turns) = 8 ln(64 / 16 pi) / (2 ln 1e4) = 0.105 -> lo 0; d(1 turn) = 1.008 -> hi 2
    ramp = torch.tensor([0.0, 0.5, 1.0, 1.0], dtype=torch.float64)
    assert torch.allclose(f, plain_f / 4.0 * ramp + plain_f * (1 - ramp))
    assert math.isclose(mult, 0.1 * math.log(4.0) + 1.0)
    assert plain.yarn_frequencies({"base": 10000.0, "dims": 8})[1] == 1.0


def _one_head(T, window, sink, scores_of=None):
    """A one-head attention layer whose queries and keys are made by hand: width 2, key i
    points along e0 with length given by the token, values are the tokens' second input."""
    m = {"heads": 1, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 1.0,
         "rot": {"base": 10.0, "dims": 2}, "mask": {"size": window}}
    eye = torch.eye(2, dtype=torch.float64)
    w = {"a.q": eye, "a.k": eye, "a.v": torch.tensor([[0.0, 1.0]], dtype=torch.float64),
         "a.q.norm": torch.ones(2, dtype=torch.float64), "a.k.norm": torch.ones(2, dtype=torch.float64),
         "a.sink": torch.tensor([sink], dtype=torch.float64),
         "a.g": torch.full((1, 2), 0.0, dtype=torch.float64),
         "a.o": torch.ones(2, 1, dtype=torch.float64)}
    return m, w


def test_plain_window_sees_exactly_its_size_and_the_sink_takes_its_share():
    T, window = 9, 4
    m, w = _one_head(T, window, sink=-1e9)
    m["rot"] = {"base": 10.0, "dims": 2}
    # every token's input: (1, t): equal queries and keys up to the rotation, which is the
    # same for q and k of equal positions only; with values t the output is a weighted mean
    h = torch.stack([torch.ones(T, dtype=torch.float64), torch.arange(T, dtype=torch.float64)], 1)
    kv = plain.attention_keys(h, w, "a.", m, 1e-6)
    out = plain.attention(h, w, "a.", m, 1e-6, kv)
    # gate = sigmoid(0) = 0.5, o = ones: out[t] = 0.5 * mean over the window, both columns
    for t in range(T):
        seen = list(range(max(0, t - window + 1), t + 1))
        assert min(seen) <= float(out[t, 0]) * 2 <= max(seen)
    # the very value: keys normed to equal length, so a score depends on the distance only
    q = plain.rotate(plain.norm_plain(h.view(T, 1, 2), w["a.q.norm"], 1e-6), m["rot"])[:, 0]
    t = 8
    s = torch.tensor([float(q[t] @ q[j]) for j in range(5, 9)], dtype=torch.float64)
    p = torch.softmax(s, 0)
    want = 0.5 * float(p @ torch.arange(5.0, 9.0, dtype=torch.float64))
    assert math.isclose(float(out[t, 0]), want, rel_tol=1e-9)
    # a sink as large as the largest score (q.k of a token with itself: the squared length
    # of a normed pair, about 2) takes its share of the weight and gives nothing back
    m2, w2 = _one_head(T, window, sink=float(q[t] @ q[t]))
    out2 = plain.attention(h, w2, "a.", m2, 1e-6, kv)
    p2 = torch.softmax(torch.cat([s, w2["a.sink"]]), 0)
    assert math.isclose(float(out2[t, 0]), 0.5 * float(p2[:4] @ torch.arange(5.0, 9.0, dtype=torch.float64)),
                        rel_tol=1e-9)
    assert float(out2[t, 0]) < float(out[t, 0])


def test_plain_recurrence_closed_form():
    """One channel a block, no convolution taps beyond the current token: with constant
    input the state is a geometric series."""
    width, T = 3, 6
    m = {"width": width, "blocks": 3, "conv": 1}
    z = lambda *s: torch.zeros(*s, dtype=torch.float64)
    w = {"r.y": z(width, 2), "r.y.b": torch.full((width,), 0.7, dtype=torch.float64),
         "r.x": z(width, 2), "r.x.b": torch.tensor([1.0, -2.0, 0.5], dtype=torch.float64),
         "r.conv": torch.full((width, 1), 2.0, dtype=torch.float64), "r.conv.b": torch.full((width,), 0.25, dtype=torch.float64),
         "r.ra": z(3, 1, 1), "r.ra.b": z(3, 1), "r.ri": z(3, 1, 1), "r.ri.b": z(3, 1),
         "r.lam": torch.tensor([-1.0, 0.0, 2.0], dtype=torch.float64),
         "r.o": torch.eye(width, dtype=torch.float64)}
    out = plain.rglru(z(T, 2), w, "r.", m)
    u = 2.0 * w["r.x.b"] + 0.25
    a = torch.exp(-8.0 * 0.5 * torch.log1p(torch.exp(w["r.lam"])))
    feed = torch.sqrt(1 - a * a) * 0.5 * u
    y = 0.7
    gelu = 0.5 * y * (1 + math.tanh(math.sqrt(2 / math.pi) * (y + 0.044715 * y ** 3)))
    for t in range(T):
        S = feed * (1 - a ** (t + 1)) / (1 - a)
        assert torch.allclose(out[t], S * gelu, rtol=1e-12, atol=1e-14)


def test_plain_convolution_starts_behind_zeros():
    x = torch.tensor([[1.0], [2.0], [3.0]], dtype=torch.float64)
    wgt = torch.tensor([[100.0, 10.0, 1.0]], dtype=torch.float64)
    out = plain.causal_conv(x, wgt, torch.tensor([0.5], dtype=torch.float64))
    assert out.view(-1).tolist() == [1.5, 12.5, 123.5]


def test_plain_experts_weigh_what_they_read():
    torch.manual_seed(0)
    W, ff, E = 4, 3, 3
    w = {"m.router": torch.tensor([[5.0, 0, 0, 0], [0, 5.0, 0, 0], [0, 0, 5.0, 0]], dtype=torch.float64)}
    for e in range(E):
        for n, shape in (("gate", (ff, W)), ("up", (ff, W)), ("down", (W, ff))):
            w[f"m.e{e}.{n}"] = torch.randn(shape, dtype=torch.float64)
    h = torch.tensor([[1.0, 0.2, -1.0, 0.3]], dtype=torch.float64)
    out = plain.routed_ff(h, w, "m.", {"router": {"experts": E, "top": 2}})
    want = torch.zeros(W, dtype=torch.float64)
    for e in (0, 1):                                   # logits 5, 1, -5: experts 0 and 1
        s = 1 / (1 + math.exp(-5.0 * float(h[0, e])))
        x = s * h[0]                                   # the score as it is, on the input
        g, u = w[f"m.e{e}.gate"] @ x, w[f"m.e{e}.up"] @ x
        want += w[f"m.e{e}.down"] @ (g / (1 + torch.exp(-g)) * u)
    assert torch.allclose(out[0], want)
    z = torch.tensor([[-1.0, 0.0, 2.0]], dtype=torch.float64)
    assert torch.allclose(plain.dense_ff(z, {"d.up": torch.eye(3, dtype=torch.float64),
                                             "d.down": torch.eye(3, dtype=torch.float64)}, "d."),
                          torch.tensor([[0.0, 0.0, 4.0]], dtype=torch.float64))


# ------------------------------------------------------------------ other arrangements


def _run_drives(cfg, seed, page, tmp_path, lengths=(9, 30, 1, 18)):
    d = write_zolorax_model(tmp_path, cfg, seed, torch.float32)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 50 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    drives.compare(drives.drive_whole(runner_for(model, page, 40), requests), ref, *TOL)
    drives.compare(drives.drive_portions(runner_for(model, page, 40), requests), ref, *TOL)
    drives.compare(drives.drive_mixed(runner_for(model, page, 40), requests), ref, *TOL)


def test_only_recurrent_layers_without_a_cache_group(tmp_path):
    cfg = zolorax_config(width=24, vocab=50, eps=1e-6, layers=[
        zolorax_rglru(width=24, blocks=3, conv=4, mlp=None),
        zolorax_rglru(width=40, blocks=5, conv=2, mlp=zolorax_dense(30))])
    _run_drives(cfg, 7, 4, tmp_path)


def test_only_attention_layers_and_a_window_wider_than_every_request(tmp_path):
    att = dict(heads=2, kv_heads=1, dim=16, vdim=16, scale=0.3, rot_dims=8, base=1000.0)
    cfg = zolorax_config(width=24, vocab=50, eps=1e-6, layers=[
        zolorax_attention(**att, window=500, mlp=zolorax_moe(ff=8, experts=4, top=2)),
        zolorax_attention(**att, window=2, kv_from=0, mlp=None)])
    _run_drives(cfg, 8, 4, tmp_path)
