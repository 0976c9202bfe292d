"""Pinedra on the CPU: configuration, the model as data, the plain implementation's own pins
(each mechanism against a closed form or a crafted case), and the engine's cache manager,
batch builder and step function (with the plain torch kernel references in place of the HIP
kernels) against the plain whole-sequence implementation, float32."""

import copy
import math

import pytest
import torch

import drives
from helpers import (PINE, PINE_A, PINE_B, PINE_C, pinedra_chunked_attention, pinedra_config,
                     pinedra_distance_attention, pinedra_moe, pinedra_plain_attention,
                     random_prompt, write_pinedra_model)
from kernel_refs import TorchOps
from plain import pinedra_plain as plain
from tokensprint_amd.config import ConfigError, PinedraConfig
from tokensprint_amd.config.registry import architecture_names, get_architecture
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import build_model, load_model
from tokensprint_amd.models.spec import EMBEDDING_OUTPUT
from tokensprint_amd.parts.base import PagedKVNeed


@pytest.fixture(scope="module", params=sorted(PINE))
def setup(request, tmp_path_factory):
    cfg, seed, page = PINE[request.param]
    d = write_pinedra_model(tmp_path_factory.mktemp(f"pine{request.param}"), cfg, seed,
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


def test_mixed_with_pages_used_again(setup):
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
    cfg = PinedraConfig.from_dict(PINE_A)
    assert (cfg.width, cfg.vocab_size, cfg.eps, cfg.embed_scale, len(cfg.layers)) == \
        (40, 97, 1e-5, 3.0, 4)
    assert (cfg.loop.start, cfg.loop.stop, cfg.loop.times) == (1, 3, 2)
    c = cfg.layers[0].mixer
    assert (c.kind, c.heads, c.kv_heads, c.dim, c.vdim, c.scale) == ("attention_3", 4, 2, 12, 20, 0.4)
    assert (c.rot_base, c.rot_dims, c.softcap, c.chunk) == (10000.0, 8, 5.0, 7)
    p = cfg.layers[1].mixer
    assert (p.kind, p.heads, p.kv_heads, p.dim, p.vdim, p.scale) == ("attention", 4, 2, 12, 12, 0.3)
    d = cfg.layers[2].mixer
    assert (d.kind, d.temp_coef, d.temp_every, d.vdim) == ("attention_2", 0.5, 4, 8)
    m = cfg.layers[0].mlp
    assert (m.ff, m.experts, m.identity, m.top, m.group_count, m.group_keep, m.scale,
            m.shared_ff) == (12, 5, 1, 2, 3, 2, 1.5, 20)
    assert cfg.layers[1].mlp is None and cfg.layers[2].mlp.shared_ff is None
    assert PinedraConfig.from_dict(PINE_C).loop is None
    assert "Pinedra" in architecture_names()


def test_run_order_and_what_enters():
    cfg = PinedraConfig.from_dict(PINE_A)
    assert cfg.run_order() == [(0, False), (1, False), (2, False), (1, True), (2, False), (3, False)]
    assert PinedraConfig.from_dict(PINE_B).run_order() == \
        [(0, False), (0, True), (0, True), (1, False), (2, False)]
    arch = get_architecture("Pinedra")
    spec = arch.build_spec(arch.parse_config(PINE_A))
    assert [run.layer for run in spec.order] == [0, 1, 2, 1, 2, 3]
    assert [run.enter for run in spec.order] == [None, None, None, EMBEDDING_OUTPUT, None, None]
    assert plain.run_order(PINE_A) == cfg.run_order()
    assert plain.run_order(PINE_B) == PinedraConfig.from_dict(PINE_B).run_order()
    assert plain.run_order(PINE_C) == [(0, False), (1, False), (2, False)]


def test_every_run_owns_a_cache_and_tensors_follow_the_mixer():
    _, model = build_model(PINE_A, "float32", "cpu", ops=TorchOps())
    needs = model.cache_needs()
    # heads are laid out in the larger of key and value size rounded up to 16
    assert needs == [PagedKVNeed(2, 32, None), PagedKVNeed(2, 16, None), PagedKVNeed(1, 16, None),
                     PagedKVNeed(2, 16, None), PagedKVNeed(1, 16, None), PagedKVNeed(2, 16, None)]
    names = set(model.tensor_decls())
    assert {"l0.mix.q.b", "l0.mix.k.b", "l0.mix.v.b", "l0.mix.g", "l0.norm1", "embed", "head",
            "final.norm", "l0.mlp.router", "l0.mlp.correction", "l0.mlp.e4.down",
            "l0.mlp.shared.gate"} <= names
    assert not {"l0.mix.o.b", "l0.mix.q.norm", "l0.mlp.e5.gate", "l1.mix.v", "l1.mix.v.b",
                "l2.mix.q.b", "l2.mix.o.b", "l2.mlp.shared.up", "l1.mlp.router", "l0.norm2"} & names
    decls = model.tensor_decls()
    assert decls["l0.norm1"].shape == () and decls["final.norm"].shape == ()
    assert decls["l0.mix.g"].shape == (4, 40) and decls["l1.mix.g"].shape == (48, 40)
    assert decls["l1.mix.q.norm"].shape == (48,) and decls["l1.mix.k.norm"].shape == (24,)
    assert decls["l2.mix.q.norm"].shape == (16,) and decls["l1.mix.o.b"].shape == (40,)
    assert decls["l0.mlp.router"].shape == (6, 40) and decls["l0.mlp.correction"].shape == (6,)


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="attention_4"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(vdim=16), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=14), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"].update(softcap=-1.0), "softcap"),
    (lambda c: c["layers"][2]["mixer"]["q_temp"].update(every=0), "q_temp"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "cannot give"),
    (lambda c: c["loop"].update(stop=9), "loop"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_config_errors(change, message):
    cfg = copy.deepcopy(PINE_A)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        PinedraConfig.from_dict(cfg)


def test_a_constant_that_is_left_out_takes_its_mechanism_along(tmp_path):
    """No cap, no chunks, no rotation, no temperature, a value size that the keys give: the
    engine and the plain implementation agree on what is left."""
    cfg = copy.deepcopy(PINE_A)
    for key in ("softcap", "mask", "rot"):
        cfg["layers"][0]["mixer"].pop(key)
    cfg["layers"][3]["mixer"].pop("softcap")
    cfg["layers"][1]["mixer"].pop("vdim")
    cfg["layers"][2]["mixer"].pop("q_temp")
    parsed = PinedraConfig.from_dict(cfg)
    assert parsed.layers[0].mixer.chunk is None and parsed.layers[0].mixer.rot_dims is None
    assert parsed.layers[1].mixer.vdim == 12 and parsed.layers[2].mixer.temp_every is None
    d = write_pinedra_model(tmp_path, cfg, 3, torch.float32)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    requests = {"a": random_prompt(30, cfg["vocab"], 1), "b": random_prompt(9, cfg["vocab"], 2)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    drives.compare(drives.drive_portions(runner_for(model, 4, 20), requests), ref, *TOL)


# ------------------------------------------------------------------ the plain implementation's pins


def test_norm_with_one_number():
    x = torch.tensor([[3.0, -4.0, 0.0, 0.0]], dtype=torch.float64)
    out = plain.norm_one_number(x, torch.tensor(2.0, dtype=torch.float64), 0.0)
    assert torch.allclose(out, torch.tensor([[2.4, -3.2, 0.0, 0.0]], dtype=torch.float64))
    # eps stands inside the root
    out = plain.norm_one_number(x, torch.tensor(1.0, dtype=torch.float64), 2.75)
    assert torch.allclose(out, x / 3.0)


def test_softmax_with_one_more_term():
    s = torch.tensor([[math.log(3.0), -50.0], [0.0, 0.0]], dtype=torch.float64)
    seen = torch.tensor([[True, False], [True, True]])
    p = plain.softmax_rows(s, seen, plus_one=True)
    assert torch.allclose(p, torch.tensor([[0.75, 0.0], [1 / 3, 1 / 3]], dtype=torch.float64))
    p = plain.softmax_rows(s, seen)
    assert torch.allclose(p, torch.tensor([[1.0, 0.0], [0.5, 0.5]], dtype=torch.float64))
    # large scores and very small ones do not overflow, and the further term still counts
    big = plain.softmax_rows(torch.tensor([[800.0]], dtype=torch.float64), torch.tensor([[True]]), True)
    small = plain.softmax_rows(torch.tensor([[-800.0]], dtype=torch.float64), torch.tensor([[True]]), True)
    assert float(big) == 1.0 and float(small) == 0.0


def test_chunks_count_from_position_zero():
    seen = plain.causal_mask(10, chunk=4)
    assert seen[3].tolist() == [True] * 4 + [False] * 6
    assert seen[4].tolist() == [False] * 4 + [True] + [False] * 5
    assert seen[9].tolist() == [False] * 8 + [True, True]
    assert plain.causal_mask(3).tolist() == [[True, False, False], [True, True, False], [True] * 3]


def test_distance_bias_temperature_and_the_further_term_by_hand():
    # one head of dim 1 (H = 1: slope 2^-8), width 1; q = k = v = h (unit weights), norms off
    # by a norm weight that undoes them: with dim 1 the unit norm of x is sign(x) (eps 0)
    T = 6
    m = {"heads": 1, "kv_heads": 1, "dim": 1, "vdim": 1, "scale": 1.0,
         "q_temp": {"coef": 2.0, "every": 3}}
    one = torch.ones(1, 1, dtype=torch.float64)
    w = {"x.q": one, "x.k": one, "x.v": one, "x.o": one, "x.g": 50.0 * one,
         "x.q.norm": torch.ones(1, dtype=torch.float64), "x.k.norm": torch.ones(1, dtype=torch.float64)}
    h = torch.tensor([[1.0], [2.0], [3.0], [4.0], [5.0], [6.0]], dtype=torch.float64)
    out = plain.attention_distance(h, w, "x.", m, 0.0)
    slope = 2.0 ** -8
    for i in range(T):
        temp = 1.0 + 2.0 * math.log((i + 1) // 3 + 1)
        e = [math.exp(temp - slope * (i - j)) for j in range(i + 1)]
        want = sum(ej * (j + 1.0) for j, ej in enumerate(e)) / (1.0 + sum(e))
        assert abs(float(out[i]) - want) < 1e-12     # (the gate's sigmoid(50 h) is 1)
    # slopes of several heads
    assert [2.0 ** (-8.0 * (j + 1) / 4) for j in range(4)] == [0.25, 0.0625, 0.015625, 0.00390625]


def test_capped_scores_and_a_gate_per_head():
    T, cap = 3, 2.0
    m = {"heads": 2, "kv_heads": 1, "dim": 2, "vdim": 1, "scale": 10.0, "softcap": cap,
         "mask": {"size": 2}, "rot": {"dims": 2, "base": 10.0}}
    z1 = torch.zeros(1, dtype=torch.float64)
    w = {"x.q": torch.zeros(4, 2, dtype=torch.float64), "x.q.b": torch.tensor([1.0, 0, 0, 1.0], dtype=torch.float64),
         "x.k": torch.zeros(2, 2, dtype=torch.float64), "x.k.b": torch.tensor([1.0, 0.0], dtype=torch.float64),
         "x.v": torch.tensor([[1.0, 0.0]], dtype=torch.float64), "x.v.b": z1,
         "x.g": torch.tensor([[0.0, 1.0], [0.0, -1.0]], dtype=torch.float64),
         "x.o": torch.tensor([[1.0, 0.0], [0.0, 1.0]], dtype=torch.float64)}
    h = torch.tensor([[1.0, 0.3], [2.0, -0.7], [4.0, 0.1]], dtype=torch.float64)
    out = plain.attention_chunked(h, w, "x.", m, 0.0)
    # head 0: q = (1, 0), k = (1, 0) rotated by the position's angle (frequency 1):
    # q . k = cos(i - j); head 1: q = (0, 1): q . k = -sin(i - j); values are h[:, 0]
    for i in range(T):
        keys = [j for j in range(i + 1) if j // 2 == i // 2]
        for head, dot in ((0, math.cos), (1, lambda d: -math.sin(d))):
            e = [math.exp(cap * math.tanh(10.0 * dot(i - j) / cap)) for j in keys]
            att = sum(ej * float(h[j, 0]) for ej, j in zip(e, keys)) / sum(e)
            gate = 1.0 / (1.0 + math.exp(-float(h[i, 1]) * (1.0 if head == 0 else -1.0)))
            assert abs(float(out[i, head]) - att * gate) < 1e-12


def test_keys_serve_as_values_before_their_norm_and_norms_run_over_all_heads():
    m = {"heads": 2, "kv_heads": 2, "dim": 1, "vdim": 1, "scale": 1.0}
    eye = torch.eye(2, dtype=torch.float64)
    w = {"x.q": eye, "x.q.b": torch.zeros(2, dtype=torch.float64), "x.k": eye,
         "x.k.b": torch.tensor([10.0, 20.0], dtype=torch.float64), "x.g": 50.0 * eye, "x.o": eye,
         "x.o.b": torch.tensor([0.5, -0.5], dtype=torch.float64),
         "x.q.norm": torch.ones(2, dtype=torch.float64), "x.k.norm": torch.ones(2, dtype=torch.float64)}
    h = torch.tensor([[3.0, 4.0]], dtype=torch.float64)
    out = plain.attention_keys_as_values(h, w, "x.", m, 0.0)
    # one token: the softmax is 1, the output is the value = the key with its bias, unnormed
    assert torch.allclose(out, torch.tensor([[13.5, 23.5]], dtype=torch.float64))
    # the norm over the whole projection: (3, 4) / sqrt(12.5), not a sign per head
    T = 2
    h = torch.tensor([[3.0, 4.0], [3.0, 4.0]], dtype=torch.float64)
    w["x.k.b"] = torch.zeros(2, dtype=torch.float64)
    out = plain.attention_keys_as_values(h, w, "x.", m, 0.0)
    assert torch.allclose(out[1] - w["x.o.b"], torch.tensor([3.0, 4.0], dtype=torch.float64))


def test_router_groups_correction_identity_and_scale():
    r = {"experts": 3, "identity": 1, "top": 2, "scale": 2.0, "groups": {"count": 2, "keep": 1}}
    z = torch.log(torch.tensor([[0.1, 0.2, 0.3, 0.4], [0.4, 0.3, 0.2, 0.1]], dtype=torch.float64))
    none = torch.zeros(4, dtype=torch.float64)
    chosen, weights = plain.route(z, none, r)
    assert chosen.tolist() == [[3, 2], [0, 1]]
    assert torch.allclose(weights, torch.tensor([[0.8, 0.6], [0.8, 0.6]], dtype=torch.float64))
    # the correction decides the choice of group and expert, not the weights; a group whose
    # choice scores are all negative can still be the best
    corr = torch.tensor([-0.2, -0.35, -5.0, -5.0], dtype=torch.float64)
    chosen, weights = plain.route(z, corr, r)
    assert chosen.tolist() == [[0, 1], [0, 1]]
    assert torch.allclose(weights, torch.tensor([[0.2, 0.4], [0.8, 0.6]], dtype=torch.float64))
    # an identity expert gives back what it reads, times its weight
    mlp = {"router": dict(r, top=1, groups={"count": 1, "keep": 1}), "shared": None}
    w = {"m.router": torch.tensor([[0.0, 0.0], [0.0, 0.0], [0.0, 0.0], [9.0, 0.0]], dtype=torch.float64),
         "m.correction": none}
    h = torch.tensor([[1.0, -2.0]], dtype=torch.float64)
    s = math.exp(9.0) / (math.exp(9.0) + 3.0)
    assert torch.allclose(plain.routed_ff(h, w, "m.", mlp), 2.0 * s * h)


def test_embedding_output_enters_every_later_pass():
    """A model of one looped layer whose mixer and feed-forward give nothing: the stream after
    pass t is (t + 1) times the embedding's output."""
    cfg = pinedra_config(width=4, vocab=5, eps=1e-6, embed_scale=2.0, loop=(0, 1, 3), layers=[
        pinedra_plain_attention(heads=1, kv_heads=1, dim=2, scale=1.0)])
    w = {"embed": torch.arange(20, dtype=torch.float64).view(5, 4), "l0.norm1": torch.tensor(1.0),
         "final.norm": torch.tensor(1.0), "head": torch.eye(4, dtype=torch.float64)[:5].repeat(2, 1)[:5],
         "l0.mix.q": torch.zeros(2, 4), "l0.mix.q.b": torch.zeros(2), "l0.mix.k": torch.zeros(2, 4),
         "l0.mix.k.b": torch.zeros(2), "l0.mix.q.norm": torch.ones(2), "l0.mix.k.norm": torch.ones(2),
         "l0.mix.g": torch.zeros(2, 4), "l0.mix.o": torch.zeros(4, 2), "l0.mix.o.b": torch.zeros(4)}
    w = {k: v.double() for k, v in w.items()}
    outs = []
    plain.forward(cfg, w, [1, 3], outs)
    x0 = 2.0 * w["embed"][[1, 3]]
    assert [torch.allclose(o, (t + 1) * x0) for t, o in enumerate(outs)] == [True] * 3
