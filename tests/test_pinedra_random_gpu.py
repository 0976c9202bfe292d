"""Pinedra configurations drawn at random on the GPU: layer orders, loops anywhere, sizes that
are no multiples of the kernels' tiles, chunks from one token to beyond the request, every
kind of attention with few and many heads, routers with and without groups, identity experts
and a shared expert, every run compared with the plain implementation in float32 however the
work is cut, and with itself in bfloat16."""

import random

import pytest
import torch

import drives
from helpers import (pinedra_chunked_attention, pinedra_config, pinedra_distance_attention,
                     pinedra_moe, pinedra_plain_attention, random_prompt, write_pinedra_model)
from plain import pinedra_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model

pytestmark = pytest.mark.gpu


def draw_mlp(rnd):
    if rnd.random() < 0.25:
        return None
    groups = rnd.choice([1, 1, 2, 3, 4])
    per = rnd.choice([1, 2, 3, 6])
    outputs = groups * per
    identity = rnd.choice([0, 0, 1, 2, outputs - 1])
    identity = min(identity, outputs - 1)
    keep = rnd.randint(1, groups)
    return pinedra_moe(ff=rnd.choice([8, 12, 40, 100]), experts=outputs - identity,
                       identity=identity, top=rnd.randint(1, min(keep * per, 4)), groups=groups,
                       keep=keep, scale=rnd.choice([1.0, 1.75, 0.3]),
                       shared=rnd.choice([None, 8, 40, 96]))


def draw_layer(rnd):
    kv = rnd.choice([1, 2, 3, 4])
    heads = kv * rnd.choice([1, 2, 4, 6])
    dim = rnd.choice([6, 16, 24, 40, 64, 96, 120, 128])
    vdim = rnd.choice([4, 16, 48, 100, 128])
    scale = rnd.choice([0.1, dim ** -0.5])
    mlp = draw_mlp(rnd)
    kind = rnd.choice(["attention", "attention_2", "attention_3"])
    if kind == "attention":
        return pinedra_plain_attention(heads=heads, kv_heads=kv, dim=dim, scale=scale, mlp=mlp)
    if kind == "attention_2":
        return pinedra_distance_attention(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale,
                                          coef=rnd.choice([0.1, 0.5, 1.0]),
                                          every=rnd.choice([1, 3, 16, 96]), mlp=mlp)
    return pinedra_chunked_attention(heads=heads, kv_heads=kv, dim=dim, vdim=vdim, scale=scale,
                                     rot_dims=rnd.choice([2, dim // 2 * 2, dim // 4 * 2 or 2]),
                                     base=rnd.choice([100.0, 1e4, 1e6]),
                                     softcap=rnd.choice([1.0, 10.0, 50.0]),
                                     chunk=rnd.choice([1, 2, 7, 16, 31, 64, 100, 1000]), mlp=mlp)


def draw(case):
    rnd = random.Random(3000 + case)
    n = rnd.choice([1, 2, 3, 4, 5])
    layers = [draw_layer(rnd) for _ in range(n)]
    loop = None
    if rnd.random() < 0.7:
        start = rnd.randrange(n)
        loop = (start, rnd.randint(start + 1, n), rnd.choice([1, 2, 3]))
    cfg = pinedra_config(width=rnd.choice([20, 36, 64, 100]), vocab=rnd.choice([50, 97, 300]),
                         eps=rnd.choice([1e-6, 1e-5]), embed_scale=rnd.choice([1.0, 8.0, 2.7]),
                         layers=layers, loop=loop)
    return cfg, rnd.choice([4, 16, 32])


@pytest.mark.parametrize("case", range(12))
def test_a_drawn_configuration(case, tmp_path, gpu_device):
    cfg, page = draw(case)
    d = write_pinedra_model(tmp_path, cfg, case, torch.float32, std=0.15, sharpen=2.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, torch.float32, gpu_device)
    lengths = [5, 17, 40, 1, 70, 131]
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}

    def runner(pages):
        return ModelRunner(model, page_size=page, num_pages=pages, num_slots=4)

    roomy = 160 // page + 4
    drives.compare(drives.drive_whole(runner(roomy), requests), ref, 3e-4, 6e-5)
    drives.compare(drives.drive_prefill_then_decode(runner(roomy), requests), ref, 3e-4, 6e-5)
    drives.compare(drives.drive_portions(runner(roomy), requests), ref, 3e-4, 6e-5)
    drives.compare(drives.drive_mixed(runner(448 // page), requests), ref, 3e-4, 6e-5)


@pytest.mark.parametrize("case", range(12))
def test_a_drawn_configuration_runs_in_bfloat16(case, tmp_path, gpu_device):
    """The same draws in bfloat16: whole prompts and mixed steps agree with each other row by
    row (what differs between them is which kernel serves a row), and stay finite."""
    cfg, page = draw(case)
    for layer in cfg["layers"]:
        # every expert in use: a choice between two experts whose scores lie within the
        # rounding of the router's bfloat16 input would decide a token's row
        if layer["mlp"]:
            r = layer["mlp"]["router"]
            r["top"], r["groups"]["keep"] = r["experts"] + r["identity"], r["groups"]["count"]
    d = write_pinedra_model(tmp_path, cfg, case, torch.bfloat16, std=0.15, sharpen=1.0)
    _, model = load_model(d, torch.bfloat16, gpu_device)
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i)
                for i, n in enumerate([5, 17, 40, 1, 70, 131])}

    def runner(pages):
        return ModelRunner(model, page_size=page, num_pages=pages, num_slots=4)

    a = drives.drive_whole(runner(160 // page + 4), requests)
    b = drives.drive_mixed(runner(448 // page), requests)
    rows = bad = 0
    for rid in requests:
        x, y = a.stacked(rid)[0], b.stacked(rid)[0]
        assert torch.isfinite(x).all() and torch.isfinite(y).all()
        scale = max(1.0, float(x.abs().max()))
        rows += x.shape[0]
        bad += int(((x - y).abs() > 0.08 * scale).any(dim=1).sum())
    assert bad <= 0.02 * rows, f"{bad} of {rows} rows differ between the two ways of cutting"
