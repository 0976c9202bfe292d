"""Zolorax configurations drawn at random on the GPU: layer orders, sizes that are no
multiples of the kernels' tiles, windows from one token to beyond the request, readers of
other layers' keys, experts from one a token to all, every run compared with the plain
implementation in float32 however the work is cut, and with itself in bfloat16."""

import random

import pytest
import torch

import drives
from helpers import (random_prompt, write_zolorax_model, zolorax_attention, zolorax_config,
                     zolorax_dense, zolorax_moe, zolorax_rglru)
from plain import zolorax_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model

pytestmark = pytest.mark.gpu


def draw_mlp(rnd):
    kind = rnd.choice(["none", "dense", "moe", "moe"])
    if kind == "none":
        return None
    if kind == "dense":
        return zolorax_dense(rnd.choice([24, 50, 96, 200]))
    experts = rnd.choice([1, 2, 3, 5, 8, 16, 24])
    return zolorax_moe(ff=rnd.choice([8, 12, 40, 100]), experts=experts,
                       top=rnd.randint(1, min(experts, 4)))


def draw_sizes(rnd):
    kv = rnd.choice([1, 2, 3, 4])
    dim = rnd.choice([6, 16, 24, 40, 64, 96, 120, 128])
    scaling = None
    if rnd.random() < 0.6:
        scaling = (rnd.choice([2.0, 8.0, 32.0]), rnd.choice([16, 64, 2048]),
                   rnd.choice([8.0, 32.0]), rnd.choice([0.5, 1.0, 2.0]))
    return dict(heads=kv * rnd.choice([1, 2, 4, 6]), kv_heads=kv, dim=dim,
                vdim=rnd.choice([4, 16, 48, 100, 128]),
                rot_dims=rnd.choice([2, dim // 2 * 2, dim // 4 * 2 or 2]),
                base=rnd.choice([100.0, 1e4, 1e6]), scale=rnd.choice([0.1, dim ** -0.5]),
                scaling=scaling)


def draw(case):
    rnd = random.Random(2000 + case)
    layers, owners = [], []
    for i in range(rnd.choice([2, 3, 4, 5])):
        mlp = draw_mlp(rnd)
        if rnd.random() < 0.45:
            blocks = rnd.choice([1, 2, 3, 4, 8])
            layers.append(zolorax_rglru(width=blocks * rnd.choice([1, 5, 16, 24, 48, 80]),
                                        blocks=blocks, conv=rnd.choice([1, 2, 4, 5]), mlp=mlp))
            continue
        window = rnd.choice([1, 2, 7, 16, 31, 64, 100, None])
        if owners and rnd.random() < 0.5:
            j, sizes = rnd.choice(owners)
            heads = sizes["kv_heads"] * rnd.choice([1, 2, 3])
            layers.append(zolorax_attention(**{**sizes, "heads": heads}, window=window, kv_from=j,
                                            mlp=mlp))
        else:
            sizes = draw_sizes(rnd)
            owners.append((i, sizes))
            layers.append(zolorax_attention(**sizes, window=window, mlp=mlp))
    cfg = zolorax_config(width=rnd.choice([20, 36, 64, 100]), vocab=rnd.choice([50, 97, 300]),
                         eps=rnd.choice([1e-6, 1e-5]), layers=layers)
    return cfg, rnd.choice([4, 16, 32])


@pytest.mark.parametrize("case", range(12))
def test_a_drawn_configuration(case, tmp_path, gpu_device):
    cfg, page = draw(case)
    d = write_zolorax_model(tmp_path, cfg, case, torch.float32, std=0.15, sharpen=2.0)
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
        # every expert in use: among two dozen experts some token's best two lie within the
        # rounding of the router's bfloat16 input, and which of the two ways of cutting meets
        # which rounding would decide that token's row and, through its keys, later ones
        if layer["mlp"] and layer["mlp"]["kind"] == "moe":
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    d = write_zolorax_model(tmp_path, cfg, case, torch.bfloat16, std=0.15, sharpen=1.0)
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
