"""Pinedra on the GPU: each new or widened HIP kernel against its plain torch reference, the
three kinds of attention and the routed feed-forward alone against the plain implementation
with crafted cases that random weights would hide (a token just inside and just outside a
chunk, a key hundreds of positions back that a distance bias has to weigh down, a further
term that carries most of a softmax), the engine against the plain whole-sequence
implementation however requests are cut into steps, in float32 and bfloat16, and greedy
generation through LLMEngine."""

import copy

import pytest
import torch

import drives
from helpers import (PINE, pinedra_chunked_attention, pinedra_config, pinedra_distance_attention,
                     pinedra_moe, pinedra_plain_attention, random_prompt, write_pinedra_model)
from kernel_refs import TorchOps
from plain import pinedra_plain as plain
from test_palelix_gpu import PART_TOL, Scene, close, compare, load_part, part_context, rnd, \
    run_part_in_steps
from test_zolorax_gpu import close_part
from tokensprint_amd.config import Config, SamplingParams
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.engine.llm_engine import LLMEngine
from tokensprint_amd.kernels import load_hip_ops
from tokensprint_amd.models.spec import PartSpec
from tokensprint_amd.parts.base import FEED_FORWARDS, MIXERS, POSITIONS, PagedKVNeed, build_part

pytestmark = pytest.mark.gpu
REF = TorchOps()


# ------------------------------------------------------------------ row kernels


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_finish_projection(gpu_device, out_dtype):
    """Biases, norms over a whole projection with padding that does not count, keys copied to
    the values' place before their norm, further columns carried along."""
    ops = load_hip_ops(gpu_device)
    for T, q_cols, k_cols, v_cols, extra, from_keys, normed, biased in (
            (5, 64, 32, 32, 8, False, False, True), (70, 48, 16, 16, 48, True, True, True),
            (1, 512, 128, 128, 0, True, True, False), (33, 16, 16, 32, 16, False, True, True),
            (9, 1280, 256, 256, 1280, True, True, True),
            # (parts that do not begin at multiples of four columns, and rows beyond what a
            # workgroup keeps in registers: the kernel that walks a row three times)
            (6, 18, 6, 6, 3, True, True, True), (3, 12288, 2048, 2048, 4096, False, True, True)):
        in_ld = q_cols + k_cols + (0 if from_keys else v_cols) + extra
        rows = rnd((T, in_ld), 1, 2.0).to(gpu_device)
        bias = rnd((in_ld - extra,), 2).to(gpu_device) if biased else None
        qn = (1 + 0.3 * rnd((q_cols,), 3)).to(gpu_device) if normed else None
        kn = (1 + 0.3 * rnd((k_cols,), 4)).to(gpu_device) if normed else None
        kw = dict(q_cols=q_cols, k_cols=k_cols, extra=extra, values_from_keys=from_keys,
                  q_norm=qn, k_norm=kn, q_count=q_cols - 5, k_count=k_cols - 3, eps=1e-3,
                  out_dtype=out_dtype)
        got = ops.finish_projection(rows, bias, **kw)
        want = REF.finish_projection(rows, bias, **kw)
        assert got.shape == (T, q_cols + k_cols + v_cols + extra)
        close(got, want, **(dict(rtol=1e-5, atol=1e-5) if out_dtype == torch.float32
                            else dict(rtol=1e-2, atol=1e-2)))


def test_bias_gate_per_head_weighted_rows_and_a_scaled_embedding(gpu_device):
    ops = load_hip_ops(gpu_device)
    for T, width, n in ((7, 40, 40), (130, 96, 50), (1, 8, 1)):
        x = rnd((T, width), 1).to(gpu_device)
        bias = rnd((n,), 2).to(gpu_device)
        want = x.clone()
        REF.add_bias(want, bias)
        ops.add_bias(x, bias)
        close(x, want, rtol=0, atol=0)
    for dtype in (torch.float32, torch.bfloat16):
        for T, heads, hd, ld, col in ((5, 4, 16, 200, 136), (40, 3, 48, 152, 144), (1, 1, 16, 8, 3)):
            x = rnd((T, heads * hd), 3).to(dtype).to(gpu_device)
            rows = rnd((T, ld), 4, 2.0).to(dtype).to(gpu_device)
            close(ops.sigmoid_gate(x, rows, col, dtype, group=hd),
                  REF.sigmoid_gate(x, rows, col, dtype, group=hd),
                  **(dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)))
        for T, width, n, col, count in ((6, 40, 7, 5, 2), (50, 72, 6, 3, 3), (1, 32, 4, 3, 1)):
            out = rnd((T, width), 5).to(gpu_device)
            h = rnd((T, width), 6).to(dtype).to(gpu_device)
            weights = torch.relu(rnd((T, n), 7)).to(gpu_device)
            want = out.clone()
            REF.add_weighted_rows(want, h, weights, col, count)
            ops.add_weighted_rows(out, h, weights, col, count)
            close(out, want, rtol=1e-6, atol=1e-6)
        table = rnd((50, 24), 8).to(dtype).to(gpu_device)
        ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32, device=gpu_device)
        close(ops.embed(table, ids, scale=5.5), REF.embed(table, ids, scale=5.5), rtol=1e-7, atol=0)
        close(ops.embed(table, ids), REF.embed(table, ids), rtol=0, atol=0)


def test_rows_that_enter_the_stream(gpu_device):
    """`stream_add` and `stream_add_norm` with a row for every token."""
    ops = load_hip_ops(gpu_device)
    for T, width in ((5, 40), (33, 2304), (1, 8)):
        for dtype in (torch.float32, torch.bfloat16):
            resid = rnd((T, width), 1).to(gpu_device)
            a = rnd((T, width), 2).to(dtype).to(gpu_device)
            b = rnd((T, width), 3).to(dtype).to(gpu_device)
            rows = rnd((T, width), 4).to(gpu_device)
            w = (1 + 0.1 * rnd((width,), 5)).to(gpu_device)
            want = resid.clone()
            want_h = REF.stream_add_norm(want, a, b, rows, w, 1e-5, dtype)
            got = resid.clone()
            got_h = ops.stream_add_norm(got, a, b, rows, w, 1e-5, dtype)
            close(got, want, rtol=1e-6, atol=1e-6)
            close(got_h, want_h, **(dict(rtol=1e-5, atol=1e-5) if dtype == torch.float32
                                    else dict(rtol=1e-2, atol=1e-2)))
            want, got = resid.clone(), resid.clone()
            REF.stream_add(want, a, None, rows)
            ops.stream_add(got, a, None, rows)
            close(got, want, rtol=1e-6, atol=1e-6)


def test_router_with_a_correction_and_experts_without_weights(gpu_device):
    ops = load_hip_ops(gpu_device)
    for T, n, top, groups, keep, scale in ((40, 15, 4, 3, 1, 1.75), (7, 6, 2, 3, 2, 1.0),
                                           (100, 64, 8, 8, 4, 0.5), (3, 4, 4, 4, 4, 2.0), (9, 5, 1, 1, 1, 1.0)):
        logits = rnd((T, n), 1, 2.0).to(gpu_device)
        corr = (rnd((n,), 2, 0.2) - 0.3).to(gpu_device)       # most choice scores are negative
        kw = dict(top=top, group_count=groups, group_keep=keep, normalize=False)
        got = ops.route_experts(logits, correction=corr, weight_scale=scale, **kw)
        want = REF.route_experts(logits, correction=corr, weight_scale=scale, **kw)
        close(got, want, rtol=1e-5, atol=1e-7)
        assert int((got != 0).sum()) == T * top
        # the correction changes who is chosen, never a chosen expert's weight
        bare = ops.route_experts(logits, **kw)
        both = (got != 0) & (bare != 0)
        close(got[both], bare[both] * scale, rtol=1e-6, atol=0)
        if n > top:
            assert bool(((got != 0) != (bare != 0)).any())
    for dtype in (torch.float32, torch.bfloat16):
        for T, experts, identity, inner, shared in ((9, 5, 1, 12, 20), (40, 8, 0, 16, 16),
                                                    (3, 2, 2, 7, 0), (130, 10, 2, 88, 104)):
            weights = torch.relu(rnd((T, experts + identity), 3)).to(gpu_device)
            gate_up = rnd((T, 2 * (experts * inner + shared)), 4).to(dtype).to(gpu_device)
            kw = dict(form="silu", experts=experts, shared_inner=shared)
            close(ops.expert_activation(gate_up, weights, inner, 0.0, dtype, **kw),
                  REF.expert_activation(gate_up, weights, inner, 0.0, dtype, **kw),
                  **(dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)))


# ------------------------------------------------------------------ attention kernels


def test_scores_with_chunks_caps_distance_and_temperature_in_every_kernel(gpu_device):
    """The float32 kernel and the matrix-core kernel (keys split and whole, decode steps, short
    portions, long portions, mixed steps) against the plain torch attention, option by option
    and all together, at head sizes 48 to 128 and chunks of 1 token to several pages."""
    ops = load_hip_ops(gpu_device)
    for dtype in (torch.float32, torch.bfloat16):
        for nq, nkv, hd, options in (
                (4, 2, 64, dict(chunk=48, softcap=15.0)), (8, 8, 128, dict(chunk=1)),
                (6, 1, 96, dict(q_temp=(0.3, 3), sink=True, slopes=True)),
                (2, 2, 48, dict(chunk=100, softcap=1.5, slopes=True, q_temp=(1.0, 96), sink=True)),
                (4, 4, 64, dict(slopes=True)), (4, 1, 128, dict(chunk=7))):
            options = dict(options)
            if options.pop("slopes", False):
                options["slopes"] = torch.tensor([2.0 ** (-8.0 * (j + 1) / nq) for j in range(nq)],
                                                 device=gpu_device)
            if options.pop("sink", False):
                options["sink"] = torch.zeros(nq, device=gpu_device)
            needs = PagedKVNeed(nkv, hd, None)
            for spans in ([[700, 0, 0, 0]], [[500, 3, 40, 1], [1, 1, 1, 1]], [[90, 1, 0, 33], [2, 40, 7, 1]],
                          [[2100, 0, 0, 0], [1, 0, 0, 0]], [[900, 1200, 0, 0]]):
                if spans[0][0] > 800 and dtype == torch.float32 and hd != 64:
                    continue         # (the long prompts are for the matrix-core kernels)
                scene = Scene(gpu_device, needs, 16, 4, dtype=dtype, num_pages=160)
                for step, sp in enumerate(spans):
                    batch = scene.step(sp)
                    T = batch.num_tokens
                    table = batch.tables[0]
                    k = rnd((T, nkv, hd), step).to(dtype).to(gpu_device)
                    v = rnd((T, nkv, hd), 50 + step).to(dtype).to(gpu_device)
                    q = rnd((T, nq, hd), 90 + step, 1.5).to(dtype).to(gpu_device)
                    ops.kv_store(k, v, batch, table, scene.view)
                    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5,
                              window=None, **options)
                    got = ops.paged_attention(q, batch, table, scene.view, **kw)
                    only = sorted({0, T - 1, T // 2, min(T - 1, 17), min(T - 1, 63), min(T - 1, 64),
                                   min(T - 1, 899), min(T - 1, 900), min(T - 1, 1999)})
                    want = REF.paged_attention(q, batch, table, scene.view, only=only, **kw)
                    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 \
                        else dict(rtol=3e-2, atol=2e-2)
                    err = (got[only].float() - want[only].float()).abs().cpu()
                    allowed = tol["atol"] + tol["rtol"] * want[only].float().abs().cpu()
                    assert bool((err <= allowed).all()), \
                        (f"{dtype}, heads {nq}/{nkv} of {hd}, {sorted(options)}, spans {spans}, "
                         f"step {step}: differ by up to {float(err.max()):.3e}")


# ------------------------------------------------------------------ the mixers alone


def mixer_part(gpu_device, dtype, kind, width, **m):
    """(part, the mixer's sizes as config.json gives them) for one of the three kinds."""
    ctx = part_context(gpu_device, dtype, width)
    p = {"prefix": "x.", "heads": m["heads"], "kv_heads": m["kv_heads"], "dim": m["dim"],
         "vdim": m["vdim"], "scale": m["scale"], "position": None, "window": None,
         "qk_norm_eps": 1e-5}
    if kind == "attention":
        p.update(values="keys", qk_norm="projection", bias=("q", "k", "o"), gate=True)
    elif kind == "attention_2":
        p.update(qk_norm=True, gate=True, sink="zero", distance_bias=8.0,
                 q_temp=(m["q_temp"]["coef"], m["q_temp"]["every"]))
    else:
        head = -(-max(m["dim"], m["vdim"]) // 16) * 16
        ctx.positions["rot"] = build_part(POSITIONS, PartSpec("rope_partial", {
            "dims": m["rot"]["dims"], "base": m["rot"]["base"], "head_dim": head,
            "max_position": 1024}), ctx)
        p.update(position="rot", bias=("q", "k", "v"), gate="head", softcap=m["softcap"],
                 chunk=m["mask"]["size"])
    return build_part(MIXERS, PartSpec("softmax_attention", p), ctx)


MIXER_CASES = [
    ("attention", dict(heads=4, kv_heads=2, dim=12, vdim=12, scale=0.3)),
    ("attention", dict(heads=6, kv_heads=3, dim=64, vdim=64, scale=0.1)),
    ("attention", dict(heads=3, kv_heads=3, dim=40, vdim=40, scale=0.2)),
    ("attention_2", dict(heads=3, kv_heads=1, dim=16, vdim=8, scale=0.25, q_temp={"coef": 0.5, "every": 4})),
    ("attention_2", dict(heads=4, kv_heads=2, dim=48, vdim=48, scale=0.15, q_temp={"coef": 0.25, "every": 96})),
    ("attention_2", dict(heads=8, kv_heads=2, dim=24, vdim=80, scale=0.2, q_temp={"coef": 1.0, "every": 1})),
    ("attention_2", dict(heads=2, kv_heads=1, dim=64, vdim=32, scale=0.12, q_temp={"coef": 0.2, "every": 50})),
    ("attention_3", dict(heads=4, kv_heads=2, dim=12, vdim=20, scale=0.4, softcap=5.0,
                         mask={"size": 7}, rot={"dims": 8, "base": 10000.0})),
    ("attention_3", dict(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.11, softcap=15.0,
                         mask={"size": 48}, rot={"dims": 32, "base": 5e5})),
    ("attention_3", dict(heads=9, kv_heads=3, dim=32, vdim=16, scale=0.3, softcap=2.0,
                         mask={"size": 100}, rot={"dims": 32, "base": 300.0})),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("kind, m", MIXER_CASES,
                         ids=[f"{k}-{m['dim']}-{m['vdim']}" for k, m in MIXER_CASES])
def test_mixers_alone_whole_and_cut_around_chunks_and_pages(gpu_device, dtype, kind, m):
    """330 tokens over pages of 16: whole, and cut at and around page and chunk borders down to
    single tokens."""
    width, T = 48, 330
    part = mixer_part(gpu_device, dtype, kind, width, **m)
    w = load_part(part, dtype, gpu_device, 40, sharpen=("x.q", "x.k"),
                  factor=2.0 if dtype == torch.float32 else 1.0)
    h = rnd((T, width), 3).to(dtype)
    want = plain.MIXERS[kind](h.double(), w, "x.", m, 1e-5).float()
    for cuts in ([T], [15, 1, 1, 31, 16, 2, 34, 28, 1, 1, 1, 36, 1, 2, 160]):
        scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=30)
        got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
        close_part(got, want, dtype, dict(rtol=5e-3, atol=5e-4))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("decoded", [False, True])
def test_a_token_just_inside_and_just_outside_a_chunk(gpu_device, dtype, decoded):
    """One token's value is far larger than the others' (through an input channel that only
    the value projection reads): it shows in every later row of its chunk, up to the chunk's
    last position, and in none behind; in a prompt and decoded, for chunks that end inside a
    page and at a page's border."""
    for chunk, marked in ((50, 103), (32, 70), (1, 9)):
        width, T = 32, 200
        m = dict(heads=2, kv_heads=1, dim=16, vdim=16, scale=0.25, softcap=8.0,
                 mask={"size": chunk}, rot={"dims": 8, "base": 100.0})
        part = mixer_part(gpu_device, dtype, "attention_3", width, **m)
        w = load_part(part, dtype, gpu_device, 7)
        for name in ("x.q", "x.k", "x.g"):
            w[name][:, 0] = 0.0
        part.load(lambda n: w[n].to(torch.float32 if n.endswith(".b") else dtype).to(gpu_device))
        h = rnd((T, width), 5).to(dtype)
        h[:, 0] = 0.0
        quiet = plain.attention_chunked(h.double(), w, "x.", m, 1e-5).float()
        h[marked, 0] = 3000.0
        want = plain.attention_chunked(h.double(), w, "x.", m, 1e-5).float()
        last_in, first_out = (marked // chunk + 1) * chunk - 1, (marked // chunk + 1) * chunk
        tol = dict(rtol=5e-3, atol=1e-3) if dtype == torch.float32 else dict(rtol=6e-2, atol=6e-2)
        # the plain side itself: the marked token matters up to last_in and is gone right after
        changed = (want[marked:last_in + 1] - quiet[marked:last_in + 1]).abs().max(-1).values
        assert float(changed.min()) > 0 and float(changed[-1]) > 3 * tol["atol"] \
            and float(changed.median()) > 50 * tol["atol"]
        assert torch.equal(want[first_out:], quiet[first_out:])
        assert torch.equal(want[:marked], quiet[:marked])
        head = min(marked + 3, last_in)
        cuts = [head] + [1] * (T - head) if decoded else [T]
        scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=20)
        got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
        lo, hi = max(marked - 2, 0), min(first_out + 3, T)
        if dtype == torch.float32:
            torch.testing.assert_close(got[lo:hi], want[lo:hi], **tol)
        # (bfloat16: a row's error is a share of the loud value's part in it)
        close_part(got, want, dtype, dict(rtol=5e-3, atol=1e-3))
        assert float((got[first_out:] - quiet[first_out:]).abs().max()) < 2 * tol["atol"] \
            + tol["rtol"] * float(quiet.abs().max())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_key_far_back_under_a_distance_bias_and_a_further_term_that_wins(gpu_device, dtype):
    """One key among hundreds matches the last queries: its score stands far above the others',
    and the distance bias of every head takes its slope times the distance off it.  With
    scores far below zero the further term of the denominator takes the whole weight."""
    width, T, far = 32, 420, 11
    m = dict(heads=4, kv_heads=2, dim=16, vdim=16, scale=1.0, q_temp={"coef": 0.4, "every": 64})
    part = mixer_part(gpu_device, dtype, "attention_2", width, **m)
    w = load_part(part, dtype, gpu_device, 9)
    for name in ("x.q", "x.k", "x.g"):       # channel 0 feeds the values only
        w[name][:, 0] = 0.0
    # a query head is projected as its key head is: a token's query points where its key does
    w["x.q"] = w["x.k"].view(2, 1, 16, width).expand(2, 2, 16, width).reshape(64, width).clone()
    w["x.q.norm"] = w["x.k.norm"].clone()
    part.load(lambda n: w[n].to(torch.float32 if n.endswith(".norm") else dtype).to(gpu_device))
    h = rnd((T, width), 5, 0.2).to(dtype)
    h[:, 0] = 0.0
    h[-3:] = h[far]                          # the last queries point where that key points
    without = plain.attention_distance(h.double(), w, "x.", m, 1e-5).float()
    h[far, 0] = 200.0                        # and only that key's value is loud
    want = plain.attention_distance(h.double(), w, "x.", m, 1e-5).float()
    assert float((want[-3:] - without[-3:]).abs().max()) > 0.5       # the far key matters
    for cuts in ([T], [T - 5] + [1] * 5, [200, 2, 150, T - 352]):
        scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=30)
        got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
        close_part(got, want, dtype, dict(rtol=5e-3, atol=5e-4))
    # keys that point away from every query: all scores far below zero
    w2 = {n: (-t if n == "x.k" else t) for n, t in w.items()}
    part.load(lambda n: w2[n].to(torch.float32 if n.endswith(".norm") else dtype).to(gpu_device))
    h2 = rnd((40, width), 8).to(dtype)
    # (sharp scores in float32; in bfloat16 a score's rounding times forty would decide a row)
    sharp = 40.0 if dtype == torch.float32 else 3.0
    m_sharp = dict(m, scale=sharp)
    part.scale = sharp
    want = plain.attention_distance(h2.double(), w2, "x.", m_sharp, 1e-5).float()
    scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=30)
    got = run_part_in_steps(part, h2.to(gpu_device), scene, [30] + [1] * 10)
    torch.testing.assert_close(got, want, **(
        dict(rtol=5e-3, atol=5e-4) if dtype == torch.float32
        else dict(rtol=6e-2, atol=0.05 * float(want.abs().max()))))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_feed_forward_alone(gpu_device, dtype):
    width, T = 40, 50
    ctx = part_context(gpu_device, dtype, width)
    h = rnd((T, width), 2).to(dtype)
    for experts, identity, top, groups, keep, scale, shared, inner in (
            (5, 1, 2, 3, 2, 1.5, 20, 12), (8, 0, 1, 1, 1, 1.0, 16, 16), (3, 3, 3, 2, 2, 0.7, 8, 20),
            (2, 2, 4, 4, 4, 2.0, None, 8), (10, 2, 3, 3, 2, 1.75, 64, 80)):
        moe = build_part(FEED_FORWARDS, PartSpec("routed_experts", {
            "prefix": "m.", "inner_dim": inner, "experts": experts, "top": top,
            "group_count": groups, "group_keep": keep, "scores": "softmax", "normalize": False,
            "gated": "silu", "identity": identity, "correction": True, "weight_scale": scale,
            "shared_inner": shared}), ctx)
        # (a router whose logits lie apart: no choice is decided by rounding)
        w = load_part(moe, dtype, gpu_device, 6, sharpen=("m.router",), factor=6.0)
        mlp = {"router": {"experts": experts, "identity": identity, "top": top, "scale": scale,
                          "groups": {"count": groups, "keep": keep}},
               "shared": {"ff": shared} if shared else None}
        close_part(moe.forward(h.to(gpu_device), None).float().cpu(),
                   plain.routed_ff(h.double(), w, "m.", mlp).float(), dtype)


# ------------------------------------------------------------------ the engine


TOL = {torch.float32: (2e-4, 5e-5), torch.bfloat16: (6e-2, 6e-2)}


def all_experts(cfg):
    """The configuration with every expert in use: in bfloat16 a choice between two experts
    whose scores lie within the rounding of the router's input changes a token's row, and
    the comparison is to show the kernels' precision (the choice itself is compared in
    float32 and part by part)."""
    cfg = copy.deepcopy(cfg)
    for layer in cfg["layers"]:
        if layer["mlp"]:
            r = layer["mlp"]["router"]
            r["top"] = r["experts"] + r["identity"]
            r["groups"]["keep"] = r["groups"]["count"]
    return cfg


@pytest.fixture(scope="module", params=[(n, d) for n in sorted(PINE)
                                        for d in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def setup(request, tmp_path_factory, gpu_device):
    name, dtype = request.param
    cfg, seed, page = PINE[name]
    if dtype == torch.bfloat16:
        cfg = all_experts(cfg)
    d = write_pinedra_model(tmp_path_factory.mktemp(f"pine{name}"), cfg, seed, dtype,
                            sharpen=3.0 if dtype == torch.float32 else 1.0, router=6.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, dtype, gpu_device)
    lengths = [5, 11, 17, 40, 64, 1, 23, 100, 210]
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    return model, page, requests, ref, TOL[dtype], (pcfg, w, d, dtype)


def runner_for(model, page, num_pages):
    return ModelRunner(model, page_size=page, num_pages=num_pages, num_slots=4)


def test_whole(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_whole(runner_for(model, page, 256 // page), requests), ref, rtol, atol)


def test_prefill_then_long_decode(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_prefill_then_decode(runner_for(model, page, 256 // page), requests,
                                             tail=150), ref, rtol, atol)


def test_portions(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_portions(runner_for(model, page, 256 // page), requests), ref, rtol, atol)


def test_mixed_with_pages_used_again(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    runner = runner_for(model, page, 480 // page)
    compare(drives.drive_mixed(runner, requests), ref, rtol, atol)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)


def test_preempted_and_recomputed(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_preempted(runner_for(model, page, 480 // page), requests), ref, rtol, atol)


def test_float32_does_not_depend_on_the_cut(setup):
    model, page, requests, ref, _, (_, _, _, dtype) = setup
    if dtype != torch.float32:
        pytest.skip("float32 only")
    a = drives.drive_whole(runner_for(model, page, 256 // page), requests)
    b = drives.drive_portions(runner_for(model, page, 256 // page), requests)
    c = drives.drive_mixed(runner_for(model, page, 480 // page), requests)
    for rid in requests:
        torch.testing.assert_close(a.stacked(rid)[0], b.stacked(rid)[0], rtol=1e-4, atol=5e-5)
        torch.testing.assert_close(a.stacked(rid)[0], c.stacked(rid)[0], rtol=1e-4, atol=5e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_layer_shapes_of_a_real_model(gpu_device, tmp_path, dtype):
    """Heads of 128 and 64, a width of 512, experts of 256 beside a shared one of 512: the
    instantiations and products the tiny configurations do not reach, whole, in portions
    and decoded."""
    moe = pinedra_moe(ff=256, experts=6, identity=2, top=2, groups=4, keep=2, scale=2.0, shared=512)
    cfg = pinedra_config(width=512, vocab=1000, eps=1e-6, embed_scale=4.0, loop=(1, 3, 2), layers=[
        pinedra_chunked_attention(heads=8, kv_heads=2, dim=128, vdim=128, scale=128 ** -0.5,
                                  rot_dims=64, base=1e6, softcap=30.0, chunk=128, mlp=moe),
        pinedra_plain_attention(heads=8, kv_heads=2, dim=64, scale=0.125, mlp=moe),
        pinedra_distance_attention(heads=4, kv_heads=4, dim=128, vdim=128, scale=128 ** -0.5,
                                   coef=0.2, every=64, mlp=moe),
        pinedra_plain_attention(heads=4, kv_heads=1, dim=128, scale=0.09, mlp=None)])
    if dtype == torch.bfloat16:
        cfg = all_experts(cfg)
    d = write_pinedra_model(tmp_path, cfg, 5, dtype, std=0.04, sharpen=1.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, dtype, gpu_device)
    requests = {"a": random_prompt(200, 1000, 1), "b": random_prompt(37, 1000, 2)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    rtol, atol = TOL[dtype]
    compare(drives.drive_whole(runner_for(model, 16, 24), requests), ref, rtol, atol)
    compare(drives.drive_prefill_then_decode(runner_for(model, 16, 24), requests, tail=20),
            ref, rtol, atol)
    compare(drives.drive_portions(runner_for(model, 16, 24), requests), ref, rtol, atol)


def plain_greedy(pcfg, w, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(plain.forward(pcfg, w, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_however_the_work_is_cut(setup):
    """LLMEngine.generate: scheduler, captured decode graphs, decode steps launched ahead,
    chunked prefill, preemption by recomputation."""
    model, page, requests, ref, _, (pcfg, w, d, dtype) = setup
    if dtype != torch.float32:
        pytest.skip("greedy tokens are compared in float32")
    prompts = [requests[r] for r in ("r0", "r1", "r2", "r5", "r6", "r3")]
    expected = [plain_greedy(pcfg, w, p, 10) for p in prompts]
    sp = SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)
    base = dict(model=str(d), max_model_len=128, dtype=dtype, kvcache_block_size=page,
                num_kvcache_blocks=64, max_num_seqs=8, max_num_batched_tokens=64,
                chunked_prefill=True)
    for kw in (dict(), dict(enforce_eager=True), dict(max_num_batched_tokens=7),
               dict(max_num_seqs=1), dict(chunked_prefill=False),
               dict(num_kvcache_blocks=-(-50 // page) + 3)):
        engine = LLMEngine(model, Config(**{**base, **kw}))
        assert engine.generate(prompts, sp, use_tqdm=False) == expected, kw
        assert all(p.num_used == 0 for p in engine.runner.manager.pools)
        if not kw:
            assert engine.runner.graphs, "decode steps were not captured"


def test_greedy_generation_in_bfloat16_through_captured_graphs(gpu_device, tmp_path):
    """The bfloat16 decode path as it serves: captured graphs against the eager step."""
    cfg, seed, page = PINE["A"]
    d = write_pinedra_model(tmp_path, all_experts(cfg), seed, torch.bfloat16, sharpen=1.0)
    _, model = load_model(d, torch.bfloat16, gpu_device)
    prompts = [random_prompt(n, cfg["vocab"], 7 + n) for n in (9, 30, 2, 17)]
    sp = SamplingParams(temperature=0.0, max_tokens=24, ignore_eos=True)
    base = dict(model=str(d), max_model_len=128, dtype=torch.bfloat16, kvcache_block_size=16,
                num_kvcache_blocks=64, max_num_seqs=8, max_num_batched_tokens=64,
                chunked_prefill=True)
    eager = LLMEngine(model, Config(**base, enforce_eager=True)).generate(prompts, sp, use_tqdm=False)
    engine = LLMEngine(model, Config(**base))
    assert engine.runner.graphs or engine.generate(prompts[:1], sp, use_tqdm=False)
    assert engine.generate(prompts, sp, use_tqdm=False) == eager


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_sizes_that_are_multiples_of_nothing(gpu_device, tmp_path, dtype):
    """Odd head sizes, a width and inner sizes that are multiples of no tile or vector width,
    one head, one expert, a loop over everything: the products fall to the multiply-add
    kernels and heads are padded."""
    cfg = pinedra_config(width=34, vocab=61, eps=1e-6, embed_scale=1.7, loop=(0, 3, 2), layers=[
        pinedra_distance_attention(heads=3, kv_heads=3, dim=7, vdim=5, scale=0.4, coef=0.7, every=2,
                                   mlp=pinedra_moe(ff=9, experts=1, identity=1, top=1, groups=1,
                                                   keep=1, scale=1.3, shared=5)),
        pinedra_chunked_attention(heads=1, kv_heads=1, dim=6, vdim=10, scale=0.4, rot_dims=2,
                                  base=500.0, softcap=3.0, chunk=11, mlp=None),
        pinedra_plain_attention(heads=5, kv_heads=1, dim=3, scale=0.6,
                                mlp=pinedra_moe(ff=5, experts=2, identity=0, top=2, groups=2,
                                                keep=2, scale=1.0, shared=None))])
    d = write_pinedra_model(tmp_path, cfg, 11, dtype, sharpen=2.0 if dtype == torch.float32 else 1.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, dtype, gpu_device)
    requests = {"a": random_prompt(90, 61, 1), "b": random_prompt(37, 61, 2), "c": random_prompt(1, 61, 3)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    rtol, atol = TOL[dtype]
    compare(drives.drive_whole(runner_for(model, 16, 12), requests), ref, rtol, atol)
    compare(drives.drive_portions(runner_for(model, 16, 12), requests), ref, rtol, atol)
    compare(drives.drive_mixed(runner_for(model, 16, 16), requests), ref, rtol, atol)
