"""Zolorax on the GPU: each new or widened HIP kernel against its plain torch reference (with
state carried over several steps and stale state in the slots), the mixers alone against the
plain implementation with crafted cases that random weights would hide (a key just inside
and just outside a window, a key far back, a sink that carries most of the weight, a state
remembered over hundreds of steps), the engine against the plain whole-sequence
implementation however requests are cut into steps, in float32 and bfloat16, and greedy
generation through LLMEngine."""

import copy

import pytest
import torch

import drives
from helpers import (ZOLO, random_prompt, write_zolorax_model, zolorax_attention, zolorax_config,
                     zolorax_dense, zolorax_moe, zolorax_rglru)
from kernel_refs import TorchOps
from plain import zolorax_plain as plain
from test_palelix_gpu import PART_TOL, Scene, close, compare, load_part, part_context, rnd, \
    run_part_in_steps
from tokensprint_amd.config import Config, SamplingParams
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.engine.llm_engine import LLMEngine
from tokensprint_amd.kernels import load_hip_ops
from tokensprint_amd.models.spec import PartSpec
from tokensprint_amd.parts.base import (FEED_FORWARDS, MIXERS, POSITIONS, PagedKVNeed,
                                        SlotStateNeed, build_part)

pytestmark = pytest.mark.gpu
REF = TorchOps()


def close_part(got, want, dtype, tol32=PART_TOL[torch.float32]):
    """float32: element by element.  bfloat16: every row's error, as a root mean square over
    the row, within 4 % of the row's own (an element's error grows with the magnitudes its
    sum ran over, not with the element that came out)."""
    if dtype == torch.float32:
        return torch.testing.assert_close(got, want, **tol32)
    err = (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-3)
    assert float(err.max()) < 4e-2, f"row {int(err.argmax())}: error {float(err.max()):.4f} of its size"
SPANS = [[7, 1, 3, 40], [1, 1, 0, 2], [2, 5, 1, 1], [1, 1, 1, 1], [150, 1, 0, 200], [1, 1, 1, 1]]


# ------------------------------------------------------------------ kernels


@pytest.mark.parametrize("w_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width, blocks", [(384, 4), (30, 6), (48, 1), (512, 2), (36, 36), (1280, 2)])
def test_gates_of_the_recurrence(gpu_device, w_dtype, width, blocks):
    ops, bw = load_hip_ops(gpu_device), width // blocks
    for T in (1, 3, 8, 77, 300):
        u = rnd((T, width), T).to(gpu_device)
        w_a = rnd((blocks, bw, bw), 1, 0.4).to(w_dtype).to(gpu_device)
        w_i = rnd((blocks, bw, bw), 2, 0.4).to(w_dtype).to(gpu_device)
        b_a, b_i = rnd((width,), 3).to(gpu_device), rnd((width,), 4).to(gpu_device)
        rate = (-8.0 * torch.nn.functional.softplus(rnd((width,), 5, 2.0))).to(gpu_device)
        a, x = ops.rglru_gates(u, w_a, w_i, b_a, b_i, rate)
        ra, rx = REF.rglru_gates(u, w_a, w_i, b_a, b_i, rate)
        close(a, ra, rtol=1e-4, atol=1e-6)
        close(x, rx, rtol=2e-4, atol=1e-5)
        # a token's operands do not depend on what else is in the step
        a1, x1 = ops.rglru_gates(u[T - 1:].contiguous(), w_a, w_i, b_a, b_i, rate)
        assert torch.equal(a1[0], a[T - 1]) and torch.equal(x1[0], x[T - 1])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("width", [48, 336, 5])
def test_recurrence_over_steps_with_stale_state(gpu_device, out_dtype, width):
    """Four requests in scattered slots over several steps: walked, and (a portion of more
    than 128 tokens) in chunks; the slots hold garbage that a request's first portion must
    not read."""
    ops = load_hip_ops(gpu_device)
    needs = SlotStateNeed((width,), torch.float32, "s")
    scene = Scene(gpu_device, needs, 16, 4, num_pages=4)
    state = scene.view.states["s"]
    state.fill_(7.0)
    ref_state = state.clone()
    for step, spans in enumerate(SPANS):
        batch = scene.step(spans)
        T = batch.num_tokens
        a = torch.rand((T, width), generator=torch.Generator().manual_seed(step)).pow(0.1).to(gpu_device)
        x = rnd((T, width), 10 + step).to(gpu_device)
        proj = rnd((T, 2 * width + 3), 20 + step).to(gpu_device)
        yb = rnd((width,), 30).to(gpu_device)
        got = ops.rglru_scan(a, x, proj, 3, yb, batch, state, out_dtype)
        want = REF.rglru_scan(a, x, proj, 3, yb, batch, ref_state, out_dtype)
        tol = dict(rtol=2e-5, atol=2e-5) if out_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
        close(got, want, **tol)
        close(state, ref_state, rtol=2e-5, atol=2e-5)


def test_a_state_is_remembered_over_hundreds_of_steps_and_forgotten(gpu_device):
    """A channel whose decay is 1 to rounding keeps what its first token wrote, token by
    token, over 400 steps; a channel whose decay is small has lost it after a few."""
    ops, width = load_hip_ops(gpu_device), 8
    scene = Scene(gpu_device, SlotStateNeed((width,), torch.float32, "s"), 16, 1, num_pages=4)
    state = scene.view.states["s"]
    proj = torch.full((1, width), 30.0, device=gpu_device)        # gelu(30) = 30
    keep = torch.tensor([1.0] * 4 + [0.5] * 4, device=gpu_device).view(1, width)
    out = None
    for t in range(400):
        batch = scene.step([1])
        x = torch.full((1, width), 3.0 if t == 0 else 0.0, device=gpu_device)
        out = ops.rglru_scan(keep, x, proj, 0, None, batch, state, torch.float32)
    assert torch.equal(out[0, :4].cpu(), torch.full((4,), 90.0))
    assert float(out[0, 4:].abs().max()) == 0.0


def test_convolution_with_a_bias_on_its_inputs_and_no_activation(gpu_device):
    ops, channels, taps = load_hip_ops(gpu_device), 37, 4
    needs = SlotStateNeed((taps - 1, channels), torch.float32, "c")
    scene = Scene(gpu_device, needs, 16, 4, num_pages=4)
    state = scene.view.states["c"]
    state.fill_(5.0)
    ref_state = state.clone()
    w, b = rnd((channels, taps), 1).to(gpu_device), rnd((channels,), 2).to(gpu_device)
    ib = rnd((channels,), 3).to(gpu_device)
    for step, spans in enumerate(SPANS):
        batch = scene.step(spans)
        proj = rnd((batch.num_tokens, channels + 9), 40 + step).to(gpu_device)
        got = ops.conv_silu(proj, 4, channels, w, b, batch, state, in_bias=ib, plain=True)
        want = REF.conv_silu(proj, 4, channels, w, b, batch, ref_state, in_bias=ib, plain=True)
        close(got, want)
        close(state, ref_state)
    # the zeros in front of a sequence are zeros, not the bias: a first token alone
    scene = Scene(gpu_device, needs, 16, 1, num_pages=4)
    batch = scene.step([1])
    proj = torch.zeros(1, channels, device=gpu_device)
    got = ops.conv_silu(proj, 0, channels, w, b, batch, scene.view.states["c"], in_bias=ib, plain=True)
    close(got[0], b + w[:, taps - 1] * ib)


def test_sigmoid_router_and_experts_that_weigh_their_input(gpu_device):
    ops = load_hip_ops(gpu_device)
    for T, E, top in ((1, 16, 1), (33, 6, 2), (200, 5, 5), (7, 3, 1)):
        logits = rnd((T, E), T, 2.0).to(gpu_device)
        got = ops.route_experts(logits, top=top, scores="sigmoid", normalize=False)
        want = REF.route_experts(logits, top=top, scores="sigmoid", normalize=False)
        close(got, want, rtol=1e-6, atol=1e-7)
        assert int((got > 0).sum()) == T * top
        for dtype in (torch.float32, torch.bfloat16):
            inner = 12
            gate_up = rnd((T, E * 2 * inner), 3).to(dtype).to(gpu_device)
            a = ops.expert_activation(gate_up, got, inner, 0.0, dtype, weighted_input=True)
            b = REF.expert_activation(gate_up, got, inner, 0.0, dtype, weighted_input=True)
            close(a, b, **(dict(rtol=1e-5, atol=1e-6) if dtype == torch.float32
                           else dict(rtol=1e-2, atol=1e-3)))
    # equal scores: the lower index
    got = ops.route_experts(torch.zeros(2, 4, device=gpu_device), top=2, scores="sigmoid",
                            normalize=False)
    assert got.cpu().tolist() == [[0.5, 0.5, 0, 0]] * 2


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_squared_relu_and_sigmoid_gate(gpu_device, dtype):
    ops = load_hip_ops(gpu_device)
    tol = dict(rtol=1e-6, atol=1e-6) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-3)
    x = rnd((37, 50), 1).to(dtype).to(gpu_device)
    close(ops.relu_squared(x, dtype), REF.relu_squared(x, dtype), **tol)
    gate = rnd((37, 70), 2).to(gpu_device)
    close(ops.sigmoid_gate(x, gate, 11, dtype), REF.sigmoid_gate(x, gate, 11, dtype), **tol)


# ------------------------------------------------------------------ attention with a sink


def attention_part(gpu_device, dtype, *, width, heads, kv_heads, dim, vdim, rot, window, base=1000.0,
                   scaling=None, scale=0.5, max_position=1024):
    ctx = part_context(gpu_device, dtype, width)
    head = -(-max(dim, vdim) // 16) * 16
    ctx.positions["rot"] = build_part(POSITIONS, PartSpec("rope_partial", {
        "dims": rot, "base": base, "head_dim": head, "max_position": max_position,
        "scaling": scaling}), ctx)
    part = build_part(MIXERS, PartSpec("softmax_attention", {
        "prefix": "x.", "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
        "scale": scale, "position": "rot", "window": window, "qk_norm": True,
        "qk_norm_eps": 1e-5, "sink": True, "gate": True}), ctx)
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
         "rot": {"dims": rot, "base": base}}
    if scaling:
        m["rot"]["scaling"] = scaling
    if window is not None:
        m["mask"] = {"size": window}
    return part, m


def plain_attention(h, w, m):
    kv = plain.attention_keys(h, w, "x.", m, 1e-5)
    return plain.attention(h, w, "x.", m, 1e-5, kv).float()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_attention_alone_whole_and_cut_around_windows_and_pages(gpu_device, dtype):
    """330 tokens over pages of 16: windows below a page, of several pages and none, value
    sizes above and below the key size (heads padded), partial and whole rotation, stretched
    frequencies; whole (the kernels for long portions), and cut at and around page and
    window borders down to single tokens (the kernels for short portions and decode steps)."""
    YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 1.0}
    for heads, kv_heads, dim, vdim, rot, window, scaling in (
            (4, 2, 12, 20, 8, 70, YARN), (2, 2, 24, 8, 24, 5, None), (3, 1, 16, 16, 4, None, YARN),
            (8, 2, 64, 64, 32, 100, None), (4, 2, 96, 80, 40, 33, YARN)):
        width, T = 48, 330
        part, m = attention_part(gpu_device, dtype, width=width, heads=heads, kv_heads=kv_heads,
                                 dim=dim, vdim=vdim, rot=rot, window=window, scaling=scaling)
        w = load_part(part, dtype, gpu_device, 40, sharpen=("x.q.norm", "x.k.norm"),
                      factor=1.5 if dtype == torch.float32 else 1.0)
        h = rnd((T, width), 3).to(dtype)
        want = plain_attention(h.double(), w, m)
        for cuts in ([T], [15, 1, 1, 31, 16, 2, 94, 1, 1, 1, 167]):
            scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=30)
            got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
            close_part(got, want, dtype, dict(rtol=5e-3, atol=5e-4))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("decoded", [False, True])
def test_a_key_just_inside_and_just_outside_the_window_and_a_loud_sink(gpu_device, dtype, decoded):
    """One token carries a value a thousand times the others'.  A query that still has it in
    its window gives an output dominated by it; the next query does not see it at all.  Then
    the sink is raised far above every score: all outputs go to zero."""
    width, T, window, marked = 32, 200, 70, 100
    part, m = attention_part(gpu_device, dtype, width=width, heads=2, kv_heads=1, dim=16, vdim=16,
                             rot=8, window=window)
    w = load_part(part, dtype, gpu_device, 7)
    h = rnd((T, width), 5).to(dtype)
    h[marked] *= 40.0           # the norms take the length out of q and k; the value keeps it
    want = plain_attention(h.double(), w, m)
    cuts = [marked + 60] + [1] * (T - marked - 60) if decoded else [T]
    scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=20)
    got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
    last_in, first_out = marked + window - 1, marked + window
    tol = dict(rtol=5e-3, atol=1e-3) if dtype == torch.float32 else dict(rtol=6e-2, atol=6e-2)
    torch.testing.assert_close(got[last_in - 2:first_out + 3], want[last_in - 2:first_out + 3], **tol)
    # the plain side itself: the marked token matters at last_in and is gone right after
    h2 = h.clone()
    h2[marked] = h[marked] / 40.0
    quiet = plain_attention(h2.double(), w, m)
    assert float((want[last_in] - quiet[last_in]).abs().max()) > 50 * tol["atol"]
    assert torch.equal(want[first_out:], quiet[first_out:])
    # a sink far above every score
    part.sink = torch.full_like(part.sink, 60.0)
    scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=20)
    loud = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
    assert float(loud.abs().max()) < 1e-12 * float(want.abs().max()) + 1e-12


def test_the_sink_in_every_attention_kernel(gpu_device):
    """The attention kernels one by one (float32 arithmetic; decode kernel with its keys split
    and whole, the kernel for short portions and mixed steps, the kernels for long portions)
    against the plain torch attention, with sinks that take a small and a large share."""
    ops = load_hip_ops(gpu_device)
    for dtype in (torch.float32, torch.bfloat16):
        for nq, nkv, hd, window in ((4, 2, 64, None), (8, 8, 128, 40), (6, 1, 96, 300), (2, 2, 48, 17)):
            needs = PagedKVNeed(nkv, hd, window)
            for spans in ([[700, 0, 0, 0]], [[500, 3, 40, 1], [1, 1, 1, 1]], [[90, 1, 0, 33], [2, 40, 7, 1]]):
                scene = Scene(gpu_device, needs, 16, 4, dtype=dtype, num_pages=80)
                sink = torch.tensor([(-2.0, 0.5, 3.0)[j % 3] for j in range(nq)], device=gpu_device)
                for step, sp in enumerate(spans):
                    batch = scene.step(sp)
                    T = batch.num_tokens
                    table = batch.tables[0]
                    k = rnd((T, nkv, hd), step).to(dtype).to(gpu_device)
                    v = rnd((T, nkv, hd), 50 + step).to(dtype).to(gpu_device)
                    q = rnd((T, nq, hd), 90 + step, 1.5).to(dtype).to(gpu_device)
                    ops.kv_store(k, v, batch, table, scene.view)
                    kw = dict(num_heads=nq, num_kv_heads=nkv, head_dim=hd, scale=hd ** -0.5,
                              window=window)
                    got = ops.paged_attention(q, batch, table, scene.view, sink=sink, **kw)
                    only = sorted({0, T - 1, T // 2, min(T - 1, 17)})
                    want = REF.paged_attention(q, batch, table, scene.view, sink=sink, only=only, **kw)
                    bare = REF.paged_attention(q, batch, table, scene.view, only=only, **kw)
                    tol = dict(rtol=1e-4, atol=1e-5) if dtype == torch.float32 \
                        else dict(rtol=3e-2, atol=2e-2)
                    err = (got[only].float() - want[only].float()).abs().cpu()
                    allowed = tol["atol"] + tol["rtol"] * want[only].float().abs().cpu()
                    assert bool((err <= allowed).all()), \
                        (f"{dtype}, heads {nq}/{nkv} of {hd}, window {window}, spans {spans}, step "
                         f"{step}: rows {[only[i] for i in (err > allowed).any(-1).any(-1).nonzero().view(-1).tolist()]}"
                         f" differ, by up to {float(err.max()):.3e}")
                    assert float((want[only].float() - bare[only].float()).abs().max()) > 0.02


def test_readers_of_one_cache_with_windows_of_their_own(gpu_device):
    """A layer that reads another's keys sees its own window of them: the owner's cache keeps
    the widest, and each kernel call masks by its caller's."""
    width, T = 32, 120
    for dtype in (torch.float32, torch.bfloat16):
        owner, m_owner = attention_part(gpu_device, dtype, width=width, heads=2, kv_heads=2, dim=16,
                                        vdim=16, rot=16, window=9)
        owner.cache_window = 50
        ctx = owner.ctx
        reader = build_part(MIXERS, PartSpec("softmax_attention", {
            "prefix": "y.", "heads": 4, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.3,
            "position": "rot", "window": 50, "qk_norm": True, "qk_norm_eps": 1e-5, "sink": True,
            "gate": True, "own_kv": False}), ctx)
        assert not {"y.k", "y.v", "y.k.norm"} & set(reader.tensors())
        w = load_part(owner, dtype, gpu_device, 3)
        w2 = load_part(reader, dtype, gpu_device, 9)
        h = rnd((T, width), 5).to(dtype)
        h2 = rnd((T, width), 6).to(dtype)
        kv = plain.attention_keys(h.double(), w, "x.", m_owner, 1e-5)
        m_reader = dict(m_owner, heads=4, scale=0.3, mask={"size": 50})
        want = plain.attention(h2.double(), w2, "y.", m_reader, 1e-5, kv).float()
        scene = Scene(gpu_device, owner.cache_need(), 16, 1, dtype=dtype, num_pages=12)
        outs, at = [], 0
        for n in [70, 1, 1, 30, 2, 16]:
            batch = scene.step([n])
            owner.forward(h[at:at + n].contiguous().to(gpu_device), batch, scene.view, True)
            outs.append(reader.forward(h2[at:at + n].contiguous().to(gpu_device), batch, scene.view,
                                       False).float().cpu())
            at += n
        close_part(torch.cat(outs), want, dtype, dict(rtol=5e-3, atol=5e-4))


# ------------------------------------------------------------------ the recurrent mixer, feed-forwards


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_recurrent_mixer_alone(gpu_device, dtype):
    for width, lru, blocks, taps in ((48, 96, 2, 4), (40, 30, 6, 1), (64, 256, 1, 3)):
        T = 300
        ctx = part_context(gpu_device, dtype, width)
        part = build_part(MIXERS, PartSpec("rglru", {"prefix": "r.", "width": lru, "blocks": blocks,
                                                     "conv": taps}), ctx)
        w = load_part(part, dtype, gpu_device, 11)
        m = {"width": lru, "blocks": blocks, "conv": taps}
        h = rnd((T, width), 2).to(dtype)
        want = plain.rglru(h.double(), w, "r.", m).float()
        for cuts in ([T], [5, 1, 1, 130, 2, 1, 160]):
            scene = Scene(gpu_device, part.cache_need(), 16, 1, num_pages=4)
            for s in scene.view.states.values():
                s.fill_(3.0)
            got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
            close_part(got, want, dtype)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_feed_forwards_alone(gpu_device, dtype):
    width, T = 40, 50
    ctx = part_context(gpu_device, dtype, width)
    h = rnd((T, width), 2).to(dtype)
    dense = build_part(FEED_FORWARDS, PartSpec("relu2_mlp", {"prefix": "d.", "inner_dim": 56}), ctx)
    w = load_part(dense, dtype, gpu_device, 4)
    close_part(dense.forward(h.to(gpu_device), None).float().cpu(),
               plain.dense_ff(h.double(), w, "d.").float(), dtype)
    for experts, top in ((6, 2), (16, 1), (3, 3)):
        moe = build_part(FEED_FORWARDS, PartSpec("routed_experts", {
            "prefix": "m.", "inner_dim": 12, "experts": experts, "top": top, "scores": "sigmoid",
            "normalize": False, "gated": "silu_on_input"}), ctx)
        # (a router whose logits lie apart: no choice is decided by rounding; many of its
        # sigmoids round to 1, and the experts are still ranked as their logits are)
        w = load_part(moe, dtype, gpu_device, 6, sharpen=("m.router",), factor=6.0)
        mlp = {"router": {"experts": experts, "top": top}}
        close_part(moe.forward(h.to(gpu_device), None).float().cpu(),
                   plain.routed_ff(h.double(), w, "m.", mlp).float(), dtype)


# ------------------------------------------------------------------ the engine


TOL = {torch.float32: (2e-4, 5e-5), torch.bfloat16: (6e-2, 6e-2)}


@pytest.fixture(scope="module", params=[(n, d) for n in sorted(ZOLO)
                                        for d in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def setup(request, tmp_path_factory, gpu_device):
    name, dtype = request.param
    cfg, seed, page = ZOLO[name]
    if dtype == torch.bfloat16:
        # every expert is used: a choice between two experts whose logits lie within the
        # rounding of the router's bfloat16 input would change the token's row and, through
        # the recurrent layers behind it, the rows after it, and the comparison is to show
        # the kernels' precision (the choice itself is compared in float32 and part by part)
        cfg = copy.deepcopy(cfg)
        for layer in cfg["layers"]:
            if layer["mlp"] and layer["mlp"]["kind"] == "moe":
                layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    d = write_zolorax_model(tmp_path_factory.mktemp(f"zolo{name}"), cfg, seed, dtype,
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


def test_mixed_with_pages_and_slots_used_again(setup):
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
    """Heads of 128, a width of 512, recurrences of 1,024 channels in blocks of 256, experts of
    256: the instantiations and products the tiny configurations do not reach, whole, in
    portions and decoded."""
    att = dict(heads=8, kv_heads=2, dim=128, vdim=128, scale=128 ** -0.5, rot_dims=64, base=1e6,
               scaling=(8.0, 128, 32.0, 1.0))
    moe = zolorax_moe(ff=256, experts=8, top=2) if dtype == torch.float32 \
        else zolorax_moe(ff=256, experts=4, top=4)
    cfg = zolorax_config(width=512, vocab=1000, eps=1e-6, layers=[
        zolorax_rglru(width=1024, blocks=4, conv=4, mlp=zolorax_dense(1536)),
        zolorax_attention(**att, window=64, mlp=moe),
        zolorax_attention(**att, window=128, kv_from=1, mlp=zolorax_dense(1024)),
        zolorax_rglru(width=512, blocks=2, conv=4, mlp=moe)])
    d = write_zolorax_model(tmp_path, cfg, 5, dtype, std=0.04, sharpen=1.0)
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
    """LLMEngine.generate: scheduler, state slots, captured decode graphs, decode steps
    launched ahead, chunked prefill, preemption by recomputation."""
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


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_sizes_that_are_multiples_of_nothing(gpu_device, tmp_path, dtype):
    """Odd head sizes, a width, blocks and inner sizes that are multiples of no tile or vector
    width: the products fall to the multiply-add kernels, heads are padded, the recurrence's
    gates take their scalar form."""
    att = dict(heads=3, kv_heads=3, dim=7, vdim=5, scale=0.4, rot_dims=4, base=500.0,
               scaling=(4.0, 32, 8.0, 1.0))
    cfg = zolorax_config(width=34, vocab=61, eps=1e-6, layers=[
        zolorax_attention(**att, window=11, mlp=zolorax_moe(ff=9, experts=3, top=3)),
        zolorax_rglru(width=75, blocks=3, conv=3, mlp=zolorax_dense(27)),
        zolorax_attention(**att, window=29, kv_from=0, mlp=None),
        zolorax_rglru(width=7, blocks=7, conv=2, mlp=zolorax_moe(ff=5, experts=2, top=2))])
    d = write_zolorax_model(tmp_path, cfg, 11, dtype, sharpen=2.0 if dtype == torch.float32 else 1.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, dtype, gpu_device)
    requests = {"a": random_prompt(90, 61, 1), "b": random_prompt(37, 61, 2), "c": random_prompt(1, 61, 3)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    rtol, atol = TOL[dtype]
    compare(drives.drive_whole(runner_for(model, 16, 12), requests), ref, rtol, atol)
    compare(drives.drive_portions(runner_for(model, 16, 12), requests), ref, rtol, atol)
    compare(drives.drive_mixed(runner_for(model, 16, 16), requests), ref, rtol, atol)
