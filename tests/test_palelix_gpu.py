"""Palelix on the GPU: each HIP kernel against its plain torch reference (with state carried
over several steps and stale state in the slots), each mixer and feed-forward alone against
the plain implementation, crafted cases that random weights would hide (a write remembered
over hundreds of steps, a key far back and at page borders), the engine against the plain
whole-sequence implementation however requests are cut into steps, in float32 and bfloat16,
and greedy generation through LLMEngine."""

import pytest
import torch

import drives
from helpers import PALE, random_prompt, write_palelix_model
from kernel_refs import TorchOps
from plain import palelix_plain as plain
from tokensprint_amd.cache import CacheManager, CacheStorage
from tokensprint_amd.config import Config, SamplingParams
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.engine.batch import BatchBuilder, StepEntry
from tokensprint_amd.engine.llm_engine import LLMEngine
from tokensprint_amd.kernels import load_hip_ops
from tokensprint_amd.models.spec import PartSpec
from tokensprint_amd.parts.base import (FEED_FORWARDS, MIXERS, POSITIONS, BuildContext,
                                        SlotStateNeed, build_part)

pytestmark = pytest.mark.gpu
REF = TorchOps()


def rnd(shape, seed, scale=1.0):
    return torch.randn(shape, generator=torch.Generator().manual_seed(seed)) * scale


class Scene:
    """A cache with the given needs, live requests in scattered slots and pages, and
    batches over them: `step(spans)` extends request i by spans[i] tokens (0: left out)."""

    def __init__(self, device, needs, page, num_requests, dtype=torch.float32, num_pages=40):
        self.device = device
        self.storage = CacheStorage([needs], page, num_pages, num_requests + 2, dtype, device)
        self.manager = CacheManager(self.storage.groups, page, num_pages, num_requests + 2)
        order = torch.randperm(num_pages, generator=torch.Generator().manual_seed(5)).tolist()
        for pool in self.manager.pools:
            pool.free = type(pool.free)((i, None) for i in order)
        self.manager.admit("spare")                      # so that slot ids do not start at 0
        self.caches = [self.manager.admit(i) for i in range(num_requests)]
        self.builder = BatchBuilder(device, len(self.storage.groups))
        self.view = self.storage.views[0]

    def step(self, spans):
        entries = []
        for rc, n in zip(self.caches, spans):
            if n:
                start = rc.num_tokens
                self.manager.extend(rc, start + n)
                entries.append(StepEntry(rc, [1] * n, start, [n - 1]))
        return self.builder.build(entries)


def close(a, b, rtol=2e-5, atol=2e-5):
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=rtol, atol=atol)


SPANS = [[7, 1, 3, 40], [1, 1, 0, 2], [2, 5, 1, 1], [1, 1, 1, 1]]


# ------------------------------------------------------------------ the recurrence


@pytest.mark.parametrize("mode", ["fixed", "per_head", "per_channel", "per_head_plain"])
@pytest.mark.parametrize("heads, kv_heads, dim, vdim", [(4, 2, 16, 64), (3, 1, 10, 6),
                                                        (2, 2, 5, 70), (1, 1, 132, 9)])
def test_recurrence_over_steps_with_stale_state(gpu_device, mode, heads, kv_heads, dim, vdim):
    ops = load_hip_ops(gpu_device)
    if mode == "fixed":
        kv_heads = heads
    qk, inner = kv_heads * dim, heads * vdim
    scene = Scene(gpu_device, SlotStateNeed((heads, dim, vdim), torch.float32, "s"), 8, 4)
    st = scene.view.states["s"]
    st.fill_(3.0)                       # stale state of whoever held the slot before
    st_ref = st.clone()
    decay = torch.rand(heads, generator=torch.Generator().manual_seed(1)).to(gpu_device)
    for i, spans in enumerate(SPANS):
        batch = scene.step(spans)
        T = batch.num_tokens
        x = rnd((T, 3 + 2 * qk + inner), 10 + i, 0.5).to(gpu_device)
        kw = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim)
        if mode == "fixed":
            kw.update(silu_inputs=True, decay=decay)
        else:
            n = heads * dim if mode == "per_channel" else heads
            gates = torch.rand(T, heads + n, generator=torch.Generator().manual_seed(20 + i))
            kw.update(silu_inputs=False, gates=gates.to(gpu_device),
                      per_channel=mode == "per_channel", delta=mode != "per_head_plain")
        got = ops.linear_recurrence(x, 3, 3 + qk, 3 + 2 * qk, batch, st, **kw)
        want = REF.linear_recurrence(x, 3, 3 + qk, 3 + 2 * qk, batch, st_ref, **kw)
        close(got, want, rtol=1e-4, atol=1e-4)
        close(st, st_ref, rtol=1e-4, atol=1e-4)


@pytest.mark.parametrize("mode", ["fixed", "per_head_plain"])
@pytest.mark.parametrize("heads, dim, vdim", [(4, 16, 64), (3, 10, 6), (2, 128, 70)])
def test_long_portions_run_in_chunks(gpu_device, mode, heads, dim, vdim):
    """Without the delta rule portions beyond 128 tokens are cut into chunks of 64 that run
    side by side; beside them short portions and single tokens, states carried on."""
    ops = load_hip_ops(gpu_device)
    qk, inner = heads * dim, heads * vdim
    scene = Scene(gpu_device, SlotStateNeed((heads, dim, vdim), torch.float32, "s"), 8, 4,
                  num_pages=200)
    st = scene.view.states["s"]
    st.fill_(3.0)
    st_ref = st.clone()
    decay = (0.9 + 0.1 * torch.rand(heads, generator=torch.Generator().manual_seed(1))).to(gpu_device)
    for i, spans in enumerate([[300, 1, 131, 5], [1, 1, 1, 1], [200, 3, 0, 129]]):
        batch = scene.step(spans)
        T = batch.num_tokens
        x = rnd((T, 2 * qk + inner), 10 + i, 0.5).to(gpu_device)
        kw = dict(heads=heads, kv_heads=heads, dim=dim, vdim=vdim)
        if mode == "fixed":
            kw.update(silu_inputs=True, decay=decay)
        else:
            gates = 0.9 + 0.1 * torch.rand(T, 2 * heads, generator=torch.Generator().manual_seed(i))
            kw.update(silu_inputs=False, gates=gates.to(gpu_device))
        got = ops.linear_recurrence(x, 0, qk, 2 * qk, batch, st, **kw)
        want = REF.linear_recurrence(x, 0, qk, 2 * qk, batch, st_ref, **kw)
        close(got, want, rtol=2e-4, atol=2e-4)
        close(st, st_ref, rtol=2e-4, atol=2e-4)


@pytest.mark.parametrize("delta", [False, True])
def test_a_write_is_remembered_over_hundreds_of_steps_and_forgotten(gpu_device, delta):
    """One token writes a value under a key; 300 tokens later, alone in their steps, a query
    for that key reads decay^300 of it: all of it without a decay, e^-0.3 of it at 0.999,
    nothing at 0.5.  With the delta rule a second write under the same key replaces it."""
    ops = load_hip_ops(gpu_device)
    heads, dim, vdim = 3, 8, 4
    scene = Scene(gpu_device, SlotStateNeed((heads, dim, vdim), torch.float32, "s"), 8, 1)
    st = scene.view.states["s"]
    st.fill_(9.0)
    decays = torch.tensor([1.0, 0.999, 0.5])
    key = torch.zeros(dim)
    key[2] = 1.0
    value = torch.tensor([1.0, -2.0, 3.0, 0.5])
    n = 301

    def row(q, k, v):
        return torch.cat([q.repeat(heads), k.repeat(heads), v.repeat(heads)])

    rows = [row(torch.zeros(dim), key, value)] + [row(torch.zeros(dim), torch.zeros(dim),
                                                      torch.zeros(vdim))] * (n - 2)
    rows.append(row(key, key if delta else torch.zeros(dim), 2 * value))
    out = None
    for t in range(n):
        batch = scene.step([40] if t == 0 else [1])
        T = batch.num_tokens
        x = torch.zeros(T, 2 * heads * dim + heads * vdim)
        x[-1] = rows[t]
        if t == 0:
            x[0], x[-1] = rows[0], rows[1]              # the write stands 40 tokens back
        kw = dict(heads=heads, kv_heads=heads, dim=dim, vdim=vdim, silu_inputs=False)
        if delta:
            gates = torch.cat([torch.ones(T, heads), decays.expand(T, heads)], dim=1)
            kw.update(gates=gates.to(gpu_device), delta=True)
        else:
            kw.update(decay=decays.to(gpu_device))
        out = ops.linear_recurrence(x.to(gpu_device), 0, heads * dim, 2 * heads * dim, batch, st,
                                    **kw)
    got = out[-1].view(heads, vdim).cpu()
    steps = 40 + n - 2                  # decays between the write and the read
    if delta:
        # beta 1: the value under the key becomes the new one whatever was left of the old
        want = (2 * value).expand(heads, vdim)
    else:
        want = (decays ** steps)[:, None] * value
    torch.testing.assert_close(got, want, rtol=1e-4, atol=1e-6)
    assert got[2].abs().max() < 1e-6 or delta


@pytest.mark.parametrize("per_channel", [False, True])
def test_delta_gates(gpu_device, per_channel):
    ops = load_hip_ops(gpu_device)
    for T, heads, kv_heads, dim, vdim in ((1, 4, 2, 64, 64), (37, 3, 1, 10, 6), (5, 2, 2, 5, 70)):
        qk = kv_heads * dim
        qkv = rnd((T, 2 * qk + heads * vdim), 1).to(gpu_device)
        proj = rnd((T, 7 + 3 * heads), 2).to(gpu_device)
        n = heads * dim if per_channel else heads
        z = rnd((T, 2 + n), 3, 2.0).to(gpu_device)
        a_log, dt_bias = rnd((heads,), 4).to(gpu_device), rnd((n,), 5).to(gpu_device)
        a, b = qkv.clone(), qkv.clone()
        kw = dict(heads=heads, kv_heads=kv_heads, dim=dim, per_channel=per_channel)
        got = ops.delta_gates(a, proj, 7, z, 2, a_log, dt_bias, **kw)
        want = REF.delta_gates(b, proj, 7, z, 2, a_log, dt_bias, **kw)
        close(got, want)
        close(a, b)
        # q and k heads are unit vectors (q over sqrt(dim)), v is untouched
        norms = a[:, :2 * qk].view(T, 2, kv_heads, dim).norm(dim=-1).cpu()
        torch.testing.assert_close(norms[:, 0], torch.full_like(norms[:, 0], dim ** -0.5),
                                   rtol=1e-4, atol=1e-5)
        torch.testing.assert_close(norms[:, 1], torch.ones_like(norms[:, 1]), rtol=1e-4, atol=1e-5)
        assert torch.equal(a[:, 2 * qk:], qkv[:, 2 * qk:])


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_norm_gate(gpu_device, out_dtype):
    ops = load_hip_ops(gpu_device)
    tol = dict(rtol=2e-5, atol=2e-5) if out_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    for T, groups, width in ((1, 1, 40), (9, 4, 64), (33, 3, 70), (5, 1, 1030)):
        inner = groups * width
        y, gate = rnd((T, inner), 1, 3.0).to(gpu_device), rnd((T, inner + 5), 2).to(gpu_device)
        for w in ((1 + 0.1 * rnd((width,), 3)).to(gpu_device), (1 + 0.1 * rnd((inner,), 4)).to(gpu_device)):
            for kind in ("sigmoid", "silu"):
                kw = dict(groups=groups, gate=kind, eps=1e-5, out_dtype=out_dtype)
                close(ops.norm_gate(y, gate, 5, w, **kw), REF.norm_gate(y, gate, 5, w, **kw), **tol)


def test_convolution_without_a_bias(gpu_device):
    ops = load_hip_ops(gpu_device)
    for taps in (1, 2, 4):
        C = 21
        scene = Scene(gpu_device, SlotStateNeed((taps - 1, C), torch.float32, "conv"), 8, 4)
        st = scene.view.states["conv"]
        st.fill_(2.0)
        st_ref = st.clone()
        w = rnd((C, taps), 1).to(gpu_device)
        for i, spans in enumerate(SPANS):
            batch = scene.step(spans)
            proj = rnd((batch.num_tokens, C + 4), 10 + i).to(gpu_device)
            close(ops.conv_silu(proj, 3, C, w, None, batch, st),
                  REF.conv_silu(proj, 3, C, w, None, batch, st_ref))
            close(st, st_ref)


# ------------------------------------------------------------------ experts, stream sums


def test_route_experts(gpu_device):
    ops = load_hip_ops(gpu_device)
    for T, E, top, count, keep in ((1, 12, 3, 3, 2), (37, 8, 2, 4, 1), (300, 64, 6, 8, 3),
                                   (5, 5, 5, 1, 1), (9, 130, 1, 1, 1), (6, 6, 2, 6, 6)):
        logits = rnd((T, E), T, 2.0).to(gpu_device)
        got = ops.route_experts(logits, top=top, group_count=count, group_keep=keep).cpu()
        close(got, REF.route_experts(logits, top=top, group_count=count, group_keep=keep))
        scores = torch.softmax(logits.double().cpu(), dim=-1)
        for t in range(min(T, 20)):
            chosen, w = plain.route(scores[t], top, count, keep)
            assert sorted(got[t].nonzero().flatten().tolist()) == sorted(chosen.tolist())
            torch.testing.assert_close(got[t][chosen].double(), w, rtol=1e-5, atol=1e-6)


def test_route_experts_at_equal_scores_takes_the_lower_index(gpu_device):
    ops = load_hip_ops(gpu_device)
    logits = torch.zeros(3, 8, device=gpu_device)
    got = ops.route_experts(logits, top=3, group_count=4, group_keep=2).cpu()
    assert got.nonzero()[:, 1].view(3, 3).tolist() == [[0, 1, 2]] * 3
    torch.testing.assert_close(got[:, :3], torch.full((3, 3), 1 / 3))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_expert_activation_and_stream_sums(gpu_device, dtype):
    ops = load_hip_ops(gpu_device)
    tol = dict(rtol=2e-5, atol=2e-5) if dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    T, E, inner = 19, 5, 12
    gate_up = rnd((T, E * 2 * inner), 1, 2.0).to(dtype).to(gpu_device)
    weights = torch.rand(T, E, generator=torch.Generator().manual_seed(2))
    weights[weights < 0.5] = 0.0
    weights = weights.to(gpu_device)
    got = ops.expert_activation(gate_up, weights, inner, 1.3, dtype)
    close(got, REF.expert_activation(gate_up, weights, inner, 1.3, dtype), **tol)
    assert (got.view(T, E, inner)[weights == 0] == 0).all()
    for rows, width in ((1, 40), (9, 257), (3, 2500)):
        resid = rnd((rows, width), 3).to(gpu_device)
        a, b = rnd((rows, width), 4).to(dtype).to(gpu_device), rnd((rows, width), 5).to(gpu_device)
        row = rnd((width,), 6).to(gpu_device)
        for args in ((a, b, None), (a, None, None), (None, None, row), (a, b, row)):
            x, y = resid.clone(), resid.clone()
            ops.stream_add(x, *args)
            REF.stream_add(y, *args)
            close(x, y)
            w = (1 + 0.1 * rnd((width,), 7)).to(gpu_device)
            if args[0] is not None:
                x, y = resid.clone(), resid.clone()
                close(ops.stream_add_norm(x, *args, w, 1e-5, dtype),
                      REF.stream_add_norm(y, *args, w, 1e-5, dtype), **tol)
                close(x, y)
        close(ops.scaled_sum(a, 0.7, b, -1.3), REF.scaled_sum(a, 0.7, b, -1.3))
        close(ops.take_columns(b, 3, width - 7, dtype), REF.take_columns(b, 3, width - 7, dtype), **tol)


# ------------------------------------------------------------------ each part alone


def part_context(gpu_device, dtype, width):
    return BuildContext(ops=load_hip_ops(gpu_device), dtype=dtype, device=gpu_device, width=width)


def load_part(part, dtype, gpu_device, seed, sharpen=(), factor=3.0):
    """Random tensors for a part's declarations; returns them in float64 for the plain side."""
    tensors = {}
    for i, (name, decl) in enumerate(sorted(part.tensors().items())):
        if decl.init is not None:
            t = decl.init[0] + torch.rand(decl.shape, generator=torch.Generator().manual_seed(
                seed + i)) * (decl.init[1] - decl.init[0])
        elif decl.role == "vector":
            t = 1 + 0.1 * rnd(decl.shape, seed + i)
        else:
            t = rnd(decl.shape, seed + i, 0.3)
        if name.endswith(sharpen):
            t = t * factor
        held = torch.float32 if decl.role == "vector" else dtype
        tensors[name] = t.to(held)
    part.load(lambda n: tensors[n].to(gpu_device))
    return {n: t.double() for n, t in tensors.items()}


def run_part_in_steps(part, h, scene, spans_list):
    """The part's output over request 0's tokens fed in the given portions."""
    outs, at = [], 0
    for n in spans_list:
        batch = scene.step([n])
        outs.append(part.forward(h[at:at + n].contiguous(), batch, scene.view, True))
        at += n
    return torch.cat([o.float() for o in outs]).cpu()


PART_TOL = {torch.float32: dict(rtol=2e-4, atol=2e-5), torch.bfloat16: dict(rtol=5e-2, atol=3e-2)}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_softmax_attention_alone_far_keys_and_page_borders(gpu_device, dtype):
    """Sharp scores (a few keys carry a query's weight), 330 tokens over pages of 16, value
    size above and below the key size, partial rotation: whole, and cut at and around page
    borders down to single tokens."""
    for heads, kv_heads, dim, vdim, rot in ((4, 2, 12, 20, 8), (2, 2, 24, 8, 24), (3, 1, 16, 16, 4)):
        width, T = 48, 330
        ctx = part_context(gpu_device, dtype, width)
        head = -(-max(dim, vdim) // 16) * 16
        ctx.positions["rot"] = build_part(POSITIONS, PartSpec("rope_partial", {
            "dims": rot, "base": 1000.0, "head_dim": head, "max_position": 512}), ctx)
        m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": 0.6,
             "rot": {"dims": rot, "base": 1000.0}}
        part = build_part(MIXERS, PartSpec("softmax_attention", {
            "prefix": "x.", "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
            "scale": 0.6, "position": "rot", "window": None}), ctx)
        # (bfloat16: scores of a few units, or the operands' rounding moves the weights)
        w = load_part(part, dtype, gpu_device, 40, sharpen=("x.q", "x.k"),
                      factor=3.0 if dtype == torch.float32 else 0.3)
        h = rnd((T, width), 3).to(dtype)
        want = plain.softmax_attention(h.double(), w, "x.", m).float()
        # (scores of some tens: a float32 angle's last bit moves a softmax weight by 1e-3 of
        # itself, a key that is lost or seen too early by all of it)
        tol = dict(rtol=5e-3, atol=5e-4) if dtype == torch.float32 else PART_TOL[dtype]
        for cuts in ([T], [15, 1, 1, 31, 16, 2, 94, 1, 1, 1, 167]):
            scene = Scene(gpu_device, part.cache_need(), 16, 1, dtype=dtype, num_pages=30)
            got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
            torch.testing.assert_close(got, want, **tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("per_channel", [False, True])
def test_gated_delta_rule_alone(gpu_device, dtype, per_channel):
    for heads, kv_heads, dim, vdim, conv in ((4, 2, 16, 8, 3), (1, 1, 9, 70, 1), (3, 3, 4, 4, 4)):
        width, T = 40, 90
        ctx = part_context(gpu_device, dtype, width)
        params = {"prefix": "x.", "heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                  "conv": conv, "eps": 1e-5, "per_channel": per_channel, "decay_rank": 6,
                  "gate_rank": 5, "state": "d"}
        part = build_part(MIXERS, PartSpec("gated_delta", params), ctx)
        w = load_part(part, dtype, gpu_device, 50)
        h = rnd((T, width), 4).to(dtype)
        want = plain.delta_mixer(h.double(), w, "x.", params, 1e-5, per_channel).float()
        for cuts in ([T], [2, 1, 1, 40, 1, 45]):
            scene = Scene(gpu_device, part.cache_need(), 16, 1)
            for st in scene.view.states.values():
                st.fill_(5.0)
            got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
            torch.testing.assert_close(got, want, **PART_TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_lightning_attention_alone(gpu_device, dtype):
    for heads, dim, vdim, decay in ((4, 8, 16, (0.5, 0.9, 0.99, 0.999)), (1, 20, 70, (1.0,))):
        width, T = 40, 120
        ctx = part_context(gpu_device, dtype, width)
        params = {"prefix": "x.", "heads": heads, "dim": dim, "vdim": vdim, "decay": decay,
                  "eps": 1e-5, "state": "l"}
        part = build_part(MIXERS, PartSpec("lightning_attention", params), ctx)
        w = load_part(part, dtype, gpu_device, 60)
        h = rnd((T, width), 5).to(dtype)
        want = plain.lightning_mixer(h.double(), w, "x.", params, 1e-5).float()
        for cuts in ([T], [1, 1, 70, 2, 46]):
            scene = Scene(gpu_device, part.cache_need(), 16, 1)
            scene.view.states["l"].fill_(5.0)
            got = run_part_in_steps(part, h.to(gpu_device), scene, cuts)
            torch.testing.assert_close(got, want, **PART_TOL[dtype])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_routed_experts_alone(gpu_device, dtype):
    for experts, top, count, keep, inner in ((6, 2, 3, 2, 12), (4, 4, 1, 1, 8), (16, 3, 4, 2, 20)):
        width, T = 40, 70
        ctx = part_context(gpu_device, dtype, width)
        part = build_part(FEED_FORWARDS, PartSpec("routed_experts", {
            "prefix": "x.", "inner_dim": inner, "experts": experts, "top": top,
            "group_count": count, "group_keep": keep, "limit": 0.9}), ctx)
        w = load_part(part, dtype, gpu_device, 70, sharpen=("x.router",))
        h = rnd((T, width), 6).to(dtype)
        mlp = {"router": {"experts": experts, "top": top, "groups": {"count": count, "keep": keep}},
               "expert": {"ff": inner, "limit": 0.9}}
        want = plain.moe_ff(h.double(), w, "x.", mlp).float()
        got = part.forward(h.to(gpu_device), None).float().cpu()
        torch.testing.assert_close(got, want, **PART_TOL[dtype])


# ------------------------------------------------------------------ the engine

TOL = {torch.float32: (2e-4, 5e-5), torch.bfloat16: (6e-2, 6e-2)}


def compare(col, ref, rtol, atol):
    """float32: every row within the tolerance.  bfloat16: a router's choice between two
    experts of nearly equal score is decided by rounding, and the token's logits then differ
    by more than rounding, so up to one row in twenty-five may lie outside; a state or a key
    that is lost puts every later row outside."""
    if rtol < 1e-2:
        return drives.compare(col, ref, rtol, atol)
    errors = []
    for rid, want in ref.items():
        got, positions = col.stacked(rid)
        assert positions == list(range(want.shape[0]))
        assert torch.isfinite(got).all()
        # a row's error as the replayed traces are judged: the root mean square of the
        # difference over the vocabulary, its mean taken off, in units of the logits' own
        diff = got - want
        diff = diff - diff.mean(dim=1, keepdim=True)
        errors.append(diff.pow(2).mean(dim=1).sqrt() / want.std())
    errors = torch.cat(errors)
    bad = int((errors > atol).sum())
    assert bad <= 0.04 * errors.numel() and float(errors.median()) < atol / 3, \
        (f"{bad} of {errors.numel()} rows outside the tolerance; median error "
         f"{float(errors.median()):.4f}, largest {float(errors.max()):.4f}")


@pytest.fixture(scope="module", params=[(n, d) for n in sorted(PALE)
                                        for d in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def setup(request, tmp_path_factory, gpu_device):
    name, dtype = request.param
    cfg, seed, page = PALE[name]
    d = write_palelix_model(tmp_path_factory.mktemp(f"pale{name}"), cfg, seed, dtype,
                            sharpen=4.0 if dtype == torch.float32 else 1.0)
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
    compare(drives.drive_whole(runner_for(model, page, 256 // page), requests),
                   ref, rtol, atol)


def test_prefill_then_long_decode(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_prefill_then_decode(runner_for(model, page, 256 // page),
                                                    requests, tail=150), ref, rtol, atol)


def test_portions(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_portions(runner_for(model, page, 256 // page), requests),
                   ref, rtol, atol)


def test_mixed_with_pages_and_slots_used_again(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    runner = runner_for(model, page, 480 // page)
    compare(drives.drive_mixed(runner, requests), ref, rtol, atol)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)


def test_preempted_and_recomputed(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    compare(drives.drive_preempted(runner_for(model, page, 480 // page), requests),
                   ref, rtol, atol)


def test_float32_does_not_depend_on_the_cut(setup):
    """A position's float32 logits are the same to rounding whether its request ran whole,
    in portions or token by token beside others."""
    model, page, requests, ref, _, (_, _, _, dtype) = setup
    if dtype != torch.float32:
        pytest.skip("float32 only")
    a = drives.drive_whole(runner_for(model, page, 256 // page), requests)
    b = drives.drive_portions(runner_for(model, page, 256 // page), requests)
    c = drives.drive_mixed(runner_for(model, page, 480 // page), requests)
    # (a long portion's recurrence adds a column's parts over sixteen lanes, a short one's over
    # eight: the same sums in another order)
    for rid in requests:
        torch.testing.assert_close(a.stacked(rid)[0], b.stacked(rid)[0], rtol=1e-4, atol=5e-5)
        torch.testing.assert_close(a.stacked(rid)[0], c.stacked(rid)[0], rtol=1e-4, atol=5e-5)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["float32", "bfloat16"])
def test_layer_shapes_of_a_real_model(gpu_device, tmp_path, dtype):
    """Heads of 128 x 128, a width of 512, experts of 256: the instantiations and products
    that the tiny configurations do not reach (sixteen rows a lane, the vendor library's
    products, attention heads of 128), whole, in portions and decoded."""
    from helpers import (palelix_config, palelix_delta, palelix_delta_sizes, palelix_dense,
                         palelix_lightning, palelix_moe, palelix_parallel)
    # (bfloat16: every expert is used, so that no choice between nearly equal scores is
    # decided by rounding and the comparison shows the kernels' precision alone)
    moe = palelix_moe(ff=256, limit=7.0, experts=8, top=2, count=4, keep=2) \
        if dtype == torch.float32 else \
        palelix_moe(ff=256, limit=7.0, experts=8, top=8, count=1, keep=1)
    cfg = palelix_config(width=512, vocab=1000, eps=1e-6, loop=(1, 3, 2), layers=[
        palelix_delta(heads=4, kv_heads=2, dim=128, vdim=128, conv=4, mlp=palelix_dense(1024)),
        palelix_lightning(heads=4, dim=128, vdim=128, decay=(0.75, 0.9, 0.99, 0.999), mlp=moe),
        palelix_parallel(heads=4, kv_heads=2, dim=128, vdim=128, rot_dims=64, base=1e6,
                         scale=128 ** -0.5, left_scale=1.0, right_scale=1.0,
                         right=palelix_delta_sizes(heads=2, kv_heads=2, dim=64, vdim=128, conv=4,
                                                   ranks=(64, 64)), mlp=moe)])
    d = write_palelix_model(tmp_path, cfg, 5, dtype, std=0.04, sharpen=1.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, dtype, gpu_device)
    requests = {"a": random_prompt(150, 1000, 1), "b": random_prompt(37, 1000, 2)}
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
