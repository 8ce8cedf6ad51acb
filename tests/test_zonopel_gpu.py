"""Zonopel on the GPU: each HIP kernel against its plain torch reference (with state
carried over two steps), crafted cases that random weights would hide (a far key, the edges
of a window), the engine against the plain whole-sequence implementation however requests
are cut into steps, in float32 and bfloat16, and greedy generation through LLMEngine."""

import pytest
import torch

import drives
from helpers import ZONO, random_prompt
from kernel_refs import TorchOps
from plain import zonopel_plain as plain
from tokensprint_amd.cache import CacheManager, CacheStorage
from tokensprint_amd.config import Config, SamplingParams
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.engine.batch import BatchBuilder, StepEntry
from tokensprint_amd.engine.llm_engine import LLMEngine
from tokensprint_amd.kernels import load_hip_ops
from tokensprint_amd.parts.base import PagedLatentNeed, SlotStateNeed
from tokensprint_amd.weights import write_random_model

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

    def clone_states(self):
        return {k: v.clone() for k, v in self.view.states.items()}


def close(a, b, rtol=2e-5, atol=2e-5):
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=rtol, atol=atol)


SPANS = [[7, 1, 3, 40], [1, 1, 0, 2], [2, 5, 1, 1], [1, 1, 1, 1]]


# ------------------------------------------------------------------ row kernels


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_bigram_embedding(gpu_device, dtype):
    ops = load_hip_ops(gpu_device)
    vocab, width, buckets = 53, 44, 19
    table, bigram = rnd((vocab, width), 1).to(dtype).to(gpu_device), \
        rnd((buckets + 1, width), 2).to(dtype).to(gpu_device)
    w = (1 + 0.1 * rnd((width,), 3)).to(gpu_device)
    scene = Scene(gpu_device, SlotStateNeed((1,), torch.int32, "prev_token"), 8, 4)
    st = scene.view.states["prev_token"]
    st.fill_(7)                         # stale state of whoever held the slot before
    st_ref = st.clone()
    kw = dict(scale=1.7, buckets=buckets, mul_prev=1000003, mul_cur=77, eps=1e-5)
    for i, spans in enumerate(SPANS):
        batch = scene.step(spans)
        batch.token_ids.copy_(torch.randint(0, vocab, (batch.num_tokens,),
                                            generator=torch.Generator().manual_seed(i)))
        got = ops.bigram_embed(table, bigram, w, batch, st, **kw)
        want = REF.bigram_embed(table, bigram, w, batch, st_ref, **kw)
        close(got, want)
        assert torch.equal(st.cpu(), st_ref.cpu())


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_postnorm_add_and_polynorm(gpu_device, out_dtype):
    ops = load_hip_ops(gpu_device)
    tol = dict(rtol=2e-5, atol=2e-5) if out_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    for rows, width in ((1, 40), (9, 257), (33, 1024)):
        resid, delta = rnd((rows, width), 1).to(gpu_device), rnd((rows, width), 2, 3.0).to(gpu_device)
        pw, nw = (1 + 0.1 * rnd((width,), 3)).to(gpu_device), (1 + 0.1 * rnd((width,), 4)).to(gpu_device)
        a, b = resid.clone(), resid.clone()
        ops.postnorm_add(a, delta, pw, 1e-5)
        REF.postnorm_add(b, delta, pw, 1e-5)
        close(a, b)
        a, b = resid.clone(), resid.clone()
        close(ops.postnorm_add_norm(a, delta, pw, 1e-5, nw, 1e-6, out_dtype),
              REF.postnorm_add_norm(b, delta, pw, 1e-5, nw, 1e-6, out_dtype), **tol)
        close(a, b)
        coef = torch.tensor([0.3, -0.2, 0.5, 0.1], device=gpu_device)
        close(ops.polynorm(delta, coef, 1e-5, out_dtype), REF.polynorm(delta, coef, 1e-5, out_dtype),
              **tol)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_norm_token_shift_carries_the_last_row(gpu_device, out_dtype):
    ops = load_hip_ops(gpu_device)
    width = 72
    scene = Scene(gpu_device, SlotStateNeed((width,), torch.float32, "shift"), 8, 4)
    st = scene.view.states["shift"]
    st.fill_(3.0)
    st_ref = st.clone()
    nw, sw = (1 + 0.1 * rnd((width,), 3)).to(gpu_device), torch.rand(width).to(gpu_device)
    tol = dict(rtol=2e-5, atol=2e-5) if out_dtype == torch.float32 else dict(rtol=1e-2, atol=1e-2)
    for i, spans in enumerate(SPANS):
        batch = scene.step(spans)
        resid = rnd((batch.num_tokens, width), 10 + i).to(gpu_device)
        close(ops.norm_token_shift(resid, nw, 1e-5, sw, batch, st, out_dtype),
              REF.norm_token_shift(resid, nw, 1e-5, sw, batch, st_ref, out_dtype), **tol)
        close(st, st_ref)


# ------------------------------------------------------------------ state-space mixer


@pytest.mark.parametrize("heads, vdim, N, groups, taps", [(4, 6, 5, 4, 4), (2, 40, 20, 1, 2),
                                                          (3, 64, 128, 3, 1), (6, 48, 48, 2, 9)])
def test_convolution_and_recurrence_over_steps(gpu_device, heads, vdim, N, groups, taps):
    ops = load_hip_ops(gpu_device)
    inner, C = heads * vdim, heads * vdim + 2 * groups * N
    ld = 2 * inner + 2 * groups * N + heads
    needs = (SlotStateNeed((taps - 1, C), torch.float32, "conv"),
             SlotStateNeed((heads, N, vdim), torch.float32, "ssm"))
    scene = Scene(gpu_device, needs, 8, 4)
    for s in scene.view.states.values():
        s.fill_(9.0)
    ref_states = scene.clone_states()
    cw, cb = rnd((C, taps), 1, 0.5).to(gpu_device), rnd((C,), 2, 0.1).to(gpu_device)
    dt_bias, a_log = rnd((heads,), 3).to(gpu_device) - 1, rnd((heads,), 4, 0.5).to(gpu_device)
    d_skip, nw = rnd((heads,), 5).to(gpu_device), (1 + 0.1 * rnd((inner,), 6)).to(gpu_device)
    for i, spans in enumerate(SPANS):
        batch = scene.step(spans)
        proj = rnd((batch.num_tokens, ld), 20 + i).to(gpu_device)
        got = ops.conv_silu(proj, inner, C, cw, cb, batch, scene.view.states["conv"])
        want = REF.conv_silu(proj, inner, C, cw, cb, batch, ref_states["conv"])
        close(got, want)
        close(scene.view.states["conv"], ref_states["conv"])
        kw = dict(heads=heads, vdim=vdim, state_rows=N, groups=groups)
        y = ops.ssm_scan(want, proj, ld - heads, dt_bias, a_log, d_skip, batch,
                         scene.view.states["ssm"], **kw)
        y_ref = REF.ssm_scan(want, proj, ld - heads, dt_bias, a_log, d_skip, batch,
                             ref_states["ssm"], **kw)
        close(y, y_ref, rtol=1e-4, atol=1e-4)
        close(scene.view.states["ssm"], ref_states["ssm"], rtol=1e-4, atol=1e-4)
        for g in (1, heads):
            close(ops.gated_group_norm(y_ref, proj, nw, g, 1e-5, torch.float32),
                  REF.gated_group_norm(y_ref, proj, nw, g, 1e-5, torch.float32))


def test_long_portions_run_in_chunks(gpu_device):
    """Portions above the chunking threshold (cut into runs of 64 tokens side by side)
    beside short ones, continued over steps: the same y and state as the plain walk."""
    ops = load_hip_ops(gpu_device)
    heads, vdim, N, groups = 3, 40, 20, 1
    inner = heads * vdim
    scene = Scene(gpu_device, SlotStateNeed((heads, N, vdim), torch.float32, "ssm"), 16, 4,
                  num_pages=80)
    state = scene.view.states["ssm"]
    state.fill_(5.0)
    ref_state = state.clone()
    dt_bias, a_log = rnd((heads,), 3).to(gpu_device) - 2, rnd((heads,), 4, 0.5).to(gpu_device) - 1
    d_skip = rnd((heads,), 5).to(gpu_device)
    for i, spans in enumerate([[300, 1, 130, 64], [1, 200, 2, 129], [129, 0, 1, 1]]):
        batch = scene.step(spans)
        assert batch.max_q_len > ops.dispatch.scan_whole_tokens
        xbc = rnd((batch.num_tokens, inner + 2 * groups * N), 50 + i, 0.5).to(gpu_device)
        proj = rnd((batch.num_tokens, heads), 60 + i).to(gpu_device)
        kw = dict(heads=heads, vdim=vdim, state_rows=N, groups=groups)
        y = ops.ssm_scan(xbc, proj, 0, dt_bias, a_log, d_skip, batch, state, **kw)
        y_ref = REF.ssm_scan(xbc, proj, 0, dt_bias, a_log, d_skip, batch, ref_state, **kw)
        close(y, y_ref, rtol=1e-4, atol=1e-4)
        close(state, ref_state, rtol=1e-4, atol=1e-4)


def test_recurrence_remembers_a_far_token(gpu_device):
    """With a decay of almost one, what one early token wrote is read hundreds of tokens
    later, across steps; with a strong decay it is gone."""
    ops = load_hip_ops(gpu_device)
    heads, vdim, N = 1, 8, 4
    needs = SlotStateNeed((heads, N, vdim), torch.float32, "ssm")
    for a_log, expect in ((-12.0, 1.0), (3.0, 0.0)):
        scene = Scene(gpu_device, needs, 8, 1)
        zeros = torch.zeros(heads, device=gpu_device)
        out = []
        for n in (300, 1, 2):
            batch = scene.step([n])
            xbc = torch.zeros(n, vdim + 2 * N, device=gpu_device)
            proj = torch.zeros(n, 1, device=gpu_device)          # dt = softplus(0)
            if not out:
                xbc[3, :vdim] = 1.0
                xbc[3, vdim] = 1.0                                # B_0 at token 3
            xbc[:, vdim + N] = 1.0                                # C_0 everywhere
            out.append(ops.ssm_scan(xbc, proj, 0, zeros, torch.full((1,), a_log, device=gpu_device),
                                    zeros, batch, scene.view.states["ssm"], heads=heads,
                                    vdim=vdim, state_rows=N, groups=1))
        last = out[-1][-1].cpu()
        want = expect * 0.6931472 * torch.ones(vdim)
        torch.testing.assert_close(last, want, rtol=2e-3, atol=1e-6)


# ------------------------------------------------------------------ latent attention


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("heads, dim, rot_dim, rot_dims, vdim, q_rank, kv_rank, window",
                         [(3, 8, 6, 4, 10, 12, 14, 5), (5, 16, 8, 8, 12, 24, 32, None),
                          (4, 32, 16, 16, 32, 96, 64, 24), (16, 128, 64, 64, 128, 256, 512, 33),
                          (2, 16, 24, 24, 16, 32, 712, 9)])
def test_latent_attention_kernels(gpu_device, cache_dtype, heads, dim, rot_dim, rot_dims, vdim,
                                  q_rank, kv_rank, window):
    ops = load_hip_ops(gpu_device)
    dl = kv_rank + rot_dim
    scene = Scene(gpu_device, PagedLatentNeed(dl, window), 8, 4, dtype=cache_dtype, num_pages=60)
    ref_pages = scene.view.k_pages.clone()
    import dataclasses
    ref_view = dataclasses.replace(scene.view, k_pages=ref_pages)
    freqs = (10000.0 ** (-2.0 * torch.arange(rot_dims // 2) / rot_dims)).float().to(gpu_device)
    qn, kn = (1 + 0.1 * rnd((q_rank,), 1)).to(gpu_device), (1 + 0.1 * rnd((kv_rank,), 2)).to(gpu_device)
    tol = dict(rtol=1e-4, atol=1e-4) if cache_dtype == torch.float32 else dict(rtol=2e-2, atol=2e-2)
    for i, spans in enumerate(SPANS):
        batch = scene.step(spans)
        table = batch.tables[0]
        T = batch.num_tokens
        proj = rnd((T, q_rank + dl), 30 + i).to(gpu_device)
        kw = dict(q_rank=q_rank, kv_rank=kv_rank, rot_dim=rot_dim, q_norm=qn, kv_norm=kn,
                  eps=1e-5, freqs=freqs, rot_dims=rot_dims, out_dtype=torch.float32)
        close(ops.latent_prepare(proj, batch, table, scene.view, **kw),
              REF.latent_prepare(proj, batch, table, ref_view, **kw))
        close(scene.view.k_pages, ref_pages, **tol)
        ref_pages.copy_(scene.view.k_pages)       # attention below reads identical pages
        qa = rnd((T, heads, dl), 40 + i).to(gpu_device)
        qb = qa.clone()
        ops.rotate_interleaved_inplace(qa, batch.positions, freqs, rot_dims, offset=kv_rank)
        REF.rotate_interleaved_inplace(qb, batch.positions, freqs, rot_dims, offset=kv_rank)
        close(qa, qb)
        kw = dict(heads=heads, kv_rank=kv_rank, rot_dim=rot_dim, scale=0.2, window=window)
        ol = REF.latent_attention(qb, batch, table, ref_view, **kw)
        # (bfloat16 pages take the matrix-core kernel, which rounds queries and softmax
        # weights to bfloat16: scores of standard deviation 5 move by a few hundredths)
        loose = dict(rtol=6e-2, atol=6e-2)
        close(ops.latent_attention(qb, batch, table, scene.view, **kw), ol,
              **(tol if cache_dtype == torch.float32 else loose))
        got = ops.latent_attention(qb, batch, table, scene.view, out_dtype=torch.bfloat16, **kw)
        assert got.dtype == torch.bfloat16
        close(got, ol, **loose)


@pytest.mark.parametrize("cache_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [None, 20, 64, 65])
@pytest.mark.parametrize("decode", [False, True])
def test_one_key_stands_out(gpu_device, window, decode, cache_dtype):
    """Rows of the pages are small noise but for one, which the query points at: the
    result is that row if the query can see it (far back without a window, or the first
    token inside one) and noise if it is the first token outside."""
    ops = load_hip_ops(gpu_device)
    heads, kv_rank, rot_dim, page = 2, 16, 8, 8      # (bfloat16 pages: the matrix-core kernel)
    dl, T = kv_rank + rot_dim, 301
    for where in ("inside", "outside"):
        if window is None and where == "outside":
            continue
        scene = Scene(gpu_device, PagedLatentNeed(dl, None), page, 1, dtype=cache_dtype,
                      num_pages=45)
        batch = scene.step([T])
        if decode:
            batch = BatchBuilder(gpu_device, 1).build(
                [StepEntry(scene.caches[0], [1], T - 1, [0])])
        pos_q = T - 1
        target = 2 if window is None else pos_q - window + (1 if where == "inside" else 0)
        rows = rnd((T, dl), 7, 0.01)
        direction = torch.nn.functional.normalize(rnd((dl,), 8), dim=0)
        rows[target] = direction * 3.0
        table = batch.tables[0][0].cpu()
        pos = torch.arange(T)
        rows = rows.to(cache_dtype).float()
        scene.view.k_pages[table[pos // page].long(), pos % page] = rows.to(cache_dtype).to(gpu_device)
        n = batch.num_tokens
        qa = torch.zeros(n, heads, dl)
        qa[-1] = direction * 40.0
        out = ops.latent_attention(qa.to(gpu_device), batch, batch.tables[0], scene.view,
                                   heads=heads, kv_rank=kv_rank, rot_dim=rot_dim, scale=1.0,
                                   window=window)[-1].cpu()
        if where == "inside":
            torch.testing.assert_close(out, rows[target, :kv_rank].expand(heads, -1),
                                       rtol=1e-3, atol=1e-3 if cache_dtype == torch.float32 else 2e-2)
        else:
            assert out.abs().max() < 0.1


# ------------------------------------------------------------------ the engine

TOL = {torch.float32: (2e-4, 5e-5), torch.bfloat16: (4e-2, 4e-2)}


@pytest.fixture(scope="module", params=[(n, d) for n in sorted(ZONO)
                                        for d in (torch.float32, torch.bfloat16)],
                ids=lambda p: f"{p[0]}-{str(p[1]).split('.')[-1]}")
def setup(request, tmp_path_factory, gpu_device):
    name, dtype = request.param
    cfg, seed, page = ZONO[name]
    d = tmp_path_factory.mktemp(f"zono{name}")
    write_random_model(d, cfg, seed, dtype, std=0.2)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, dtype, gpu_device)
    lengths = [5, 11, 17, 40, 64, 1, 23, 100]
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}
    return model, page, requests, ref, TOL[dtype], (pcfg, w, d, dtype)


def runner_for(model, page, num_pages):
    return ModelRunner(model, page_size=page, num_pages=num_pages, num_slots=4)


def test_whole(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    drives.compare(drives.drive_whole(runner_for(model, page, 128 // page), requests),
                   ref, rtol, atol)


def test_prefill_then_decode(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    drives.compare(drives.drive_prefill_then_decode(runner_for(model, page, 128 // page),
                                                    requests, tail=40), ref, rtol, atol)


def test_portions(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    drives.compare(drives.drive_portions(runner_for(model, page, 128 // page), requests),
                   ref, rtol, atol)


def test_mixed_with_pages_and_slots_used_again(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    runner = runner_for(model, page, 224 // page)
    drives.compare(drives.drive_mixed(runner, requests), ref, rtol, atol)
    assert all(pool.num_used == 0 for pool in runner.manager.pools)


def test_preempted_and_recomputed(setup):
    model, page, requests, ref, (rtol, atol), _ = setup
    drives.compare(drives.drive_preempted(runner_for(model, page, 224 // page), requests),
                   ref, rtol, atol)


def test_float32_does_not_depend_on_the_cut(setup):
    """A position's float32 logits are the same to rounding whether its request ran whole,
    in portions or token by token beside others."""
    model, page, requests, ref, _, (_, _, _, dtype) = setup
    if dtype != torch.float32:
        pytest.skip("float32 only")
    a = drives.drive_whole(runner_for(model, page, 128 // page), requests)
    b = drives.drive_portions(runner_for(model, page, 128 // page), requests)
    c = drives.drive_mixed(runner_for(model, page, 224 // page), requests)
    for rid in requests:
        torch.testing.assert_close(a.stacked(rid)[0], b.stacked(rid)[0], rtol=1e-4, atol=2e-5)
        torch.testing.assert_close(a.stacked(rid)[0], c.stacked(rid)[0], rtol=1e-4, atol=2e-5)


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
