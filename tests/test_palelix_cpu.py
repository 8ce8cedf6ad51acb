"""Palelix on the CPU: configuration, the model as data, the plain implementation's own
pins, and the engine's cache manager, state slots, batch builder and step function (with the
plain torch kernel references in place of the HIP kernels) against the plain whole-sequence
implementation, float32."""

import json
import math

import pytest
import torch

import drives
from helpers import (PALE, PALE_A, PALE_B, PALE_C, palelix_config, palelix_delta, palelix_dense,
                     palelix_lightning, palelix_moe, random_prompt, write_palelix_model)
from kernel_refs import TorchOps
from plain import palelix_plain as plain
from tokensprint_amd.config import ConfigError, PalelixConfig
from tokensprint_amd.config.registry import get_architecture
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import build_model, load_model


def plain_logits(cfg, w, tokens):
    return plain.forward(cfg, w, tokens).float()


@pytest.fixture(scope="module", params=sorted(PALE))
def setup(request, tmp_path_factory):
    cfg, seed, page = PALE[request.param]
    d = write_palelix_model(tmp_path_factory.mktemp(f"pale{request.param}"), cfg, seed,
                            torch.float32)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    lengths = [5, 11, 17, 40, 64, 1, 23]
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain_logits(pcfg, w, t) for rid, t in requests.items()}
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


def test_config_reads_every_size_and_the_loop_repeats_runs():
    cfg = PalelixConfig.from_dict(PALE_A)
    assert (cfg.width, cfg.vocab_size, cfg.eps) == (40, 97, 1e-5)
    assert [l.type for l in cfg.layers] == ["parallel", "lightning", "delta"]
    left, right = cfg.layers[0].mixer.left, cfg.layers[0].mixer.right
    assert (left.heads, left.kv_heads, left.dim, left.vdim, left.rot_dims) == (4, 2, 12, 20, 8)
    assert (left.scale, left.rot_base) == (0.35, 10000.0)
    assert right.per_channel and (right.decay_rank, right.gate_rank) == (5, 7)
    assert cfg.layers[1].mixer.decay == (0.4, 0.93, 0.999)
    assert not cfg.layers[2].mixer.per_channel and cfg.layers[2].mlp is None
    moe = cfg.layers[0].mlp
    assert (moe.experts, moe.top, moe.group_count, moe.group_keep, moe.limit) == (6, 2, 3, 2, 0.8)
    arch = get_architecture("Palelix")
    spec = arch.build_spec(cfg)
    assert [r.layer for r in spec.order] == [0, 1, 0, 1, 0, 1, 2]
    assert [r.enter for r in spec.order] == [("loop.step", 0), None, ("loop.step", 1), None,
                                             ("loop.step", 2), None, None]
    assert all(r.cache_of is None for r in spec.order)       # every pass owns cache and state
    assert "feed_forward" not in spec.layers[2].parts
    plain_order = plain.run_order(PALE_A)
    assert [i for i, _ in plain_order] == [r.layer for r in spec.order]
    no_loop = arch.build_spec(arch.parse_config(PALE_C))
    assert [r.enter for r in no_loop.order] == [None] * 3 and not no_loop.enter_tables


def test_cache_needs_name_pages_and_states():
    _, model = build_model(PALE_B, "float32", "cpu", ops=TorchOps())
    needs = model.cache_needs()
    assert len(needs) == 5                                    # delta, (lightning, parallel) x 2
    kinds = [sorted(type(n).__name__ + ":" + getattr(n, "name", "") for n in
                    (need if isinstance(need, tuple) else (need,))) for need in needs]
    assert kinds[0] == ["SlotStateNeed:delta", "SlotStateNeed:delta.conv"]
    assert kinds[1] == kinds[3] == ["SlotStateNeed:lightning"]
    assert kinds[2] == kinds[4] == ["PagedKVNeed:", "SlotStateNeed:delta", "SlotStateNeed:delta.conv"]
    runner = ModelRunner(model, page_size=8, num_pages=6, num_slots=3)
    groups = runner.storage.groups
    # one head size serves keys (16) and values (8), rounded up to the kernels' step
    assert [(g.kind, g.num_kv_heads, g.head_dim, g.window, g.runs) for g in groups] == \
        [("kv", 3, 16, None, (2, 4))]
    assert runner.storage.views[0].states["delta"].shape == (4, 6, 20, 12)
    assert runner.storage.views[0].states["delta.conv"].shape == (4, 2, 2 * 40 + 72)
    assert runner.storage.views[2].states["delta.conv"].shape == (4, 0, 2 * 18 + 48)
    assert runner.storage.views[1].states["lightning"].shape == (4, 2, 24, 16)
    assert runner.storage.views[2].states["delta"].data_ptr() != \
        runner.storage.views[4].states["delta"].data_ptr()


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="mamba2"), "type"),
    (lambda c: c["layers"][1]["mlp"].update(kind="glu"), "dense and moe"),
    (lambda c: c["layers"][1]["mixer"].update(decay=[0.5]), "decay"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(kv_heads=2), "kv_heads"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=5), "cannot give"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "cannot give"),
    (lambda c: c["loop"].update(stop=4), "loop"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["layers"][2]["mixer"].pop("conv"), "conv"),
])
def test_config_errors(change, message):
    raw = json.loads(json.dumps(PALE_A))
    change(raw)
    with pytest.raises(ConfigError, match=message):
        PalelixConfig.from_dict(raw)


def test_random_weights_fit_the_declarations(tmp_path):
    from tokensprint_amd.weights.random_init import declared_tensors
    decls = declared_tensors(PALE_A)
    assert decls["loop.step"].shape == (3, 40) and decls["embed"].shape == (97, 40)
    assert decls["l0.mix.left.q"].shape == (48, 40) and decls["l0.mix.left.o"].shape == (40, 80)
    assert decls["l0.mix.right.a2"].shape == (30, 5) and decls["l0.mix.right.g2"].shape == (18, 7)
    assert decls["l0.mix.right.dt_bias"].shape == (30,) and decls["l2.mix.dt_bias"].shape == (2,)
    assert decls["l0.mix.right.norm"].shape == (6,) and decls["l1.mix.norm"].shape == (27,)
    assert decls["l0.mlp.e5.down"].shape == (40, 12) and "l2.mlp.gate" not in decls
    assert "loop.step" not in declared_tensors(PALE_C)
    d = write_palelix_model(tmp_path / "m", PALE_A, 3, torch.bfloat16)
    load_model(d, "bfloat16", "cpu", ops=TorchOps())
    # the two-step projections' inner sizes may be left to the file
    raw = json.loads(json.dumps(PALE_A))
    for key in ("decay_rank", "gate_rank"):
        raw["layers"][0]["mixer"]["right"].pop(key)
    (d / "config.json").write_text(json.dumps(raw))
    _, model = load_model(d, "bfloat16", "cpu", ops=TorchOps())
    assert model.blocks[0].mixer.right.decay_rank == 5
    with pytest.raises(ValueError, match="random weights need it"):
        declared = declared_tensors(raw)
        from tokensprint_amd.weights.random_init import random_tensors
        random_tensors(raw, 1)


def test_the_architecture_is_registered_beside_the_others():
    from model_registry import listing
    from tokensprint_amd.config import architecture_names
    assert {"Qwen3ForCausalLM", "Zonopel", "Palelix"} <= set(architecture_names())
    assert "Palelix" in listing()


# ------------------------------------------------------------------ the plain mechanisms


def test_plain_route_keeps_the_best_groups_only():
    s = torch.tensor([0.05, 0.30, 0.02, 0.03, 0.25, 0.20, 0.01, 0.14], dtype=torch.float64)
    # groups of two: bests 0.30, 0.03, 0.25, 0.14 -> groups 0 and 2 are kept
    chosen, w = plain.route(s, 3, 4, 2)
    assert sorted(chosen.tolist()) == [1, 4, 5]
    assert torch.allclose(w.sum(), torch.tensor(1.0, dtype=torch.float64))
    assert math.isclose(float(w[chosen.tolist().index(1)]), 0.30 / 0.75)
    # expert 7 (0.14) beats expert 0 (0.05), but its group is out
    chosen, _ = plain.route(s, 4, 4, 2)
    assert sorted(chosen.tolist()) == [0, 1, 4, 5]
    # every group kept: the plain top
    chosen, _ = plain.route(s, 4, 4, 4)
    assert sorted(chosen.tolist()) == [1, 4, 5, 7]


def test_plain_delta_rule_overwrites_a_key_and_lightning_decays():
    k = torch.tensor([[[1.0, 0.0]], [[1.0, 0.0]], [[0.0, 1.0]]], dtype=torch.float64)   # [T,1,2]
    v = torch.tensor([[[2.0]], [[5.0]], [[7.0]]], dtype=torch.float64)
    ones = torch.ones(3, 1, dtype=torch.float64)
    o = plain.gated_delta_rule(k, k, v, ones, ones)
    # beta = 1, no decay: the second write to the same key replaces the first value
    assert o.flatten().tolist() == [2.0, 5.0, 7.0]
    o = plain.gated_delta_rule(k, k, v, 0.5 * ones, ones)
    assert o.flatten().tolist() == [1.0, 1.0 + 0.5 * (5.0 - 1.0), 3.5]
    # a decay per key channel acts on the rows of S: the first channel forgets, the second not
    g = torch.tensor([1.0, 1.0]).expand(3, 1, 2).clone().double()
    g[2, 0, 0] = 0.0
    q = torch.tensor([[[1.0, 1.0]]], dtype=torch.float64).expand(3, 1, 2)
    o = plain.gated_delta_rule(q, k, v, ones, g)
    assert o.flatten().tolist() == [2.0, 5.0, 7.0]
    o = plain.lightning_attention(q, k, v, torch.tensor([0.5], dtype=torch.float64))
    assert o.flatten().tolist() == [2.0, 1.0 + 5.0, 3.0 + 7.0]


def test_plain_rotation_is_a_complex_multiplication_of_the_paired_dimensions():
    x = torch.randn(3, 2, 10, dtype=torch.float64)
    pos = torch.tensor([0, 4, 9])
    out = plain.rotate_half(x, pos, 6, 100.0)
    assert torch.equal(out[0], x[0]) and torch.equal(out[..., 6:], x[..., 6:])
    for i in range(3):
        z = torch.complex(x[:, :, i], x[:, :, i + 3])
        ang = pos.double() * 100.0 ** (-2.0 * i / 6)
        r = z * torch.polar(torch.ones(3, dtype=torch.float64), ang).unsqueeze(1)
        assert torch.allclose(out[:, :, i], r.real) and torch.allclose(out[:, :, i + 3], r.imag)


def test_plain_short_convolution_and_expert():
    x = torch.arange(8, dtype=torch.float64).view(4, 2)
    taps = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    out = plain.short_conv(x, taps)
    assert out[:, 1].tolist() == [1.0, 3.0, 5.0, 7.0]
    assert out[:, 0].tolist() == [0.0, 200.0, 400.0 + 20.0, 600.0 + 40.0 + 2.0]
    w = {"gate": torch.tensor([[10.0], [-1.0]], dtype=torch.float64),
         "up": torch.tensor([[10.0], [-10.0]], dtype=torch.float64),
         "down": torch.eye(2, dtype=torch.float64)}
    y = plain.expert_ff(torch.ones(1, 1, dtype=torch.float64), w, "", 2.0)
    g0 = 2.0 / (1 + math.exp(-1.702 * 2.0)) * 3.0                  # both clamped from above
    g1 = -1.0 / (1 + math.exp(1.702)) * (-2.0 + 1.0)               # gate has no lower clamp
    assert torch.allclose(y, torch.tensor([[g0, g1]], dtype=torch.float64))


# ------------------------------------------------------------------ unusual layer lists


def _run_drives(cfg, seed, page, tmp_path, lengths=(9, 30, 1, 18)):
    d = write_palelix_model(tmp_path / "m", cfg, seed, torch.float32)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 300 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain_logits(pcfg, w, t) for rid, t in requests.items()}
    drives.compare(drives.drive_portions(runner_for(model, page, 10), requests), ref, *TOL)
    drives.compare(drives.drive_mixed(runner_for(model, page, 10), requests), ref, *TOL)


def test_only_recurrent_layers_looped_whole(tmp_path):
    """No layer keeps pages (the cache manager has no group at all) and the loop covers every
    layer, once."""
    cfg = palelix_config(width=24, vocab=50, eps=1e-5, loop=(0, 2, 1), layers=[
        palelix_lightning(heads=2, dim=4, vdim=4, decay=(1.0, 0.5), mlp=palelix_dense(16)),
        palelix_delta(heads=2, kv_heads=1, dim=4, vdim=6, conv=1,
                      mlp=palelix_moe(ff=8, limit=1.0, experts=2, top=1, count=2, keep=1))])
    _run_drives(cfg, 21, 8, tmp_path)


def test_layers_without_any_feed_forward(tmp_path):
    cfg = palelix_config(width=24, vocab=50, eps=1e-5, layers=[
        palelix_delta(heads=1, kv_heads=1, dim=12, vdim=12, conv=5, mlp=None),
        palelix_lightning(heads=3, dim=2, vdim=2, decay=(0.9, 0.8, 0.7), mlp=None)])
    _run_drives(cfg, 22, 8, tmp_path)
