"""Zonopel on the CPU: configuration, the model as data, and the engine's cache manager,
state slots, batch builder and step function (with the plain torch kernel references in
place of the HIP kernels) against the plain whole-sequence implementation, float32."""

import json

import pytest
import torch

import drives
from helpers import ZONO, ZONO_A, ZONO_B, random_prompt
from kernel_refs import TorchOps
from plain import zonopel_plain as plain
from tokensprint_amd.config import ConfigError, ZonopelConfig
from tokensprint_amd.config.registry import get_architecture
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model
from tokensprint_amd.weights import write_random_model


def plain_logits(cfg, w, tokens):
    return plain.forward(cfg, w, tokens).float()


@pytest.fixture(scope="module", params=sorted(ZONO))
def setup(request, tmp_path_factory):
    cfg, seed, page = ZONO[request.param]
    d = tmp_path_factory.mktemp(f"zono{request.param}")
    write_random_model(d, cfg, seed, torch.float32, std=0.2)
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


def test_config_reads_every_size_and_the_spec_shares_weights():
    cfg = ZonopelConfig.from_dict(ZONO_A)
    assert (cfg.width, cfg.vocab_size, cfg.eps, cfg.embed_scale) == (40, 97, 1e-5, 2.5)
    assert (cfg.bigram_buckets, cfg.bigram_mul_prev, cfg.bigram_mul_cur) == (61, 31, 5)
    assert [l.type for l in cfg.layers] == ["latent_attention", "mamba2", "mamba2",
                                            "latent_attention", "mamba2"]
    assert [l.weights_of for l in cfg.layers] == [None, None, 1, 0, None]
    assert cfg.layers[0].mixer.window == 5 and cfg.layers[0].mixer.rot_dims == 4
    assert cfg.layers[4].ff is None and cfg.layers[1].ff == 48
    arch = get_architecture("Zonopel")
    spec = arch.build_spec(arch.parse_config(ZONO_A))
    assert len(spec.layers) == 3 and [r.layer for r in spec.order] == [0, 1, 1, 0, 2]
    assert all(r.cache_of is None for r in spec.order)      # every run owns its cache and state
    assert "feed_forward" not in spec.layers[2].parts


def test_cache_needs_name_pages_and_states():
    from tokensprint_amd.engine.assemble import build_model
    _, model = build_model(ZONO_B, "float32", "cpu", ops=TorchOps())
    needs = model.cache_needs()
    assert len(needs) == len(ZONO_B["layers"]) + 1           # the embedding's state comes last
    kinds = [sorted(type(n).__name__ + ":" + getattr(n, "name", "") for n in
                    (need if isinstance(need, tuple) else (need,))) for need in needs]
    assert kinds[0] == ["SlotStateNeed:conv", "SlotStateNeed:shift", "SlotStateNeed:ssm"]
    assert kinds[1] == ["PagedLatentNeed:", "SlotStateNeed:shift"]
    assert kinds[-1] == ["SlotStateNeed:prev_token"]
    runner = ModelRunner(model, page_size=8, num_pages=6, num_slots=3)
    groups = runner.storage.groups
    assert [(g.kind, g.head_dim, g.window, g.runs) for g in groups] == \
        [("latent", 40, None, (1,)), ("latent", 28, 17, (2,))]
    assert runner.storage.views[1].k_pages.shape == (6, 8, 40)
    assert runner.storage.views[0].states["ssm"].shape == (4, 2, 20, 40)
    assert runner.storage.views[4].states["prev_token"].dtype == torch.int32
    with pytest.raises(ValueError, match="keep all keys|fixed-size state"):
        runner.manager.enable_prefix_cache()


@pytest.mark.parametrize("change, message", [
    (lambda c: c["layers"][0].update(type="rwkv"), "type"),
    (lambda c: c["layers"][1]["mlp"].update(kind="moe"), "dense"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=3), "no tensors of its own"),
    (lambda c: c["layers"][1]["mixer"].update(groups=3), "groups"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c["embedding"]["bigram"].pop("buckets"), "buckets"),
])
def test_config_errors(change, message):
    raw = json.loads(json.dumps(ZONO_A))
    change(raw)
    with pytest.raises(ConfigError, match=message):
        ZonopelConfig.from_dict(raw)


def test_random_weights_fit_the_declarations(tmp_path):
    from tokensprint_amd.weights.random_init import declared_tensors
    decls = declared_tensors(ZONO_A)
    assert decls["bigram"].shape == (62, 40) and decls["l1.mix.conv"].shape == (6 * 4 + 40, 4)
    assert "l2.mix.in" not in decls and "l3.mix.dq" not in decls     # borrowed weights
    assert decls["l4.mix.in"].shape == (2 * 24 + 2 * 9 + 2, 40) and "l4.mlp.up" not in decls
    d = write_random_model(tmp_path / "m", ZONO_A, 3, torch.bfloat16)
    load_model(d, "bfloat16", "cpu", ops=TorchOps())


# ------------------------------------------------------------------ unusual layer lists


def _run_drives(cfg, seed, page, tmp_path):
    d = write_random_model(tmp_path / "m", cfg, seed, torch.float32, std=0.2)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, "float32", "cpu", ops=TorchOps())
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 300 + i) for i, n in enumerate([9, 30, 1, 18])}
    ref = {rid: plain_logits(pcfg, w, t) for rid, t in requests.items()}
    drives.compare(drives.drive_portions(runner_for(model, page, 10), requests), ref, *TOL)
    drives.compare(drives.drive_mixed(runner_for(model, page, 10), requests), ref, *TOL)


def test_only_recurrent_layers_and_weights_borrowed_from_a_later_layer(tmp_path):
    """No layer keeps pages (the cache manager has no group at all); the first layer runs
    with the second one's weights."""
    from helpers import zonopel_config, zonopel_mamba
    cfg = zonopel_config(width=24, vocab=50, eps=1e-5, scale=1.5, buckets=11, mul_prev=5,
                         mul_cur=2, layers=[
                             zonopel_mamba(heads=0, vdim=0, state=0, groups=0, conv=0,
                                           norm_groups=0, weights_of=1),
                             zonopel_mamba(heads=3, vdim=8, state=6, groups=3, conv=3,
                                           norm_groups=3, ff=32)])
    _run_drives(cfg, 21, 8, tmp_path)


def test_only_attention_layers(tmp_path):
    from helpers import zonopel_config, zonopel_latent
    cfg = zonopel_config(width=24, vocab=50, eps=1e-5, scale=1.5, buckets=11, mul_prev=5,
                         mul_cur=2, layers=[
                             zonopel_latent(heads=2, dim=6, rot_dim=4, vdim=5, q_rank=10,
                                            kv_rank=12, window=7, ff=None),
                             zonopel_latent(heads=2, dim=6, rot_dim=4, vdim=5, q_rank=10,
                                            kv_rank=12, window=7, ff=20)])
    _run_drives(cfg, 22, 8, tmp_path)


def test_the_architecture_is_registered_beside_the_others():
    from model_registry import listing
    from tokensprint_amd.config import architecture_names
    assert {"Qwen3ForCausalLM", "Zonopel"} <= set(architecture_names())
    assert "Zonopel" in listing()
    # config.json names it with a single 'architecture' string
    from tokensprint_amd.config.model_config import architecture_of
    assert architecture_of(ZONO_B) == "Zonopel"
    with pytest.raises(ConfigError, match="architecture"):
        architecture_of({"width": 8})
