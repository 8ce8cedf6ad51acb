"""Randomly drawn small Palelix configurations through the drives on the GPU against the
plain implementation: widths that are no multiple of eight, key sizes from 3 to 200, value
sizes above and below the kernels' column blocks, any grouping of heads, convolutions of 1
to 5 taps, expert counts and groups of any kind, loops anywhere.  The draws are seeded, so a
run is repeatable; what they are for is the sizes nobody thought of."""

import random

import pytest
import torch

import drives
from helpers import (palelix_config, palelix_delta, palelix_delta_sizes, palelix_dense,
                     palelix_lightning, palelix_moe, palelix_parallel, random_prompt,
                     write_palelix_model)
from plain import palelix_plain as plain
from tokensprint_amd.engine import ModelRunner
from tokensprint_amd.engine.assemble import load_model

pytestmark = pytest.mark.gpu


def draw_mlp(rnd):
    kind = rnd.choice(["none", "dense", "moe", "moe"])
    if kind == "none":
        return None
    if kind == "dense":
        return palelix_dense(rnd.choice([24, 50, 96]))
    count = rnd.choice([1, 2, 3, 4])
    per = rnd.choice([1, 2, 3, 5])
    keep = rnd.randint(1, count)
    return palelix_moe(ff=rnd.choice([8, 12, 40]), limit=rnd.choice([0.5, 1.5, 7.0]),
                       experts=count * per, top=rnd.randint(1, keep * per), count=count, keep=keep)


def draw_delta(rnd, ranks):
    kv = rnd.choice([1, 2, 3])
    return dict(heads=kv * rnd.choice([1, 2, 3]), kv_heads=kv,
                dim=rnd.choice([3, 8, 20, 33, 64, 200]), vdim=rnd.choice([4, 10, 64, 72, 130]),
                conv=rnd.choice([1, 2, 4, 5]), ranks=ranks)


def draw(case):
    rnd = random.Random(1000 + case)
    layers = []
    for _ in range(rnd.choice([2, 3, 4])):
        kind = rnd.choice(["lightning", "delta", "parallel"])
        mlp = draw_mlp(rnd)
        if kind == "lightning":
            heads = rnd.choice([1, 2, 5])
            layers.append(palelix_lightning(
                heads=heads, dim=rnd.choice([4, 9, 32, 128]), vdim=rnd.choice([6, 16, 70]),
                decay=[rnd.choice([1.0, 0.999, 0.9, 0.3]) for _ in range(heads)], mlp=mlp))
        elif kind == "delta":
            layers.append(palelix_delta(mlp=mlp, **draw_delta(rnd, None)))
        else:
            kv = rnd.choice([1, 2, 3])
            dim = rnd.choice([6, 16, 24, 40, 64, 120])
            layers.append(palelix_parallel(
                heads=kv * rnd.choice([1, 2, 4]), kv_heads=kv, dim=dim,
                vdim=rnd.choice([4, 16, 48, 100]), rot_dims=rnd.choice([2, dim // 2 * 2, dim // 4 * 2 or 2]),
                base=rnd.choice([100.0, 1e4, 1e6]), scale=rnd.choice([0.1, dim ** -0.5]),
                left_scale=rnd.choice([1.0, 0.3]), right_scale=rnd.choice([1.0, 2.0]),
                right=palelix_delta_sizes(**draw_delta(rnd, (rnd.choice([1, 6, 16]),
                                                            rnd.choice([2, 8])))), mlp=mlp))
    loop = None
    if rnd.random() < 0.6:
        start = rnd.randrange(len(layers))
        loop = (start, rnd.randint(start + 1, len(layers)), rnd.choice([1, 2, 3]))
    cfg = palelix_config(width=rnd.choice([20, 36, 64, 100]), vocab=rnd.choice([50, 97, 300]),
                         eps=rnd.choice([1e-6, 1e-5]), layers=layers, loop=loop)
    return cfg, rnd.choice([4, 16, 32])


@pytest.mark.parametrize("case", range(10))
def test_a_drawn_configuration(case, tmp_path, gpu_device):
    cfg, page = draw(case)
    d = write_palelix_model(tmp_path, cfg, case, torch.float32, std=0.15, sharpen=2.0)
    pcfg, w = plain.read_model_dir(d)
    _, model = load_model(d, torch.float32, gpu_device)
    lengths = [5, 17, 40, 1, 70]
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate(lengths)}
    ref = {rid: plain.forward(pcfg, w, t).float() for rid, t in requests.items()}

    def runner(pages):
        return ModelRunner(model, page_size=page, num_pages=pages, num_slots=4)

    roomy = 96 // page + 4
    drives.compare(drives.drive_whole(runner(roomy), requests), ref, 3e-4, 6e-5)
    drives.compare(drives.drive_prefill_then_decode(runner(roomy), requests), ref, 3e-4, 6e-5)
    drives.compare(drives.drive_portions(runner(roomy), requests), ref, 3e-4, 6e-5)
    drives.compare(drives.drive_mixed(runner(224 // page), requests), ref, 3e-4, 6e-5)


@pytest.mark.parametrize("case", range(10))
def test_a_drawn_configuration_runs_in_bfloat16(case, tmp_path, gpu_device):
    """The same draws in bfloat16: whole prompts and mixed steps agree with each other row by
    row (what differs between them is which kernel serves a row), and stay finite."""
    cfg, page = draw(case)
    d = write_palelix_model(tmp_path, cfg, case, torch.bfloat16, std=0.15, sharpen=1.0)
    _, model = load_model(d, torch.bfloat16, gpu_device)
    requests = {f"r{i}": random_prompt(n, cfg["vocab"], 100 + i) for i, n in enumerate([5, 17, 40, 1, 70])}

    def runner(pages):
        return ModelRunner(model, page_size=page, num_pages=pages, num_slots=4)

    a = drives.drive_whole(runner(96 // page + 4), requests)
    b = drives.drive_mixed(runner(224 // page), requests)
    rows = bad = 0
    for rid in requests:
        x, y = a.stacked(rid)[0], b.stacked(rid)[0]
        assert torch.isfinite(x).all() and torch.isfinite(y).all()
        scale = max(1.0, float(x.abs().max()))
        rows += x.shape[0]
        bad += int(((x - y).abs() > 0.08 * scale).any(dim=1).sum())
    assert bad <= 0.05 * rows, f"{bad} of {rows} rows differ between the two ways of cutting"
