"""Tarunex configurations drawn at random, each replayed whole, in portions and mixed against the plain implementation:
any order of the two mixers, loops anywhere (or none) walked one to three times, head sizes that are and are not whole
MFMA tiles, value heads larger and smaller than key heads, latents that the MFMA kernel takes and refuses, widths that are
and are not multiples of 128, layers without feed-forward, pages of 8 to 32 tokens.  float32 holds every logit; bfloat16
is held by the rows' error in the median and at the ninth decile."""
import random

import pytest
import torch

from tests import replay_cases as rc
from tests import tarunex_cases as tc
from tests.gpu_util import require_gpu
from tests.test_gpu_tarunex import compare

pytestmark = pytest.mark.gpu


def draw_config(seed):
    rng = random.Random(7000 + seed)
    width = rng.choice([128, 256, 384]) if seed % 3 == 0 else 8 * rng.randint(5, 40)
    n = rng.randint(1, 5)
    layers = []
    for _ in range(n):
        mlp = None
        if rng.random() < 0.85:
            experts = rng.choice([1, 2, 4, 6, 8, 16])
            mlp = dict(kind="moe", expert=dict(ff=8 * rng.randint(1, 20)), router=dict(experts=experts, top=rng.randint(1, min(experts, 4))),
                       shared=dict(ff=8 * rng.randint(1, 20)))
        if rng.random() < 0.5:
            kv = rng.choice([1, 2, 3])
            dim = rng.choice([8, 16, 24, 32, 48, 64, 80, 96, 128])
            vdim = dim if rng.random() < 0.5 else rng.choice([8, 16, 40, 64, 96, 112])
            mixer = dict(heads=kv * rng.choice([1, 2, 3, 4]), kv_heads=kv, dim=dim, vdim=vdim, scale=dim ** -0.5 * rng.choice([0.5, 1.0]),
                         softcap=rng.choice([5.0, 20.0, 50.0]), q_temp=dict(coef=rng.choice([0.1, 0.3, 0.6]), every=rng.choice([1, 3, 16, 64, 500])))
            layers.append(dict(type="attention", mixer=mixer, mlp=mlp))
        else:
            rot_dim = rng.choice([2, 8, 16, 32, 64])
            dim = rng.choice([4, 8, 16, 32, 64, 128])
            mixer = dict(heads=rng.randint(1, 6), dim=dim, rot_dim=rot_dim, vdim=rng.choice([8, 16, 40, 64, 80]), kv_rank=rng.choice([8, 12, 32, 64, 96]),
                         q_rank=rng.choice([8, 24, 48, 96]), scale=(dim + rot_dim) ** -0.5,
                         rot=dict(base=rng.choice([100.0, 1e4, 1e6]), dims=rot_dim if rng.random() < 0.7 else 2 * rng.randint(1, rot_dim // 2)))
            layers.append(dict(type="latent_attention", mixer=mixer, mlp=mlp))
    cfg = dict(architecture="Tarunex", vocab=rng.randint(90, 700), width=width, norm=dict(eps=rng.choice([1e-6, 1e-5, 3e-6])),
               embedding=dict(scale=rng.choice([1.0, 4.0, 12.0])), logit_scale=rng.choice([0.3, 1.0, 2.0]), logit_softcap=rng.choice([10.0, 40.0]),
               layers=layers)
    if rng.random() < 0.8:
        start = rng.randint(0, n - 1)
        cfg["loop"] = dict(start=start, stop=rng.randint(start + 1, n), times=rng.randint(1, 3))
    return cfg, rng.choice([8, 16, 32])


@pytest.mark.parametrize("seed", range(12))
def test_random_configuration(seed, tmp_path):
    require_gpu()
    cfg, page = draw_config(seed)
    print("seed %d: width %d, page %d, loop %s, layers %s" % (seed, cfg["width"], page, cfg.get("loop"),
                                                               [(l["type"], l["mixer"], l["mlp"] and l["mlp"]["router"]) for l in cfg["layers"]]), flush=True)
    folder = tc.write_model(str(tmp_path / "m"), cfg, 300 + seed, tc.decisive_router(3.0))
    rng = random.Random(seed)
    reqs = rc.random_requests(cfg["vocab"], [rng.randint(1, 150) for _ in range(5)] + [70, 140], seed=seed)
    ref = tc.plain_logits(folder, reqs)
    for dtype in ("float32", "bfloat16"):
        for name, steps in (("whole", rc.whole(reqs)), ("portions", rc.portions(reqs)), ("mixed", rc.mixed(reqs, seed=seed))):
            out = str(tmp_path / (dtype + name))
            rc.run_replay_inprocess(folder, dtype, out, steps, rc.max_live_tokens(steps), ["--kvcache-block-size", str(page), "--poison-cache"])
            compare(rc.collect(out, steps, cfg["vocab"]), ref, dtype, "seed %d/%s/%s" % (seed, name, dtype))
