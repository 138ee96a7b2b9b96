"""Ruvalorn configurations drawn at random (widths, head counts and sizes also beside the
multiples of 16, how much of a head rotates, windows shorter and longer than the sequences and the
16-token pages or none, dense feed-forwards, mixtures with and without groups, identity outputs
and a shared expert, feed-forward widths beside the multiples of 8, layers without a feed-forward, loops anywhere in the stack): mixed batches
through the engine against the plain implementation, float32 tight and bfloat16 by the root mean
square."""
import random

import pytest
import torch

import helpers as H
import ruvalorn_cases as R
from emu_ops import EmuOps

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]


def draw_mlp(rng):
    kind = rng.choice(["none", "dense", "moe", "moe"])
    if kind == "none":
        return None
    if kind == "dense":
        return R.dense(rng.choice([8 * rng.randint(2, 20), 20, 36, 100]))
    per, count = rng.choice([1, 2, 3, 5]), rng.choice([1, 2, 4])
    outputs = per * count
    identity = rng.choice([0, 0, 1, per]) if outputs > 1 else 0
    identity = min(identity, outputs - 1)
    keep = rng.randint(1, count)
    top = rng.randint(1, min(keep * per, 4))
    return R.moe(rng.choice([8 * rng.randint(1, 6), 12, 20]), outputs - identity, top, identity=identity, scale=rng.choice([0.5, 1.0, 2.5]),
                 groups=None if count == 1 and rng.random() < 0.5 else (count, keep),
                 shared=rng.choice([None, 8 * rng.randint(1, 8), 28]))


def draw_config(seed):
    rng = random.Random(seed)
    layers = []
    for _ in range(rng.randint(1, 4)):
        kv = rng.choice([1, 2, 3])
        dim = rng.choice([8, 16, 24, 32, 40, 64, 96, 128])
        rot = rng.choice([None, 2, dim // 2 // 2 * 2, dim])
        layers.append(R.attention(kv * rng.choice([1, 2, 4]), kv, dim, rng.choice([0.05, 0.1, 0.3]),
                                  size=rng.choice([None, 1, 2, 5, 16, 17, 31, 40, 64, 500]),
                                  rot=None if not rot else (rot, rng.choice([10.0, 1000.0, 50000.0])),
                                  mlp=draw_mlp(rng)))
    raw = dict(architecture="Ruvalorn", vocab=rng.choice([50, 131, 256]), width=rng.choice([32, 48, 64, 96, 128]),
               norm=dict(eps=rng.choice([1e-6, 1e-5, 1e-3])), layers=layers)
    if rng.random() < 0.7:
        start = rng.randrange(len(layers))
        raw["loop"] = dict(start=start, stop=rng.randint(start + 1, len(layers)), times=rng.randint(1, 3))
    return raw


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("seed", range(12))
def test_drawn_configuration(backend, seed):
    raw = draw_config(seed)
    cfg = H.lab.RuvalornConfig.from_dict(raw)
    tensors = R.make_tensors(cfg, seed)
    seqs = {f"r{i}": R.random_ids(cfg, n, 100 * seed + i) for i, n in enumerate([3, 45, 70, 20])}
    want = {rid: R.plain_of(cfg.to_dict(), tensors, ids) for rid, ids in seqs.items()}
    for dtype in ("f32", "bf16"):
        kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=40,
                              max_requests=3, max_batch_tokens=128, max_seq_len=128, **kw)
        got = H.run_trace(engine, seqs, H.steps_mixed(seqs, seed=seed, max_live=3, budget=64))
        diff = torch.cat([got[rid].double() - want[rid] for rid in got])
        assert not torch.isnan(diff).any()
        size = max(1.0, float(torch.cat(list(want.values())).std()))
        if dtype == "f32":
            bad = H.first_wrong(got, want, 2e-4 * size)
            assert bad is None, f"{raw}\nfirst wrong logits at (request, position, error) = {bad}"
        else:
            rms = float(diff.pow(2).mean().sqrt())
            assert rms < 0.2 * size, (raw, rms)
        engine.cache.check()
        assert engine.cache.metrics()["rows_used"] == 0


# Two configurations at the sizes of small real models (hundreds of channels, windows of hundreds
# of positions over pages of 64, dozens of experts), with sequences that cross several windows.
LARGER = {
    "X": dict(architecture="Ruvalorn", vocab=701, width=384, norm=dict(eps=1e-6), loop=dict(start=0, stop=2, times=3),
              layers=[R.attention(6, 3, 80, 0.11, size=150, rot=(40, 20000.0),
                                  mlp=R.moe(48, 24, 6, identity=8, scale=1.5, groups=(8, 4), shared=136)),
                      R.attention(8, 2, 64, 0.125, size=70, rot=(64, 500.0), mlp=R.dense(320)),
                      R.attention(3, 1, 128, 0.09, size=300, rot=(32, 100.0),
                                  mlp=R.moe(104, 70, 3, identity=2, scale=2.0, groups=(8, 3)))]),
    "Y": dict(architecture="Ruvalorn", vocab=330, width=192, norm=dict(eps=1e-5), loop=dict(start=1, stop=2, times=2),
              layers=[R.attention(2, 2, 112, 0.1, size=257, rot=(56, 1e6), mlp=R.dense(512)),
                      R.attention(12, 4, 32, 0.2, size=64, rot=(8, 10.0),
                                  mlp=R.moe(32, 62, 5, identity=2, scale=3.0, groups=(16, 5), shared=64)),
                      R.attention(4, 1, 48, 0.15, rot=(48, 10000.0), mlp=None)]),
}


@pytest.mark.gpu
@pytest.mark.parametrize("name", list(LARGER))
def test_sizes_of_small_real_models(name):
    raw = LARGER[name]
    cfg = H.lab.RuvalornConfig.from_dict(raw)
    tensors = R.make_tensors(cfg, 11)
    seqs = {f"r{i}": R.random_ids(cfg, n, 50 + i) for i, n in enumerate([420, 97, 333, 1])}
    want = {rid: R.plain_of(cfg.to_dict(), tensors, ids) for rid, ids in seqs.items()}
    size = max(1.0, float(torch.cat(list(want.values())).std()))
    for dtype in ("f32", "bf16"):
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=64, num_pages=16,
                              max_requests=3, max_batch_tokens=512, max_seq_len=512)
        for steps in (H.steps_prefill_then_decode(seqs, tail=40), H.steps_mixed(seqs, seed=1, max_live=3, budget=150)):
            got = H.run_trace(engine, seqs, steps)
            diff = torch.cat([got[rid].double() - want[rid] for rid in got])
            assert not torch.isnan(diff).any()
            if dtype == "f32":
                bad = H.first_wrong(got, want, 3e-4 * size)
                assert bad is None, f"first wrong logits at (request, position, error) = {bad}"
            else:
                assert float(diff.pow(2).mean().sqrt()) < 0.2 * size
            engine.cache.check()
            assert engine.cache.metrics()["rows_used"] == 0
