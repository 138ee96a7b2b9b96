"""Vivevik configurations drawn at random (widths, head counts, key and value widths, layer
order, which layers read whose keys, windows and kept prefixes shorter and longer than the
sequences and the 16-token pages, decay ranks and temperatures, feed-forwards present or not):
mixed batches through the engine against the plain implementation, float32 tight and bfloat16
by the root mean square."""
import random

import pytest
import torch

import helpers as H
import vivevik_cases as V
import plain_vivevik
from emu_ops import EmuOps

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]


def draw_config(seed):
    rng = random.Random(seed)
    width = rng.choice([32, 48, 64, 96, 128])
    layers, owners = [], []
    for i in range(rng.randint(2, 6)):
        ff = rng.choice([None, 8 * rng.randint(2, 20)])
        if rng.random() < 0.4:
            heads = rng.choice([1, 2, 3, 4, 6])
            vdim = rng.choice([8, 16, 24, 32, 64, 80])
            while heads * vdim % 8:
                vdim += 8
            layers.append(V._gla(heads, rng.choice([8, 16, 24, 32, 48, 64, 72]), vdim, rng.choice([1.0, 4.0, 16.0, 64.0]),
                                 rank=rng.choice([1, 3, 8, 16, 20]), ff=ff))
            continue
        mask = dict(size=rng.choice([1, 2, 5, 16, 17, 31, 40, 64, 500]), keep_first=rng.choice([0, 0, 1, 4, 15, 16, 33]))
        if owners and rng.random() < 0.5:
            src = rng.choice(owners)
            m = layers[src]["mixer"]
            group = m["heads"] // m["kv_heads"]
            layers.append(V._attention(m["kv_heads"] * rng.choice([1, group, 2 * group] if group > 1 else [1, 2]),
                                       m["kv_heads"], m["dim"], m["vdim"], rng.choice([0.1, 0.5, 1.0]),
                                       kv_from=src, ff=ff, **mask))
            continue
        kv = rng.choice([1, 2, 3])
        vdim = rng.choice([8, 16, 32, 48, 64, 128])
        heads = kv * rng.choice([1, 2, 4, 7])
        while heads * vdim % 8:
            vdim += 8
        layers.append(V._attention(heads, kv, rng.choice([8, 16, 32, 40, 64, 96, 128]), vdim, rng.choice([0.1, 0.5, 1.0]),
                                   ff=ff, **(mask if rng.random() < 0.85 else {})))
        owners.append(i)
    return dict(architecture="Vivevik", vocab=rng.choice([50, 131, 256]), width=width,
                norm=dict(eps=rng.choice([1e-6, 1e-5, 1e-3])), layers=layers)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("seed", range(20))
def test_drawn_configuration(backend, seed):
    raw = draw_config(seed)
    cfg = H.lab.VivevikConfig.from_dict(raw)
    tensors = V.make_tensors(cfg, seed)
    seqs = {f"r{i}": V.random_ids(cfg, n, 100 * seed + i) for i, n in enumerate([3, 45, 70, 20])}
    want = {rid: plain_vivevik.forward(ids, tensors, cfg.to_dict()) for rid, ids in seqs.items()}
    for dtype in ("f32", "bf16"):
        kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
        engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype=dtype, page_size=16, num_pages=16,
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
            assert rms < 0.06 * size, (raw, rms)
        engine.cache.check()
        assert engine.cache.metrics()["rows_used"] == 0
