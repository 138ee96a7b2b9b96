"""Each mechanism of Ruvalorn alone, against the plain implementation's function for it: the
kernel set's operation (or the part that owns the mechanism) once as the PyTorch reference on
the CPU and once as the HIP kernel on the GPU.  Where random numbers would hide a fault (a key at
a window's edge, a far key among hundreds, a router output that is left out), the inputs are made
so that it shows."""
import types

import pytest
import torch

import helpers as H          # noqa: F401
import plain_ruvalorn as P
import ruvalorn_cases as R
from emu_ops import EmuOps
from llm_inference_lab_amd.parts import RMSNorm, RotaryEmbedding, RoutedExperts
from llm_inference_lab_amd.config.spec import PartSpec

BACKENDS = ["emu", pytest.param("hip", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
F64 = torch.float64


def ops_of(backend):
    if backend == "emu":
        return EmuOps()
    from llm_inference_lab_amd.kernels.hip_ops import HipOps
    return HipOps("cuda:0")


def randn(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(got, want, dtype, what="", f32=2e-5, bf16=2e-2):
    err = float((got.detach().cpu().double() - want.double()).abs().max())
    size = max(1.0, float(want.abs().max()))
    assert err <= (f32 if dtype == torch.float32 else bf16) * size, f"{what}: off by {err} (values up to {size})"


class Scratch:
    """The least a part needs of a step: named scratch buffers and no sums owed."""

    def __init__(self, device):
        self.device, self.pending, self.memo = device, None, {}

    def scratch(self, name, shape, dtype):
        return torch.zeros(shape, dtype=dtype, device=self.device)


# ------------------------------------------------------------------ norm, gate, offset
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden", [8, 72, 1000])
def test_norm_with_a_weight_stored_around_zero(backend, dtype, hidden):
    ops = ops_of(backend)
    x = (randn(9, hidden, seed=1, scale=3.0) + 0.5).to(ops.device)
    w = randn(hidden, seed=2, scale=0.4).to(torch.bfloat16)
    norm = RMSNorm(hidden, 1e-3, dict(weight="w"), weight_offset=1.0)
    norm.bind({"w": w.to(ops.device) if dtype == torch.bfloat16 else w.float().to(ops.device)}, ops, dtype)
    out = torch.empty(9, hidden, dtype=dtype, device=ops.device)
    norm.forward(x, out)
    close(out, P.norm(x.cpu().to(F64), w.to(F64), 1e-3), dtype, "x / rms * (1 + w)")


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim", [(1, 16), (4, 96), (7, 48)])
def test_one_gate_per_head(backend, dtype, heads, dim):
    ops = ops_of(backend)
    out = randn(11, heads * dim, seed=3).to(dtype)
    gate = randn(11, heads, seed=4, scale=3.0)
    want = P.gate_heads(out.to(F64).view(11, heads, dim), gate.to(F64)).reshape(11, -1)
    got = out.clone().to(ops.device)
    ops.gate_heads(got, gate.to(ops.device), heads, dim)
    close(got, want, dtype, "heads times sigmoid")


@pytest.mark.parametrize("backend", BACKENDS)
def test_a_vector_added_to_every_row(backend):
    ops = ops_of(backend)
    x, table = randn(13, 40, seed=5), randn(3, 40, seed=6)
    got = x.clone().to(ops.device)
    ops.add_row_vector(got, table.to(ops.device), 2)
    close(got, x.to(F64) + table[2].to(F64), torch.float32, "stream + vector", f32=1e-6)


# ------------------------------------------------------------------ rotation of part of a head
@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dim,rot,padded", [(16, 16, 16), (16, 8, 16), (96, 32, 96), (24, 12, 32), (40, 40, 48),
                                            (20, 2, 32)])
def test_rotation_of_the_first_channels_of_a_head(backend, dim, rot, padded):
    """The part's table and channel order, applied by the kernel set's rotation in the kernels'
    pairing (place j with place j + padded/2), are the rotation of channel i with channel i + rot/2
    of the head as the model file has it; channels that do not turn, and the zeros behind a head,
    come back as they went in."""
    ops = ops_of(backend)
    part = RotaryEmbedding(dim, 300.0, rotary_dim=rot, padded_dim=padded)
    part.bind({}, ops, torch.float32)
    order = part.channel_order() or list(range(dim))
    assert sorted(c for c in order if c >= 0) == list(range(dim)) and len(order) == padded
    x = randn(7, 3, dim, seed=7)
    positions = torch.tensor([0, 1, 2, 17, 100, 1000, 5000], dtype=torch.int32)
    want = P.rotate(x.to(F64), positions, rot, 300.0)
    laid = torch.zeros(7, 3, padded)
    for place, c in enumerate(order):
        if c >= 0:
            laid[:, :, place] = x[:, :, c]
    got = laid.to(ops.device)
    ops.rope_inplace(got, positions.to(ops.device), part.rotary_table())
    got = got.cpu()
    for place, c in enumerate(order):
        if c >= 0:
            close(got[:, :, place], want[:, :, c], torch.float32, f"channel {c}", f32=3e-4)
        else:
            assert float(got[:, :, place].abs().max()) == 0.0


# ------------------------------------------------------------------ the router's choice
def choice_by_plain(logits, correction, groups, keep, top, scale, identity=0):
    """The plain implementation's choice for given router logits: its router is fed the logits
    themselves through an identity matrix."""
    outputs = logits.shape[1]
    weights = {"router": torch.eye(outputs, dtype=F64), "correction": correction.to(F64)}
    router = dict(experts=outputs - identity, identity=identity, top=top, scale=scale,
                  groups=dict(count=groups, keep=keep))
    return P.route(logits.to(F64), weights, "", router)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("outputs,groups,keep,top", [(20, 4, 3, 4), (8, 1, 1, 8), (6, 6, 2, 2), (12, 3, 1, 4),
                                                     (64, 8, 4, 6), (5, 1, 1, 1), (300, 4, 2, 9)])
def test_the_routers_choice(backend, outputs, groups, keep, top):
    ops = ops_of(backend)
    logits = randn(50, outputs, seed=outputs, scale=2.0)
    correction = randn(outputs, seed=outputs + 1, scale=0.3) - 0.2
    chosen = torch.zeros(50, top, dtype=torch.int32, device=ops.device)
    weights = torch.zeros(50, top, device=ops.device)
    ops.moe_select(logits.to(ops.device), correction.to(ops.device), groups, keep, 2.5, chosen, weights)
    want = choice_by_plain(logits, correction, groups, keep, top, 2.5)
    for r in range(50):
        assert chosen[r].tolist() == [e for e, _ in want[r]], f"row {r}"
        close(weights[r], torch.stack([w for _, w in want[r]]), torch.float32, f"weights of row {r}", f32=1e-5)


@pytest.mark.parametrize("backend", BACKENDS)
def test_an_output_of_a_dropped_group_counts_as_minus_infinity(backend):
    """All choice values negative: if the outputs of a dropped group counted as 0 they would win."""
    ops = ops_of(backend)
    logits = torch.zeros(1, 6)                                         # scores of 1/6 each
    correction = torch.tensor([-0.9, -0.8, -0.3, -0.7, -0.5, -0.6])    # groups (0,1) (2,3) (4,5); (0,1) is dropped
    chosen = torch.zeros(1, 3, dtype=torch.int32, device=ops.device)
    weights = torch.zeros(1, 3, device=ops.device)
    ops.moe_select(logits.to(ops.device), correction.to(ops.device), 3, 2, 1.0, chosen, weights)
    assert chosen[0].tolist() == [2, 4, 5]
    # the weights are the scores without the correction, times the scale, and are not renormalised
    close(weights[0], torch.full((3,), 1.0 / 6), torch.float32, "weights", f32=1e-6)
    # equal values: the smaller index
    ops.moe_select(logits.to(ops.device), torch.zeros(6, device=ops.device), 1, 1, 1.0, chosen, weights)
    assert chosen[0].tolist() == [0, 1, 2]


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
def test_the_weighted_sum_takes_the_chosen_only(backend, dtype):
    ops = ops_of(backend)
    resid, src = randn(6, 24, seed=8), randn(6, 24, seed=9).to(dtype)
    chosen = torch.tensor([[0, 3], [3, 1], [2, 2], [5, 4], [1, 0], [3, 3]], dtype=torch.int32)
    weights = randn(6, 2, seed=10).abs()
    got = resid.clone().to(ops.device)
    ops.moe_add_chosen(got, src.to(ops.device), chosen.to(ops.device), weights.to(ops.device), 3, 5)
    w = (weights * ((chosen >= 3) & (chosen < 5))).sum(-1, keepdim=True)
    close(got, resid.to(F64) + w.to(F64) * src.to(F64), torch.float32, "resid + w src", f32=1e-6)


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 5, 70, 300])
@pytest.mark.parametrize("shape", [dict(experts=6, identity=2, top=3, groups=(4, 2), shared=40, ff=24, width=64),
                                   dict(experts=5, identity=0, top=1, groups=None, shared=None, ff=16, width=48),
                                   dict(experts=12, identity=3, top=5, groups=(5, 3), shared=48, ff=32, width=128)])
def test_the_mixture_of_experts_alone(backend, dtype, rows, shape):
    """The part with its own tensors against the plain implementation's mixture, on inputs whose
    choice is not close (the margin of every row's choice is checked in the plain implementation)."""
    ops = ops_of(backend)
    width, ff, n = shape["width"], shape["ff"], shape["experts"]
    raw = R.moe(ff, n, shape["top"], identity=shape["identity"], scale=1.5, groups=shape["groups"], shared=shape["shared"])
    names = dict(router="m.router", correction="m.correction", expert_gate="m.e{}.gate", expert_up="m.e{}.up",
                 expert_down="m.e{}.down")
    shared = None if shape["shared"] is None else PartSpec(
        "swiglu", params=dict(hidden_size=width, intermediate_size=shape["shared"]),
        tensors=dict(gate_weight="m.shared.gate", up_weight="m.shared.up", down_weight="m.shared.down"))
    groups = shape["groups"] or (1, 1)
    part = RoutedExperts(width, ff, n, shape["top"], names, identity=shape["identity"], scale=1.5, groups=groups[0],
                         groups_keep=groups[1], shared=shared)
    tensors = {}
    for i, (name, spec) in enumerate(part.tensor_specs().items()):
        if name.endswith("correction"):
            t = randn(*spec.shape, seed=100 + i, scale=0.3) - 0.1
        elif name.endswith("router"):
            t = randn(*spec.shape, seed=100 + i, scale=3.0 / width ** 0.5)
        else:
            t = randn(*spec.shape, seed=100 + i, scale=1.0 / spec.shape[1] ** 0.5)
        tensors[name] = t.to(torch.bfloat16)
    # rows whose choice rests on a close call are left out of the comparison (not of the batch)
    h = randn(rows, width, seed=11).to(torch.bfloat16)
    plain_w = {k[2:]: v.to(F64) for k, v in tensors.items()}
    want = P.mixture(h.to(F64), plain_w, "", raw)
    z = h.to(F64) @ plain_w["router"].T
    c = torch.softmax(z, -1) + plain_w["correction"]
    gaps = (c[:, :, None] - c[:, None, :]).abs() + torch.eye(c.shape[1], dtype=F64)[None] * 9.0
    # (the part is handed activations of 16 bits in both dtypes, so the router's products are exact
    # and its choice values differ from these by the order of 32-bit sums only)
    sure = gaps.flatten(1).min(-1).values > 1e-5
    assert int(sure.sum()) >= rows // 2
    kept = {k: (v.to(ops.device) if dtype == torch.bfloat16 or v.dim() != 2 else v.float().to(ops.device))
            for k, v in tensors.items()}
    part.bind(kept, ops, dtype)
    resid = randn(rows, width, seed=12)
    got = resid.clone().to(ops.device)
    part.forward(h.to(dtype).to(ops.device), got, Scratch(ops.device))
    close(got.cpu()[sure], (resid.to(F64) + want)[sure], dtype, "stream + mixture", f32=5e-5, bf16=4e-2)
    if backend == "hip" and dtype == torch.bfloat16:
        # the same with the experts one after the other over all rows (what float32 does) instead
        # of grouped products over rows sorted by expert
        assert ops.moe_grouped(dtype)
        with ops.debug.force(experts_one_by_one=True):
            again = resid.clone().to(ops.device)
            part.forward(h.to(dtype).to(ops.device), again, Scratch(ops.device))
        close(again.cpu()[sure], (resid.to(F64) + want)[sure], dtype, "stream + mixture, expert by expert", bf16=4e-2)


# ------------------------------------------------------------------ window edges, far keys
def one_layer_with_a_key_that_stands_out(window, dim=16, rot=(4, 50.0), heads=2, kv_heads=1, width=64, vocab=40):
    """A model of one attention layer in which the key of token 1 takes nearly all the weight of the
    query of token 2 whenever it is seen: a channel that does not turn carries a large product for
    that pair and nearly nothing for the filler tokens.  Returns (raw config, tensors)."""
    raw = dict(architecture="Ruvalorn", vocab=vocab, width=width, norm=dict(eps=1e-6),
               layers=[R.attention(heads, kv_heads, dim, 1.0, size=window, rot=rot, mlp=None)])
    cfg = H.lab.RuvalornConfig.from_dict(raw)
    tensors = R.make_tensors(cfg, 3)
    emb = tensors["embed"].double()
    normed = P.norm(emb, tensors["l0.norm1"].double(), 1e-6)
    channel = dim - 1                                  # (beyond the channels that turn)
    for name, token, n_heads in (("l0.mix.k", 1, kv_heads), ("l0.mix.q", 2, heads)):
        w = tensors[name].double() * 0.2
        u = normed[token]
        for head in range(n_heads):
            w[head * dim + channel] = 7.0 * u / (u @ u)
        tensors[name] = w.to(torch.bfloat16)
        tensors[name + ".b"] = torch.zeros_like(tensors[name + ".b"])
    return raw, tensors


def run_prompt_or_decode(raw, tensors, ids, backend, decode_from, page_size=16):
    cfg = H.lab.RuvalornConfig.from_dict(raw)
    kw = dict(ops=EmuOps(), device="cpu") if backend == "emu" else {}
    engine = H.lab.Engine(config=cfg, tensors=tensors.items(), dtype="f32", page_size=page_size, num_pages=40,
                          max_requests=1, max_batch_tokens=512, max_seq_len=512, **kw)
    req = engine.open("r")
    if decode_from >= len(ids):
        out = engine.step([H.lab.StepEntry(req, ids, [len(ids) - 1])])
    else:
        engine.step([H.lab.StepEntry(req, ids[:decode_from], [])])
        for i in range(decode_from, len(ids)):
            out = engine.step([H.lab.StepEntry(req, [ids[i]], [0])])
    return out.float().cpu()[0].double()


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoded", [False, True])
@pytest.mark.parametrize("window", [1, 5, 16, 17, 40])
def test_a_key_just_inside_and_just_outside_the_window(backend, decoded, window):
    """The query at position i sees the keys i - window + 1 .. i.  With the key that stands out
    at the window's last seen place, one beyond it, next to the query, and on both sides of the
    borders of the 16-token pages, the logits are the plain implementation's, and the plain
    implementation itself says whether the key was seen (its logits with and without differ)."""
    raw, tensors = one_layer_with_a_key_that_stands_out(window)
    plain = lambda ids, r=raw: R.plain_of(r, tensors, ids)[-1]
    wider = {**raw, "layers": [R.attention(2, 1, 16, 1.0, size=window + 1, rot=(4, 50.0), mlp=None)]}
    for back in sorted({0, 1, window - 1, window, window + 1, 15, 16, 17}):
        for at in (20, 31, 32, 47):                    # the query's position, around page borders
            if back > at:
                continue
            ids = [3 + (7 * i) % 30 for i in range(at + 1)]
            ids[at] = 2
            if back > 0:
                ids[at - back] = 1
            want = plain(ids)
            got = run_prompt_or_decode(raw, tensors, ids, backend, at if decoded else at + 1)
            assert float((got - want).abs().max()) < 2e-4, (window, back, at)
            if back == window and back > 0:            # the first key that is out of sight: one position more would see it
                assert float((plain(ids, wider) - want).abs().max()) > 0.3, "the test would not see a window one too wide"


@pytest.mark.parametrize("backend", BACKENDS)
@pytest.mark.parametrize("decoded", [False, True])
def test_a_far_key_among_hundreds(backend, decoded):
    raw, tensors = one_layer_with_a_key_that_stands_out(300, dim=32, rot=(16, 10000.0), heads=4, kv_heads=2)
    for back in (250, 299, 300):
        ids = [3 + (11 * i) % 31 for i in range(330)]
        ids[-1] = 2
        ids[-1 - back] = 1
        want = R.plain_of(raw, tensors, ids)[-1]
        without = list(ids)
        without[-1 - back] = 5
        seen = float((R.plain_of(raw, tensors, without)[-1] - want).abs().max()) > 0.3
        assert seen == (back < 300)
        got = run_prompt_or_decode(raw, tensors, ids, backend, 300 if decoded else 330, page_size=64)
        assert float((got - want).abs().max()) < 2e-4, back


@pytest.mark.parametrize("backend", BACKENDS)
def test_the_first_tokens_of_a_sequence(backend):
    """Positions 0, 1, 2 as a prompt and token by token: the first has one key, its own."""
    raw, tensors = one_layer_with_a_key_that_stands_out(4)
    for ids in ([2], [1, 2], [1, 7, 2], [9, 1, 2, 2]):
        want = R.plain_of(raw, tensors, ids)[-1]
        for decode_from in (len(ids), 1):
            got = run_prompt_or_decode(raw, tensors, ids, backend, decode_from)
            assert float((got - want).abs().max()) < 2e-4, (ids, decode_from)
