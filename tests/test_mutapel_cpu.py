"""Mutapel without a GPU: its configuration reader and the specification built from it, the order in which layers run,
the tensor names a checkpoint must hold, and the plain implementation's mechanisms against closed forms written out
token by token."""

import copy
import math

import pytest
import torch

from tests.mutapel_configs import ALONE, MUTA_A, MUTA_B, MUTA_C
from tests.plain import mutapel_plain as plain


def build(cfg):
    from paged_llm_amd.config.registry import lookup_architecture
    from paged_llm_amd.models.decoder import DecoderModel
    arch = lookup_architecture(cfg)
    spec = arch.build_spec(arch.read_config(cfg))
    return spec, DecoderModel(spec, torch.float32, "cpu", max_positions=64)


def test_architecture_is_registered():
    from paged_llm_amd.config.registry import lookup_architecture
    assert lookup_architecture(MUTA_A).name == "Mutapel"


def test_repeated_layers_are_steps_of_one_layer_with_a_cache_each():
    spec, model = build(MUTA_A)
    # layer 0, then layers 1 and 2 three times, then layer 3; a pass of the repeated range starts at the steps marked
    assert [s.layer for s in spec.schedule] == [0, 1, 2, 1, 2, 1, 2, 3] and len(spec.layers) == 4
    assert [s.entry is not None for s in spec.schedule] == [False, True, False, True, False, True, False, False]
    assert [(s.layer, enters) for s, (_, enters) in zip(spec.schedule, plain.run_order(MUTA_A))] == plain.run_order(MUTA_A)
    # every step that convolves over time owns a state: the three runs of layer 1 (four taps) and layer 3 (two taps)
    assert sorted(model.state_specs()) == [1, 3, 5, 7]
    assert model.state_specs()[1].shape == (3 * (4 * 24 + 2 * 24 + 2 * 40),) and model.state_specs()[7].shape == (1 * (3 * 48 + 3 * 48 + 3 * 16),)
    groups = list(model.cache_groups().values())
    # pages per step; the runs of one layer share a group (equal shapes, mask and size), other layers have their own
    assert sorted(sorted(g.owners) for g in groups) == [[0], [1, 3, 5], [2, 4, 6], [7]]
    by_owner = {tuple(sorted(g.owners)): g.spec for g in groups}
    assert (by_owner[(0,)].kind, by_owner[(0,)].window) == ("window", 19) and (by_owner[(1, 3, 5)].kind, by_owner[(1, 3, 5)].window) == ("chunk", 21)
    names = set(model.weight_specs())
    assert {"embed", "head", "final.norm", "loop.in", "l0.norm1", "l0.norm1b", "l0.norm2", "l0.norm2b", "l0.mix.q", "l0.mix.g", "l0.mix.o",
            "l1.mix.q.b", "l1.mix.o.b", "l1.mix.k.conv", "l1.mix.sink", "l1.mlp.router", "l1.mlp.correction", "l1.mlp.e3.down",
            "l0.mlp.e3.gate", "l0.mlp.e3.up"} <= names
    assert not {"l2.norm2", "l2.mlp.router", "l0.mix.q.b", "l0.mix.sink", "l1.mix.g", "l1.mlp.e5.gate", "l0.mlp.e6.up"} & names


def test_sizes_come_from_the_configuration():
    _, model = build(MUTA_B)
    specs = model.weight_specs()
    assert "loop.in" not in specs                                               # no repeated range, no product in front of a pass
    assert specs["l0.mix.q"].shape == (3 * 10, 50) and specs["l0.mix.v"].shape == (3 * 6, 50) and specs["l0.mix.o"].shape == (50, 3 * 6)
    assert specs["l0.mix.v.conv"].shape == (18, 1) and specs["l2.mix.q.conv"].shape == (40, 7)
    assert specs["l1.mix.g"].shape == (5, 50) and specs["l1.mix.k"].shape == (6, 50) and specs["l1.mix.v"].shape == (10, 50)
    assert specs["l1.mlp.router"].shape == (8, 50) and specs["l1.mlp.correction"].shape == (8,) and "l1.mlp.e4.gate" not in specs
    assert specs["l2.mlp.e6.down"].shape == (50, 65) and specs["l2.mlp.router"].shape == (8, 50)
    assert sorted(model.state_specs()) == [2] and model.state_specs()[2].shape == (6 * (40 + 20 + 20),)    # one tap keeps nothing
    _, model = build(MUTA_C)
    assert model.weight_specs()["loop.in"].shape == (64, 128)
    assert [s.layer for s in build(MUTA_C)[0].schedule] == [0, 1, 2, 0, 1, 2]


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="attention_3"), "mixer type"),
    (lambda c: c["layers"][1]["mlp"].update(kind="dense"), "feed-forward kind"),
    (lambda c: c["loop"].update(stop=7), "loop"),
    (lambda c: c["loop"].update(times=0), "loop"),
])
def test_bad_configurations_are_refused(change, message):
    cfg = copy.deepcopy(MUTA_A)
    change(cfg)
    with pytest.raises(ValueError, match=message):
        build(cfg)


def test_missing_and_unexpected_tensors_are_named(tmp_path):
    from safetensors.torch import load_file, save_file
    from paged_llm_amd.weights import write_random_model
    from paged_llm_amd.weights.loader import WeightsError, load_weights
    cfg = ALONE["blocks"]
    folder = write_random_model(str(tmp_path), cfg, seed=1, dtype="float32", std=0.1)
    file = str(tmp_path / "model.safetensors")
    tensors = load_file(file)
    tensors["l0.mix.sinks"] = tensors.pop("l0.mix.sink")
    save_file(tensors, file)
    _, model = build(cfg)
    with pytest.raises(WeightsError) as err:
        load_weights(model, folder)
    assert err.value.missing == ["l0.mix.sink"] and err.value.unexpected == ["l0.mix.sinks"]


# --------------------------------------------------------------------------- the plain implementation against closed forms
def _weights(names_shapes, seed):
    g = torch.Generator().manual_seed(seed)
    return {n: torch.randn(shape, generator=g, dtype=torch.float64) * 0.3 for n, shape in names_shapes.items()}


def _turn(u, v, angle):
    return u * math.cos(angle) - v * math.sin(angle), v * math.cos(angle) + u * math.sin(angle)


def test_plain_rotation_pairs():
    x = torch.randn(5, 1, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(1))
    pos = torch.tensor([0, 1, 2, 7, 300])
    halves, neighbours = plain.rotate(x, pos, 50.0, 6, False), plain.rotate(x, pos, 50.0, 6, True)
    for t, p in enumerate(pos.tolist()):
        for i in range(3):
            angle = float(torch.tensor(float(p), dtype=torch.float32) * torch.tensor(50.0 ** (-2.0 * i / 6), dtype=torch.float32))
            a, b = _turn(x[t, 0, i], x[t, 0, i + 3], angle)                    # (i, i + 3) of the first six
            assert abs(halves[t, 0, i] - a) < 1e-12 and abs(halves[t, 0, i + 3] - b) < 1e-12
            a, b = _turn(x[t, 0, 2 * i], x[t, 0, 2 * i + 1], angle)            # (2i, 2i + 1)
            assert abs(neighbours[t, 0, 2 * i] - a) < 1e-12 and abs(neighbours[t, 0, 2 * i + 1] - b) < 1e-12
        assert torch.equal(halves[t, 0, 6:], x[t, 0, 6:]) and torch.equal(neighbours[t, 0, 6:], x[t, 0, 6:])
    assert torch.equal(plain.rotate(x, pos, 50.0, 0, True), x)


def test_plain_convolution_over_time():
    u = torch.randn(6, 3, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    w = torch.randn(3, 4, dtype=torch.float64, generator=torch.Generator().manual_seed(3))
    got = plain.time_convolution(u, w)
    for t in range(6):
        want = torch.zeros(3, dtype=torch.float64)
        for j in range(4):                                    # tap j meets the token 3 - j places back; the last tap the token itself
            if t - (3 - j) >= 0:
                want += w[:, j] * u[t - (3 - j)]
        assert torch.allclose(got[t], want, rtol=0, atol=1e-14)
    assert torch.allclose(plain.time_convolution(u, w[:, :1]), u * w[:, 0])    # one tap: a factor per channel


def test_plain_masks():
    assert [j for j in range(12) if plain.visible(7, j, "window", 3)] == [5, 6, 7]
    assert [j for j in range(12) if plain.visible(7, j, "window", 1)] == [7]
    assert [j for j in range(12) if plain.visible(7, j, "block", 3)] == [6, 7]           # blocks 0-2, 3-5, 6-8
    assert [j for j in range(12) if plain.visible(6, j, "block", 3)] == [6]
    assert [j for j in range(12) if plain.visible(8, j, "block", 3)] == [6, 7, 8]
    assert [j for j in range(12) if plain.visible(5, j, "block", 100)] == [0, 1, 2, 3, 4, 5]


@pytest.mark.parametrize("kind", ["attention", "attention_2"])
def test_plain_attention_token_by_token(kind):
    """Either mixer written out for one query at a time over exactly the keys it sees."""
    first = kind == "attention"
    T, width, H, G, d, dv, size, r = 11, 9, 4, 2, 6, 5, 4, 4
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": 3, "mask": {"size": size}, "rot": {"base": 30.0, "dims": r}, "scale": 0.7}
    shapes = {"l.q": (H * d, width), "l.k": (G * d, width), "l.v": (G * dv, width), "l.o": (width, H * dv)}
    if first:
        shapes.update({"l.q.b": (H * d,), "l.k.b": (G * d,), "l.v.b": (G * dv,), "l.o.b": (width,), "l.q.conv": (H * d, 3),
                       "l.k.conv": (G * d, 3), "l.v.conv": (G * dv, 3), "l.sink": (H,)})
    else:
        shapes["l.g"] = (H, width)
    W = _weights(shapes, 7)
    h = torch.randn(T, width, dtype=torch.float64, generator=torch.Generator().manual_seed(8))
    got = plain.attention_mixer(h, W, "l", m, kind, 1e-5, torch.float64)

    def rows(name, heads, size_):
        u = h @ W[f"l.{name}"].T
        if first:
            u = u + W[f"l.{name}.b"]
            u = torch.stack([sum(W[f"l.{name}.conv"][:, j] * u[t - 2 + j] for j in range(3) if t - 2 + j >= 0) for t in range(T)])
        return u.reshape(T, heads, size_)
    unit = lambda x: x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5)
    q = unit(plain.rotate(rows("q", H, d), torch.arange(T), 30.0, r, not first))
    k = unit(plain.rotate(rows("k", G, d), torch.arange(T), 30.0, r, not first))
    v = rows("v", G, dv)
    out = torch.zeros(T, H, dv, dtype=torch.float64)
    for a in range(H):
        g = a // (H // G)
        for t in range(T):
            keys = [n for n in range(t + 1) if (t // size == n // size if first else t - n < size)]
            e = torch.stack([torch.exp((q[t, a] @ k[n, g]) * 0.7) for n in keys])
            denom = e.sum() + (torch.exp(W["l.sink"][a]) if first else 0.0)
            out[t, a] = sum(e[i] / denom * v[n, g] for i, n in enumerate(keys))
            if not first:
                out[t, a] = out[t, a] * torch.sigmoid(W["l.g"][a] @ h[t])
    want = out.reshape(T, H * dv) @ W["l.o"].T + (W["l.o.b"] if first else 0.0)
    assert torch.allclose(got, want, rtol=1e-10, atol=1e-12)


def test_plain_router_by_hand():
    """Six router outputs in three groups of two, two groups kept, two chosen; the last output is a pass-through."""
    r = {"experts": 5, "identity": 1, "top": 2, "groups": {"count": 3, "keep": 2}}
    z = torch.log(torch.tensor([[0.30, 0.05, 0.10, 0.20, 0.25, 0.10]], dtype=torch.float64))     # softmax(z) is the row itself
    router = torch.eye(6, dtype=torch.float64)
    # without a correction: groups' marks 0.30, 0.20, 0.25 -> groups 0 and 2; chosen 0 (0.30) and 4 (0.25)
    chosen, weights = plain.route(z, router, torch.zeros(6, dtype=torch.float64), r)
    assert sorted(chosen[0].tolist()) == [0, 4] and torch.allclose(weights.sum(), torch.tensor(0.55, dtype=torch.float64))
    # a correction lifts expert 3 and the pass-through: marks 0.30, 0.50, 0.40 -> groups 1 and 2, chosen 3 and 5; the
    # weights are the scores without it, and they are not made to sum to one
    corr = torch.tensor([0.0, 0.0, 0.0, 0.30, 0.0, 0.30], dtype=torch.float64)
    chosen, weights = plain.route(z, router, corr, r)
    order = chosen[0].argsort()
    assert chosen[0][order].tolist() == [3, 5] and torch.allclose(weights[0][order], torch.tensor([0.20, 0.10], dtype=torch.float64))
    # corrections below zero everywhere: a group that is shut out counts as minus infinity, not as zero
    corr = torch.tensor([-1.0, -1.0, -3.0, -3.0, -1.1, -1.2], dtype=torch.float64)
    chosen, _ = plain.route(z, router, corr, {**r, "top": 3})
    assert sorted(chosen[0].tolist()) == [0, 1, 4]


def test_plain_experts_sum_the_chosen_and_hand_rows_back():
    width, ff = 6, 4
    mlp = {"expert": {"ff": ff}, "router": {"experts": 2, "identity": 2, "top": 2, "groups": {"count": 2, "keep": 2}}}
    W = _weights({"m.router": (4, width), "m.correction": (4,), "m.e0.gate": (ff, width), "m.e0.up": (ff, width), "m.e0.down": (width, ff),
                  "m.e1.gate": (ff, width), "m.e1.up": (ff, width), "m.e1.down": (width, ff)}, 9)
    h = torch.randn(20, width, dtype=torch.float64, generator=torch.Generator().manual_seed(10))
    got = plain.routed_experts(h, W, "m", mlp, torch.float64)
    s = torch.softmax(h @ W["m.router"].T, dim=-1)
    seen = set()
    for t in range(20):
        chosen = torch.topk(s[t] + W["m.correction"], 2).indices.tolist()
        seen.update(chosen)
        want = torch.zeros(width, dtype=torch.float64)
        for e in chosen:
            if e >= 2:
                want += s[t, e] * h[t]
            else:
                a = h[t] @ W[f"m.e{e}.gate"].T
                want += s[t, e] * ((a * torch.sigmoid(a) * (h[t] @ W[f"m.e{e}.up"].T)) @ W[f"m.e{e}.down"].T)
        assert torch.allclose(got[t], want, rtol=1e-10, atol=1e-12)
    assert seen == {0, 1, 2, 3}


def test_plain_model_repeats_layers_behind_a_product_with_the_embedding():
    """Two passes over one layer written out with the plain mixer: x <- W_in [x ; x0] in front of each, norms with
    1 + stored weight on both sides of the mixer, the sum times the constant."""
    cfg = ALONE["repeated"]
    cfg = {**cfg, "loop": {"start": 0, "stop": 1, "times": 2}}
    from paged_llm_amd.weights.random_init import _declared_weights, draw_weights
    W = {n: t.to(torch.float64) for n, t in draw_weights(_declared_weights(cfg), 5, torch.float32, 0.2, norm_jitter=True)}
    tokens = [3, 9, 9, 40, 2, 7]
    logits, streams = plain.forward(cfg, W, tokens, dtype=torch.float64, want_layers=True)
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    norm = lambda x, w: x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w)
    x0 = W["embed"][tokens]
    x = x0
    for run in range(2):
        x = torch.cat([x, x0], dim=1) @ W["loop.in"].T
        a = plain.attention_mixer(norm(x, W["l0.norm1"]), W, "l0.mix", cfg["layers"][0]["mixer"], "attention_2", eps, torch.float64)
        x = x + mult * norm(a, W["l0.norm1b"])
        assert torch.allclose(streams[run], x, rtol=1e-12, atol=1e-12)
    assert torch.allclose(logits, norm(x, W["final.norm"]) @ W["head"].T, rtol=1e-12, atol=1e-12)
