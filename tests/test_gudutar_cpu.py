"""Gudutar without a GPU: its configuration reader and the specification built from it, the tensor names a checkpoint
must hold, and the plain implementation's recurrent mixers against closed forms of the same sums."""

import copy

import pytest
import torch

from tests.gudutar_configs import ALONE, GUDU_A, GUDU_B
from tests.plain import gudutar_plain as plain


def build(cfg):
    from paged_llm_amd.config.registry import lookup_architecture
    from paged_llm_amd.models.decoder import DecoderModel
    arch = lookup_architecture(cfg)
    spec = arch.build_spec(arch.read_config(cfg))
    return spec, DecoderModel(spec, torch.float32, "cpu", max_positions=64)


def test_architecture_is_found_by_the_singular_key():
    from paged_llm_amd.config.registry import lookup_architecture
    assert lookup_architecture(GUDU_A).name == "Gudutar"
    with pytest.raises(ValueError):
        lookup_architecture({"architecture": "NoSuchModel"})


def test_layers_that_share_weights_are_steps_of_one_layer():
    spec, model = build(GUDU_A)
    assert [s.layer for s in spec.schedule] == [0, 1, 2, 0, 2, 1] and len(spec.layers) == 3
    # every step owns its state or cache: six steps, four with state, two with pages (in one group: equal shapes and window)
    assert sorted(model.state_specs()) == [0, 1, 3, 5]
    groups = model.cache_groups()
    assert len(groups) == 1 and list(groups.values())[0].owners == [2, 4] and list(groups.values())[0].spec.window == 21
    names = set(model.weight_specs())
    assert {"embed", "head", "final.norm", "final.norm.b", "l0.norm1", "l0.norm1.b", "l0.norm2.b", "l0.mix.in", "l0.mix.conv",
            "l0.mix.conv.b", "l0.mix.A_log", "l0.mlp.gate", "l1.mix.g", "l2.mix.dkv.norm", "l2.mix.uk"} <= names
    assert not any(n.startswith(("l3.", "l4.", "l5.")) for n in names) and "l1.norm2" not in names


def test_sizes_come_from_the_configuration():
    _, model = build(GUDU_B)
    specs = model.weight_specs()
    assert specs["l1.mix.in"].shape == (2 * 144 + 2 * 80 + 2, 64) and specs["l1.mix.conv"].shape == (144 + 160, 2)
    assert specs["l0.mix.dkv"].shape == (272 + 32, 64) and specs["l0.mix.uv"].shape == (2 * 48, 272)
    assert specs["l2.mix.q"].shape == (2 * 144, 64) and specs["l2.mix.o"].shape == (64, 2 * 16)
    groups = {g.spec.window: g for g in model.cache_groups().values()}
    assert sorted(groups) == [0, 16]                          # one full group (no mask in the configuration), one window
    # a latent too wide for the paged attention kernels keeps key rows only; the other one keys and transposed values
    assert [t.name for t in groups[0].spec.tensors] == ["k"] and [t.name for t in groups[16].spec.tensors] == ["k", "v"]
    assert model.state_specs()[1].shape == (2 * 80 * 72 + (144 + 160) * 1,)


@pytest.mark.parametrize("change,message", [
    (lambda c: c["layers"][0].update(type="hyena"), "mixer type"),
    (lambda c: c["layers"][2]["mlp"].update(kind="experts"), "feed-forward kind"),
    (lambda c: c["layers"][3].update(weights_of=4), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=1), "another type"),
])
def test_bad_configurations_are_refused(change, message):
    cfg = copy.deepcopy(GUDU_A)
    change(cfg)
    with pytest.raises(ValueError, match=message):
        build(cfg)


def test_missing_and_unexpected_tensors_are_named(tmp_path):
    from safetensors.torch import load_file, save_file
    from paged_llm_amd.weights import write_random_model
    from paged_llm_amd.weights.loader import WeightsError, load_weights
    cfg = ALONE["retention"]
    folder = write_random_model(str(tmp_path), cfg, seed=1, dtype="float32", std=0.1)
    file = str(tmp_path / "model.safetensors")
    tensors = load_file(file)
    tensors["l0.norm1.bias"] = tensors.pop("l0.norm1.b")
    save_file(tensors, file)
    _, model = build(cfg)
    with pytest.raises(WeightsError) as err:
        load_weights(model, folder)
    assert err.value.missing == ["l0.norm1.b"] and err.value.unexpected == ["l0.norm1.bias"]


# --------------------------------------------------------------------------- the plain implementation against closed forms
def _weights(names_shapes, seed):
    g = torch.Generator().manual_seed(seed)
    return {n: torch.randn(shape, generator=g, dtype=torch.float64) * 0.3 for n, shape in names_shapes.items()}


def test_plain_retention_is_the_decayed_sum_over_earlier_tokens():
    m = {"heads": 2, "dim": 6, "vdim": 5, "rot": {"base": 50.0, "dims": 4}, "decay": [0.7, 0.95]}
    w = _weights({"q": (12, 8), "k": (12, 8), "v": (10, 8), "g": (10, 8), "o": (8, 10)}, 1)
    h = torch.randn(9, 8, dtype=torch.float64, generator=torch.Generator().manual_seed(2))
    got = plain.retention_mixer(h, w, m, 1e-6)
    pos = torch.arange(9)
    q = plain.rotate((h @ w["q"].T).reshape(9, 2, 6), pos, 50.0, 4, False)
    k = plain.rotate((h @ w["k"].T).reshape(9, 2, 6), pos, 50.0, 4, False) * 6 ** -0.5
    v = (h @ w["v"].T).reshape(9, 2, 5)
    o = torch.zeros(9, 2, 5, dtype=torch.float64)
    for a in range(2):
        for t in range(9):
            for s in range(t + 1):                             # o_t = sum_s decay^(t - s) (q_t . k_s) v_s
                o[t, a] += m["decay"][a] ** (t - s) * (q[t, a] @ k[s, a]) * v[s, a]
    want = (plain.unit_rms(o, 1e-6).reshape(9, 10) * plain.silu(h @ w["g"].T)) @ w["o"].T
    assert torch.allclose(got, want, rtol=1e-10, atol=1e-12)


def test_plain_state_space_layer_is_the_weighted_sum_over_earlier_tokens():
    m = {"heads": 4, "vdim": 3, "state": 5, "groups": 2, "conv": 3, "norm_groups": 2}
    inner, gn = 12, 10
    w = _weights({"in": (2 * inner + 2 * gn + 4, 7), "conv": (inner + 2 * gn, 3), "conv.b": (inner + 2 * gn,), "dt_bias": (4,),
                  "A_log": (4,), "D": (4,), "norm": (inner,), "o": (7, inner)}, 3)
    h = torch.randn(8, 7, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    got = plain.mamba2_mixer(h, w, m, 1e-5)
    proj = h @ w["in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:inner + inner + 2 * gn], proj[:, 2 * inner + 2 * gn:]
    conv = torch.zeros_like(xbc)
    for t in range(8):
        for j in range(3):                                    # tap j meets the token 2 - j places back
            if t - (2 - j) >= 0:
                conv[t] += w["conv"][:, j] * xbc[t - (2 - j)]
    xbc = plain.silu(conv + w["conv.b"])
    x, B, C = xbc[:, :inner].reshape(8, 4, 3), xbc[:, inner:inner + gn].reshape(8, 2, 5), xbc[:, inner + gn:].reshape(8, 2, 5)
    dt = torch.log1p(torch.exp(dt + w["dt_bias"]))
    log_decay = -torch.exp(w["A_log"]) * dt                   # [8, 4]
    y = torch.zeros(8, 4, 3, dtype=torch.float64)
    for a in range(4):
        g = a // 2
        for t in range(8):
            for s in range(t + 1):                             # y_t = sum_s exp(sum of log decays after s) (C_t . B_s) dt_s x_s
                y[t, a] += torch.exp(log_decay[s + 1:t + 1, a].sum()) * (C[t, g] @ B[s, g]) * dt[s, a] * x[s, a]
            y[t, a] += w["D"][a] * x[t, a]
    y = y.reshape(8, inner) * plain.silu(z)
    y = plain.unit_rms(y.reshape(8, 2, 6), 1e-5).reshape(8, inner) * w["norm"]
    assert torch.allclose(got, y @ w["o"].T, rtol=1e-10, atol=1e-12)


def test_plain_latent_attention_window_and_shared_rotated_key():
    m = {"heads": 2, "dim": 4, "rot_dim": 2, "vdim": 3, "kv_rank": 5, "rot": {"base": 20.0, "dims": 2}, "scale": 0.4, "mask": {"size": 3}}
    w = _weights({"q": (12, 6), "dkv": (7, 6), "dkv.norm": (5,), "uk": (8, 5), "uv": (6, 5), "o": (6, 6)}, 5)
    h = torch.randn(7, 6, dtype=torch.float64, generator=torch.Generator().manual_seed(6))
    got = plain.latent_attention_mixer(h, w, m, 1e-5)
    # token by token, every key expanded from the latent, only the keys at distance 0, 1, 2
    out = torch.zeros(7, 6, dtype=torch.float64)
    down = h @ w["dkv"].T
    c = down[:, :5] / torch.sqrt((down[:, :5] ** 2).mean(-1, keepdim=True) + 1e-5) * w["dkv.norm"]
    kr = plain.rotate(down[:, 5:], torch.arange(7), 20.0, 2, True)
    qs = (h @ w["q"].T).reshape(7, 2, 6)
    for a in range(2):
        for t in range(7):
            q_rot = plain.rotate(qs[t:t + 1, a, 4:], torch.tensor([t]), 20.0, 2, True)[0]
            keys = list(range(max(0, t - 2), t + 1))
            scores = torch.stack([(qs[t, a, :4] @ (w["uk"][4 * a:4 * a + 4] @ c[n]) + q_rot @ kr[n]) * 0.4 for n in keys])
            p = torch.softmax(scores, 0)
            out[t, 3 * a:3 * a + 3] = sum(p[i] * (w["uv"][3 * a:3 * a + 3] @ c[n]) for i, n in enumerate(keys))
    assert torch.allclose(got, out @ w["o"].T, rtol=1e-10, atol=1e-12)
