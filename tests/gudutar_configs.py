"""Small Gudutar configurations for the tests: sizes, layer orders and constants that differ from one another in
every field, and single-layer ones that show one mechanism alone."""

import copy


def _mamba(heads=4, vdim=24, state=16, groups=2, conv=3, norm_groups=2):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _retention(heads=3, dim=32, vdim=40, rot_dims=16, base=5000.0, decay=(0.9, 0.97, 0.995)):
    return {"heads": heads, "dim": dim, "vdim": vdim, "rot": {"base": base, "dims": rot_dims}, "decay": list(decay)}


def _latent(heads=6, dim=24, rot_dim=8, vdim=20, kv_rank=48, window=21, base=300.0, scale=0.2):
    out = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
           "rot": {"base": base, "dims": rot_dim}, "scale": scale}
    if window:
        out["mask"] = {"size": window}
    return out


def _layer(kind, mixer, ff=None, weights_of=None):
    out = {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}
    if weights_of is not None:
        out["weights_of"] = weights_of
    return out


def model(width, vocab, layers, eps=1e-5, scale=1.0):
    layers = copy.deepcopy(layers)
    for l in layers:                       # an entry that shares weights repeats the rest of the entry it names
        if "weights_of" in l:
            src = layers[l["weights_of"]]
            l["type"], l["mixer"], l["mlp"] = src["type"], copy.deepcopy(src["mixer"]), copy.deepcopy(src["mlp"])
    return {"architecture": "Gudutar", "vocab": vocab, "width": width, "embedding": {"scale": scale}, "norm": {"eps": eps},
            "layers": layers}


# Every mixer, feed-forwards on some layers, layers that run with another layer's weights, a window of 21 positions
# (not a multiple of a page), groups and norm parts other than 1, a partial rotation in the retention layer.
GUDU_A = model(96, 300, [
    _layer("mamba2", _mamba(), ff=160),
    _layer("retention", _retention()),
    _layer("latent_attention", _latent(), ff=72),
    _layer("mamba2", None, weights_of=0),
    _layer("latent_attention", None, weights_of=2),
    _layer("retention", None, weights_of=1),
], eps=1e-6, scale=3.3)

# Other sizes everywhere: more than 64 value channels and more than 64 state rows per head (several blocks and waves in
# the recurrence kernel), one group, two taps, a latent too wide for the paged attention kernels and without a window,
# a second latent layer with a window of one page exactly, a whole-head rotation in the retention layer.
GUDU_B = model(64, 131, [
    _layer("latent_attention", _latent(heads=2, dim=16, rot_dim=32, vdim=48, kv_rank=272, window=0, base=10000.0, scale=0.11)),
    _layer("mamba2", _mamba(heads=2, vdim=72, state=80, groups=1, conv=2, norm_groups=1)),
    _layer("retention", _retention(heads=2, dim=144, vdim=16, rot_dims=144, base=100.0, decay=(0.5, 0.999)), ff=96),
    _layer("latent_attention", _latent(heads=3, dim=8, rot_dim=4, vdim=8, kv_rank=40, window=16, base=50.0, scale=0.35), ff=40),
], eps=1e-4, scale=0.7)

# Sizes that fit no vector load and no tile: a width that is no multiple of 4, odd head sizes, three norm parts of ten
# channels, twelve state rows, a latent of 22 + 4 elements (padded to 32 in the pages), eight taps, a window of five.
GUDU_C = model(50, 77, [
    _layer("retention", _retention(heads=3, dim=10, vdim=6, rot_dims=6, base=33.0, decay=(0.6, 0.9, 0.99)), ff=34),
    _layer("mamba2", _mamba(heads=3, vdim=10, state=12, groups=1, conv=8, norm_groups=3)),
    _layer("latent_attention", _latent(heads=3, dim=6, rot_dim=4, vdim=10, kv_rank=22, window=5, base=7.0, scale=0.3)),
    _layer("mamba2", None, weights_of=1),
], eps=1e-3, scale=1.5)

# One mechanism alone, each in the smallest model that holds it.
ALONE = {
    "mamba2": model(48, 90, [_layer("mamba2", _mamba(heads=3, vdim=16, state=24, groups=3, conv=4, norm_groups=1))], scale=2.0),
    "mamba2_one_tap": model(48, 90, [_layer("mamba2", _mamba(heads=2, vdim=8, state=8, groups=1, conv=1, norm_groups=4))], scale=2.0),
    "mamba2_many_state_rows": model(48, 90, [_layer("mamba2", _mamba(heads=2, vdim=8, state=272, groups=2, conv=9, norm_groups=1))], scale=2.0),
    "retention": model(48, 90, [_layer("retention", _retention(heads=2, dim=16, vdim=24, rot_dims=8, decay=(0.8, 0.99)))], scale=2.0),
    "latent_attention": model(48, 90, [_layer("latent_attention", _latent(heads=4, dim=16, rot_dim=16, vdim=12, kv_rank=32, window=9))], scale=2.0),
    "latent_attention_full": model(48, 90, [_layer("latent_attention", _latent(heads=1, dim=8, rot_dim=2, vdim=8, kv_rank=16, window=0))], scale=2.0),
    "feed_forward": model(48, 90, [_layer("retention", _retention(heads=1, dim=8, vdim=8, rot_dims=2, decay=(0.9,)), ff=56)], scale=2.0),
}
