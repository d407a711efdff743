"""Small Mutapel configurations for the tests: sizes, layer orders and constants that differ from one another in every
field, and single-layer ones that show one mechanism alone."""

import copy


def _blocks(heads=4, kv_heads=2, dim=24, vdim=40, conv=4, size=21, rot_dims=16, base=1e4, scale=0.3):
    """The attention layer with biases, a convolution over time, blocks of ``size`` positions and sinks."""
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "conv": conv, "mask": {"size": size},
            "rot": {"base": base, "dims": rot_dims}, "scale": scale}


def _window(heads=6, kv_heads=3, dim=32, vdim=16, size=19, rot_dims=32, base=500.0, scale=0.2):
    """The attention layer with a sliding window and a gate per head."""
    return {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": size},
            "rot": {"base": base, "dims": rot_dims}, "scale": scale}


def _moe(experts=6, identity=2, top=3, count=4, keep=2, ff=40):
    return {"kind": "moe", "expert": {"ff": ff},
            "router": {"experts": experts, "identity": identity, "top": top, "groups": {"count": count, "keep": keep}}}


def _layer(kind, mixer, mlp=None):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


def model(width, vocab, layers, loop=None, eps=1e-5, mult=0.5):
    out = {"architecture": "Mutapel", "vocab": vocab, "width": width, "norm": {"eps": eps}, "residual_mult": mult,
           "layers": copy.deepcopy(layers)}
    if loop is not None:
        out["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return out


# Both mixers, key and value sizes that differ either way, a partial rotation, groups of heads on a key head, a window and
# a block size that are no multiples of a page, a layer without a feed-forward, two layers that run three times, a layer
# behind the repeated ones.
MUTA_A = model(96, 300, [
    _layer("attention_2", _window(), _moe()),
    _layer("attention", _blocks(), _moe(experts=5, identity=1, top=2, count=3, keep=2, ff=24)),
    _layer("attention_2", _window(heads=2, kv_heads=1, dim=16, vdim=48, size=33, rot_dims=8, base=77.0, scale=0.4)),
    _layer("attention", _blocks(heads=3, kv_heads=3, dim=48, vdim=16, conv=2, size=50, rot_dims=48, base=3e5, scale=0.1), _moe(top=1)),
], loop=(1, 3, 3), eps=1e-6, mult=0.5)

# No repeated layers; as many key heads as heads; no pass-through experts, one group, one chosen expert; a block and a
# window of exactly one page; head sizes that fit no tile; a width that is no multiple of 4; one tap.
MUTA_B = model(50, 77, [
    _layer("attention", _blocks(heads=3, kv_heads=3, dim=10, vdim=6, conv=1, size=16, rot_dims=6, base=33.0, scale=0.5),
           _moe(experts=3, identity=0, top=1, count=1, keep=1, ff=34)),
    _layer("attention_2", _window(heads=5, kv_heads=1, dim=6, vdim=10, size=16, rot_dims=2, base=7.0, scale=0.6),
           _moe(experts=4, identity=4, top=4, count=2, keep=1, ff=10)),
    _layer("attention", _blocks(heads=2, kv_heads=1, dim=20, vdim=20, conv=7, size=5, rot_dims=20, base=1e6, scale=0.25),
           _moe(experts=7, identity=1, top=8, count=8, keep=8, ff=65)),
], eps=1e-3, mult=1.0)

# Every layer repeated (twice), a window and blocks of one position (a query sees itself alone), eight taps, head sizes
# beyond 64 and 128, every expert chosen.
MUTA_C = model(64, 131, [
    _layer("attention", _blocks(heads=2, kv_heads=1, dim=80, vdim=144, conv=8, size=1, rot_dims=40, base=100.0, scale=0.11),
           _moe(experts=2, identity=2, top=4, count=1, keep=1, ff=16)),
    _layer("attention_2", _window(heads=4, kv_heads=2, dim=16, vdim=16, size=1, rot_dims=16, base=50.0, scale=0.35), _moe(ff=72)),
    _layer("attention_2", _window(heads=1, kv_heads=1, dim=160, vdim=32, size=70, rot_dims=64, base=1e4, scale=0.09), None),
], loop=(0, 3, 2), eps=1e-4, mult=0.3)

# One mechanism alone, each in the smallest model that holds it.
ALONE = {
    "blocks": model(48, 90, [_layer("attention", _blocks(heads=4, kv_heads=2, dim=16, vdim=16, conv=3, size=9, rot_dims=16))]),
    "blocks_no_rotation": model(48, 90, [_layer("attention", _blocks(heads=1, kv_heads=1, dim=8, vdim=24, conv=2, size=40, rot_dims=0))]),
    "window": model(48, 90, [_layer("attention_2", _window(heads=4, kv_heads=1, dim=16, vdim=16, size=9, rot_dims=16))]),
    "window_wide_values": model(48, 90, [_layer("attention_2", _window(heads=2, kv_heads=2, dim=8, vdim=40, size=30, rot_dims=4))]),
    "experts": model(48, 90, [_layer("attention_2", _window(heads=1, kv_heads=1, dim=8, vdim=8, size=4, rot_dims=2),
                                     _moe(experts=9, identity=3, top=3, count=4, keep=2, ff=56))]),
    "repeated": model(48, 90, [_layer("attention_2", _window(heads=2, kv_heads=1, dim=8, vdim=8, size=12, rot_dims=8))], loop=(0, 1, 4)),
}
