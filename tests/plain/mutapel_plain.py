"""A plain, slow Mutapel: whole sequences, no cache, no paging, no batches, one function per mechanism.

Mutapel is a decoder with two kinds of attention layers and a routed mixture of small gated feed-forwards.  A layer
norms what a sublayer reads and what it returns (RMS norms whose weights are stored as w - 1) and adds the result times
a constant m:   x <- x + m * N1b(mixer(N1(x))),   x <- x + m * N2b(ff(N2(x))).   A range of layers may run several times
in a row with the same weights; in front of every such pass the stream is mixed with the embedding output x0 by one
product, x <- W_in [x ; x0].

* ``attention``: q, k, v with biases, a short causal convolution over time on every channel of q, k and v, rotary
  angles on pairs (i, i + r/2), q and k of every head divided by their root mean square, keys visible inside the
  query's own block of ``mask.size`` positions only, a learned logit per head in the softmax's denominator, an output
  product with a bias.
* ``attention_2``: no biases, pairs (2i, 2i + 1), the same division, a sliding window of ``mask.size`` positions, and
  each head's output times the sigmoid of one number that a product of the mixer's input gives for that head.

Everything is computed in one floating type chosen by the caller (float32 by default; float64 to judge which of two
float32 results is closer).  It shares no code with the engine under ``paged-llm_amd/`` and reads ``config.json`` and
the safetensors file on its own.
"""

from __future__ import annotations

import json
import math
import os

import torch


def read_config(model_dir: str) -> dict:
    with open(os.path.join(model_dir, "config.json")) as f:
        return json.load(f)


def load_weights(model_dir: str) -> dict:
    from safetensors import safe_open
    out = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt", device="cpu") as f:
        for name in f.keys():
            out[name] = f.get_tensor(name)
    return out


# --------------------------------------------------------------------------- small pieces
_NOISE = None      # a function applied to every product's operand rows and result (see ``rounding_noise``), or None


def product(x, w, b=None):
    """x W^T (+ b); with ``_NOISE`` set, rows and result are disturbed as a 16-bit compute type would round them."""
    if _NOISE is None:
        y = x @ w.T
        return y if b is None else y + b
    y = _NOISE(x) @ w.T
    return _NOISE(y if b is None else y + b)


class rounding_noise:
    """Inside ``with rounding_noise(seed):`` every product's rows and result are multiplied by 1 + u * 2^-8 with u uniform
    in (-1, 1), drawn from ``seed``: the relative error of two roundings to bfloat16, at random.  Several seeds show how
    far the logits of one position move under the compute type's rounding alone; norms, scores, the router and the
    residual stream stay exact, as the design keeps them in 32 bits."""

    def __init__(self, seed: int, amplitude: float = 2.0 ** -8):
        self.gen = torch.Generator().manual_seed(seed)
        self.amplitude = amplitude

    def __call__(self, t):
        return t * (1.0 + (torch.rand(t.shape, generator=self.gen, dtype=t.dtype) * 2.0 - 1.0) * self.amplitude)

    def __enter__(self):
        global _NOISE
        _NOISE = self
        return self

    def __exit__(self, *exc):
        global _NOISE
        _NOISE = None


def root_mean_square_norm(x, eps, stored_weight=None):
    """x / sqrt(mean(x^2) + eps) over the last dimension, times (1 + stored weight) when there is one."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if stored_weight is None else y * (1.0 + stored_weight)


def silu(z):
    return z * torch.sigmoid(z)


def time_convolution(u, taps_weight):
    """y_t = sum_j w[:, j] u_(t - taps + 1 + j) per channel, zeros in front of the sequence.  u [T, C], w [C, taps]."""
    T, C = u.shape
    taps = taps_weight.shape[1]
    padded = torch.cat([u.new_zeros((taps - 1, C)), u], dim=0)
    y = u.new_zeros((T, C))
    for j in range(taps):
        y = y + padded[j:j + T] * taps_weight[:, j]
    return y


def rotate(x, positions, base, dims, interleaved):
    """x [T, heads, d]: the first ``dims`` elements of every head turn in pairs by the angle p * base^(-2i/dims):
    pairs (i, i + dims/2), or (2i, 2i + 1) when ``interleaved``.  Angles in float32, as positions times frequencies."""
    if dims == 0:
        return x
    half = dims // 2
    freq = torch.tensor([float(base) ** (-2.0 * i / dims) for i in range(half)], dtype=torch.float32)
    angle = (positions.to(torch.float32)[:, None] * freq[None, :]).to(x.dtype)           # [T, half]
    c, s = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    out = x.clone()
    if interleaved:
        a, b = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = a * c - b * s
        out[..., 1:dims:2] = b * c + a * s
    else:
        a, b = x[..., :half], x[..., half:dims]
        out[..., :half] = a * c - b * s
        out[..., half:dims] = b * c + a * s
    return out


def visible(i, j, kind, size):
    """Whether the query at position i sees the key at position j."""
    if j > i:
        return False
    if kind == "block":
        return i // size == j // size
    if kind == "window":
        return i - j < size
    return True


def softmax_attention(q, k, v, positions, scale, kind, size, sink=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv] of one sequence -> [T, H, dv].  ``sink`` [H]: a logit per head that stands
    in the denominator only."""
    T, H, d = q.shape
    G = k.shape[1]
    per = H // G
    mask = torch.tensor([[visible(int(positions[a]), int(positions[b]), kind, size) for b in range(T)] for a in range(T)])
    out = q.new_zeros((T, H, v.shape[2]))
    for h in range(H):
        g = h // per
        s = (q[:, h] @ k[:, g].T) * scale
        s = s.masked_fill(~mask, float("-inf"))
        top = s.max(dim=1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].expand_as(top))
        e = torch.exp(s - top)
        denom = e.sum(dim=1, keepdim=True)
        if sink is not None:
            denom = denom + torch.exp(sink[h] - top)
        out[:, h] = (e / denom) @ v[:, g]
    return out


# --------------------------------------------------------------------------- mixers
def attention_mixer(h, W, prefix, m, kind, eps, dtype):
    """Either attention layer on the normed rows h [T, width] of one sequence from position 0."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    w = lambda n: W[f"{prefix}.{n}"].to(dtype)
    positions = torch.arange(T)
    if kind == "attention":
        q, k, v = (product(h, w(n), w(n + ".b")) for n in ("q", "k", "v"))
        q, k, v = (time_convolution(t, w(n + ".conv")) for t, n in ((q, "q"), (k, "k"), (v, "v")))
    else:
        q, k, v = (product(h, w(n)) for n in ("q", "k", "v"))
    q, k, v = q.view(T, H, d), k.view(T, G, d), v.view(T, G, dv)
    rot = m["rot"]
    q = rotate(q, positions, rot["base"], int(rot["dims"]), kind == "attention_2")
    k = rotate(k, positions, rot["base"], int(rot["dims"]), kind == "attention_2")
    q, k = root_mean_square_norm(q, eps), root_mean_square_norm(k, eps)
    size = int(m["mask"]["size"])
    if kind == "attention":
        o = softmax_attention(q, k, v, positions, float(m["scale"]), "block", size, sink=w("sink"))
        return product(o.reshape(T, H * dv), w("o"), w("o.b"))
    o = softmax_attention(q, k, v, positions, float(m["scale"]), "window", size)
    gate = torch.sigmoid(product(h, w("g")))                       # [T, H]
    return product((o * gate[:, :, None]).reshape(T, H * dv), w("o"))


def route(h, router_weight, correction, r):
    """(chosen [T, top] expert numbers, weights [T, top]).  Scores are the softmax of the router's outputs over plain
    and pass-through experts together; the choice looks at score + correction, only inside the best ``keep`` of
    ``count`` groups of neighbours (a group's mark is its largest corrected score); the weights are the uncorrected
    scores of the chosen, as they are."""
    z = h.to(torch.float32) @ router_weight.to(torch.float32).T if h.dtype != torch.float64 else h @ router_weight.to(h.dtype).T
    s = torch.softmax(z, dim=-1)
    choice = s + correction.to(s.dtype)
    n = choice.shape[1]
    count, keep = int(r["groups"]["count"]), int(r["groups"]["keep"])
    per = n // count
    marks = choice.view(-1, count, per).max(dim=2).values
    best = torch.topk(marks, keep, dim=1).indices
    allowed = torch.zeros_like(marks, dtype=torch.bool).scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(-1, count, per).reshape(-1, n)
    limited = choice.masked_fill(~allowed, float("-inf"))
    chosen = torch.topk(limited, int(r["top"]), dim=1).indices
    return chosen, torch.gather(s, 1, chosen)


def routed_experts(h, W, prefix, mlp, dtype):
    """sum over the chosen experts of weight * expert(h); an expert is down(silu(gate h) * (up h)), and the last
    ``identity`` router outputs stand for experts that hand h back."""
    r = mlp["router"]
    experts = int(r["experts"])
    chosen, weights = route(h, W[f"{prefix}.router"], W[f"{prefix}.correction"], r)
    weights = weights.to(dtype)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, wt in zip(chosen[t].tolist(), weights[t]):
            if e >= experts:
                out[t] = out[t] + wt * h[t]
                continue
            p = f"{prefix}.e{e}"
            a = silu(product(h[t:t + 1], W[p + ".gate"].to(dtype))) * product(h[t:t + 1], W[p + ".up"].to(dtype))
            out[t] = out[t] + wt * product(a, W[p + ".down"].to(dtype))[0]
    return out


# --------------------------------------------------------------------------- the model
def run_order(cfg):
    """[(layer, first of a repeated pass?)] in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    order = [(i, False) for i in range(start)]
    for _ in range(times):
        order += [(i, i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward(cfg, W, tokens, dtype=torch.float32, want_layers=False):
    """Logits [T, vocab] of one sequence from position 0 (and the stream after every layer run, when asked)."""
    eps, mult = float(cfg["norm"]["eps"]), float(cfg["residual_mult"])
    x0 = W["embed"].to(dtype)[torch.as_tensor(tokens, dtype=torch.long)]
    x = x0
    streams = []
    for i, enters_pass in run_order(cfg):
        layer, p = cfg["layers"][i], f"l{i}"
        if enters_pass:
            x = product(torch.cat([x, x0], dim=1), W["loop.in"].to(dtype))
        h = root_mean_square_norm(x, eps, W[p + ".norm1"].to(dtype))
        a = attention_mixer(h, W, p + ".mix", layer["mixer"], layer["type"], eps, dtype)
        x = x + mult * root_mean_square_norm(a, eps, W[p + ".norm1b"].to(dtype))
        if layer.get("mlp") is not None:
            h = root_mean_square_norm(x, eps, W[p + ".norm2"].to(dtype))
            f = routed_experts(h, W, p + ".mlp", layer["mlp"], dtype)
            x = x + mult * root_mean_square_norm(f, eps, W[p + ".norm2b"].to(dtype))
        streams.append(x)
    logits = product(root_mean_square_norm(x, eps, W["final.norm"].to(dtype)), W["head"].to(dtype))
    return (logits, torch.stack(streams)) if want_layers else logits
