"""A plain, slow Gudutar: whole sequences, token by token where the design is recurrent, no cache, no
paging, no batches, one function per mechanism.

Gudutar is a decoder whose layers each hold one of three mixers (a Mamba-2 state-space layer, a retention
layer, an attention layer over a compressed key/value latent with a sliding window) and optionally a dense
gated feed-forward.  A sublayer reads the residual stream x itself and its output passes a layer norm before
it is added:  x <- x + LN(mixer(x)),  x <- x + LN(ff(x)).

Everything is computed in one floating type chosen by the caller (float32 by default; float64 to judge
which of two float32 results is closer).  It shares no code with the engine under ``paged-llm_amd/`` and
reads ``config.json`` and the safetensors file on its own.
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


def product(x, w):
    """x W^T; with ``_NOISE`` set, rows and result are disturbed as a 16-bit compute type would round them."""
    if _NOISE is None:
        return x @ w.T
    return _NOISE(_NOISE(x) @ w.T)


class rounding_noise:
    """Inside ``with rounding_noise(seed):`` every product's rows and result are multiplied by 1 + u * 2^-8 with u uniform
    in (-1, 1), drawn from ``seed``: the relative error of two roundings to bfloat16, at random (an engine that computes
    in bfloat16 rounds the rows, the result, and what it computes element by element between two products).  Several
    seeds show how far the logits of one position move under the compute type's rounding alone; the state, the norms and
    everything else that the design keeps in 32 bits stay exact."""

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


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    """log(1 + e^z) without overflow."""
    return torch.where(z > 20.0, z, torch.log1p(torch.exp(torch.clamp(z, max=20.0))))


def unit_rms(x, eps):
    """x divided by its root mean square over the last dimension, eps inside the root."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mean = x.mean(dim=-1, keepdim=True)
    dev = x - mean
    var = (dev * dev).mean(dim=-1, keepdim=True)
    return dev / torch.sqrt(var + eps) * w + b


def rotate(vec, positions, base: float, dims: int, interleaved: bool):
    """Turns the first ``dims`` elements of the last dimension of ``vec`` [L, ..., d] by the angle
    position * base^(-2i/dims) of pair i: (u, v) -> (u cos - v sin, v cos + u sin).  The partners are
    (i, i + dims/2), or (2i, 2i + 1) when ``interleaved``."""
    half = dims // 2
    i = torch.arange(half, dtype=torch.float64)
    freq = (float(base) ** (-2.0 * i / dims)).to(vec.dtype)
    ang = positions.to(vec.dtype)[:, None] * freq[None, :]             # [L, half]
    shape = [vec.shape[0]] + [1] * (vec.dim() - 2) + [half]
    cos, sin = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    out = vec.clone()
    if interleaved:
        u, v = vec[..., 0:dims:2], vec[..., 1:dims:2]
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
    else:
        u, v = vec[..., :half], vec[..., half:dims]
        out[..., :half] = u * cos - v * sin
        out[..., half:dims] = v * cos + u * sin
    return out


# --------------------------------------------------------------------------- mixers
def mamba2_mixer(h, w: dict, m: dict, eps: float):
    """h [L, width] -> [L, width].  ``w``: the mixer's tensors by their short names, ``m``: its sizes."""
    L = h.shape[0]
    H, P, N, G, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = H * P
    proj = product(h, w["in"])
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    # causal convolution per channel: the last column of the filter meets the current token
    padded = torch.cat([torch.zeros(taps - 1, xbc.shape[1], dtype=h.dtype), xbc], dim=0)
    conv = torch.zeros_like(xbc)
    for j in range(taps):
        conv = conv + padded[j:j + L] * w["conv"][:, j]
    xbc = silu(conv + w["conv.b"])
    x = xbc[:, :inner].reshape(L, H, P)
    B = xbc[:, inner:inner + G * N].reshape(L, G, N)
    C = xbc[:, inner + G * N:].reshape(L, G, N)
    dt = softplus(dt + w["dt_bias"])                                   # [L, H]
    decay = torch.exp(-torch.exp(w["A_log"]) * dt)                      # [L, H]
    per_group = H // G
    S = torch.zeros(H, N, P, dtype=h.dtype)
    y = torch.zeros(L, H, P, dtype=h.dtype)
    for t in range(L):
        for a in range(H):
            g = a // per_group
            S[a] = decay[t, a] * S[a] + dt[t, a] * torch.outer(B[t, g], x[t, a])
            y[t, a] = S[a].T @ C[t, g] + w["D"][a] * x[t, a]
    y = y.reshape(L, inner) * silu(z)
    parts = m["norm_groups"]
    y = unit_rms(y.reshape(L, parts, inner // parts), eps).reshape(L, inner) * w["norm"]
    return product(y, w["o"])


def retention_mixer(h, w: dict, m: dict, eps: float):
    L = h.shape[0]
    H, d, P = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(L)
    q = product(h, w["q"]).reshape(L, H, d)
    k = product(h, w["k"]).reshape(L, H, d)
    v = product(h, w["v"]).reshape(L, H, P)
    q = rotate(q, pos, m["rot"]["base"], m["rot"]["dims"], interleaved=False)
    k = rotate(k, pos, m["rot"]["base"], m["rot"]["dims"], interleaved=False) * d ** -0.5
    S = torch.zeros(H, d, P, dtype=h.dtype)
    o = torch.zeros(L, H, P, dtype=h.dtype)
    for t in range(L):
        for a in range(H):
            S[a] = float(m["decay"][a]) * S[a] + torch.outer(k[t, a], v[t, a])
            o[t, a] = S[a].T @ q[t, a]
    o = unit_rms(o, eps).reshape(L, H * P)
    return product(o * silu(product(h, w["g"])), w["o"])


def latent_attention_mixer(h, w: dict, m: dict, eps: float):
    L = h.shape[0]
    H, d, r, P, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(L)
    q = product(h, w["q"]).reshape(L, H, d + r)
    q_plain, q_rot = q[..., :d], q[..., d:]
    down = product(h, w["dkv"])
    c = unit_rms(down[:, :rank], eps) * w["dkv.norm"]
    k_rot = down[:, rank:]                                              # [L, r], one for all heads
    base, dims = m["rot"]["base"], m["rot"]["dims"]
    q_rot = rotate(q_rot, pos, base, dims, interleaved=True)
    k_rot = rotate(k_rot, pos, base, dims, interleaved=True)
    k_plain = product(c, w["uk"]).reshape(L, H, d)
    v = product(c, w["uv"]).reshape(L, H, P)
    i_idx, j_idx = pos[:, None], pos[None, :]
    hidden = j_idx > i_idx
    if m.get("mask"):                                                   # a sliding window: query i sees 0 <= i - j < size
        hidden = hidden | (i_idx - j_idx >= m["mask"]["size"])
    out = torch.zeros(L, H, P, dtype=h.dtype)
    for a in range(H):
        s = (q_plain[:, a] @ k_plain[:, a].T + q_rot[:, a] @ k_rot.T) * m["scale"]
        s = s.masked_fill(hidden, float("-inf"))
        out[:, a] = torch.softmax(s, dim=-1) @ v[:, a]
    return product(out.reshape(L, H * P), w["o"])


def dense_ff(h, w: dict):
    return product(gelu_tanh(product(h, w["gate"])) * product(h, w["up"]), w["down"])


MIXERS = {"mamba2": mamba2_mixer, "retention": retention_mixer, "latent_attention": latent_attention_mixer}


# --------------------------------------------------------------------------- the model
def forward(cfg: dict, weights: dict, tokens: list, dtype=torch.float32, layers_out: list | None = None):
    """Logits [L, vocab] of one whole sequence.  ``layers_out``: a list that receives the residual stream
    after every layer run."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        src = layer.get("weights_of", i)
        pre = f"l{src}."
        mix = {k[len(pre) + 4:]: v for k, v in W.items() if k.startswith(pre + "mix.")}
        a = MIXERS[layer["type"]](x, mix, layer["mixer"], eps)
        x = x + layer_norm(a, W[pre + "norm1"], W[pre + "norm1.b"], eps)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            ff = {k[len(pre) + 4:]: v for k, v in W.items() if k.startswith(pre + "mlp.")}
            x = x + layer_norm(dense_ff(x, ff), W[pre + "norm2"], W[pre + "norm2.b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = layer_norm(x, W["final.norm"], W["final.norm.b"], eps)
    return product(x, W["head"])
