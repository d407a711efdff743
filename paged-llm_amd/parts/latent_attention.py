"""Causal attention whose keys and values are expanded from one cached latent vector per token.

One product gives every head's query [plain | rot] and the down-projection [rank | rot]; the first ``rank`` elements,
RMS-normed with a weight, are the latent c, the last ``rot`` one rotated key part that all heads share.  A head's key
is [W_uk c ; rotated part] and its value W_uv c, so only c and the rotated part are kept per token, in pages of their own
shapes.  The kernels never expand the cache: the query is carried into the latent space (qa = W_uk^T q_plain, one small
product per head), the softmax runs over (qa . c + q_rot . k_rot) * scale and weighs the latents themselves, and W_uv is
applied to the weighted latent of each head.  A window (the last ``window`` positions) makes the pages a windowed group.
"""

from __future__ import annotations

import torch

from ..csrc import ops
from .base import BLOCK, CacheSpec, Mixer, PageTensor
from .linear import Weight, linear
from .registry import BuildEnv, register_mixer
from .spec import PartSpec, WeightSpec


class LatentAttention(Mixer):
    """params: ``heads``, ``plain_dim``, ``rot_dim`` (per head), ``head_dim`` (of the values), ``rank``, ``scale``,
    ``window`` (0: none), ``position`` (the rotary spec of the rot part), ``eps`` (of the latent's norm).
    Tensors ``q`` [heads (plain + rot), width], ``dkv`` [rank + rot, width], ``dkv.norm`` [rank], ``uk`` [heads plain,
    rank], ``uv`` [heads head_dim, rank], ``o`` [width, heads head_dim]."""
    graph_capturable = True
    graph_capturable_prompts = True

    def __init__(self, params: dict, env: BuildEnv):
        self.hidden = env.hidden_size
        self.heads, self.plain, self.rot = int(params["heads"]), int(params["plain_dim"]), int(params["rot_dim"])
        self.P, self.rank = int(params["head_dim"]), int(params["rank"])
        self.scale, self.window, self.eps = float(params["scale"]), int(params.get("window") or 0), float(params["eps"])
        if self.rank > ops.MAX_LATENT_RANK or self.rot > ops.MAX_LATENT_ROT or self.rot % 2 or self.rot <= 0 or self.plain <= 0:
            raise ValueError(f"latent attention takes a rank up to {ops.MAX_LATENT_RANK}, an even rotated width up to "
                             f"{ops.MAX_LATENT_ROT} and a plain width of at least 1; got {self.rank}, {self.rot}, {self.plain}")
        pos = params["position"]
        self.position = env.position_encoding(PartSpec(**pos) if isinstance(pos, dict) else pos)
        if (self.position.rotary_dim or self.rot) != self.rot:
            raise ValueError(f"the rotated part of {self.rot} elements turns as a whole, not {self.position.rotary_dim} of it")
        self.dtype, self.device = env.dtype, env.device
        self._w: dict = {}
        self.w_in = self.w_o = self.w_uk_t = self.w_uv = self.norm_w = None

    def weight_specs(self):
        H = self.heads
        return {"q": WeightSpec((H * (self.plain + self.rot), self.hidden)), "dkv": WeightSpec((self.rank + self.rot, self.hidden)),
                "dkv.norm": WeightSpec((self.rank,), role="vector", init="ones"), "uk": WeightSpec((H * self.plain, self.rank)),
                "uv": WeightSpec((H * self.P, self.rank)), "o": WeightSpec((self.hidden, H * self.P))}

    def assign(self, name, tensor):
        spec = self.weight_specs().get(name)
        if spec is None:
            raise KeyError(name)
        self._w[name] = tensor.to(device=self.device, dtype=torch.float32 if spec.role == "vector" else self.dtype).contiguous()

    def finalize(self):
        w, H = self._w, self.heads
        self.w_in = Weight(torch.cat([w.pop("q"), w.pop("dkv")], dim=0).contiguous())
        self.w_o = Weight(w.pop("o"))
        self.w_uk_t = w.pop("uk").view(H, self.plain, self.rank).transpose(1, 2).contiguous()     # [heads, rank, plain]: qa = W_uk^T q
        self.w_uv = w.pop("uv").view(H, self.P, self.rank).contiguous()
        self.norm_w = w.pop("dkv.norm")

    def cache_spec(self):
        kind = "window" if self.window > 0 else "full"
        return CacheSpec(kind, (PageTensor("c", (BLOCK, self.rank)), PageTensor("kr", (BLOCK, self.rot))), self.window)

    def forward(self, h, ctx, cache, state):
        H, d, r = self.heads, self.plain, self.rot
        view = ctx.groups[cache.group]
        rows = linear(h, self.w_in)
        if not rows.is_contiguous():
            rows = rows.contiguous()
        pe = self.position
        ops.latent_prepare(rows, H * (d + r), ctx.positions, pe.cos, pe.sin, self.norm_w, self.eps,
                           view.slot_mapping if cache.writable else None, cache["c"], cache["kr"], H, d, r, self.rank, bool(pe.interleaved))
        qa = ops.gemm_heads(rows[:, :H * (d + r)].unflatten(1, (H, d + r))[:, :, :d], self.w_uk_t)
        mixed = ops.latent_attention(qa, rows, d, r, cache["c"], cache["kr"], view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k,
                                     self.scale, self.window)
        values = ops.gemm_heads(mixed, self.w_uv)
        return linear(values.view(values.shape[0], H * self.P), self.w_o,
                      out_dtype=torch.float32 if getattr(ctx, "float_branch", False) else None)


register_mixer("latent_attention", LatentAttention)
