"""Causal attention whose keys and values are expanded from one cached latent vector per token.

One product gives every head's query [plain | rot] and the down-projection [rank | rot]; the first ``rank`` elements,
RMS-normed with a weight, are the latent c, the last ``rot`` one rotated key part that all heads share.  A head's key
is [W_uk c ; rotated part] and its value W_uv c, so only c and the rotated part are kept per token.  The kernels never
expand the cache: the query is carried into the latent space (qa = W_uk^T q_plain, one small product per head), the
softmax runs over (qa . c + q_rot . k_rot) * scale and weighs the latents themselves, and W_uv is applied to the weighted
latent of each head.  That is attention with ONE key/value head shared by all query heads, key row [c | rotated part],
value c: the pages hold the key rows (padded to a multiple of 16 elements) and, transposed inside the page, the latents
once more as values, in the layouts of ``paged_attention``, whose kernels (the matrix-core ones in bfloat16, the plain one
in float32) then serve this mixer as they serve the grouped-head attention.  Latents wider than those kernels take keep
the key rows alone and use a plain kernel of this mixer.  A window (the last ``window`` positions) makes the pages a
windowed group.
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
        self.width = -(-(self.rank + self.rot) // 16) * 16            # of a key row in the pages
        self.paged = self.width <= ops.MAX_HEAD_DIM_GENERIC           # the paged attention kernels take it
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
        tensors = (PageTensor("k", (1, BLOCK, self.width)),) + ((PageTensor("v", (1, self.width, BLOCK)),) if self.paged else ())
        return CacheSpec(kind, tensors, self.window)

    def graph_step_arrays(self, layout):
        """The prompt kernel's work list of the paged attention (all heads are one group) for a replayed step."""
        if not self.paged:
            return {}
        first, group = layout.num_single_rows, self.heads
        pairs = ops.prompt_tiles_capacity(layout.num_portions, layout.portion_tokens, group)
        return {("prompt_tiles", first, group): (2 * pairs, lambda q_lens, k_lens: ops.prompt_tiles(q_lens, k_lens, first, group, pairs))}

    def forward(self, h, ctx, cache, state):
        H, d, r, rank, width = self.heads, self.plain, self.rot, self.rank, self.width
        view = ctx.groups[cache.group]
        rows = linear(h, self.w_in)
        T = rows.shape[0]
        pe = self.position
        k_pages, v_pages = cache["k"], (cache["v"] if self.paged else None)
        q = torch.empty((T, H, width), dtype=rows.dtype, device=rows.device)
        ops.latent_prepare(rows, H * (d + r), ctx.positions, pe.cos, pe.sin, self.norm_w, self.eps,
                           view.slot_mapping if cache.writable else None, k_pages, v_pages, q, H, d, r, rank, bool(pe.interleaved))
        ops.gemm_heads(rows[:, :H * (d + r)].unflatten(1, (H, d + r))[:, :, :d], self.w_uk_t, out=q[:, :, :rank])
        if self.paged:
            mixed = ops.paged_attention(q.view(T, H * width), k_pages, v_pages, view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k,
                                        H, 1, width, self.scale, self.window, ctx).view(T, H, width)[:, :, :rank]
        else:
            mixed = ops.latent_attention(q, rank, r, k_pages, view.block_tables, ctx.cu_seqlens_q, ctx.seq_lens_k, self.scale, self.window)
        values = ops.gemm_heads(mixed, self.w_uv)
        return linear(values.view(T, H * self.P), self.w_o, out_dtype=torch.float32 if getattr(ctx, "float_branch", False) else None)


register_mixer("latent_attention", LatentAttention)
