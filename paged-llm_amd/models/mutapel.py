"""Mutapel: a decoder of two kinds of attention layers over a residual stream kept in float, each layer with a routed
mixture of small gated feed-forwards.  Norms stand in front of and behind every sublayer (RMS norms whose weights are
stored as w - 1) and a sublayer's normed output enters the stream times a constant:

    x <- x + m * norm1b(mixer(norm1(x)));   x <- x + m * norm2b(ff(norm2(x))).

A range of layers may run several times in a row with the same weights (a cache and state of its own per pass); in front
of every pass the stream is mixed with the embedding's output by one product, x <- W_in [x ; x0].

* ``attention``: q/k/v with biases, a short causal convolution over time on their channels, rotary pairs (i, i + r/2),
  q and k divided by their root mean square per head, keys visible inside the query's own block of ``mask.size``
  positions, a learned logit per head in the softmax's denominator, an output product with a bias.
* ``attention_2``: no biases, rotary pairs (2i, 2i + 1), the same division, a sliding window of ``mask.size``
  positions, every head's output times the sigmoid of a gate that one more product of the mixer's input gives.

``config.json``: ``architecture`` "Mutapel", ``vocab``, ``width``, ``norm.eps``, ``residual_mult``, ``layers`` (a list of
{``type``, ``mixer``, ``mlp`` or null}) and optionally ``loop`` {``start``, ``stop``, ``times``}.  Layer i's tensors are
``l<i>.norm1``, ``l<i>.norm1b``, ``l<i>.norm2``, ``l<i>.norm2b``, ``l<i>.mix.*``, ``l<i>.mlp.*``; outside the layers
``embed``, ``loop.in``, ``final.norm`` and ``head``.  Importing this module registers the architecture."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleStep, StreamOpSpec

MIXER_TYPES = ("attention", "attention_2")


@dataclass
class MutapelLayer:
    type: str
    mixer: dict
    mlp: dict | None


@dataclass
class MutapelConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: list = field(default_factory=list)
    loop: dict | None = None                 # {"start", "stop", "times"}
    max_positions: int = 4096
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_json(cls, cfg: dict) -> "MutapelConfig":
        layers = [MutapelLayer(str(l["type"]), dict(l["mixer"]), (dict(l["mlp"]) if l.get("mlp") is not None else None)) for l in cfg["layers"]]
        loop = cfg.get("loop")
        out = cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), norm_eps=float(cfg["norm"]["eps"]),
                  residual_mult=float(cfg.get("residual_mult", 1.0)), layers=layers,
                  loop={k: int(loop[k]) for k in ("start", "stop", "times")} if loop else None,
                  max_positions=int(cfg.get("max_positions", 4096)), torch_dtype=str(cfg.get("torch_dtype") or "bfloat16"))
        out.validate()
        return out

    def validate(self) -> None:
        problems = []
        if self.vocab <= 0 or self.width <= 0 or not self.layers:
            problems.append("vocab, width and the number of layers must be positive")
        for i, l in enumerate(self.layers):
            if l.type not in MIXER_TYPES:
                problems.append(f"layer {i}: mixer type {l.type!r} is none of {MIXER_TYPES}")
            if l.mlp is not None and l.mlp.get("kind") != "moe":
                problems.append(f"layer {i}: feed-forward kind {l.mlp.get('kind')!r} (moe only)")
        if self.loop is not None and not (0 <= self.loop["start"] < self.loop["stop"] <= len(self.layers) and self.loop["times"] >= 1):
            problems.append(f"loop {self.loop}: 0 <= start < stop <= {len(self.layers)} layers, times >= 1")
        if problems:
            raise ValueError("bad Mutapel config: " + "; ".join(problems))

    def run_order(self) -> list:
        """[(layer, whether a pass of the repeated range starts here)] in the order the layers run."""
        n = len(self.layers)
        if self.loop is None:
            return [(i, False) for i in range(n)]
        start, stop, times = self.loop["start"], self.loop["stop"], self.loop["times"]
        order = [(i, False) for i in range(start)]
        for _ in range(times):
            order += [(i, i == start) for i in range(start, stop)]
        return order + [(i, False) for i in range(stop, n)]


def _mixer_spec(kind: str, m: dict, eps: float) -> PartSpec:
    first = kind == "attention"
    rot = m.get("rot")
    position = None
    if rot and int(rot["dims"]) > 0:
        position = {"kind": "rotary", "params": {"head_dim": int(m["dim"]), "theta": float(rot["base"]), "rotary_dim": int(rot["dims"]),
                                                 "interleaved": not first, "scaling": None}}
    size = int((m.get("mask") or {}).get("size") or 0)
    return PartSpec("normed_attention", {
        "heads": int(m["heads"]), "kv_heads": int(m["kv_heads"]), "key_dim": int(m["dim"]), "value_dim": int(m["vdim"]),
        "scale": float(m["scale"]), "eps": eps, "position": position,
        "mask": ("chunk" if first else "window") if size > 0 else "full", "mask_size": size,
        "conv": int(m.get("conv") or 0) if first else 0, "bias": first, "sinks": first, "head_gate": not first})


def _mlp_spec(mlp: dict) -> PartSpec:
    r = mlp["router"]
    groups = r.get("groups") or {}
    return PartSpec("routed_experts", {"experts": int(r["experts"]), "identity": int(r.get("identity") or 0), "top": int(r["top"]),
                                       "groups": int(groups.get("count") or 1), "keep": int(groups.get("keep") or 1),
                                       "intermediate_size": int(mlp["expert"]["ff"]), "activation": "silu", "correction": True})


def build_spec(cfg: MutapelConfig) -> ModelSpec:
    eps = cfg.norm_eps
    norm = PartSpec("rmsnorm", {"eps": eps, "weight_name": "", "unit_offset": True})
    layers = []
    for i, l in enumerate(cfg.layers):
        parts = {"mixer_norm": norm, "mixer": _mixer_spec(l.type, l.mixer, eps), "mixer_out_norm": norm}
        names = {"mixer_norm": "norm1", "mixer": "mix", "mixer_out_norm": "norm1b", "feed_forward": l.mlp is not None,
                 "residual_mult": cfg.residual_mult}
        if l.mlp is not None:
            parts.update({"feed_forward_norm": norm, "feed_forward": _mlp_spec(l.mlp), "feed_forward_out_norm": norm})
            names.update({"feed_forward_norm": "norm2", "feed_forward": "mlp", "feed_forward_out_norm": "norm2b"})
        layers.append(LayerSpec(f"l{i}", PartSpec("sandwich_norm", names), parts))
    stream_ops = [StreamOpSpec("loop.in", PartSpec("concat_projection", {"tensor_name": ""}))] if cfg.loop is not None else []
    schedule = [ScheduleStep(i, entry=0 if enters else None) for i, enters in cfg.run_order()]
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "float_stream": True, "tensor_name": ""}),
        layers=layers, final_norm=norm, head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "tied": False, "tensor_name": ""}),
        schedule=schedule, stream_ops=stream_ops, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_id=None, stored_dtype=cfg.torch_dtype)


register_architecture(Architecture("Mutapel", MutapelConfig.from_json, build_spec))
