"""Gudutar: a decoder whose layers each hold one of three mixers (a Mamba-2 state-space layer, a retention layer, an
attention layer over a compressed key/value latent with a sliding window) and, some of them, a dense gated feed-forward
(tanh-form GELU).  A sublayer reads the residual stream itself and a layer norm (weight and bias) stands behind it:
x <- x + LN(mixer(x)), x <- x + LN(ff(x)); the stream is kept in float.  The embedding is scaled; a layer may run with
another layer's weights (``weights_of``) and a cache or state of its own.

``config.json``: ``architecture`` "Gudutar", ``vocab``, ``width``, ``embedding.scale``, ``norm.eps`` and ``layers``, a list
of {``type``, ``mixer`` (the mixer's sizes), ``mlp`` ({``kind``: "dense", ``ff``} or null), optionally ``weights_of``}.
Layer i's tensors are ``l<i>.norm1[.b]``, ``l<i>.mix.*``, ``l<i>.norm2[.b]``, ``l<i>.mlp.{gate,up,down}``; outside the
layers ``embed``, ``final.norm[.b]`` and ``head``.  Importing this module registers the architecture."""

from __future__ import annotations

from dataclasses import dataclass, field

from ..config.registry import Architecture, register_architecture
from ..parts.spec import LayerSpec, ModelSpec, PartSpec, ScheduleStep

MIXER_TYPES = ("mamba2", "retention", "latent_attention")


@dataclass
class GudutarLayer:
    type: str
    mixer: dict
    mlp: dict | None
    weights_of: int | None = None


@dataclass
class GudutarConfig:
    vocab: int
    width: int
    embedding_scale: float
    norm_eps: float
    layers: list = field(default_factory=list)
    max_positions: int = 4096
    torch_dtype: str = "bfloat16"

    @classmethod
    def from_json(cls, cfg: dict) -> "GudutarConfig":
        layers = [GudutarLayer(str(l["type"]), dict(l["mixer"]), (dict(l["mlp"]) if l.get("mlp") is not None else None),
                               (int(l["weights_of"]) if l.get("weights_of") is not None else None)) for l in cfg["layers"]]
        out = cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), embedding_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                  norm_eps=float(cfg["norm"]["eps"]), layers=layers,
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
            if l.mlp is not None and l.mlp.get("kind") != "dense":
                problems.append(f"layer {i}: feed-forward kind {l.mlp.get('kind')!r} (dense only)")
            if l.weights_of is not None:
                if not 0 <= l.weights_of < len(self.layers) or self.layers[l.weights_of].weights_of is not None:
                    problems.append(f"layer {i}: weights_of names layer {l.weights_of}, which is no layer with weights of its own")
                elif self.layers[l.weights_of].type != l.type:
                    problems.append(f"layer {i}: weights_of names a layer of another type")
        if problems:
            raise ValueError("bad Gudutar config: " + "; ".join(problems))


def _rotary(rot: dict, width: int, interleaved: bool) -> dict:
    return {"kind": "rotary", "params": {"head_dim": width, "theta": float(rot["base"]), "rotary_dim": int(rot["dims"]),
                                         "interleaved": interleaved, "scaling": None}}


def _mixer_spec(kind: str, m: dict, eps: float) -> PartSpec:
    if kind == "mamba2":
        return PartSpec("mamba2", {"heads": m["heads"], "head_dim": m["vdim"], "state": m["state"], "groups": m.get("groups", 1),
                                   "conv": m["conv"], "norm_groups": m.get("norm_groups", 1), "eps": eps})
    if kind == "retention":
        return PartSpec("retention", {"heads": m["heads"], "key_dim": m["dim"], "head_dim": m["vdim"], "decay": list(m["decay"]),
                                      "position": _rotary(m["rot"], m["dim"], False) if m.get("rot") else None, "eps": eps})
    return PartSpec("latent_attention", {"heads": m["heads"], "plain_dim": m["dim"], "rot_dim": m["rot_dim"], "head_dim": m["vdim"],
                                         "rank": m["kv_rank"], "scale": m["scale"], "window": int((m.get("mask") or {}).get("size") or 0),
                                         "position": _rotary(m["rot"], m["rot_dim"], True), "eps": eps})


def build_spec(cfg: GudutarConfig) -> ModelSpec:
    eps = cfg.norm_eps
    norm = PartSpec("layernorm", {"eps": eps, "weight_name": "", "bias_name": "b"})
    layers, index_of, schedule = [], {}, []
    for i, l in enumerate(cfg.layers):
        if l.weights_of is None:
            parts = {"mixer": _mixer_spec(l.type, l.mixer, eps), "mixer_norm": norm}
            names = {"mixer": "mix", "mixer_norm": "norm1", "feed_forward": l.mlp is not None}
            if l.mlp is not None:
                parts["feed_forward"] = PartSpec("gated_mlp", {"intermediate_size": int(l.mlp["ff"]), "activation": "gelu_tanh",
                                                               "tensor_names": {"gate": "gate", "up": "up", "down": "down"}})
                parts["feed_forward_norm"] = norm
                names.update({"feed_forward": "mlp", "feed_forward_norm": "norm2"})
            index_of[i] = len(layers)
            layers.append(LayerSpec(f"l{i}", PartSpec("branch_norm", names), parts))
    for i, l in enumerate(cfg.layers):
        schedule.append(ScheduleStep(index_of[i if l.weights_of is None else l.weights_of]))
    return ModelSpec(
        hidden_size=cfg.width, vocab_size=cfg.vocab,
        embedding=PartSpec("token_embedding", {"vocab_size": cfg.vocab, "scale": cfg.embedding_scale, "float_stream": True, "tensor_name": ""}),
        layers=layers, final_norm=norm, head=PartSpec("lm_head", {"vocab_size": cfg.vocab, "tied": False, "tensor_name": ""}),
        schedule=schedule, embedding_name="embed", final_norm_name="final.norm", head_name="head",
        max_positions=cfg.max_positions, eos_token_id=None, stored_dtype=cfg.torch_dtype)


register_architecture(Architecture("Gudutar", GudutarConfig.from_json, build_spec))
