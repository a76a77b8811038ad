"""Pamunex: a decoder whose layers norm what a sublayer GIVES, not what it reads:
x <- x + norm1(mixer(x)); x <- x + norm2(ffn(x)), the norms being layer norms with weight and bias.  A layer's
mixer is grouped-query attention over the keys of the query's own block of positions (`attention`) or latent
attention over a sliding window (`latent_attention`), both with a sink in the softmax; its feed-forward is dense
or a mixture of experts with group-limited routing, the activation relu(x)^2; a layer may have none.  The output
is the final layer norm, the embedding table as the head, and a factor on the logits.  This class knows the
config.json keys and the tensor names and nothing else: every size and constant goes through a spec to a
registered part.

config.json: `architecture` (the name), `vocab`, `width`, `norm.eps`, `logit_scale`, and `layers`, a list of
{`type`: attention | latent_attention, `mixer`: sizes and constants (`heads`, `dim`, `vdim`, `scale`, `rot.base`,
`rot.dims`, `mask.size`; `kv_heads` / `kv_rank`, `rot_dim`), `mlp`: null, {`kind`: dense, `ff`} or {`kind`: moe,
`expert.ff`, `router.experts`, `router.top`, `router.groups.count`, `router.groups.keep`}}.  Positions are not
bounded by the model; `max_positions`, when a file gives it, bounds what the engine plans for.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Tuple

from .registry import ConfigError, register_architecture
from .specs import (HeadSpec, LatentAttentionSpec, LayerRun, LayerSpec, MaskSpec, ModelSpec, NormSpec, PlainMlpSpec,
                    PositionSpec, RoutedMlpSpec, SinkAttentionSpec)
from .taletar import DEFAULT_MAX_POSITIONS, _freeze, _int, _num, _thaw


def _object(d, key, where):
    v = d.get(key)
    if not isinstance(v, dict):
        raise ConfigError(f"config.json: {where}`{key}` must be an object")
    return v


def _rotation(m, where, dims=None):
    rot = _object(m, "rot", where)
    n = _int(rot, "dims", where + "rot.")
    if n % 2 != 0 or (dims is not None and n != dims):
        raise ConfigError(f"config.json: {where}rot.dims {n} must be even" + (f" and equal rot_dim {dims}" if dims else ""))
    return PositionSpec("rope_split_half", n, _num(rot, "base", where + "rot.", positive=True))


def _mask(m, kind, where):
    return MaskSpec(kind, _int(_object(m, "mask", where), "size", where + "mask."))


def _attention(m, width, eps, where):
    heads, kv = _int(m, "heads", where), _int(m, "kv_heads", where)
    if heads % kv != 0:
        raise ConfigError(f"config.json: {where}heads {heads} is no multiple of kv_heads {kv}")
    dim = _int(m, "dim", where)
    position = _rotation(m, where)
    if position.dim > dim:
        raise ConfigError(f"config.json: {where}rot.dims {position.dim} exceeds dim {dim}")
    return SinkAttentionSpec(kind="sink_attention", hidden=width, q_heads=heads, kv_heads=kv, head_dim=dim,
                             value_dim=_int(m, "vdim", where), scale=_num(m, "scale", where),
                             qk_norm=NormSpec("rmsnorm", dim, eps), position=position, mask=_mask(m, "chunk", where),
                             sink=True, bias=True)


def _latent_attention(m, width, eps, where):
    rot_dim = _int(m, "rot_dim", where)
    return LatentAttentionSpec(kind="latent_attention", hidden=width, heads=_int(m, "heads", where),
                               head_dim=_int(m, "dim", where), rot_dim=rot_dim, value_dim=_int(m, "vdim", where),
                               rank=_int(m, "kv_rank", where), scale=_num(m, "scale", where), eps=eps,
                               position=_rotation(m, where, rot_dim), mask=_mask(m, "window", where), sink=True)


def _mlp(mlp, width, where):
    if mlp is None:
        return None
    if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
        raise ConfigError(f"config.json: {where} must be null or an object of kind `dense` or `moe`")
    if mlp["kind"] == "dense":
        return PlainMlpSpec("plain_mlp", width, _int(mlp, "ff", where + "."), "relu_squared")
    router = _object(mlp, "router", where + ".")
    groups = router.get("groups") or {"count": 1, "keep": 1}
    experts, top = _int(router, "experts", where + ".router."), _int(router, "top", where + ".router.")
    count, keep = _int(groups, "count", where + ".router.groups."), _int(groups, "keep", where + ".router.groups.")
    if experts % count != 0 or keep > count or top > keep * (experts // count):
        raise ConfigError(f"config.json: {where}.router: {experts} experts in {count} groups of which {keep} stay "
                          f"cannot give {top} choices")
    return RoutedMlpSpec("routed_mlp", width, _int(_object(mlp, "expert", where + "."), "ff", where + ".expert."),
                         experts, top, count, keep, "relu_squared", "sigmoid", False)


_MIXERS = {"attention": _attention, "latent_attention": _latent_attention}


@register_architecture("Pamunex")
@dataclass(frozen=True)
class PamunexConfig:
    vocab: int
    width: int
    eps: float
    logit_scale: float
    layers: Tuple            # the `layers` list of config.json, frozen
    max_positions: int = DEFAULT_MAX_POSITIONS
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, data):
        for key in ("vocab", "width", "norm", "layers"):
            if key not in data:
                raise ConfigError(f"config.json: missing `{key}`")
        if not isinstance(data["norm"], dict):
            raise ConfigError("config.json: `norm` must be an object with `eps`")
        layers = data["layers"]
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json: `layers` must be a non-empty list")
        width = _int(data, "width", "")
        for i, layer in enumerate(layers):
            where = f"layers[{i}]."
            if not isinstance(layer, dict) or not isinstance(layer.get("mixer"), dict):
                raise ConfigError(f"config.json: {where}mixer must be an object")
            if layer.get("type") not in _MIXERS:
                raise ConfigError(f"config.json: {where}type {layer.get('type')!r} is none of {sorted(_MIXERS)}")
            _MIXERS[layer["type"]](layer["mixer"], width, 1e-6, where + "mixer.")      # (checks the keys)
            _mlp(layer.get("mlp"), width, where + "mlp")
        eos = data.get("eos_token_id")
        eos_ids = () if eos is None else (eos,) if isinstance(eos, int) else tuple(eos)
        return cls(vocab=_int(data, "vocab", ""), width=width, eps=_num(data["norm"], "eps", "norm.", positive=True),
                   logit_scale=_num(data, "logit_scale", "", default=1.0), layers=_freeze(layers),
                   max_positions=_int(data, "max_positions", "") if "max_positions" in data else DEFAULT_MAX_POSITIONS,
                   eos_token_ids=eos_ids)

    def to_dict(self):
        out = {"architecture": self.architecture, "layers": _thaw(self.layers), "logit_scale": self.logit_scale,
               "norm": {"eps": self.eps}, "vocab": self.vocab, "width": self.width}
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        if self.eos_token_ids:
            out["eos_token_id"] = list(self.eos_token_ids)
        return out

    # ---- the model as parts -------------------------------------------------------------------
    def model_spec(self):
        norm = NormSpec("layernorm", self.width, self.eps)
        specs = []
        for i, layer in enumerate(_thaw(self.layers)):
            mixer = _MIXERS[layer["type"]](layer["mixer"], self.width, self.eps, f"layers[{i}].mixer.")
            ffn = _mlp(layer.get("mlp"), self.width, f"layers[{i}].mlp")
            specs.append(LayerSpec("postnorm", norm, mixer, None if ffn is None else norm, ffn))
        n = len(specs)
        return ModelSpec(architecture=self.architecture, vocab_size=self.vocab, hidden=self.width, layers=tuple(specs),
                         schedule=tuple(LayerRun(i, i) for i in range(n)), final_norm=norm, tie_embeddings=True,
                         max_positions=self.max_positions, eos_token_ids=self.eos_token_ids,
                         head=HeadSpec("scaled_head", self.vocab, self.width, tied=True, scale=self.logit_scale))

    # ---- tensor names ----------------------------------------------------------------------------
    @staticmethod
    def global_tensor_name(local):
        return {"embed.weight": "embed", "final_norm.weight": "final.norm", "final_norm.bias": "final.norm.b",
                "head.weight": "head"}[local]

    @staticmethod
    def layer_tensor_name(layer, part, local):
        if part in ("norm1", "norm2"):
            return f"l{layer}.{part}" + ("" if local == "weight" else ".b")
        return f"l{layer}.{'mix' if part == 'mixer' else 'mlp'}.{local}"
