"""The configuration of the Fadutar decoder, read from its own config.json keys.

    architecture   "Fadutar"
    vocab, width   sizes of the vocabulary and of the residual stream
    norm.eps       of every RMS norm
    layers         one entry a layer, in the order they run: `type` ("attention", "latent_attention",
                   "rglru"), `mixer` (that mixer's sizes and constants) and `mlp` (null: the layer has no
                   feed-forward; else `kind` "dense", `ff`, `limit`)

    attention        heads, kv_heads, dim, vdim, scale, mask.size (a token sees its own chunk of so many
                     positions; no mask: every earlier position), kv_from (the layer whose keys and values
                     this one reads; it then has none of its own)
    latent_attention heads, dim, rot_dim, vdim, kv_rank, scale, rot.base, rot.dims (= rot_dim; fewer: the rest of
                     the rot_dim part passes unrotated)
    rglru            width, blocks, conv (taps)

Every size and every constant that can differ between two models of the design is read from here; what
the design fixes for all of them (the recurrence's decay factor 8, the gate's 1.702, norms whose stored
weight w acts as 1 + w, the tensors' names) is written down in `to_spec`.  The design sets no bound on
positions: the cache pool's size is the only one.
"""
from __future__ import annotations

import copy
import math
from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import invalid_config
from .spec import LayerSpec, ModelSpec, PartSpec, Run

RECURRENCE_DECAY = 8.0          # log a = -8 * r * softplus(lambda)
GATE_ALPHA = 1.702              # g * sigmoid(1.702 g) * (u + 1)
LAYER_TYPES = ("attention", "latent_attention", "rglru")


def _number(where: str, raw: Mapping[str, Any], key: str, kind=int, positive: bool = True):
    if not isinstance(raw, Mapping) or key not in raw or raw[key] is None:
        raise invalid_config(f"config.json lacks '{key}' in {where}")
    value = raw[key]
    if isinstance(value, bool) or not isinstance(value, (int, float) if kind is float else int):
        raise invalid_config(f"'{key}' in {where} must be {'a number' if kind is float else 'an integer'}, not {value!r}")
    value = kind(value)
    if positive and not value > 0:
        raise invalid_config(f"'{key}' in {where} must be positive, not {value!r}")
    if kind is float and not math.isfinite(value):
        raise invalid_config(f"'{key}' in {where} must be finite")
    return value


@dataclass(frozen=True)
class FadutarConfig:
    raw: Mapping[str, Any]          # config.json as read (validated)
    architecture: str = "Fadutar"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "FadutarConfig":
        config = cls(raw=copy.deepcopy(dict(raw)), architecture=str(raw.get("architecture", "Fadutar")))
        config.validate()
        return config

    def to_dict(self) -> dict:
        return copy.deepcopy(dict(self.raw))

    # ---- checks -----------------------------------------------------------------------------------
    def validate(self) -> None:
        raw = self.raw
        _number("the model", raw, "vocab")
        _number("the model", raw, "width")
        _number("norm", raw.get("norm"), "eps", float)
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise invalid_config("'layers' must be a list with at least one layer")
        for index, layer in enumerate(layers):
            where = f"layer {index}"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                kind = layer.get("type") if isinstance(layer, Mapping) else layer
                raise invalid_config(f"{where}: type {kind!r} is not one of {', '.join(LAYER_TYPES)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, Mapping):
                raise invalid_config(f"{where} lacks 'mixer'")
            getattr(self, "_check_" + layer["type"])(index, mixer, f"{where}'s mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, Mapping) or mlp.get("kind") != "dense":
                    raise invalid_config(f"{where}: an mlp must be null or of kind 'dense'")
                _number(f"{where}'s mlp", mlp, "ff")
                _number(f"{where}'s mlp", mlp, "limit", float)

    def _check_attention(self, index, mixer, where):
        heads, kv_heads = _number(where, mixer, "heads"), _number(where, mixer, "kv_heads")
        _number(where, mixer, "dim"), _number(where, mixer, "vdim"), _number(where, mixer, "scale", float)
        if heads % kv_heads != 0:
            raise invalid_config(f"{where}: heads {heads} is not a multiple of kv_heads {kv_heads}")
        if mixer.get("mask") is not None:
            _number(f"{where}'s mask", mixer["mask"], "size")
        source = mixer.get("kv_from")
        if source is not None:
            layers = self.raw["layers"]
            if isinstance(source, bool) or not isinstance(source, int) or not 0 <= source < index:
                raise invalid_config(f"{where}: kv_from {source!r} must name an earlier layer")
            other = layers[source]
            if other.get("type") != "attention" or other["mixer"].get("kv_from") is not None:
                raise invalid_config(f"{where}: layer {source} has no keys and values of its own to read")
            for key in ("kv_heads", "dim", "vdim"):
                if other["mixer"].get(key) != mixer.get(key):
                    raise invalid_config(f"{where}: '{key}' differs from layer {source}'s, whose keys and values it reads")

    def _check_latent_attention(self, index, mixer, where):
        for key in ("heads", "dim", "vdim", "kv_rank"):
            _number(where, mixer, key)
        rot_dim = _number(where, mixer, "rot_dim")
        _number(where, mixer, "scale", float)
        rot = mixer.get("rot")
        _number(f"{where}'s rot", rot, "base", float)
        dims = _number(f"{where}'s rot", rot, "dims")
        if dims > rot_dim or dims % 2 != 0:
            raise invalid_config(f"{where}: rot.dims must be even and at most rot_dim (the dims past it pass unrotated)")

    def _check_rglru(self, index, mixer, where):
        width, blocks = _number(where, mixer, "width"), _number(where, mixer, "blocks")
        _number(where, mixer, "conv")
        if width % blocks != 0:
            raise invalid_config(f"{where}: width {width} is not a multiple of blocks {blocks}")

    # ---- the model as data ----------------------------------------------------------------------------
    def to_spec(self) -> ModelSpec:
        raw = self.raw
        width, vocab, eps = int(raw["width"]), int(raw["vocab"]), float(raw["norm"]["eps"])
        # the tensor is named by the place alone ("l3.norm1"), and its weight w acts as 1 + w
        norm = PartSpec("rms_norm", {"size": width, "eps": eps, "offset": True, "tensor": ""})
        layers, runs = [], []
        for index, layer in enumerate(raw["layers"]):
            mixer = getattr(self, "_spec_" + layer["type"])(index, layer["mixer"], width, eps)
            mlp = layer.get("mlp")
            feed_forward = None
            if mlp is not None:
                feed_forward = PartSpec("gated_mlp", {
                    "hidden_size": width, "intermediate_size": int(mlp["ff"]), "activation": "clamped_swish",
                    "alpha": GATE_ALPHA, "limit": float(mlp["limit"]), "bias": True,
                    "names": {"gate": "gate", "up": "up", "down": "down", "gate_bias": "gate.b", "up_bias": "up.b",
                              "down_bias": "down.b"}})
            layers.append(LayerSpec(
                prefix=f"l{index}.", block="sandwich_norm", mixer=mixer, feed_forward=feed_forward,
                mixer_norm=norm, feed_forward_norm=norm if mlp is not None else None,
                mixer_post_norm=norm, feed_forward_post_norm=norm if mlp is not None else None,
                mixer_norm_place="norm1", mixer_post_norm_place="norm1b", feed_forward_norm_place="norm2",
                feed_forward_post_norm_place="norm2b", mixer_place="mix.", feed_forward_place="mlp."))
            source = layer["mixer"].get("kv_from") if layer["type"] == "attention" else None
            runs.append(Run(layer=index, cache_of=index if source is None else int(source)))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=width, vocab_size=vocab, max_positions=None,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": width}),
            layers=tuple(layers), runs=tuple(runs), final_norm=norm,
            head=PartSpec("lm_head", {"vocab_size": vocab, "hidden_size": width, "tied": False}),
            embedding_name="embed", final_norm_prefix="final.norm", head_name="head")
        spec.validate()
        return spec

    def _reach(self, mixer) -> int | None:
        """How far back a token of this attention layer reads at most (None: to the start)."""
        mask = mixer.get("mask")
        return int(mask["size"]) if mask is not None else None

    def _spec_attention(self, index, mixer, width, eps) -> PartSpec:
        mask = mixer.get("mask")
        # the owner of a cache keeps its pages for as long as any layer reads them: itself and every layer
        # that names it in kv_from, each with a mask of its own
        readers = [other["mixer"] for other in self.raw["layers"]
                   if other["type"] == "attention" and other["mixer"].get("kv_from") == index]
        reaches = [self._reach(user) for user in [mixer, *readers]]
        return PartSpec("attention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "num_kv_heads": int(mixer["kv_heads"]),
            "head_dim": int(mixer["dim"]), "value_dim": int(mixer["vdim"]), "scale": float(mixer["scale"]),
            "bias": False, "window": None, "chunk": int(mask["size"]) if mask is not None else None, "sink": True,
            "cache_window": None if any(reach is None for reach in reaches) else max(reaches),
            "reads_other_cache": mixer.get("kv_from") is not None, "position": PartSpec("none"),
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "sink": "sink"}})

    def _spec_latent_attention(self, index, mixer, width, eps) -> PartSpec:
        return PartSpec("latent_attention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "head_dim": int(mixer["dim"]),
            "rot_dim": int(mixer["rot_dim"]), "value_dim": int(mixer["vdim"]), "rank": int(mixer["kv_rank"]),
            "scale": float(mixer["scale"]), "norm_eps": eps, "sink": True,
            "position": PartSpec("rotary", {"head_dim": int(mixer["rot"]["dims"]), "theta": float(mixer["rot"]["base"]),
                                            "max_positions": None}),
            "names": {"q": "q", "down": "dkv", "down_norm": "dkv.norm", "up_keys": "uk", "up_values": "uv", "o": "o",
                      "sink": "sink"}})

    def _spec_rglru(self, index, mixer, width, eps) -> PartSpec:
        return PartSpec("gated_recurrence", {
            "hidden_size": width, "width": int(mixer["width"]), "blocks": int(mixer["blocks"]), "taps": int(mixer["conv"]),
            "decay": RECURRENCE_DECAY,
            "names": {"gate_branch": "y", "gate_branch_bias": "y.b", "input": "x", "input_bias": "x.b", "conv": "conv",
                      "conv_bias": "conv.b", "recurrence_gate": "ra", "recurrence_gate_bias": "ra.b", "input_gate": "ri",
                      "input_gate_bias": "ri.b", "decay": "lam", "o": "o"}})
