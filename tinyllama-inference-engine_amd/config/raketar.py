"""The configuration of the Raketar decoder, read from its own config.json keys.

    architecture    "Raketar"
    vocab, width    sizes of the vocabulary and of the residual stream
    norm.eps        of every RMS norm
    residual_mult   what a layer's sublayers (and its token input) are multiplied by before they join the residual
    token_side.dim  the size of a layer's part of the per-layer token table (absent: no such input)
    loop            start, stop, times: layers start .. stop - 1 run `times` times in a row, each pass on a cache
                    and state of its own (absent: every layer runs once)
    layers          one entry a layer: `type` ("attention", "mlstm"), `mixer` (that mixer's sizes and constants)
                    and `mlp` (null: no feed-forward)

    attention   heads, kv_heads, dim, vdim, scale, diff, rot (base, dims, scaling.factor; absent: no positions)
    mlstm       heads, dim, vdim, gate_cap
    mlp         kind "dense": ff; kind "moe": expert.ff, router.experts, router.top, shared.ff (absent: no shared expert)

A layer norms the residual once and runs its mixer and its feed-forward side by side on that.  Every size and
every constant that can differ between two models of the design is read from here; what the design fixes (the
layer's arrangement, the interleaved rotation pairs, sigmoid scores that are not renormalized and weigh an
expert's input, the tensors' names) is written down in `to_spec`.  The design sets no bound on positions.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Any, Mapping

from ..errors import invalid_config
from .fadutar import _number
from .spec import LayerSpec, ModelSpec, PartSpec, Run, TensorSpec

LAYER_TYPES = ("attention", "mlstm")


@dataclass(frozen=True)
class RaketarConfig:
    raw: Mapping[str, Any]          # config.json as read (validated)
    architecture: str = "Raketar"

    @classmethod
    def from_dict(cls, raw: Mapping[str, Any]) -> "RaketarConfig":
        config = cls(raw=copy.deepcopy(dict(raw)), architecture=str(raw.get("architecture", "Raketar")))
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
        _number("the model", raw, "residual_mult", float, positive=False)
        if raw.get("token_side") is not None:
            _number("token_side", raw["token_side"], "dim")
        layers = raw.get("layers")
        if not isinstance(layers, list) or not layers:
            raise invalid_config("'layers' must be a list with at least one layer")
        loop = raw.get("loop")
        if loop is not None:
            start, stop = _number("loop", loop, "start", positive=False), _number("loop", loop, "stop")
            _number("loop", loop, "times")
            if not 0 <= start < stop <= len(layers):
                raise invalid_config(f"loop: layers {start} .. {stop - 1} are not a stretch of the model's {len(layers)}")
        for index, layer in enumerate(layers):
            where = f"layer {index}"
            if not isinstance(layer, Mapping) or layer.get("type") not in LAYER_TYPES:
                kind = layer.get("type") if isinstance(layer, Mapping) else layer
                raise invalid_config(f"{where}: type {kind!r} is not one of {', '.join(LAYER_TYPES)}")
            mixer = layer.get("mixer")
            if not isinstance(mixer, Mapping):
                raise invalid_config(f"{where} lacks 'mixer'")
            getattr(self, "_check_" + layer["type"])(mixer, f"{where}'s mixer")
            mlp = layer.get("mlp")
            if mlp is not None:
                self._check_mlp(mlp, f"{where}'s mlp")

    def _check_attention(self, mixer, where):
        heads, kv_heads = _number(where, mixer, "heads"), _number(where, mixer, "kv_heads")
        dim = _number(where, mixer, "dim")
        _number(where, mixer, "vdim"), _number(where, mixer, "scale", float)
        _number(where, mixer, "diff", float, positive=False)
        if heads % kv_heads != 0:
            raise invalid_config(f"{where}: heads {heads} is not a multiple of kv_heads {kv_heads}")
        rot = mixer.get("rot")
        if rot is not None:
            _number(f"{where}'s rot", rot, "base", float)
            dims = _number(f"{where}'s rot", rot, "dims")
            if dims > dim or dims % 2 != 0:
                raise invalid_config(f"{where}: rot.dims must be even and at most dim (the dims past it pass unrotated)")
            if rot.get("scaling") is not None:
                _number(f"{where}'s rot.scaling", rot["scaling"], "factor", float)

    def _check_mlstm(self, mixer, where):
        for key in ("heads", "dim", "vdim"):
            _number(where, mixer, key)
        _number(where, mixer, "gate_cap", float)

    def _check_mlp(self, mlp, where):
        if not isinstance(mlp, Mapping) or mlp.get("kind") not in ("dense", "moe"):
            raise invalid_config(f"{where}: an mlp must be null or of kind 'dense' or 'moe'")
        if mlp["kind"] == "dense":
            _number(where, mlp, "ff")
            return
        _number(f"{where}'s expert", mlp.get("expert"), "ff")
        experts = _number(f"{where}'s router", mlp.get("router"), "experts")
        top = _number(f"{where}'s router", mlp.get("router"), "top")
        if top > experts:
            raise invalid_config(f"{where}: a token cannot use {top} of {experts} experts")
        if mlp.get("shared") is not None:
            _number(f"{where}'s shared expert", mlp["shared"], "ff")

    # ---- the model as data ----------------------------------------------------------------------------
    def to_spec(self) -> ModelSpec:
        raw = self.raw
        width, vocab, eps = int(raw["width"]), int(raw["vocab"]), float(raw["norm"]["eps"])
        mult = float(raw["residual_mult"])
        norm = PartSpec("rms_norm", {"size": width, "eps": eps, "tensor": ""})      # (the tensor is named by the place alone)
        side = raw.get("token_side")
        side_dim = int(side["dim"]) if side is not None else 0
        count = len(raw["layers"])
        layers = []
        for index, layer in enumerate(raw["layers"]):
            mixer = getattr(self, "_spec_" + layer["type"])(layer["mixer"], width, eps)
            mlp = layer.get("mlp")
            layer_input = None
            if side is not None:
                layer_input = PartSpec("token_side", {
                    "hidden_size": width, "dim": side_dim, "table": "side.embed", "table_width": count * side_dim,
                    "offset": index * side_dim, "eps": eps, "scale": mult,
                    "names": {"gate": "gate", "proj": "proj", "norm": "norm"}})
            layers.append(LayerSpec(
                prefix=f"l{index}.", block="parallel", mixer=mixer,
                feed_forward=self._spec_mlp(mlp, width) if mlp is not None else None,
                mixer_norm=norm, feed_forward_norm=None, mixer_norm_place="norm1", mixer_place="mix.",
                feed_forward_place="mlp.", residual_scale=mult, layer_input=layer_input, layer_input_place="side."))
        runs, shared = [], []
        loop = raw.get("loop")
        if loop is None:
            runs = [Run(layer=index, cache_of=index) for index in range(count)]
        else:
            start, stop, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
            shared.append(TensorSpec("loop.step", (times, width)))
            order = [(index, None) for index in range(start)]
            for t in range(times):
                order += [(index, t if index == start else None) for index in range(start, stop)]
            order += [(index, None) for index in range(stop, count)]
            for layer, enters in order:
                # a pass of the loop begins: all passes but the first take the embedding's output again, each its own vector
                runs.append(Run(layer=layer, cache_of=len(runs), add_embedding=enters is not None and enters > 0,
                                add_vector=("loop.step", enters) if enters is not None else None))
        if side is not None:
            shared.append(TensorSpec("side.embed", (vocab, count * side_dim)))
        spec = ModelSpec(
            architecture=self.architecture, hidden_size=width, vocab_size=vocab, max_positions=None,
            embedding=PartSpec("token_embedding", {"vocab_size": vocab, "hidden_size": width}),
            layers=tuple(layers), runs=tuple(runs), final_norm=norm,
            head=PartSpec("lm_head", {"vocab_size": vocab, "hidden_size": width, "tied": False}),
            embedding_name="embed", final_norm_prefix="final.norm", head_name="head", shared_tensors=tuple(shared))
        spec.validate()
        return spec

    def _spec_attention(self, mixer, width, eps) -> PartSpec:
        rot = mixer.get("rot")
        position = PartSpec("none")
        if rot is not None:
            scaling = rot.get("scaling")
            position = PartSpec("rotary", {
                "head_dim": int(mixer["dim"]), "rot_dim": int(rot["dims"]), "theta": float(rot["base"]),
                "linear_factor": float(scaling["factor"]) if scaling is not None else 1.0})
        return PartSpec("differential_attention", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "num_kv_heads": int(mixer["kv_heads"]),
            "head_dim": int(mixer["dim"]), "value_dim": int(mixer["vdim"]), "scale": float(mixer["scale"]),
            "diff": float(mixer["diff"]), "norm_eps": eps, "output_gate": True, "pairing": "interleaved", "position": position,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "lambda_q1": "lq1", "lambda_k1": "lk1",
                      "lambda_q2": "lq2", "lambda_k2": "lk2"}})

    def _spec_mlstm(self, mixer, width, eps) -> PartSpec:
        return PartSpec("mlstm", {
            "hidden_size": width, "num_heads": int(mixer["heads"]), "head_dim": int(mixer["dim"]),
            "value_dim": int(mixer["vdim"]), "gate_cap": float(mixer["gate_cap"]), "norm_eps": eps,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "norm": "norm", "input_gate": "i",
                      "input_gate_bias": "i.b", "forget_gate": "f", "forget_gate_bias": "f.b"}})

    def _spec_mlp(self, mlp, width) -> PartSpec:
        names = {"gate": "gate", "up": "up", "down": "down"}
        if mlp["kind"] == "dense":
            return PartSpec("gated_mlp", {"hidden_size": width, "intermediate_size": int(mlp["ff"]), "activation": "silu",
                                          "names": names})
        shared = mlp.get("shared")
        return PartSpec("routed_mlp", {
            "hidden_size": width, "experts": int(mlp["router"]["experts"]), "top": int(mlp["router"]["top"]),
            "expert_size": int(mlp["expert"]["ff"]), "shared_size": int(shared["ff"]) if shared is not None else 0,
            "score": "sigmoid", "renormalize": False, "weigh": "input",
            "names": {"router": "router", "expert": "e{}.", "shared": "shared.", **names}})
