"""Typed configuration of the Menerax decoder, read from config.json.

A decoder whose layers put their norms on the sublayers' OUTPUTS: x <- x + norm1(mixer(x)), x <- x + norm2(ff(x)), both
sublayers reading the stream itself.  Every norm of the model (those, the one behind the embedding, the final one) is an RMS
norm whose weight is stored as its distance from one.  A layer has one of two mixers:
  "latent_attention"  causal softmax attention whose queries, keys and values go through latents; a head's key is a part made
                      from the cached latent beside a rotated part that all heads share (pairs 2i, 2i + 1); a sigmoid gate per
                      head on the output;
  "parallel"          `left`: grouped-query attention with biases, a short convolution on q, k and v, per-head norms on q and k,
                      a rotation of the head's first numbers (i with i + dims / 2, long wavelengths stretched), capped
                      scores, a window that keeps the first tokens and a gate on every output number; beside it `right`: time
                      mixing with a token shift (a decaying matrix state per head, read before the token's write, with a bonus
                      for the token itself); the result is left_scale * left + right_scale * right;
and a dense feed-forward whose gate and up branches are limited (or none).  A layer with `weights_of: j` has no tensors of its
own: it runs layer j's parts again, with a cache and state of its own.

Keys: architecture, vocab, width, norm.eps, layers: [{"type", "mixer": {...}, "mlp": {...} or null, "weights_of": j}].
The inner size of the time mixing's decay projections is not in the file: it is the first size of `l<i>.mix.right.w1`
(`with_tensor_shapes`); a model made without a file names it itself (`decay_rank`).

Tensor names: embed, embed.norm, head, final.norm, and per layer i that owns weights under `l<i>.`: norm1, norm2, mix.*, mlp.*.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List, Optional

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec
from .tigutar import _float, _int, _obj

MAX_POSITIONS = 1 << 20        # config.json gives no limit; this bounds a sequence where nothing else does
TYPES = ("latent_attention", "parallel")
GATE_ALPHA = 1.702             # the feed-forward's gate is g * sigmoid(1.702 g): fixed by the design


def _rot(m: Dict[str, Any], where: str, limit: int) -> Dict[str, Any]:
    rot = _obj(m, "rot", where)
    dims = _int(rot, "dims", f"{where} rot", zero_ok=True)
    if not _float(rot, "base", f"{where} rot") > 0:
        raise ConfigError(f"{where} rot: base must be positive")
    if dims % 2 != 0 or dims > limit:
        raise ConfigError(f"{where}: rot.dims must be even and at most {limit}, found {dims}")
    scaling = rot.get("scaling")
    if scaling is not None:
        if not isinstance(scaling, dict):
            raise ConfigError(f"{where} rot: 'scaling' must be an object")
        for key in ("factor", "low", "high", "original"):
            _float(scaling, key, f"{where} rot scaling")
        if scaling["high"] == scaling["low"] or scaling["factor"] <= 0:
            raise ConfigError(f"{where} rot scaling: high and low must differ and factor be positive")
    return rot


@dataclass
class MeneraxConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: List[Dict[str, Any]] = field(default_factory=list)
    max_positions: int = MAX_POSITIONS

    architecture = "Menerax"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "MeneraxConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config: 'layers' must be a list with at least one layer")
        cfg = cls(vocab=_int(d, "vocab", "config"), width=_int(d, "width", "config"),
                  norm_eps=_float(_obj(d, "norm", "config"), "eps", "norm"), layers=copy.deepcopy(layers),
                  max_positions=_int(d, "max_positions", "config", MAX_POSITIONS))
        cfg.check()
        return cfg

    # ------------------------------------------------------------------ checks
    def owner(self, i: int) -> int:
        """The layer whose tensors layer i uses (itself, unless it names another)."""
        seen = set()
        while self.layers[i].get("weights_of") is not None:
            if i in seen:
                raise ConfigError(f"layer {i}: weights_of leads back to the layer itself")
            seen.add(i)
            i = self.layers[i]["weights_of"]
        return i

    def check(self) -> None:
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            if not isinstance(layer, dict) or layer.get("type") not in TYPES:
                raise ConfigError(f"{where}: type must be one of {', '.join(TYPES)}, found "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = _obj(layer, "mixer", where)
            if layer["type"] == "latent_attention":
                for key in ("heads", "dim", "vdim", "q_rank", "kv_rank"):
                    _int(m, key, where)
                _int(m, "rot_dim", where, zero_ok=True)
                _float(m, "scale", where)
                if (m["rot_dim"] or m.get("rot") is not None) and _rot(m, where, m["rot_dim"])["dims"] != m["rot_dim"]:
                    raise ConfigError(f"{where}: the rotated part has rot_dim = {m['rot_dim']} numbers and all of them are rotated, "
                                      f"found rot.dims = {m['rot']['dims']}")
            else:
                left, right = _obj(m, "left", where), _obj(m, "right", where)
                lw = f"{where} left"
                for key in ("heads", "kv_heads", "dim", "vdim", "conv"):
                    _int(left, key, lw)
                if left["heads"] % left["kv_heads"] != 0:
                    raise ConfigError(f"{lw}: {left['heads']} heads cannot share {left['kv_heads']} key/value heads")
                _float(left, "scale", lw)
                _rot(left, lw, left["dim"])
                if left.get("softcap") is not None and not _float(left, "softcap", lw) > 0:
                    raise ConfigError(f"{lw}: softcap must be positive")
                if left.get("mask") is not None:
                    mask = _obj(left, "mask", lw)
                    _int(mask, "size", f"{lw} mask")
                    _int(mask, "keep_first", f"{lw} mask", 0, zero_ok=True)
                for key in ("heads", "dim"):
                    _int(right, key, f"{where} right")
                _float(m, "left_scale", where)
                _float(m, "right_scale", where)
            mlp = layer.get("mlp")
            if mlp is not None:
                if not isinstance(mlp, dict) or mlp.get("kind") != "dense":
                    raise ConfigError(f"{where}: mlp must be null or of kind 'dense', found {mlp!r}")
                _int(mlp, "ff", f"{where} mlp")
                if not _float(mlp, "limit", f"{where} mlp") > 0:
                    raise ConfigError(f"{where} mlp: limit must be positive")
            j = layer.get("weights_of")
            if j is not None:
                if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < len(self.layers) or j == i:
                    raise ConfigError(f"{where}: weights_of must name another layer, found {j!r}")
        for i in range(len(self.layers)):
            j = self.owner(i)
            if self.layers[j]["type"] != self.layers[i]["type"]:
                raise ConfigError(f"layer {i}: it uses layer {j}'s weights, but is of another type")

    def to_dict(self) -> Dict[str, Any]:
        out = {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": copy.deepcopy(self.layers)}
        if self.max_positions != MAX_POSITIONS:
            out["max_positions"] = self.max_positions
        return out

    # ------------------------------------------------------------------ sizes only the weights know
    def with_tensor_shapes(self, shapes: Dict[str, Any]) -> "MeneraxConfig":
        out = copy.deepcopy(self)
        for i, layer in enumerate(out.layers):
            name = f"l{out.owner(i)}.mix.right.w1"
            if layer["type"] == "parallel" and name in shapes and len(shapes[name]) == 2:
                layer["mixer"]["right"]["decay_rank"] = int(shapes[name][0])
        return out

    # ------------------------------------------------------------------ the spec
    def _position(self, rot: Dict[str, Any], style: str) -> PartSpec:
        params = {"head_dim": rot["dims"], "theta": rot["base"], "style": style, "max_positions": self.max_positions}
        s = rot.get("scaling")
        if s is not None:
            params["scaling"] = {"rope_type": "llama3", "factor": s["factor"], "low_freq_factor": s["low"],
                                 "high_freq_factor": s["high"], "original_max_position_embeddings": s["original"]}
        return PartSpec("rope", params)

    def _latent(self, m: Dict[str, Any]) -> PartSpec:
        return PartSpec("latent_attention", {
            "heads": m["heads"], "dim": m["dim"], "vdim": m["vdim"], "q_rank": m["q_rank"], "kv_rank": m["kv_rank"],
            "scale": m["scale"], "eps": self.norm_eps, "rot_dim": m["rot_dim"],
            "position": self._position(m["rot"], "interleaved") if m["rot_dim"] else None, "sink": False, "head_gate": True})

    def _left(self, m: Dict[str, Any]) -> PartSpec:
        mask = m.get("mask")
        rot = m["rot"]
        position = self._position(rot, "half") if rot["dims"] else PartSpec("none", {"max_positions": self.max_positions})
        return PartSpec("attention", {
            "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
            "scale": m["scale"], "window": None if mask is None else mask["size"],
            "keep_first": 0 if mask is None else mask.get("keep_first", 0), "softcap": m.get("softcap"),
            "bias": True, "conv": m["conv"], "qk_norm": {"eps": self.norm_eps, "weight": True}, "gate": "elementwise",
            "position": position,
            "names": {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b",
                      "q_conv": "q.conv", "k_conv": "k.conv", "v_conv": "v.conv", "q_norm": "q.norm", "k_norm": "k.norm"}})

    def to_spec(self) -> ModelSpec:
        def norm() -> PartSpec:
            return PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "one_plus": True, "names": {"weight": ""}})
        owners = [i for i in range(len(self.layers)) if self.owner(i) == i]
        index = {i: n for n, i in enumerate(owners)}
        layers = []
        for i in owners:
            layer = self.layers[i]
            m = layer["mixer"]
            if layer["type"] == "latent_attention":
                mixer = self._latent(m)
            else:
                right = m["right"]
                if "decay_rank" not in right:
                    raise ConfigError(f"layer {i}: decay_rank is neither in the configuration nor given by a weight file")
                mixer = PartSpec("pair", {
                    "combine": "weighted", "left_scale": m["left_scale"], "right_scale": m["right_scale"], "left": self._left(m["left"]),
                    "right": PartSpec("time_mix", {"heads": right["heads"], "dim": right["dim"], "decay_rank": right["decay_rank"],
                                                   "eps": self.norm_eps})})
            mlp = layer.get("mlp")
            ff = None if mlp is None else PartSpec("clamped_glu", {"intermediate_size": mlp["ff"], "limit": mlp["limit"],
                                                                   "alpha": GATE_ALPHA})
            layers.append(LayerSpec(prefix=f"l{i}", block="outnorm", mixer=mixer, feed_forward=ff, norm1=norm(),
                                    norm2=None if ff is None else norm(),
                                    segments={"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"}))
        return ModelSpec(
            architecture=self.architecture, hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            layers=layers, schedule=[index[self.owner(i)] for i in range(len(self.layers))],
            embedding=PartSpec("table", {"name": "embed", "vocab_size": self.vocab, "norm": norm(), "norm_name": "embed.norm"}),
            head=PartSpec("linear", {"norm": norm(), "norm_name": "final.norm", "name": "head", "vocab_size": self.vocab}))

