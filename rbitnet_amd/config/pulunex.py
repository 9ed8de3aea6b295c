"""Typed configuration of the Pulunex decoder, read from config.json.

A pre-norm decoder with learned positions: x = embed[id] * embedding.scale + pos[p]; per layer
x <- x + mixer(shift(norm1(x))), x <- x + ff(norm2(x)); logits = head(norm(x)) * logit_scale.  Every norm is an RMS
norm whose gain is one number.  `shift` moves every channel of the mixer's input towards the token before by the layer's
tensor `shift` (the block's token shift).  The order of layers is the file's; every layer's mixer is
  "attention"  grouped-query causal softmax attention without a rotation: biases on q, k, v; query and key heads divided
               by their root mean square; the heads' scores mixed by the tensor `talk` before the softmax; keys limited to
               the query's chunk of `mask.size` positions; `kv_from: j` reads layer j's keys and values;
and its feed-forward is dense (the tanh form of GELU, no gate), a mixture of experts (softmax scores over the experts and
`router.identity` outputs that stand for the token's own input; the `top` largest of score + correction; weights on the
experts' outputs; a shared expert behind a sigmoid gate), or absent.

Keys: architecture, vocab, width, max_positions, embedding.scale, logit_scale, norm.eps,
layers: [{"type", "mixer": {heads, kv_heads, dim, vdim, scale, mask: {size} or null, kv_from}, "mlp": {...} or null}].

Tensor names: embed, pos, head, final.norm, and per layer i under `l<i>.`: norm1, norm2, shift, mix.*, mlp.*.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass, field
from typing import Any, Dict, List

from ..errors import ConfigError
from .spec import LayerSpec, ModelSpec, PartSpec
from .tigutar import _float, _int, _obj

TYPES = ("attention",)


@dataclass
class PulunexConfig:
    vocab: int
    width: int
    max_positions: int
    norm_eps: float
    embedding_scale: float
    logit_scale: float
    layers: List[Dict[str, Any]] = field(default_factory=list)

    architecture = "Pulunex"

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "PulunexConfig":
        layers = d.get("layers")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config: 'layers' must be a list with at least one layer")
        cfg = cls(vocab=_int(d, "vocab", "config"), width=_int(d, "width", "config"),
                  max_positions=_int(d, "max_positions", "config"),
                  norm_eps=_float(_obj(d, "norm", "config"), "eps", "norm"),
                  embedding_scale=_float(_obj(d, "embedding", "config"), "scale", "embedding"),
                  logit_scale=_float(d, "logit_scale", "config"), layers=copy.deepcopy(layers))
        cfg.check()
        return cfg

    # ------------------------------------------------------------------ checks
    def check(self) -> None:
        for i, layer in enumerate(self.layers):
            where = f"layer {i}"
            if not isinstance(layer, dict) or layer.get("type") not in TYPES:
                raise ConfigError(f"{where}: type must be one of {', '.join(TYPES)}, found "
                                  f"{layer.get('type') if isinstance(layer, dict) else layer!r}")
            m = _obj(layer, "mixer", where)
            for key in ("heads", "kv_heads", "dim", "vdim"):
                _int(m, key, where)
            if m["heads"] % m["kv_heads"] != 0:
                raise ConfigError(f"{where}: {m['heads']} heads cannot share {m['kv_heads']} key/value heads")
            _float(m, "scale", where)
            if m.get("mask") is not None:
                _int(_obj(m, "mask", where), "size", f"{where} mask")
            j = m.get("kv_from")
            if j is not None:
                if isinstance(j, bool) or not isinstance(j, int) or not 0 <= j < i:
                    raise ConfigError(f"{where}: kv_from must name an earlier layer, found {j!r}")
                other = self.layers[j]["mixer"]
                if other.get("kv_from") is not None:
                    raise ConfigError(f"{where}: kv_from = {j}, but layer {j} keeps no keys and values of its own")
                for key in ("kv_heads", "dim", "vdim"):
                    if other.get(key) != m[key]:
                        raise ConfigError(f"{where}: {key} {m[key]} differs from layer {j}'s {other.get(key)}")
            mlp = layer.get("mlp")
            if mlp is None:
                continue
            if not isinstance(mlp, dict) or mlp.get("kind") not in ("dense", "moe"):
                raise ConfigError(f"{where}: mlp must be null or of kind 'dense' or 'moe', found {mlp!r}")
            if mlp["kind"] == "dense":
                _int(mlp, "ff", where)
                continue
            expert, router = _obj(mlp, "expert", f"{where} mlp"), _obj(mlp, "router", f"{where} mlp")
            _int(expert, "ff", f"{where} expert")
            n = _int(router, "experts", f"{where} router") + _int(router, "identity", f"{where} router", 0, zero_ok=True)
            if _int(router, "top", f"{where} router") > n:
                raise ConfigError(f"{where} router: top {router['top']} of {n} outputs")
            if mlp.get("shared") is not None:
                _int(_obj(mlp, "shared", f"{where} mlp"), "ff", f"{where} shared")

    def to_dict(self) -> Dict[str, Any]:
        return {"architecture": self.architecture, "vocab": self.vocab, "width": self.width, "max_positions": self.max_positions,
                "embedding": {"scale": self.embedding_scale}, "logit_scale": self.logit_scale, "norm": {"eps": self.norm_eps},
                "layers": copy.deepcopy(self.layers)}

    # ------------------------------------------------------------------ the spec
    def _norm(self) -> PartSpec:
        return PartSpec("rmsnorm", {"size": self.width, "eps": self.norm_eps, "scalar": True, "names": {"weight": ""}})

    def to_spec(self) -> ModelSpec:
        layers = []
        for i, layer in enumerate(self.layers):
            m = layer["mixer"]
            mask = m.get("mask")
            mixer = PartSpec("attention", {
                "num_heads": m["heads"], "num_kv_heads": m["kv_heads"], "head_dim": m["dim"], "value_dim": m["vdim"],
                "scale": m["scale"], "window": None, "chunk": None if mask is None else mask["size"],
                "cache_from": m.get("kv_from"), "bias": True, "qk_norm": {"eps": self.norm_eps}, "talk": True,
                "position": PartSpec("none", {"max_positions": self.max_positions}),
                "names": {"q": "q", "k": "k", "v": "v", "o": "o", "q_bias": "q.b", "k_bias": "k.b", "v_bias": "v.b", "talk": "talk"}})
            mlp = layer.get("mlp")
            if mlp is None:
                ff = None
            elif mlp["kind"] == "dense":
                ff = PartSpec("dense_gelu", {"intermediate_size": mlp["ff"], "names": {"up": "up", "down": "down"}})
            else:
                router, shared = mlp["router"], mlp.get("shared")
                ff = PartSpec("routed_experts", {
                    "experts": router["experts"], "top": router["top"], "identity": router.get("identity", 0),
                    "intermediate_size": mlp["expert"]["ff"], "limit": None, "score": "softmax", "correction": True,
                    "weight_on": "output", "shared": None if shared is None else {"intermediate_size": shared["ff"]}})
            layers.append(LayerSpec(prefix=f"l{i}", block="prenorm", mixer=mixer, feed_forward=ff, norm1=self._norm(),
                                    norm2=None if ff is None else self._norm(),
                                    segments={"norm1": "norm1", "mixer": "mix", "norm2": "norm2", "feed_forward": "mlp"},
                                    params={"token_shift": {"name": "shift"}}))
        return ModelSpec(
            architecture=self.architecture, hidden_size=self.width, vocab_size=self.vocab, max_positions=self.max_positions,
            layers=layers,
            embedding=PartSpec("table", {"name": "embed", "vocab_size": self.vocab, "scale": self.embedding_scale,
                                         "positions": {"name": "pos", "max_positions": self.max_positions}}),
            head=PartSpec("linear", {"norm": self._norm(), "norm_name": "final.norm", "name": "head", "vocab_size": self.vocab,
                                     "logit_scale": self.logit_scale}))
