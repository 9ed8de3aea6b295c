"""The Pulunex configuration on the CPU: keys, errors, the spec it turns into, tensor names and shapes against the plain
implementation's, a folder written with random weights read back."""
import copy

import pytest

import plain_pulunex as P
from rbitnet_amd.config import load_config
from rbitnet_amd.engine.model import expected_tensors
from rbitnet_amd.errors import ConfigError


def _mix(**more):
    return dict(dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, mask={"size": 5}), **more)


def _moe(ff, experts, top, identity, shared):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


CFG = {"architecture": "Pulunex", "vocab": 50, "width": 32, "max_positions": 96, "embedding": {"scale": 1.5}, "logit_scale": 0.5,
       "norm": {"eps": 1e-5}, "layers": [
           {"type": "attention", "mixer": _mix(), "mlp": {"kind": "dense", "ff": 40}},
           {"type": "attention", "mixer": _mix(heads=2, kv_heads=2, mask=None), "mlp": _moe(12, 5, 2, 1, 20)},
           {"type": "attention", "mixer": _mix(heads=6, kv_from=0), "mlp": None},
           {"type": "attention", "mixer": _mix(kv_from=0, mask={"size": 64}), "mlp": _moe(8, 3, 3, 0, None)}]}


def test_tensor_names_and_shapes_are_the_plain_implementations():
    shapes = P.tensor_shapes(CFG)
    cfg, spec = load_config(copy.deepcopy(CFG), tensor_shapes=shapes)
    want = expected_tensors(spec)
    assert set(want) == set(shapes)
    assert all(tuple(want[n].shape) == tuple(shapes[n]) for n in want)
    assert "l2.mix.k" not in want and "l2.mix.q.b" in want and "l2.norm2" not in want and want["l0.norm1"].shape == ()
    assert want["l1.mlp.router"].shape == (6, 32) and want["l3.mlp.correction"].shape == (3,) and "l3.mlp.shared.sg" not in want
    layers = spec.layers
    assert all(layer.block == "prenorm" and layer.params["token_shift"] == {"name": "shift"} for layer in layers)
    assert layers[0].mixer["chunk"] == 5 and layers[1].mixer["chunk"] is None and layers[3].mixer["chunk"] == 64
    assert layers[2].mixer["cache_from"] == 0 and layers[2].feed_forward is None and layers[2].norm2 is None
    assert layers[1].feed_forward.kind == "routed_experts" and layers[1].feed_forward["identity"] == 1
    assert layers[0].feed_forward.kind == "dense_gelu" and layers[0].mixer["scale"] == 0.3
    assert spec.embedding["scale"] == 1.5 and spec.embedding["positions"]["max_positions"] == 96 and spec.head["logit_scale"] == 0.5
    again, _ = load_config(cfg.to_dict())
    assert again.to_dict() == cfg.to_dict()


@pytest.mark.parametrize("change,message", [
    (lambda c: c.pop("logit_scale"), "logit_scale"),
    (lambda c: c.pop("max_positions"), "max_positions"),
    (lambda c: c["embedding"].pop("scale"), "scale"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="conv"), "type must be one of"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "cannot share"),
    (lambda c: c["layers"][0]["mixer"].pop("scale"), "scale"),
    (lambda c: c["layers"][0]["mixer"].update(mask={"size": 0}), "size"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=2), "keeps no keys"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=3), "earlier layer"),
    (lambda c: c["layers"][3]["mixer"].update(vdim=8), "differs from layer 0"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=7), "top 7 of 6"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "mlp must be"),
    (lambda c: c["layers"][1]["mlp"]["shared"].pop("ff"), "ff"),
    (lambda c: c.update(layers=[]), "at least one layer"),
])
def test_errors_name_the_key(change, message):
    cfg = copy.deepcopy(CFG)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        load_config(cfg)


def test_a_folder_of_random_weights_has_every_tensor(tmp_path):
    import torch
    import rbitnet_amd
    from rbitnet_amd.weights.safetensors_io import SafetensorsFile
    rbitnet_amd.write_random_model(str(tmp_path / "m"), copy.deepcopy(CFG), seed=3, dtype=torch.bfloat16)
    f = SafetensorsFile(str(tmp_path / "m" / "model.safetensors"))
    got = {n: tuple(f.info(n)[1]) for n in f.names()}
    f.close()
    assert got == {n: tuple(s) for n, s in P.tensor_shapes(CFG).items()}
