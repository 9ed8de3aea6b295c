"""The Menerax configuration without a GPU: keys and errors, the order of layers with layers that run another layer's
weights, tensor names and shapes against the plain implementation's, the size read off the weights, and the pages that a
window with kept first tokens gives back."""
import copy

import pytest
import torch

import plain_menerax as P
from rbitnet_amd.cache.pages import PAGE_SIZE, PageTable
from rbitnet_amd.config import load_config
from rbitnet_amd.engine.model import expected_tensors
from rbitnet_amd.errors import ConfigError


def latent(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=12, kv_rank=10, scale=0.3, base=100.0):
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale,
                rot={"base": base, "dims": rot_dim})


def left(heads=4, kv_heads=2, dim=8, vdim=6, conv=3, dims=4, base=50.0, scale=0.35, softcap=9.0, mask=None, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = scaling
    out = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, rot=rot, scale=scale, softcap=softcap)
    if mask:
        out["mask"] = mask
    return out


def parallel(l, heads=2, dim=6, left_scale=0.7, right_scale=1.2, decay_rank=None):
    right = dict(heads=heads, dim=dim)
    if decay_rank:
        right["decay_rank"] = decay_rank
    return {"left": l, "right": right, "left_scale": left_scale, "right_scale": right_scale}


CFG = {"architecture": "Menerax", "vocab": 40, "width": 24, "norm": {"eps": 1e-5}, "layers": [
    {"type": "parallel", "mixer": parallel(left(mask={"size": 5, "keep_first": 2}), decay_rank=4), "mlp": {"kind": "dense", "ff": 20, "limit": 1.5}},
    {"type": "latent_attention", "mixer": latent(), "mlp": None},
    {"type": "parallel", "mixer": parallel(left(mask={"size": 5, "keep_first": 2}), decay_rank=4), "mlp": {"kind": "dense", "ff": 20, "limit": 1.5},
     "weights_of": 0},
    {"type": "latent_attention", "mixer": latent(heads=2, vdim=8), "mlp": {"kind": "dense", "ff": 12, "limit": 0.5}},
    {"type": "latent_attention", "mixer": latent(), "mlp": None, "weights_of": 1}]}


def test_layers_that_run_another_layers_weights_keep_places_of_their_own():
    cfg, spec = load_config(copy.deepcopy(CFG))
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l3"]
    assert spec.schedule == [0, 1, 0, 2, 1]
    assert spec.layers[0].block == "outnorm" and spec.layers[1].feed_forward is None
    assert cfg.to_dict()["layers"][2]["weights_of"] == 0


def test_tensor_names_and_shapes_are_the_plain_implementations():
    _, spec = load_config(copy.deepcopy(CFG))
    got = {k: tuple(v.shape) for k, v in expected_tensors(spec).items()}
    assert got == P.tensor_shapes(CFG)


def test_the_decay_rank_is_read_off_the_weights():
    raw = copy.deepcopy(CFG)
    for layer in raw["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["right"].pop("decay_rank")
    with pytest.raises(ConfigError, match="decay_rank"):
        load_config(copy.deepcopy(raw))
    _, spec = load_config(copy.deepcopy(raw), tensor_shapes={"l0.mix.right.w1": (7, 24)})
    assert expected_tensors(spec)["l0.mix.right.w2"].shape == (12, 7)


@pytest.mark.parametrize("edit,match", [
    (lambda c: c.pop("vocab"), "vocab"),
    (lambda c: c["norm"].pop("eps"), "eps"),
    (lambda c: c["layers"][0].update(type="attention"), "type"),
    (lambda c: c["layers"][1]["mixer"].update(rot={"base": 10.0, "dims": 2}), "rot"),
    (lambda c: c["layers"][1]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=3), "share"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=10), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(softcap=-1.0), "softcap"),
    (lambda c: c["layers"][0]["mixer"].pop("left_scale"), "left_scale"),
    (lambda c: c["layers"][0]["mlp"].update(limit=0), "limit"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "dense"),
    (lambda c: c["layers"][2].update(weights_of=7), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=1), "another type"),
    (lambda c: c["layers"][0]["mixer"]["left"]["mask"].pop("size"), "size"),
])
def test_errors_name_the_key(edit, match):
    raw = copy.deepcopy(CFG)
    edit(raw)
    with pytest.raises(ConfigError, match=match):
        load_config(raw)


def test_the_rotation_and_the_mask_reach_the_parts():
    raw = copy.deepcopy(CFG)
    raw["layers"][0]["mixer"]["left"]["rot"]["scaling"] = {"factor": 4.0, "low": 1.0, "high": 2.0, "original": 16}
    _, spec = load_config(raw)
    p = spec.layers[0].mixer.params
    assert p["combine"] == "weighted" and (p["left_scale"], p["right_scale"]) == (0.7, 1.2)
    a = p["left"].params
    assert (a["window"], a["keep_first"], a["softcap"], a["conv"], a["gate"]) == (5, 2, 9.0, 3, "elementwise")
    assert a["position"].params["style"] == "half" and a["position"].params["scaling"]["rope_type"] == "llama3"
    from rbitnet_amd.parts.position import rope_inverse_frequencies
    f = rope_inverse_frequencies(4, 50.0, a["position"].params["scaling"])
    assert torch.allclose(f, P.frequencies(4, 50.0, raw["layers"][0]["mixer"]["left"]["rot"]["scaling"]), rtol=1e-12, atol=0)
    b = spec.layers[1].mixer.params
    assert b["position"].params["style"] == "interleaved" and b["rot_dim"] == 4 and b["head_gate"] and not b["sink"]


def test_a_window_gives_pages_back_but_keeps_those_of_the_first_tokens():
    t = PageTable(12, window=70, keep_first=PAGE_SIZE + 3)
    t.open(0)
    t.ensure(0, 6 * PAGE_SIZE)
    assert t.release_behind(0, 6 * PAGE_SIZE) == 2              # pages 2 and 3; 0 and 1 hold kept tokens, 4 and 5 the window
    assert [p >= 0 for p in t.pages(0)] == [True, True, False, False, True, True]
    t.check()
    plain = PageTable(12, window=70)
    plain.open(0)
    plain.ensure(0, 6 * PAGE_SIZE)
    assert plain.release_behind(0, 6 * PAGE_SIZE) == 4


def test_the_plain_implementations_own_properties():
    # pairs and halves rotate the same numbers when the columns are permuted
    x = torch.randn(5, 2, 8, dtype=torch.float64)
    f = P.frequencies(8, 100.0)
    perm = torch.tensor([0, 2, 4, 6, 1, 3, 5, 7])
    assert torch.allclose(P.rotate(x, f, "pairs")[..., perm], P.rotate(x[..., perm], f, "halves"), atol=1e-12)
    # a window of the whole length with kept tokens is plain causal sight
    assert torch.equal(P.visible(6, 6, 2), P.visible(6))
    seen = P.visible(9, 3, 2)
    assert seen[8].tolist() == [True, True, False, False, False, False, True, True, True]
    # the time mixing's first token sees only its own bonus term
    w = P.random_menerax_tensors(CFG, 3)
    h = torch.randn(1, 24, dtype=torch.float64)
    r = P.sub(w, "l0.mix.right.")
    out = P.time_mix(h, r, CFG["layers"][0]["mixer"]["right"], 1e-5)
    m = {s: h * (1 - r["mu." + s]) for s in "rkvg"}
    rr, kk, vv = (m[s] @ r[s].T for s in "rkv")
    o = (rr.view(2, 6) * kk.view(2, 6) * r["u"]).sum(-1, keepdim=True) * vv.view(2, 6)
    want = (P.unit_rms(o, 1e-5).reshape(1, 12) * r["norm"] * P.silu(m["g"] @ r["g"].T)) @ r["o"].T
    assert torch.allclose(out, want, atol=1e-12)
