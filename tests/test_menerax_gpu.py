"""The Menerax parts and whole models on the GPU against the plain implementation of `plain_menerax.py`: each mechanism
alone; a prompt whole, in pieces down to two tokens and token by token; batches of unequal requests against each alone;
slots and pages used again; keys far away, at page borders, just inside and outside the window and among the kept first
tokens, in prompts and in decoding; the first tokens of a sequence; long decoding; sizes that differ in everything (and
values that a model may happen to make equal or 1); greedy generation through `Engine.generate`.  Configurations and
weights are made here."""
import copy
import io
import json
import os
import tempfile

import pytest
import torch

import plain_menerax as P
from rbitnet_amd.cache import Cache
from rbitnet_amd.config.menerax import MeneraxConfig
from rbitnet_amd.config.spec import PartSpec
from rbitnet_amd.engine.context import StepBatch, StepContext
from rbitnet_amd.parts import BuildEnv, build_part

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
EPS = 1e-5


@pytest.fixture(autouse=True)
def _same_numbers_every_run():
    torch.manual_seed(20250311)


@pytest.fixture(scope="module")
def lib():
    from rbitnet_amd.csrc.lib import kernels
    return kernels()


def _env(lib, hidden, dtype):
    return BuildEnv(hidden_size=hidden, dtype=dtype, device=torch.device(DEV), lib=lib)


def _rel(got, want):
    want = want.double().cpu()
    return float((got.double().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-30))


def _rms(got, want):
    want = want.double().cpu()
    return float(((got.double().cpu() - want) ** 2).mean().sqrt() / want.abs().max().clamp_min(1e-30))


def _close(got, want, dtype) -> bool:
    """float32: every value within 2e-5 of the largest.  bfloat16 rounds activations at every product's input, and a
    recurrent state carries such errors on for hundreds of tokens: the root mean square error is bounded tightly (a
    wrong formula, window, state or kept token moves it by far more), the largest single error loosely."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    return _rms(got, want) < 1e-2 and _rel(got, want) < 1e-1


def _close_rows(got, want, dtype) -> bool:
    """Whole models: every sublayer's output is normed to unit size before it is added, so what bfloat16 rounds off a small
    output is scaled up with it, and the roundings of seven layer runs at tiny widths add up, for some sequences far more
    than for others (measured: medians over a sequence's rows of 0.002 to 0.025 of the largest logit, the worst row 0.16;
    logits of a broken mechanism are 0.3 to 0.5 off).  So the bound is on the rows: the median row, and at most one row in
    ten further off.  The float32 runs of the same models in the same schedules are held to 2e-5."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    want = want.double().cpu()
    err = ((got.double().cpu() - want) ** 2).mean(-1).sqrt() / want.abs().max()
    return float(err.median()) < 4e-2 and float((err > 1.2e-1).double().mean()) <= 0.1


def _bf(t):
    return t.to(torch.bfloat16).to(F64)


def _step(lib, cache, slots, q_lens):
    past = [cache.length(s) for s in slots]
    cache.reserve(slots, q_lens)
    return StepContext.for_batch(DEV, StepBatch(slots, past, [[0] * q for q in q_lens], [], cache.block_tables(slots)),
                                 n_compute_units=lib.n_compute_units)


def _place(part, w, dtype):
    specs = part.tensor_specs()
    return {n: w[n].to(DEV, torch.float32 if specs[n].role == "gain" else dtype).contiguous() for n in specs}


def _requests(part):
    many = getattr(part, "cache_requests", None)
    return [many()] if many else [part.cache_request()]


def _run_mixer(lib, part, x, cuts, dtype, pages=8, **kw):
    """The mixer on x [T, E] fed in pieces of the given sizes, through a cache of its own."""
    cache = Cache(_requests(part), 2, 64 * pages, dtype, DEV)
    cache.alloc_slot()                                    # slot 0 stays idle: the sequence lives in slot 1
    slot = cache.alloc_slot()
    outs, at = [], 0
    for n in cuts:
        ctx = _step(lib, cache, [slot], [n])
        outs.append(part.forward(x[at:at + n].to(DEV, dtype).contiguous(), ctx, cache.view(0, ctx.block_tables), **kw))
        cache.commit([slot], [n])
        at += n
    return outs


def _config(hidden, kind, mixer):
    return MeneraxConfig(vocab=4, width=hidden, norm_eps=EPS, layers=[{"type": kind, "mixer": mixer, "mlp": None}], max_positions=2048)


def _mixer_weights(kind, hidden, mixer, seed):
    cfg = {"vocab": 4, "width": hidden, "layers": [{"type": kind, "mixer": mixer, "mlp": None}]}
    t = P.random_menerax_tensors(cfg, seed)
    return {k[len("l0.mix."):]: v for k, v in t.items() if k.startswith("l0.mix.")}


# ---------------------------------------------------------------------------- small kernels
def test_the_norm_on_a_sublayers_output_with_the_residual_sum(lib):
    for e, dtype in ((40, torch.float32), (256, torch.bfloat16), (50, torch.float32), (4100, torch.bfloat16)):
        x, a, b = (torch.randn(9, e, dtype=F64) for _ in range(3))
        w = _bf(0.3 * torch.randn(e, dtype=F64))
        part = build_part("norm", PartSpec("rmsnorm", {"size": e, "eps": 1e-4, "one_plus": True, "names": {"weight": ""}}),
                          _env(lib, e, dtype))
        part.load({"": w.float().to(DEV)})
        for second, sa, sb in ((None, 1.0, 0.0), (b, 0.7, 1.3)):
            y = sa * a + (sb * second if second is not None else 0)
            want = x + P.norm_around_zero(y, w, 1e-4)
            xd = x.float().to(DEV)
            h = torch.empty(9, e, dtype=dtype, device=DEV)
            part.add_normed(xd, a.float().to(DEV), None if second is None else second.float().to(DEV), sa, sb, h_out=h)
            assert _rel(xd, want) < 2e-6
            assert _rel(h, want) < (2e-6 if dtype == torch.float32 else 5e-3)
        xd = torch.full((9, e), 7.0, device=DEV)
        part.add_normed(xd, a.float().to(DEV), assign=True)                   # behind an embedding: the normed rows alone
        assert _rel(xd, P.norm_around_zero(a, w, 1e-4)) < 2e-6
        rows = torch.tensor([8, 0], dtype=torch.int32, device=DEV)            # as the final norm: chosen rows, 1 + w
        assert _rel(part.forward(x.float().to(DEV), None, rows), P.norm_around_zero(x[[8, 0]], w, 1e-4)) < (
            2e-6 if dtype == torch.float32 else 5e-3)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,ff,limit", [(64, 96, 1.0), (50, 31, 0.4), (128, 256, 7.0)])
def test_the_gated_unit_with_limits(lib, dtype, hidden, ff, limit):
    part = build_part("feed_forward", PartSpec("clamped_glu", {"intermediate_size": ff, "limit": limit, "alpha": 1.702}),
                      _env(lib, hidden, dtype))
    w = {k: _bf(torch.randn(s, dtype=F64) * 0.3) for k, s in (("gate", (ff, hidden)), ("up", (ff, hidden)), ("down", (hidden, ff)))}
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(70, hidden, dtype=F64))
    reached = ((x @ w["gate"].T) > limit).double().mean()
    assert limit > 5 or 0.02 < float(reached) < 0.98                            # the limits are met, and not everywhere
    assert _close(part.forward(x.to(DEV, dtype)), P.feed_forward(x, w, limit), dtype)


# ---------------------------------------------------------------------------- attention through a latent
LATENTS = [
    dict(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=12, kv_rank=10, scale=0.3, rot={"base": 100.0, "dims": 4}),
    dict(heads=4, dim=32, rot_dim=32, vdim=16, q_rank=48, kv_rank=96, scale=0.1, rot={"base": 1e4, "dims": 32}),    # 128 numbers a token
    dict(heads=16, dim=16, rot_dim=16, vdim=24, q_rank=32, kv_rank=40, scale=0.15, rot={"base": 5e5, "dims": 16}),   # 56: padded to 64
    dict(heads=1, dim=5, rot_dim=2, vdim=7, q_rank=3, kv_rank=9, scale=0.5, rot={"base": 7.0, "dims": 2}),           # one head, odd sizes
    dict(heads=20, dim=24, rot_dim=8, vdim=8, q_rank=64, kv_rank=64, scale=0.12, rot={"base": 300.0, "dims": 8}),   # more heads than a decode group takes
    dict(heads=2, dim=64, rot_dim=64, vdim=64, q_rank=128, kv_rank=192, scale=0.08, rot={"base": 1e4, "dims": 64}),  # 256: beyond the matrix cores' sizes
    dict(heads=32, dim=16, rot_dim=16, vdim=8, q_rank=32, kv_rank=48, scale=0.2, rot={"base": 1e3, "dims": 16}),     # 64 a token, two groups of 16 heads
    dict(heads=20, dim=8, rot_dim=16, vdim=16, q_rank=24, kv_rank=112, scale=0.1, rot={"base": 50.0, "dims": 16}),   # 128 a token, two groups of 10
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", LATENTS)
def test_latent_attention_whole_in_pieces_and_token_by_token(lib, p, dtype):
    hidden, t_len = 64, 200
    spec = _config(hidden, "latent_attention", p)._latent(p)
    part = build_part("mixer", spec, _env(lib, hidden, dtype))
    w = _mixer_weights("latent_attention", hidden, p, seed=p["heads"] + p["dim"])
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.latent_attention(x, w, p, EPS)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 72], [130] + [1] * 70, [2] * 5 + [190]):
        assert _close(torch.cat(_run_mixer(lib, part, x, cuts, dtype)), want, dtype), cuts


def test_a_far_key_among_hundreds_through_the_latent(lib):
    """Position 2's input is made so that a query 600 tokens later finds its key above all others; at that distance the
    rotated part must be turned by the true positions."""
    hidden, t_len = 64, 640
    p = dict(heads=4, dim=32, rot_dim=32, vdim=32, q_rank=64, kv_rank=96, scale=0.18, rot={"base": 1e4, "dims": 32})
    w = _mixer_weights("latent_attention", hidden, p, seed=9)
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    x[2] = x[2] * 4
    want = P.latent_attention(x, w, p, EPS)
    base = P.latent_attention(torch.cat([x[:2], x[3:]]), w, p, EPS)
    assert _rel(want[630:], base[629:]) > 1e-2                                  # the far token matters to the last ones
    for dtype in (torch.float32, torch.bfloat16):
        part = build_part("mixer", _config(hidden, "latent_attention", p)._latent(p), _env(lib, hidden, dtype))
        part.load(_place(part, w, dtype))
        for cuts in ([t_len], [600] + [1] * 40):
            assert _close(torch.cat(_run_mixer(lib, part, x, cuts, dtype, pages=11)), want, dtype), (dtype, cuts)


# ---------------------------------------------------------------------------- the windowed attention of a parallel layer
def _left(heads, kv_heads, dim, vdim, conv, dims, base, scale, softcap=None, mask=None, scaling=None):
    rot = {"base": base, "dims": dims}
    if scaling:
        rot["scaling"] = scaling
    out = dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, conv=conv, rot=rot, scale=scale)
    if softcap:
        out["softcap"] = softcap
    if mask:
        out["mask"] = mask
    return out


LEFTS = [
    _left(4, 2, 16, 24, 3, 8, 100.0, 0.3, softcap=5.0, mask={"size": 36, "keep_first": 12}),
    _left(3, 3, 24, 8, 1, 24, 5000.0, 0.2, mask={"size": 70, "keep_first": 0}),                              # one tap, nothing kept
    _left(8, 2, 64, 64, 4, 64, 1e4, 0.11, softcap=20.0, mask={"size": 64, "keep_first": 64},
          scaling={"factor": 4.0, "low": 1.0, "high": 2.0, "original": 64}),                                  # the matrix cores' sizes
    _left(6, 3, 64, 128, 2, 32, 5e5, 0.1, softcap=2.0, mask={"size": 129, "keep_first": 65}),                 # padded to 128
    _left(1, 1, 6, 5, 5, 0, 10.0, 1.0, softcap=1.0, mask={"size": 1, "keep_first": 3}),                       # no rotation, itself and three
    _left(2, 1, 128, 64, 3, 128, 300.0, 0.05),                                                                # no cap, no mask
    _left(5, 5, 7, 9, 9, 6, 20.0, 0.4, softcap=12.0, mask={"size": 3, "keep_first": 130}),                    # odd sizes, kept tokens past a page
]


def _left_part(lib, hidden, p, dtype):
    return build_part("mixer", _config(hidden, "parallel", {"left": p, "right": dict(heads=1, dim=4), "left_scale": 1.0,
                                                          "right_scale": 1.0})._left(p), _env(lib, hidden, dtype))


def _left_weights(hidden, p, seed):
    mixer = {"left": p, "right": dict(heads=1, dim=4, decay_rank=2), "left_scale": 1.0, "right_scale": 1.0}
    return P.sub(_mixer_weights("parallel", hidden, mixer, seed), "left.")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", LEFTS)
def test_windowed_attention_whole_in_pieces_and_token_by_token(lib, p, dtype):
    hidden, t_len = 64, 200
    part = _left_part(lib, hidden, p, dtype)
    w = _left_weights(hidden, p, seed=p["heads"] + p["dim"])
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.windowed_attention(x, w, p, EPS)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 72], [130] + [1] * 70, [2] * 5 + [190]):
        assert _close(torch.cat(_run_mixer(lib, part, x, cuts, dtype)), want, dtype), cuts


@pytest.mark.parametrize("splits", [1, 3, 16])
def test_long_decoding_past_the_window_with_the_pages_dealt_to_several_workgroups(lib, splits):
    """1,300 tokens, the last 60 one by one: the window's pages and the kept tokens' pages are far apart, and the step's
    workgroups share them out (the number of shares forced, as a long context would choose it)."""
    from rbitnet_amd.engine import context as C
    hidden, t_len = 64, 1300
    p = _left(4, 2, 64, 64, 3, 32, 1e4, 0.125, softcap=20.0, mask={"size": 200, "keep_first": 70})
    w = _left_weights(hidden, p, seed=11)
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.windowed_attention(x, w, p, EPS)
    part = _left_part(lib, hidden, p, torch.bfloat16)
    part.load(_place(part, w, torch.bfloat16))
    C.FORCED_DECODE_SPLITS = splits
    try:
        got = torch.cat(_run_mixer(lib, part, x, [t_len - 60] + [1] * 60, torch.bfloat16, pages=22))
    finally:
        C.FORCED_DECODE_SPLITS = None
    assert _close(got, want, torch.bfloat16)
    assert _close(got[-60:], want[-60:], torch.bfloat16)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window,keep,dim,vdim", [(36, 12, 16, 12), (64, 64, 64, 64), (65, 3, 64, 128), (7, 70, 8, 12)])
def test_a_key_that_stands_out_at_every_edge_of_the_mask(lib, dtype, window, keep, dim, vdim):
    """The query's own input is also given to one earlier token, and keys are made from the matrix that makes queries, so that
    this token's key shares the query's softmax with the query's own key wherever the mask lets it: just inside and just outside the window, and as the
    last kept token and the first that is not kept, in a prompt and in decoding.  One tap, no biases, strong norms."""
    hidden = 64
    p = _left(2, 1, dim, vdim, 1, 2, 1000.0, 8.0 / dim, softcap=40.0, mask={"size": window, "keep_first": keep})
    w = _left_weights(hidden, p, seed=window)
    w["k"] = w["q"][:dim].clone()
    for name, rows in (("q", 2 * dim), ("k", dim), ("v", vdim)):
        w[name + ".b"] = torch.zeros(rows, dtype=F64)
        w[name + ".conv"] = torch.ones(rows, 1, dtype=F64)
    w["q.norm"] = w["k.norm"] = torch.full((dim,), 2.0, dtype=F64)
    w["q.norm"][:2] = 0.125                  # the rotated pair turns by a radian a token: it is kept small, so that the copy's score is the query's own
    part = _left_part(lib, hidden, p, dtype)
    part.load(_place(part, w, dtype))
    t_len = keep + window + 70
    query = t_len - 3
    for at, seen in ((query - window + 1, True), (query - window, False), (keep - 1, True), (keep, False)):
        x = _bf(torch.randn(t_len, hidden, dtype=F64))
        x[at] = x[query]
        q = P.norm_plain((x @ w["q"].T).view(t_len, 2, dim), w["q.norm"], EPS)
        k = P.norm_plain((x @ w["k"].T).view(t_len, 1, dim), w["k.norm"], EPS)
        f = P.frequencies(2, 1000.0)
        a = P.attention_weights(P.rotate(q, f, "halves"), P.rotate(k, f, "halves"), p["scale"], P.visible(t_len, window, keep), 40.0)
        if seen:
            assert float(a[0, query, at]) > 0.3                     # the edge shows in the plain weights
        else:
            assert float(a[:, query, at].max()) == 0.0
        want = P.windowed_attention(x, w, p, EPS)
        for cuts in ([t_len], [query] + [1] * 3, [at + 1, query - at - 1, 1, 2]):
            got = torch.cat(_run_mixer(lib, part, x, cuts, dtype))
            assert _close(got, want, dtype), (at, cuts)
            assert _close(got[query - 1:query + 2], want[query - 1:query + 2], dtype), (at, cuts)


# ---------------------------------------------------------------------------- time mixing
TIME_MIXES = [dict(heads=2, dim=32, decay_rank=8), dict(heads=3, dim=12, decay_rank=5), dict(heads=1, dim=64, decay_rank=16),
              dict(heads=6, dim=5, decay_rank=1), dict(heads=2, dim=128, decay_rank=24)]


def _time_mix(lib, hidden, p, dtype, seed):
    part = build_part("mixer", PartSpec("time_mix", dict(p, eps=EPS)), _env(lib, hidden, dtype))
    mixer = {"left": _left(1, 1, 4, 4, 1, 0, 10.0, 1.0), "right": p, "left_scale": 1.0, "right_scale": 1.0}
    w = P.sub(_mixer_weights("parallel", hidden, mixer, seed), "right.")
    return part, w


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("p", TIME_MIXES)
def test_time_mixing_whole_in_pieces_and_token_by_token(lib, p, dtype):
    hidden, t_len = 48, 150
    part, w = _time_mix(lib, hidden, p, dtype, seed=p["heads"] + p["dim"])
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.time_mix(x, w, p, EPS)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 22], [100] + [1] * 50, [2] * 5 + [140], [1] * 20 + [130]):
        assert _close(torch.cat(_run_mixer(lib, part, x, cuts, dtype)), want, dtype), cuts


def test_what_the_first_token_wrote_is_read_much_later_beside_another_sequence(lib):
    """Decays of nearly 1 (w0 far below zero): the state keeps the first token's k v^T for 260 tokens; a second sequence in
    another slot, fed in the same steps, keeps its own."""
    hidden, p, t_len = 32, dict(heads=2, dim=16, decay_rank=4), 260
    part, w = _time_mix(lib, hidden, p, torch.float32, seed=3)
    w["w0"] = torch.full_like(w["w0"], -12.0)
    part.load(_place(part, w, torch.float32))
    xs = [_bf(torch.randn(t_len, hidden, dtype=F64)) for _ in range(2)]
    xs[0][0] = xs[0][0] * 6
    wants = [P.time_mix(x, w, p, EPS) for x in xs]
    gone = P.time_mix(torch.cat([torch.zeros(1, hidden, dtype=F64), xs[0][1:]]), w, p, EPS)
    assert _rel(wants[0][-1:], gone[-1:]) > 1e-2                                # the first token still matters at the end
    cache = Cache(_requests(part), 3, 64, torch.float32, DEV)
    cache.alloc_slot()
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    outs, at = [[], []], 0
    for n in [100, 1, 1, 2, 156]:
        ctx = _step(lib, cache, slots, [n, n])
        x = torch.cat([xs[0][at:at + n], xs[1][at:at + n]]).to(DEV, torch.float32)
        y = part.forward(x, ctx, cache.view(0, ctx.block_tables))
        outs[0].append(y[:n])
        outs[1].append(y[n:])
        cache.commit(slots, [n, n])
        at += n
    for i in range(2):
        assert _close(torch.cat(outs[i]), wants[i], torch.float32), i


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_two_mixers_side_by_side_as_a_weighted_sum(lib, dtype):
    hidden, t_len = 64, 90
    mixer = {"left": _left(4, 2, 16, 8, 3, 8, 100.0, 0.3, softcap=4.0, mask={"size": 30, "keep_first": 4}),
             "right": dict(heads=2, dim=16, decay_rank=4), "left_scale": 0.35, "right_scale": 1.6}
    cfg = _config(hidden, "parallel", mixer)
    part = build_part("mixer", cfg.to_spec().layers[0].mixer, _env(lib, hidden, dtype))
    w = _mixer_weights("parallel", hidden, mixer, seed=2)
    part.load(_place(part, w, dtype))
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = P.parallel_mixer(x, w, mixer, EPS)
    for cuts in ([t_len], [2, 63, 1, 24]):
        terms = _run_mixer(lib, part, x, cuts, dtype, weighted_terms=True)
        got = torch.cat([t.sa * t.a + t.sb * t.b for t in terms])
        assert _close(got, want, dtype), cuts
    from rbitnet_amd.errors import ConfigError
    with pytest.raises(ConfigError, match="weighted sum"):
        _run_mixer(lib, part, x, [t_len], dtype)


# ---------------------------------------------------------------------------- whole models
def _lat(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base):
    return dict(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, scale=scale,
                rot={"base": base, "dims": rot_dim})


def _par(left, heads, dim, rank, ls, rs):
    return {"left": left, "right": dict(heads=heads, dim=dim, decay_rank=rank), "left_scale": ls, "right_scale": rs}


def _ff(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


# everything different from layer to layer; the parallel layer first; layers that run another layer's weights between others
MODEL_A = {"architecture": "Menerax", "vocab": 96, "width": 64, "norm": {"eps": 1e-5}, "layers": [
    {"type": "parallel", "mixer": _par(_left(4, 2, 16, 24, 3, 8, 100.0, 0.3, softcap=6.0, mask={"size": 44, "keep_first": 10}), 2, 16, 4, 0.55, 1.2),
     "mlp": _ff(96, 1.0)},
    {"type": "latent_attention", "mixer": _lat(3, 8, 4, 6, 12, 10, 0.3, 100.0), "mlp": None},
    {"type": "parallel", "mixer": _par(_left(4, 2, 16, 24, 3, 8, 100.0, 0.3, softcap=6.0, mask={"size": 44, "keep_first": 10}), 2, 16, 4, 0.55, 1.2),
     "mlp": _ff(96, 1.0), "weights_of": 0},
    {"type": "latent_attention", "mixer": _lat(4, 16, 8, 12, 24, 40, 0.2, 5e4), "mlp": _ff(40, 0.5)},
    {"type": "parallel", "mixer": _par(_left(2, 1, 8, 8, 2, 8, 5e5, 0.4, mask={"size": 9, "keep_first": 0},
                                              scaling={"factor": 4.0, "low": 1.0, "high": 4.0, "original": 32}), 4, 8, 3, 1.3, 0.4),
     "mlp": _ff(24, 3.0)},
    {"type": "latent_attention", "mixer": _lat(3, 8, 4, 6, 12, 10, 0.3, 100.0), "mlp": None, "weights_of": 1},
    {"type": "latent_attention", "mixer": _lat(3, 8, 4, 6, 12, 10, 0.3, 100.0), "mlp": None, "weights_of": 1}]}
# values that a model may happen to make equal or 1: one head everywhere, one tap, nothing kept, scales of 1, one layer of each
MODEL_B = {"architecture": "Menerax", "vocab": 50, "width": 32, "norm": {"eps": 1e-6}, "layers": [
    {"type": "latent_attention", "mixer": _lat(1, 32, 32, 32, 32, 32, 1.0, 1e4), "mlp": _ff(32, 1.0)},
    {"type": "parallel", "mixer": _par(_left(1, 1, 32, 32, 1, 32, 1e4, 1.0, mask={"size": 1, "keep_first": 1}), 1, 32, 1, 1.0, 1.0),
     "mlp": None}]}
# sizes on the matrix cores' grid: 128 numbers a token through the latent, heads of 64 and 128, a window of whole pages
MODEL_C = {"architecture": "Menerax", "vocab": 320, "width": 128, "norm": {"eps": 1e-5}, "layers": [
    {"type": "latent_attention", "mixer": _lat(8, 32, 32, 32, 64, 96, 0.12, 1e4), "mlp": _ff(256, 2.0)},
    {"type": "parallel", "mixer": _par(_left(8, 2, 64, 64, 4, 32, 2e5, 0.11, softcap=25.0, mask={"size": 128, "keep_first": 64},
                                              scaling={"factor": 6.0, "low": 1.0, "high": 3.0, "original": 256}), 2, 64, 16, 0.5, 1.2),
     "mlp": _ff(128, 1.5)},
    {"type": "latent_attention", "mixer": _lat(8, 32, 32, 32, 64, 96, 0.12, 1e4), "mlp": _ff(256, 2.0), "weights_of": 0},
    {"type": "parallel", "mixer": _par(_left(4, 4, 128, 64, 3, 64, 1e4, 0.09, softcap=10.0, mask={"size": 70, "keep_first": 5}), 4, 32, 8, 1.0, 0.7),
     "mlp": _ff(256, 4.0)}]}
# sizes off every grid: a width that is no multiple of 4, odd heads, nine taps and one
MODEL_D = {"architecture": "Menerax", "vocab": 37, "width": 50, "norm": {"eps": 1e-4}, "layers": [
    {"type": "parallel", "mixer": _par(_left(3, 1, 10, 14, 9, 6, 33.0, 0.3, softcap=3.0, mask={"size": 3, "keep_first": 2}), 3, 5, 3, 0.9, 0.8),
     "mlp": _ff(31, 0.8)},
    {"type": "latent_attention", "mixer": _lat(5, 6, 2, 7, 9, 11, 0.4, 7.0), "mlp": None},
    {"type": "parallel", "mixer": _par(_left(5, 5, 6, 6, 1, 2, 7.0, 0.4, mask={"size": 67, "keep_first": 66}), 1, 3, 2, 1.0, 2.0),
     "mlp": _ff(9, 5.0)}]}
MODELS = {"A": (MODEL_A, 21), "B": (MODEL_B, 22), "C": (MODEL_C, 23), "D": (MODEL_D, 24)}
_TMP = tempfile.TemporaryDirectory(prefix="menerax_models_")
_MADE = {}


def _model(name):
    """(folder, oracle) of a model written once per session: config.json (without the size that only the weights know)
    and bfloat16 weights."""
    if name not in _MADE:
        from rbitnet_amd.weights.safetensors_io import save_file
        cfg, seed = MODELS[name]
        tensors = P.random_menerax_tensors(cfg, seed)
        stored = copy.deepcopy(cfg)
        for layer in stored["layers"]:
            if layer["type"] == "parallel":
                layer["mixer"]["right"].pop("decay_rank")
        folder = os.path.join(_TMP.name, name)
        os.makedirs(folder)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(stored, f)
        save_file(os.path.join(folder, "model.safetensors"), [(k, v.to(torch.bfloat16)) for k, v in tensors.items()])
        _MADE[name] = (folder, P.PlainMenerax(copy.deepcopy(cfg), tensors))
    return _MADE[name]


def _tokens(name, n, seed):
    g = torch.Generator().manual_seed(100 * seed + n)
    return torch.randint(0, MODELS[name][0]["vocab"], (n,), generator=g).tolist()


def _engine(name, dtype, **kw):
    import rbitnet_amd
    return rbitnet_amd.Engine.load_path(_model(name)[0], dtype=dtype, max_seq_len=1024, **kw)


def test_every_layer_of_a_model_against_the_plain_stream():
    """The residual stream after every layer run (float32), so that a fault names its layer."""
    from rbitnet_amd.parts import block as B
    eng = _engine("A", "float32", max_tokens=64 * 4, max_batch=1)
    toks = _tokens("A", 90, 4)
    want = _model("A")[1].streams(toks)[1:]
    seen = []
    orig = B.OutNormBlock.forward

    def traced(self, x, pending, ctx, view, next_norm=None):
        out = orig(self, x, pending, ctx, view, next_norm)
        seen.append(x.detach().clone().cpu())
        return out

    B.OutNormBlock.forward = traced
    try:
        slot = eng.alloc_slot()
        eng.use_plans = False
        eng.step([(slot, toks)], "last")
    finally:
        B.OutNormBlock.forward = orig
    assert len(seen) == len(want) == 7
    for i, (g, w) in enumerate(zip(seen, want)):
        assert _rel(g, w) < 2e-5, i


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_model_whole_in_pieces_and_decoded(name, dtype):
    eng = _engine(name, dtype, max_tokens=64 * 12, max_batch=3)
    toks = _tokens(name, 200, 1)
    want = _model(name)[1].logits(toks)
    for cuts in ([200], [130] + [1] * 70, [2, 2, 3, 57, 64, 1, 65, 6], [1] * 5 + [195]):
        slot = eng.alloc_slot()
        out, at = [], 0
        for n in cuts:
            out.append(eng.step([(slot, toks[at:at + n])], "all"))
            at += n
        eng.free_slot(slot)
        assert _close_rows(torch.cat(out), want, dtype), cuts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])
def test_batches_of_unequal_requests_and_slots_used_again(name, dtype):
    """Four requests of 1 to 150 tokens start together and are decoded together, the short ones leaving early; then two
    new requests take the freed slots and pages.  Every request's logits are those it has alone."""
    eng = _engine(name, dtype, max_tokens=64 * 8, max_batch=4)
    oracle = _model(name)[1]
    for wave, lens in enumerate(([1, 150, 67, 30], [64, 129])):
        seqs = [_tokens(name, n + 12, 7 + wave) for n in lens]
        want = [oracle.logits(s) for s in seqs]
        slots = [eng.alloc_slot() for _ in seqs]
        got = [[] for _ in seqs]
        logits = eng.step([(sl, s[:n]) for sl, s, n in zip(slots, seqs, lens)], "all")
        off = 0
        for i, n in enumerate(lens):
            got[i].append(logits[off:off + n])
            off += n
        ends = [n + (3 + 4 * i if i < 3 else 12) for i, n in enumerate(lens)]       # they leave at different steps
        at = list(lens)
        live = list(range(len(seqs)))
        while live:
            logits = eng.step([(slots[i], [seqs[i][at[i]]]) for i in live], "last")
            for row, i in enumerate(live):
                got[i].append(logits[row:row + 1])
                at[i] += 1
            for i in [i for i in live if at[i] >= min(ends[i], len(seqs[i]))]:
                eng.free_slot(slots[i])
                live.remove(i)
        for i in range(len(seqs)):
            g = torch.cat(got[i])
            assert _close_rows(g, want[i][:g.shape[0]], dtype), (wave, i)
        eng.cache.check()


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_long_decoding_and_greedy_generation_through_the_engine(name, dtype):
    """Greedy generation through `Engine.generate` (its scheduler, its captured decode step) gives the plain
    implementation's greedy tokens for a batch of unequal prompts, past every window of the model."""
    eng = _engine(name, dtype, max_tokens=64 * 16, max_batch=5)
    oracle = _model(name)[1]
    limits = (150, 40, 90, 12, 25)
    prompts = [_tokens(name, n, 3) for n in (5, 70, 1, 33, 64)]
    results = eng.generate(prompts, max_tokens=list(limits), temperature=0.0)
    margin = 1e-4 if dtype == "float32" else 0.15
    for p, r, n in zip(prompts, results, limits):
        assert len(r.tokens) == n and r.finish_reason == "length"
        seq = list(p) + r.tokens
        logits = oracle.logits(seq[:-1])
        top2 = logits[len(p) - 1:].topk(2, dim=-1)
        greedy = top2.indices[:, 0].tolist()
        clear = (top2.values[:, 0] - top2.values[:, 1]) > margin          # a tie within rounding may go either way
        same = sum(1 for g, t, c in zip(greedy, r.tokens, clear.tolist()) if c and g == t)
        assert same >= (1.0 if dtype == "float32" else 0.95) * int(clear.sum())
        assert int(clear.sum()) > (0.9 if dtype == "float32" else 0.5) * n
    assert eng.stats["decode_tokens"] > 0 and eng.model.graph_safe and eng.model.plan_safe


def _random_config(rng):
    """A model whose every size, constant, layer order and shared layer is drawn: what no hand-made model thought of."""
    def latent():
        rot = rng.choice([0, 2, 4, 8, 16, 32, 64])
        out = dict(heads=rng.choice([1, 2, 3, 4, 8, 16, 24, 32]), dim=rng.choice([8, 16, 32, 64, 128]), rot_dim=rot, vdim=rng.choice([8, 16, 32, 64]),
                   q_rank=rng.choice([16, 24, 64, 128]), kv_rank=rng.choice([8, 24, 32, 48, 64, 96, 112, 128]), scale=rng.choice([0.05, 0.125, 0.2]))
        if rot:
            out["rot"] = {"base": rng.choice([100.0, 1e4, 5e5]), "dims": rot}
        return out

    def parallel():
        dim, kvh, group = rng.choice([8, 16, 32, 64, 128]), rng.choice([1, 2, 4]), rng.choice([1, 2, 3, 4, 8, 20])
        dims = rng.choice([0, 2, dim // 2, dim])
        rot = {"base": rng.choice([1e4, 2e5]), "dims": dims - dims % 2}
        if rot["dims"] and rng.random() < 0.5:
            rot["scaling"] = {"factor": rng.choice([2.0, 6.0]), "low": 1.0, "high": rng.choice([2.0, 3.0]), "original": rng.choice([16, 64, 1024])}
        left = dict(heads=kvh * group, kv_heads=kvh, dim=dim, vdim=rng.choice([8, 16, 48, 64, 128]), conv=rng.choice([1, 2, 3, 4, 7]), rot=rot,
                    scale=rng.choice([0.1, 0.125, 0.3]))
        if rng.random() < 0.8:
            left["softcap"] = rng.choice([5.0, 25.0, 50.0])
        if rng.random() < 0.85:
            left["mask"] = {"size": rng.choice([1, 7, 36, 64, 100, 128, 200]), "keep_first": rng.choice([0, 1, 4, 12, 64, 70, 130])}
        right = dict(heads=rng.choice([1, 2, 6, 8]), dim=rng.choice([8, 16, 32, 64]), decay_rank=rng.choice([1, 4, 16, 24]))
        return {"left": left, "right": right, "left_scale": rng.choice([0.5, 1.0, 1.5]), "right_scale": rng.choice([0.4, 1.2])}

    layers = []
    for _ in range(rng.choice([2, 3, 4])):
        kind = rng.choice(["latent_attention", "parallel"])
        mlp = None if rng.random() < 0.2 else {"kind": "dense", "ff": rng.choice([16, 40, 64, 96, 256]), "limit": rng.choice([0.5, 2.0, 7.0])}
        layers.append({"type": kind, "mixer": latent() if kind == "latent_attention" else parallel(), "mlp": mlp})
    for _ in range(rng.choice([0, 1, 2])):               # layers that run another layer's weights, anywhere behind it
        owners = [i for i, l in enumerate(layers) if "weights_of" not in l]
        j = rng.choice(owners)
        at = rng.randrange(j + 1, len(layers) + 1)
        for l in layers:                                  # the layers behind the new one move on by one
            if l.get("weights_of") is not None and l["weights_of"] >= at:
                l["weights_of"] += 1
        layers.insert(at, dict(copy.deepcopy({k: v for k, v in layers[j].items() if k != "weights_of"}), weights_of=j))
    return {"architecture": "Menerax", "vocab": rng.choice([37, 96, 300]), "width": rng.choice([32, 48, 64, 96, 128, 160, 256]),
            "norm": {"eps": rng.choice([1e-5, 1e-6])}, "layers": layers}


@pytest.mark.parametrize("seed", [16, 17, 19, 27, 29, 38])
def test_models_drawn_at_random_whole_in_pieces_decoded_and_batched(seed, tmp_path):
    import random
    import rbitnet_amd
    from rbitnet_amd.weights.safetensors_io import save_file
    cfg = _random_config(random.Random(seed))
    tensors = P.random_menerax_tensors(cfg, seed)
    oracle = P.PlainMenerax(copy.deepcopy(cfg), tensors)
    stored = copy.deepcopy(cfg)
    for layer in stored["layers"]:
        if layer["type"] == "parallel":
            layer["mixer"]["right"].pop("decay_rank")
    with open(tmp_path / "config.json", "w") as f:
        json.dump(stored, f)
    save_file(str(tmp_path / "model.safetensors"), [(k, v.to(torch.bfloat16)) for k, v in tensors.items()])
    g = torch.Generator().manual_seed(seed)
    seqs = [torch.randint(0, cfg["vocab"], (n,), generator=g).tolist() for n in (210, 75, 9)]
    want = [oracle.logits(s) for s in seqs]

    def rows(got, ref):
        ref = ref.double().cpu()
        return ((got.double().cpu() - ref) ** 2).mean(-1).sqrt() / ref.abs().max()

    for dtype in ("float32", "bfloat16"):
        eng = rbitnet_amd.Engine.load_path(str(tmp_path), dtype=dtype, max_seq_len=512, max_tokens=64 * 12, max_batch=4)
        slot = eng.alloc_slot()
        whole = eng.step([(slot, seqs[0])], "all")
        eng.free_slot(slot)
        slot, parts, at = eng.alloc_slot(), [], 0
        for n in [3, 61, 2, 64, 40] + [1] * 40:
            parts.append(eng.step([(slot, seqs[0][at:at + n])], "all"))
            at += n
        eng.free_slot(slot)
        slots, heads = [eng.alloc_slot() for _ in seqs], [180, 60, 1]
        logits = eng.step([(sl, q[:h]) for sl, q, h in zip(slots, seqs, heads)], "all")
        got = [[logits[sum(heads[:i]):sum(heads[:i + 1])]] for i in range(3)]
        at, live = list(heads), [0, 1, 2]
        while live:
            logits = eng.step([(slots[i], [seqs[i][at[i]]]) for i in live], "last")
            for r, i in enumerate(live):
                got[i].append(logits[r:r + 1])
                at[i] += 1
            for i in [i for i in live if at[i] >= len(seqs[i])]:
                eng.free_slot(slots[i])
                live.remove(i)
        eng.cache.check()
        errs = [rows(whole, want[0]), rows(torch.cat(parts), want[0])] + [rows(torch.cat(got[i]), want[i]) for i in range(3)]
        for e in errs:
            if dtype == "float32":
                assert float(e.max()) < 5e-5, (seed, dtype)
            else:
                assert float(e.median()) < 4e-2 and float((e > 1.2e-1).double().mean()) <= 0.1, (seed, dtype)
        del eng


def test_replay_and_command_line_on_a_model_of_this_design(tmp_path, capsys):
    import numpy as np
    from rbitnet_amd import cli
    from rbitnet_amd.replay import replay
    folder, oracle = _model("D")
    eng = _engine("D", "float32", max_tokens=64 * 6, max_batch=4)
    a, b = _tokens("D", 70, 5), _tokens("D", 9, 6)
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]},
                                                {"id": "b", "tokens": b[:8], "want": []}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]},
                                                {"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": a[67:], "want": [2]}], "end": ["a"]})]
    log = io.StringIO()
    assert replay(eng, io.StringIO("\n".join(lines) + "\n"), str(tmp_path / "out"), log=log) == 3
    wa, wb = oracle.logits(a), oracle.logits(b)
    vocab = MODELS["D"][0]["vocab"]
    got = [np.fromfile(tmp_path / "out" / f"{i}.f32", dtype="<f4").reshape(-1, vocab) for i in range(3)]
    assert _close(torch.from_numpy(got[0]), wa[[0, 65]], "float32")
    assert _close(torch.from_numpy(got[1]), torch.stack([wa[66], wb[8]]), "float32")
    assert _close(torch.from_numpy(got[2]), wa[[69]], "float32")
    assert eng.cache.live_slots == []
    del eng
    capsys.readouterr()
    assert cli.main(["generate", "--model", folder, "--dtype", "float32", "--prompt-ids", ",".join(str(t) for t in b),
                     "--max-tokens", "5", "--temperature", "0"]) == 0
    rec = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert len(rec["tokens"]) == 5 and rec["tokens"][0] == int(oracle.logits(b)[-1].argmax())
