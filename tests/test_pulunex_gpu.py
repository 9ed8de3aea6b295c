"""The Pulunex parts and whole models on the GPU against the plain implementation of `plain_pulunex.py`: each mechanism
alone; a prompt whole, in pieces down to two tokens and token by token; batches of unequal requests against each alone;
slots and pages used again; keys far away, at page borders and just inside and outside a chunk, in prompts and in
decoding; the first tokens of a sequence; long decoding; sizes that differ in everything (and values that a model may
happen to make equal or 1); greedy generation through `Engine.generate`.  Configurations and weights are made here."""
import copy
import io
import json
import os
import tempfile

import pytest
import torch

import plain_pulunex as P
from rbitnet_amd.cache import Cache
from rbitnet_amd.config import load_config
from rbitnet_amd.config.spec import PartSpec
from rbitnet_amd.engine.context import StepBatch, StepContext
from rbitnet_amd.parts import BuildEnv, build_part
from rbitnet_amd.parts.short_conv import ACT_NONE, ShortConv

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F64 = torch.float64
EPS = 1e-5


@pytest.fixture(autouse=True)
def _same_numbers_every_run():
    torch.manual_seed(20240911)


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
    """float32: every value within 2e-5 of the largest.  bfloat16 rounds activations at every product's input: the root
    mean square error is bounded tightly (a wrong formula, chunk, state or bias moves it by far more), the largest
    single error loosely."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    return _rms(got, want) < 1e-2 and _rel(got, want) < 1e-1


def _close_rows(got, want, dtype) -> bool:
    """Whole models with routed experts: in bfloat16 a router's close call may go the other way for a token now and
    then (its input is rounded), which moves that token's logits and, through the shift, the next one's.  So the bound
    is on the rows: the median row as close as bfloat16 allows, and at most one row in ten further off."""
    if dtype in (torch.float32, "float32"):
        return _rel(got, want) < 2e-5
    want = want.double().cpu()
    err = ((got.double().cpu() - want) ** 2).mean(-1).sqrt() / want.abs().max()
    return float(err.median()) < 6e-3 and float((err > 3e-2).double().mean()) <= 0.1


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


def _run_mixer(lib, part, x, cuts, dtype, pages=8):
    """The mixer on x [T, E] fed in pieces of the given sizes, through a cache of its own."""
    cache = Cache([part.cache_request()], 2, 64 * pages, dtype, DEV)
    cache.alloc_slot()                                    # slot 0 stays idle: the sequence lives in slot 1
    slot = cache.alloc_slot()
    outs, at = [], 0
    for n in cuts:
        ctx = _step(lib, cache, [slot], [n])
        outs.append(part.forward(x[at:at + n].to(DEV, dtype).contiguous(), ctx, cache.view(0, ctx.block_tables)))
        cache.commit([slot], [n])
        at += n
    return torch.cat(outs)


def _one_layer(hidden, mixer, mlp=None, vocab=8):
    return {"architecture": "Pulunex", "vocab": vocab, "width": hidden, "max_positions": 16, "embedding": {"scale": 1.0},
            "logit_scale": 1.0, "norm": {"eps": EPS}, "layers": [{"type": "attention", "mixer": mixer, "mlp": mlp}]}


def _mixer(lib, hidden, m, dtype, seed, change=None):
    """(part, weights by the part's own names) of an attention mixer with random weights."""
    cfg = _one_layer(hidden, m)
    spec = load_config(copy.deepcopy(cfg))[1].layers[0].mixer
    t = P.random_tensors(cfg, seed)
    w = {k[len("l0.mix."):]: v.to(F64) for k, v in t.items() if k.startswith("l0.mix.")}
    if change:
        change(w)
    part = build_part("mixer", spec, _env(lib, hidden, dtype))
    part.load(_place(part, w, dtype))
    return part, w


def _plain_mixer(x, w, m):
    k, v = P.attention_keys_values(x, w, m, EPS)
    return P.talking_attention(x, w, m, EPS, k, v)


# ---------------------------------------------------------------------------- small kernels
def test_norm_with_one_gain_for_all_coordinates(lib):
    for e, dtype in ((40, torch.float32), (256, torch.bfloat16), (50, torch.float32)):
        x, d = torch.randn(9, e, dtype=F64), torch.randn(9, e, dtype=F64)
        g = torch.tensor(1.3, dtype=F64)
        part = build_part("norm", PartSpec("rmsnorm", {"size": e, "eps": 1e-4, "scalar": True, "names": {"weight": ""}}),
                          _env(lib, e, dtype))
        assert part.tensor_specs()[""].shape == ()
        part.load({"": g.float().to(DEV)})
        tol = 5e-6 if dtype == torch.float32 else 8e-3
        assert _rel(part.forward(x.float().to(DEV)), P.scalar_rmsnorm(x, g, 1e-4)) < tol
        xd = x.float().to(DEV)
        assert _rel(part.forward(xd, d.float().to(DEV), out_dtype=torch.float32), P.scalar_rmsnorm(x + d, g, 1e-4)) < 5e-6
        assert _rel(xd, x + d) < 1e-6                       # the sum went into the stream


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_embedding_with_a_scale_and_learned_positions(lib, dtype):
    vocab, e, n_pos = 19, 36, 140
    spec = PartSpec("table", {"name": "embed", "vocab_size": vocab, "scale": 2.5, "positions": {"name": "pos", "max_positions": n_pos}})
    part = build_part("embedding", spec, _env(lib, e, dtype))
    table, pos = _bf(torch.randn(vocab, e, dtype=F64)), _bf(torch.randn(n_pos, e, dtype=F64))
    assert {k: tuple(v.shape) for k, v in part.tensor_specs().items()} == {"embed": (vocab, e), "pos": (n_pos, e)}
    part.load({"embed": table.to(DEV, dtype), "pos": pos.to(DEV, dtype)})
    # two sequences: one starts at its first token, one goes on at position 126 over a page's border
    ids = [[3, 0, 18, 3], [7, 7, 1, 2, 5]]
    ctx = StepContext.for_batch(DEV, StepBatch([0, 1], [0, 126], ids, [], {}), n_compute_units=lib.n_compute_units)
    got = part.forward(ctx)
    want = torch.cat([P.embedding(table, pos, ids[0], 2.5, 0), P.embedding(table, pos, ids[1], 2.5, 126)])
    assert got.dtype == torch.float32 and _rel(got, want) < 1e-6


def test_token_shift_in_pieces_batches_and_a_slot_used_again(lib):
    """h_t + (h_(t-1) - h_t) s as a convolution of two taps whose state is the row before: three sequences in unequal
    pieces down to one token, channels with s = 0 (the row itself) and s = 1 (the row before), zeros before a first token."""
    c = 37
    s = torch.rand(c, dtype=F64)
    s[0], s[1] = 0.0, 1.0
    conv = ShortConv(c, 2, _env(lib, c, torch.float32), residual=True, act=ACT_NONE)
    conv.load(torch.stack([s, -s], dim=1).float().to(DEV))
    cache = Cache([conv.cache_request("token_shift")], 3, 64 * 8, torch.float32, DEV)
    lens = [23, 5, 12]
    xs = [torch.randn(n, c, dtype=F64) for n in lens]
    slots = [cache.alloc_slot() for _ in lens]
    cuts = [[9, 1, 1, 2, 10], [1, 2, 2], [3, 1, 8]]
    got = [[] for _ in lens]
    for r in range(5):
        live = [i for i in range(3) if r < len(cuts[i])]
        q = [cuts[i][r] for i in live]
        at = [sum(cuts[i][:r]) for i in live]
        ctx = _step(lib, cache, [slots[i] for i in live], q)
        x = torch.cat([xs[i][a:a + n] for i, a, n in zip(live, at, q)]).float().to(DEV)
        out = conv.forward(x, ctx, cache.view(0, ctx.block_tables).states["token_shift"], torch.float32)
        cache.commit([slots[i] for i in live], q)
        off = 0
        for i, n in zip(live, q):
            got[i].append(out[off:off + n])
            off += n
    for i in range(3):
        g, want = torch.cat(got[i]), P.token_shift(xs[i], s)
        assert _rel(g, want) < 2e-6, i
        assert _rel(g[1:, 1], xs[i][:-1, 1]) < 1e-6 and float(g[0, 1]) == 0.0 and _rel(g[:, 0], xs[i][:, 0]) < 1e-6
    cache.free_slot(slots[0])
    again = cache.alloc_slot()
    ctx = _step(lib, cache, [again], [4])
    out = conv.forward(xs[2][:4].float().to(DEV), ctx, cache.view(0, ctx.block_tables).states["token_shift"], torch.float32)
    assert _rel(out, P.token_shift(xs[2][:4], s)) < 2e-6


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_biases_unit_heads_and_the_pages(lib, dtype):
    """bias_norm_store alone: first positions, a page's border, keys and values of different sizes laid out with the
    larger one, unit heads on and off, a layer without keys of its own."""
    from rbitnet_amd.parts import CacheRequest
    hq, hk, dim, vdim, pad, n = 3, 1, 12, 20, 20, 70
    cache = Cache([CacheRequest("kv", heads=hk, head_dim=pad)], 1, 128, dtype, DEV)
    slot = cache.alloc_slot()
    ctx = _step(lib, cache, [slot], [n])
    view = cache.view(0, ctx.block_tables)
    width = hq * dim + hk * dim + hk * vdim
    qkv, bias = torch.randn(n, width, dtype=F64), torch.randn(width, dtype=F64)
    tol = 1e-6 if dtype == torch.float32 else 5e-3
    for norm in (True, False):
        q_out = torch.empty(n, hq, pad, dtype=dtype, device=DEV)
        lib.bias_norm_store(qkv.float().to(DEV), bias.float().to(DEV), norm, 1e-3, q_out, view.k_pages, view.v_pages, ctx.tok_pos,
                            ctx.tok_seq, view.block_table, hq, hk, dim, vdim, pad)
        y = qkv + bias
        unit = (lambda a: P.unit_rms(a, 1e-3)) if norm else (lambda a: a)
        want_q, want_k = unit(y[:, :hq * dim].view(n, hq, dim)), unit(y[:, hq * dim:(hq + hk) * dim].view(n, hk, dim))
        assert _rel(q_out[:, :, :dim], want_q) < tol and float(q_out[:, :, dim:].abs().max()) == 0.0
        pages = view.block_table[0].tolist()
        for t in (0, 1, 63, 64, 69):
            kp, vp = view.k_pages[pages[t // 64], :, t % 64], view.v_pages[pages[t // 64], :, t % 64]
            assert _rel(kp[:, :dim], want_k[t]) < tol and float(kp[:, dim:].abs().max()) == 0.0
            assert _rel(vp[:, :vdim], y[t, (hq + hk) * dim:].view(hk, vdim)) < tol
    # queries only (a layer that reads another layer's keys and values): the pages stay as they are
    before = view.k_pages.clone()
    q_out = torch.empty(n, hq, pad, dtype=dtype, device=DEV)
    lib.bias_norm_store(qkv[:, :hq * dim].contiguous().float().to(DEV), bias[:hq * dim].float().to(DEV), True, 1e-3, q_out, None, None,
                        ctx.tok_pos, ctx.tok_seq, view.block_table, hq, hk, dim, vdim, pad)
    assert _rel(q_out[:, :, :dim], P.unit_rms((qkv + bias)[:, :hq * dim].view(n, hq, dim), 1e-3)) < tol
    bits = torch.int32 if dtype == torch.float32 else torch.int16            # pages beyond the sequence hold anything
    assert torch.equal(before.view(bits), view.k_pages.view(bits))


# ---------------------------------------------------------------------------- attention with mixed heads
ATTENTIONS = [
    dict(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.3, mask={"size": 37}),              # values larger, a chunk inside a page
    dict(heads=3, kv_heads=3, dim=24, vdim=8, scale=0.2),                                  # values smaller, no sharing, no chunks
    dict(heads=8, kv_heads=2, dim=64, vdim=64, scale=0.125, mask={"size": 64}),            # the matrix cores' sizes, a chunk a page
    dict(heads=4, kv_heads=1, dim=128, vdim=128, scale=0.09, mask={"size": 100}),
    dict(heads=6, kv_heads=2, dim=64, vdim=128, scale=0.1, mask={"size": 70}),
    dict(heads=1, kv_heads=1, dim=6, vdim=5, scale=1.0, mask={"size": 1}),                 # sees itself only
    dict(heads=2, kv_heads=1, dim=128, vdim=64, scale=0.05, mask={"size": 129}),
    dict(heads=2, kv_heads=1, dim=7, vdim=9, scale=0.4, mask={"size": 65}),                # odd sizes
    dict(heads=34, kv_heads=2, dim=32, vdim=32, scale=0.2, mask={"size": 1000}),           # 17 heads on one, a chunk never left
    dict(heads=16, kv_heads=4, dim=64, vdim=64, scale=0.125),
    dict(heads=32, kv_heads=8, dim=64, vdim=64, scale=0.125, mask={"size": 150}),          # the most heads the matrix cores' kernel takes
    dict(heads=24, kv_heads=3, dim=128, vdim=64, scale=0.09, mask={"size": 96}),
    dict(heads=12, kv_heads=12, dim=64, vdim=32, scale=0.15),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m", ATTENTIONS)
def test_attention_whole_in_pieces_and_token_by_token(lib, m, dtype):
    hidden, t_len = 64, 200
    part, w = _mixer(lib, hidden, m, dtype, seed=m["heads"] + m["dim"])
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = _plain_mixer(x, w, m)
    for cuts in ([t_len], [63, 1, 1, 2, 61, 72], [130] + [1] * 70, [2] * 5 + [190]):
        assert _close(_run_mixer(lib, part, x, cuts, dtype), want, dtype), cuts


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_mixing_the_heads_moves_every_head(lib, dtype):
    """A mixing matrix far from the identity (a head whose weights follow another head's scores alone, one that takes the
    negative of its own): the plain implementation with the identity instead is far away, the part is not."""
    hidden, t_len = 48, 90
    m = dict(heads=4, kv_heads=2, dim=16, vdim=16, scale=0.5, mask={"size": 50})

    def talk(w):
        w["talk"] = torch.tensor([[0, 1, 0, 0], [0.5, 0.5, 0, 0], [0, 0, -1, 0], [1, 1, 1, 1]], dtype=F64)

    part, w = _mixer(lib, hidden, m, dtype, seed=2, change=talk)
    x = _bf(torch.randn(t_len, hidden, dtype=F64))
    want = _plain_mixer(x, w, m)
    unmixed = _plain_mixer(x, dict(w, talk=torch.eye(4, dtype=F64)), m)
    assert _rel(unmixed, want) > 0.2
    for cuts in ([t_len], [40] + [1] * 50):
        assert _close(_run_mixer(lib, part, x, cuts, dtype), want, dtype), cuts


def _aligned(w, heads, zero_bias=True):
    """Every query head's matrix is the key head's, and no biases on q and k: a token whose input is a positive multiple
    of a query's input has the largest score that query can have (unit heads: dim * scale)."""
    w["q"] = w["k"].repeat(heads, 1)
    w["q.b"], w["k.b"] = torch.zeros_like(w["q.b"]), torch.zeros_like(w["k.b"])
    w["talk"] = torch.eye(heads, dtype=F64) + 0.05 * torch.randn(heads, heads, dtype=F64)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("chunk,dim,vdim", [(64, 64, 64), (65, 16, 16), (7, 8, 12), (130, 64, 128), (128, 128, 128)])
def test_a_key_that_stands_out_just_inside_and_just_outside_the_chunk(lib, dtype, chunk, dim, vdim):
    """The first key of a chunk scores as high as a key can with the chunk's last query, whose output then holds its
    value (three times that query's own); the first query of the next chunk has the same input and must not see it.  In a
    prompt and in decoding, the chunk being the sequence's first or a later one."""
    hidden = 64
    m = dict(heads=2, kv_heads=1, dim=dim, vdim=vdim, scale=20.0 / dim, mask={"size": chunk})
    part, w = _mixer(lib, hidden, m, dtype, seed=chunk, change=lambda w: _aligned(w, 2))
    for nth in (0, 1, 2):
        at, inside, outside = chunk * nth, chunk * nth + chunk - 1, chunk * (nth + 1)
        if inside == at:
            continue
        t_len = outside + 5
        x = _bf(torch.randn(t_len, hidden, dtype=F64))
        x[at], x[outside] = _bf(3 * x[inside]), x[inside]
        k, v = P.attention_keys_values(x, w, m, EPS)
        a = P.mixed_weights(x, w, m, EPS, k)
        assert float(a[:, inside, at].min()) > 0.3 and float(a[:, outside, at].max()) == 0.0       # the edge shows in the plain weights
        assert float(a[:, outside, outside].min()) == 1.0
        want = P.talking_attention(x, w, m, EPS, k, v)
        for cuts in ([t_len], [at + 1] + [1] * (t_len - at - 1), [inside, 1, 1, t_len - inside - 2], [outside, 1, 4]):
            got = _run_mixer(lib, part, x, cuts, dtype)
            assert _close(got, want, dtype), (nth, cuts)
            assert _close(got[[inside, outside]], want[[inside, outside]], dtype), (nth, cuts)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_a_far_key_among_hundreds(lib, dtype):
    """Every query is, through its bias, nearly the key of position 2: queries 600 tokens later still find that key among
    all others and give its value, in a prompt and in decoding; with chunks of 256 they do not see it."""
    hidden, t_len = 64, 660
    x = _bf(torch.randn(t_len, hidden, dtype=F64))

    def towards_key_2(w):
        w["q"] = 0.05 * w["q"]
        w["q.b"] = (x[2] @ w["k"].T + w["k.b"]).repeat(4)

    for mask in (None, {"size": 256}):
        m = dict(heads=4, kv_heads=1, dim=64, vdim=64, scale=0.5, mask=mask)
        part, w = _mixer(lib, hidden, m, dtype, seed=5, change=towards_key_2)
        k, v = P.attention_keys_values(x, w, m, EPS)
        a = P.mixed_weights(x, w, m, EPS, k)
        if mask is None:
            assert float(a[:, 600:, 2].min()) > 0.9
        else:
            assert float(a[:, 600:, 2].max()) == 0.0 and float(a[:, 3:256, 2].min()) > 0.9
        want = P.talking_attention(x, w, m, EPS, k, v)
        for cuts in ([t_len], [610] + [1] * 50):
            got = _run_mixer(lib, part, x, cuts, dtype, pages=11)
            assert _close(got, want, dtype), (mask, cuts)
            assert _close(got[600:], want[600:], dtype), (mask, cuts)


@pytest.mark.parametrize("heads,kv_heads,dim,chunk", [(6, 3, 64, 100), (16, 4, 64, 0), (32, 8, 64, 70), (8, 1, 128, 0), (20, 4, 128, 200)])
def test_matrix_core_kernel_for_any_number_of_splits_against_the_kernel_for_any_sizes(lib, heads, kv_heads, dim, chunk):
    """The two kernels on the same bfloat16 queries and pages: three sequences that go on at unequal lengths with unequal
    numbers of new tokens (a page's border, one token, more than 16), the pages dealt out to 1, 2, 3 and 16 workgroups."""
    from rbitnet_amd.parts import CacheRequest
    cache = Cache([CacheRequest("kv", heads=kv_heads, head_dim=dim)], 3, 64 * 24, torch.bfloat16, DEV)
    slots = [cache.alloc_slot() for _ in range(3)]
    past, new = [130, 0, 447], [40, 1, 17]
    cache.reserve(slots, past)
    cache.commit(slots, past)
    ctx = _step(lib, cache, slots, new)
    view = cache.view(0, ctx.block_tables)
    view.k_pages.normal_()
    view.v_pages.normal_()
    n = sum(new)
    q = torch.randn(n, heads, dim, device=DEV).to(torch.bfloat16)
    talk = (torch.eye(heads, device=DEV) + 0.3 * torch.randn(heads, heads, device=DEV)).contiguous()
    want = torch.empty(n, heads * dim, dtype=torch.float32, device=DEV)
    lib.attention_mixed(q.float(), view.k_pages.float(), view.v_pages.float(), want, ctx.tok_pos, ctx.tok_seq, view.block_table, heads,
                        kv_heads, dim, 0.11, talk, chunk, 0)
    for n_splits in (1, 2, 3, 16):
        got = torch.full((n, heads * dim), float("nan"), dtype=torch.bfloat16, device=DEV)
        ws = torch.empty(n_splits * n * heads * (dim + 2), dtype=torch.float32, device=DEV) if n_splits > 1 else None
        lib.attention_mixed_bf16(q, view.k_pages, view.v_pages, got, ctx, view.block_table, heads, kv_heads, dim, 0.11, talk, chunk, 0,
                                 n_splits, ws)
        assert _rel(got, want) < 6e-3, n_splits            # the output's rounding to bfloat16


# ---------------------------------------------------------------------------- feed-forwards
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,ff", [(64, 172), (48, 20), (128, 256)])
def test_dense_feed_forward_with_the_tanh_form_of_gelu(lib, dtype, hidden, ff):
    cfg = _one_layer(hidden, dict(heads=1, kv_heads=1, dim=8, vdim=8, scale=1.0), {"kind": "dense", "ff": ff})
    spec = load_config(copy.deepcopy(cfg))[1].layers[0].feed_forward
    w = {k[len("l0.mlp."):]: v.to(F64) for k, v in P.random_tensors(cfg, ff).items() if k.startswith("l0.mlp.")}
    part = build_part("feed_forward", spec, _env(lib, hidden, dtype))
    assert set(part.tensor_specs()) == {"up", "down"}
    part.load(_place(part, w, dtype))
    for n in (1, 7, 150):
        x = _bf(3 * torch.randn(n, hidden, dtype=F64))                 # large enough for both tails of the activation
        got = part.forward(x.to(DEV, dtype).contiguous(), None)
        assert _close(got, P.dense_gelu(x, w), dtype), n


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("hidden,ff,experts,top,identity,shared", [
    (64, 32, 12, 1, 0, None), (64, 64, 5, 2, 2, 48), (48, 20, 3, 3, 1, 20), (96, 96, 40, 4, 3, 32), (32, 32, 1, 1, 0, 32),
    (32, 32, 1, 2, 1, None), (128, 64, 130, 2, 6, 64), (64, 32, 2, 3, 4, None)])
def test_softmax_router_with_outputs_that_stand_for_the_input(lib, dtype, hidden, ff, experts, top, identity, shared):
    mlp = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity}}
    if shared:
        mlp["shared"] = {"ff": shared}
    cfg = _one_layer(hidden, dict(heads=1, kv_heads=1, dim=8, vdim=8, scale=1.0), mlp)
    spec = load_config(copy.deepcopy(cfg))[1].layers[0].feed_forward
    w = {k[len("l0.mlp."):]: v.to(F64) for k, v in P.random_tensors(cfg, experts + top).items() if k.startswith("l0.mlp.")}
    w["correction"] = w["correction"] * 3        # large enough to change who is chosen: the weights must not hold it
    part = build_part("feed_forward", spec, _env(lib, hidden, dtype))
    part.load(_place(part, w, dtype))
    for n in (1, 7, 16, 150):
        x = _bf(torch.randn(n, hidden, dtype=F64))
        want = P.softmax_experts(x, w, mlp)
        got = part.forward(x.to(DEV, dtype).contiguous(), None)
        if dtype == torch.float32:
            assert _rel(got, want) < 2e-5, n
        else:
            c = (torch.softmax(x @ w["router"].T, dim=-1) + w["correction"]).sort(dim=-1, descending=True).values
            clear = (c[:, top - 1] - c[:, top]) > 2e-3 if top < experts + identity else torch.ones(n, dtype=torch.bool)
            assert int(clear.sum()) >= 0.8 * n - 1
            assert _rms(got[clear], want[clear]) < 1e-2 and _rel(got[clear], want[clear]) < 1e-1, n
        alone = part.forward(x[n // 2:n // 2 + 1].to(DEV, dtype).contiguous(), None)
        assert _rel(alone[0], got[n // 2]) < (1e-5 if dtype == torch.float32 else 2e-2)
    if identity and dtype == torch.float32:
        # the correction lifts the last output above all: every token's result holds s_last * x, and s_last has no correction in it
        w2 = dict(w, correction=torch.cat([torch.zeros(experts + identity - 1, dtype=F64), torch.tensor([50.0], dtype=F64)]))
        part.load(_place(part, w2, dtype))
        x = _bf(torch.randn(9, hidden, dtype=F64))
        assert _rel(part.forward(x.float().to(DEV), None), P.softmax_experts(x, w2, mlp)) < 2e-5


# ---------------------------------------------------------------------------- whole models
def _mix(heads, kv_heads, dim, vdim, scale, chunk=None, **more):
    return dict(heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, mask=None if chunk is None else {"size": chunk}, **more)


def _moe(ff, experts, top, identity, shared=None):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top, "identity": identity}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def _dense(ff):
    return {"kind": "dense", "ff": ff}


def _model_config(vocab, width, positions, emb, logit, eps, layers):
    return {"architecture": "Pulunex", "vocab": vocab, "width": width, "max_positions": positions, "embedding": {"scale": emb},
            "logit_scale": logit, "norm": {"eps": eps}, "layers": [{"type": "attention", "mixer": m, "mlp": f} for m, f in layers]}


# everything different: keys and values of different sizes both ways, chunks that end inside a page, layers that read
# another layer's keys and values with chunks (and head counts) of their own, a layer without a feed-forward
MODEL_A = _model_config(70, 48, 1024, 2.0, 0.5, 1e-5, [
    (_mix(4, 2, 12, 20, 0.3, 37), _dense(64)),
    (_mix(6, 2, 16, 8, 0.25), _moe(24, 6, 2, 2, 40)),
    (_mix(6, 2, 16, 8, 0.2, 64, kv_from=1), None),
    (_mix(4, 2, 16, 8, 0.35, 5, kv_from=1), _moe(16, 3, 3, 0)),
    (_mix(3, 1, 8, 8, 0.5, 129), _dense(40))])
# what a model may happen to have: one head, one expert, all outputs chosen, sizes equal everywhere, factors 1, a chunk of 1
MODEL_B = _model_config(33, 32, 1024, 1.0, 1.0, 1e-6, [
    (_mix(1, 1, 32, 32, 1.0, 1), _moe(32, 1, 1, 0, 32)),
    (_mix(1, 1, 32, 32, 1.0), _dense(32)),
    (_mix(1, 1, 32, 32, 1.0, 32, kv_from=1), None),
    (_mix(2, 2, 32, 32, 1.0, 64), _moe(32, 1, 2, 1))])
# sizes on the matrix cores' grid: heads of 64 and 128, keys of 64 beside values of 128, experts on the matrix cores
MODEL_C = _model_config(320, 128, 1024, 3.0, 2.0, 1e-5, [
    (_mix(4, 1, 128, 128, 0.09, 100), _dense(256)),
    (_mix(8, 2, 64, 64, 0.125, 192), _moe(96, 8, 2, 1, 64)),
    (_mix(4, 2, 64, 128, 0.11, 80), _moe(32, 24, 1, 0, 32)),
    (_mix(4, 1, 128, 128, 0.07, kv_from=0), _dense(128)),
    (_mix(8, 2, 64, 64, 0.1, 64, kv_from=1), _moe(64, 4, 3, 2))])
# sizes off every grid: a width that is no multiple of 4, odd heads, seven experts of ten channels
MODEL_D = _model_config(37, 50, 1024, 0.7, 1.7, 1e-4, [
    (_mix(3, 1, 10, 14, 0.3, 3), _moe(10, 7, 3, 3, 11)),
    (_mix(5, 5, 6, 6, 0.4), None),
    (_mix(6, 2, 9, 3, 0.6, 66), _dense(31)),
    (_mix(5, 5, 6, 6, 0.6, 63, kv_from=1), _moe(9, 2, 1, 1)),
    (_mix(1, 1, 3, 11, 0.9, 130), None)])
MODELS = {"A": (MODEL_A, 31), "B": (MODEL_B, 32), "C": (MODEL_C, 33), "D": (MODEL_D, 34)}
_TMP = tempfile.TemporaryDirectory(prefix="pulunex_models_")
_MADE = {}


def _model(name):
    """(folder, oracle) of a model written once per session: config.json and bfloat16 weights."""
    if name not in _MADE:
        from rbitnet_amd.weights.safetensors_io import save_file
        cfg, seed = MODELS[name]
        tensors = P.random_tensors(cfg, seed)
        if name == "B":           # shifts of exactly 0 and 1: the mixer reads the row itself, or the row before alone
            tensors["l0.shift"] = torch.zeros_like(tensors["l0.shift"])
            tensors["l1.shift"] = torch.ones_like(tensors["l1.shift"])
        folder = os.path.join(_TMP.name, name)
        os.makedirs(folder)
        with open(os.path.join(folder, "config.json"), "w") as f:
            json.dump(cfg, f)
        save_file(os.path.join(folder, "model.safetensors"), list(tensors.items()))
        _MADE[name] = (folder, P.PlainPulunex(copy.deepcopy(cfg), tensors))
    return _MADE[name]


def _tokens(name, n, seed):
    g = torch.Generator().manual_seed(100 * seed + n)
    return torch.randint(0, MODELS[name][0]["vocab"], (n,), generator=g).tolist()


def _engine(name, dtype, **kw):
    import rbitnet_amd
    return rbitnet_amd.Engine.load_path(_model(name)[0], dtype=dtype, max_seq_len=1024, **kw)


@pytest.mark.parametrize("name", ["A", "D"])
def test_every_layer_of_a_model_against_the_plain_stream(name):
    """The residual stream after every layer (float32), so that a fault names its layer."""
    import rbitnet_amd.engine.model as M
    eng = _engine(name, "float32", max_tokens=64 * 4, max_batch=1)
    toks = _tokens(name, 90, 4)
    want = []
    _model(name)[1].logits(toks, want)
    seen = []
    orig = M.run_blocks

    def traced(blocks, schedule, x, ctx, cache, last_norm=None):
        pending = None
        for place, i in enumerate(schedule):
            pending = blocks[i].forward(x, pending, ctx, cache.view(place, ctx.block_tables), next_norm=None)
            seen.append((x + pending if isinstance(pending, torch.Tensor) else x).cpu())
        return pending

    M.run_blocks = traced
    try:
        slot = eng.alloc_slot()
        eng.use_plans = False
        eng.step([(slot, toks)], "last")
    finally:
        M.run_blocks = orig
    assert len(seen) == len(want)
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
    new requests take the freed slots and pages (and the shifted rows those slots held).  Every request's logits are
    those it has alone."""
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
    assert eng.plans.stats["replayed"] > 0          # steps of a shape that came back were issued from their recording


@pytest.mark.parametrize("name,dtype", [("A", "float32"), ("C", "bfloat16")])
def test_long_decoding_and_greedy_generation_through_the_engine(name, dtype):
    """Greedy generation through `Engine.generate` (its scheduler, its decode step) gives the plain implementation's
    greedy tokens for a batch of unequal prompts, past every chunk's end of the model."""
    eng = _engine(name, dtype, max_tokens=64 * 16, max_batch=5)
    oracle = _model(name)[1]
    limits = (150, 40, 90, 12, 25)
    prompts = [_tokens(name, n, 3) for n in (5, 70, 1, 33, 64)]
    results = eng.generate(prompts, max_tokens=list(limits), temperature=0.0)
    for p, r, n in zip(prompts, results, limits):
        assert len(r.tokens) == n and r.finish_reason == "length"
        seq = list(p) + r.tokens
        logits = oracle.logits(seq[:-1])
        margin = 1e-4 if dtype == "float32" else 0.03 * float(logits.abs().max())
        top2 = logits[len(p) - 1:].topk(2, dim=-1)
        greedy = top2.indices[:, 0].tolist()
        clear = (top2.values[:, 0] - top2.values[:, 1]) > margin          # a tie within rounding may go either way
        same = sum(1 for g, t, c in zip(greedy, r.tokens, clear.tolist()) if c and g == t)
        assert same >= (1.0 if dtype == "float32" else 0.9) * int(clear.sum())
        assert int(clear.sum()) > (0.9 if dtype == "float32" else 0.4) * n
    assert eng.stats["decode_tokens"] > 0 and eng.model.graph_safe and eng.model.plan_safe


def test_replay_and_command_line_on_a_model_of_this_design(tmp_path, capsys):
    import numpy as np
    from rbitnet_amd import cli
    from rbitnet_amd.replay import replay
    folder, oracle = _model("B")
    eng = _engine("B", "float32", max_tokens=64 * 6, max_batch=4)
    a, b = _tokens("B", 70, 5), _tokens("B", 9, 6)
    lines = [json.dumps({"step": 0, "entries": [{"id": "a", "tokens": a[:66], "want": [0, 65]},
                                                {"id": "b", "tokens": b[:8], "want": []}], "end": []}),
             json.dumps({"step": 1, "entries": [{"id": "a", "tokens": a[66:67], "want": [0]},
                                                {"id": "b", "tokens": b[8:9], "want": [0]}], "end": ["b"]}),
             json.dumps({"step": 2, "entries": [{"id": "a", "tokens": a[67:], "want": [2]}], "end": ["a"]})]
    log = io.StringIO()
    assert replay(eng, io.StringIO("\n".join(lines) + "\n"), str(tmp_path / "out"), log=log) == 3
    wa, wb = oracle.logits(a), oracle.logits(b)
    vocab = MODELS["B"][0]["vocab"]
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
