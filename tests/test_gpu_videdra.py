"""The Videdra design on the GPU against the plain implementation: every mechanism alone (the
two-map attention, a layer that reads another's keys and values, retention, the norms around a
sublayer, routed experts beside a gated shared one, the tanh-gelu gate), masks whose edges are
made to show, then whole models replayed whole, with a decoded tail, in portions down to two
tokens, from the first token on, mixed in a pool so small that pages and slots are used again,
configurations nobody chose, and greedy generation through the engine's entry point, its
scheduler and the command line."""

from __future__ import annotations

import pytest
import torch

from tests import helpers, replay_schedules as schedules
from tests.plain import videdra_plain as plain
from tests.test_gpu_larozen import bind_random, rnd, run_mixer_in_portions, settle
from tests.videdra_cases import (CASES, attention, dense, folder_for, layer, moe, retention,
                                 write_folder)

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BOTH = [torch.float32, torch.bfloat16]
ATT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "gate": "g", "lq1": "lq1", "lk1": "lk1",
             "lq2": "lq2", "lk2": "lk2"}
RET_NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o"}
FF_NAMES = {"gate": "gate", "up": "up", "down": "down"}


def plain_names(params, prefix="p."):
    """The part's local names ('q.weight', 'lq1') as the plain implementation calls them."""
    return {prefix + (n[:-len(".weight")] if n.endswith(".weight") else n): t
            for n, t in params.items()}


def sharpen(part, params, dtype, names, factor):
    """Scales the named tensors and binds again: with larger queries a map sits on few keys."""
    for n in names:
        params[n] = (params[n] * factor).to(dtype).float()
    part.bind({n: t.to(dtype).to(DEV) for n, t in params.items()}, dtype, DEV)


# float32 results are held to float32 tolerances relative to the size of the outputs.  The
# bfloat16 bound is derived: the plain implementation run with bfloat16 roundings between its
# products says what the format costs on that input; the engine, which rounds at other places
# (the activations of an expert, a head's gated output), may be off by BF16_SLACK times that.
BF16_SLACK = 2.0


def close(got, want, dtype, rounded=None):
    if dtype == torch.float32:
        size = max(1.0, float(want.abs().max()))
        torch.testing.assert_close(got, want, atol=2e-5 * size, rtol=2e-5)
        return
    cost = float((rounded - want).abs().max())
    worst = float((got - want).abs().max())
    assert worst <= BF16_SLACK * cost + 1e-3, f"off by {worst:.3e}; bfloat16 costs the plain run {cost:.3e}"


def compare(got, run, dtype):
    """`run(to, r)` is the plain result with inputs and weights cast by `to` and roundings `r`.
    The truth is the float64 run.  float32: float32 tolerances relative to the size of the
    outputs, plus three times what float32 costs the plain implementation (the difference of
    two maps is divided by its own root mean square: where the maps nearly cancel, the last
    bits show).  bfloat16: BF16_SLACK times what the format costs the plain run."""
    want = run(torch.Tensor.double, plain.same).float()
    assert got.shape == want.shape and torch.isfinite(got).all()
    worst = float((got - want).abs().max())
    if dtype == torch.float32:
        own = float((run(torch.Tensor.float, plain.same) - want).abs().max())
        bound = 2e-5 * max(1.0, float(want.abs().max())) + 3.0 * own
    else:
        bound = BF16_SLACK * float((run(torch.Tensor.float, plain.to_bf16) - want).abs().max()) + 1e-3
    assert worst <= bound, f"off by {worst:.3e}, allowed {bound:.3e}"
    return want


# ------------------------------------------------------------------- mechanisms, one by one


def two_map_attention(hidden, heads, kv_heads, dim, vdim, scale, diff, mask, rot, **more):
    from mercury_amd.parts import Attention, NoPosition, RotaryPosition

    position = RotaryPosition(dim, rot[0], rotary_dim=rot[1]) if rot and rot[1] else NoPosition()
    return Attention(hidden, heads, kv_heads, 2 * dim, position, qkv_bias=False, o_bias=False,
                     scale=scale, window=mask[0] if mask else None, names=ATT_NAMES, value_dim=vdim,
                     norm_eps=1e-5, keep_first=mask[1] if mask else 0, maps=2, diff_init=diff,
                     head_gate=True, **more)


ATTENTION_SIZES = {
    "grouped-window-partly-turned": (64, 4, 2, 16, 24, 0.2, 0.25, (12, 3), (10000.0, 8)),
    "odd-one-group-whole-turn": (100, 3, 1, 10, 12, 0.3, 0.35, (7, 2), (300.0, 10)),
    "no-window-no-turn": (64, 2, 2, 8, 16, 0.35, 0.1, None, None),
    "window-that-keeps-nothing": (72, 6, 3, 16, 16, 0.25, 0.5, (9, 0), (5000.0, 16)),
    "keeps-more-than-the-window": (64, 2, 1, 16, 40, 0.25, 0.3, (4, 11), (800.0, 4)),
    "sized": (128, 8, 2, 64, 128, 0.125, 0.3, (20, 4), (10000.0, 64)),
    "window-of-one": (64, 4, 4, 32, 8, 0.2, 0.2, (1, 1), (10000.0, 32)),
    "maps-of-32-grouped": (64, 6, 2, 32, 64, 0.2, 0.3, (14, 2), (10000.0, 16)),
    "maps-of-128-no-window": (128, 2, 1, 128, 64, 0.1, 0.2, None, (10000.0, 128)),
}


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("sizes", ATTENTION_SIZES.values(), ids=ATTENTION_SIZES.keys())
def test_two_map_attention_alone(dtype, sizes):
    """Two softmax maps a head over the same values, combined, normed and gated per head; over
    portions of 21, 2, 9, 1, 1 and 6 tokens (pages of 16)."""
    hidden, heads, kv_heads, dim, vdim, scale, diff, mask, rot = sizes
    part = two_map_attention(hidden, heads, kv_heads, dim, vdim, scale, diff, mask, rot)
    params = bind_random(part, dtype, scale=0.25, seed=3)
    sharpen(part, params, dtype, ["q.weight"], 3.0)
    x = rnd(40, hidden, seed=30).to(dtype)
    got = run_mixer_in_portions(part, x, dtype, hidden)
    m = attention(heads, kv_heads, dim, vdim, scale, diff, mask, rot)
    at = torch.arange(40)

    def run(to, r):
        names = {k: to(v) for k, v in plain_names(params).items()}
        return plain.differential_attention(to(x), names, "p.", m, 1e-5, at, r=r).float()

    want = compare(got, run, dtype)
    # the second map and the gate matter: with another lambda, or no gate, the result is another
    other = dict(plain_names(params))
    other["p.lq2"] = other["p.lq2"] + 0.3
    assert (plain.differential_attention(x.float(), other, "p.", m, 1e-5, at) - want).abs().max() > 1e-2
    other = dict(plain_names(params))
    other["p.g"] = torch.zeros_like(other["p.g"])
    assert (plain.differential_attention(x.float(), other, "p.", m, 1e-5, at) - want).abs().max() > 1e-2


@pytest.mark.parametrize("dim", [32, 64, 128])
@pytest.mark.parametrize("vdim", [32, 64, 128])
@pytest.mark.parametrize("page", [16, 64])
def test_every_width_the_matrix_core_attention_is_compiled_for(dim, vdim, page):
    """Maps of 32, 64 and 128 dims over values of 32, 64 and 128 in bfloat16 (one of the nine
    pairs runs in float32 arithmetic), pages of 16 and of 64 tokens: 75 tokens in a window of
    40 that keeps 3, in two portions, then token by token."""
    hidden, heads, kv_heads = 64, 4, 2
    mask, rot = (40, 3), (10000.0, dim // 2)
    part = two_map_attention(hidden, heads, kv_heads, dim, vdim, dim ** -0.5, 0.3, mask, rot)
    params = bind_random(part, torch.bfloat16, scale=0.25, seed=dim + vdim)
    sharpen(part, params, torch.bfloat16, ["q.weight"], 4.0)
    n = 75
    x = rnd(n, hidden, seed=31).to(torch.bfloat16)
    portions = ((0, 37), (37, 21)) + tuple((i, 1) for i in range(58, n))
    got = run_mixer_in_portions(part, x, torch.bfloat16, hidden, pages=8 * 64 // page, page=page,
                                portions=portions)
    m = attention(heads, kv_heads, dim, vdim, dim ** -0.5, 0.3, mask, rot)
    at = torch.arange(n)

    def run(to, r):
        names = {k: to(v) for k, v in plain_names(params).items()}
        return plain.differential_attention(to(x), names, "p.", m, 1e-5, at, r=r).float()

    compare(got, run, torch.bfloat16)


EDGE_MASKS = [(12, 3), (16, 1), (17, 16), (33, 2), (5, 0)]


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("widths", [(16, 24), (32, 32), (64, 128)], ids=["maps16", "maps32", "maps64"])
@pytest.mark.parametrize("mask", EDGE_MASKS, ids=[f"window{w}-keeps{k}" for w, k in EDGE_MASKS])
def test_the_edges_of_a_window_and_of_the_kept_tokens_show(dtype, mask, widths):
    """Queries so large that a map sits on one or two keys: among a few hundred (query, head,
    map) some sit on the key just inside the window, on the one just outside, on the last kept
    token, on the first one not kept.  A mask one token wider or narrower, or one that keeps
    one token more or fewer, gives the plain implementation another result, in the prompt
    (58 tokens, two portions) and in the 38 tokens decoded one by one; the kernels give the
    mask's own.  Maps of 32 and of 64 dims run on the matrix cores in bfloat16 (blocks of 32
    keys, four wavefronts taking them in turn), maps of 16 in float32 arithmetic."""
    hidden, heads, kv_heads, (dim, vdim) = 64, 4, 2, widths
    part = two_map_attention(hidden, heads, kv_heads, dim, vdim, 0.25, 0.3, mask, (10000.0, 8))
    params = bind_random(part, dtype, scale=0.25, seed=11)
    sharpen(part, params, dtype, ["q.weight"], 12.0)
    n, prompt = 96, 58
    x = rnd(n, hidden, seed=12).to(dtype)
    portions = ((0, 37), (37, prompt - 37)) + tuple((i, 1) for i in range(prompt, n))
    got = run_mixer_in_portions(part, x, dtype, hidden, portions=portions)
    at = torch.arange(n)
    names = plain_names(params)

    def run(size, keep, r=plain.same, to=torch.Tensor.float):
        m = attention(heads, kv_heads, dim, vdim, 0.25, 0.3, (size, keep), (10000.0, 8))
        return plain.differential_attention(to(x), {k: to(v) for k, v in names.items()}, "p.", m,
                                            1e-5, at, r=r).float()

    want = compare(got, lambda to, r: run(*mask, r=r, to=to), dtype)
    size, keep = mask
    wrong = [(size + 1, keep), (size - 1, keep), (size, keep + 1)] + ([(size, keep - 1)] if keep else [])
    for other in wrong:
        if other[0] == 0:
            continue
        off = (run(*other) - want).abs().amax(-1)
        assert off[:prompt].max() > 0.05 and off[prompt:].max() > 0.05, f"mask {other} looks like {mask}"


@pytest.mark.parametrize("dtype", [torch.bfloat16])
@pytest.mark.parametrize("mask", [None, (700, 40)], ids=["sees-all", "window700-keeps40"])
def test_decoding_over_many_keys_splits_them_over_workgroups(dtype, mask):
    """A prompt of 1,900 tokens, then 24 decoded ones: a step of single tokens deals a
    sequence's key blocks over up to eight workgroups and merges their parts."""
    hidden, heads, kv_heads, dim, vdim = 64, 4, 2, 32, 64
    part = two_map_attention(hidden, heads, kv_heads, dim, vdim, 0.2, 0.3, mask, (10000.0, 32))
    params = bind_random(part, dtype, scale=0.25, seed=23)
    sharpen(part, params, dtype, ["q.weight"], 8.0)
    n, prompt = 1924, 1900
    x = rnd(n, hidden, seed=24).to(dtype)
    portions = ((0, prompt),) + tuple((i, 1) for i in range(prompt, n))
    got = run_mixer_in_portions(part, x, dtype, hidden, pages=128, portions=portions)
    m = attention(heads, kv_heads, dim, vdim, 0.2, 0.3, mask, (10000.0, 32))
    at = torch.arange(n)

    def run(to, r):
        names = {k: to(v) for k, v in plain_names(params).items()}
        return plain.differential_attention(to(x), names, "p.", m, 1e-5, at, r=r).float()

    compare(got, run, dtype)


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("widths", [(16, 24), (32, 64)], ids=["maps16", "maps32"])
def test_keys_far_back_and_at_page_borders(dtype, widths):
    """No window, 330 tokens, queries so large that a map sits on one or two keys anywhere in
    the sequence: a prompt of 290, then decoding across two page borders.  The keys far back
    carry the result: without the first 200 it is another."""
    hidden, heads, kv_heads, (dim, vdim) = 64, 6, 2, widths
    part = two_map_attention(hidden, heads, kv_heads, dim, vdim, 0.25, 0.3, None, (10000.0, 16))
    params = bind_random(part, dtype, scale=0.25, seed=21)
    sharpen(part, params, dtype, ["q.weight"], 12.0)
    n, prompt = 330, 290
    x = rnd(n, hidden, seed=22).to(dtype)
    portions = ((0, prompt),) + tuple((i, 1) for i in range(prompt, n))
    got = run_mixer_in_portions(part, x, dtype, hidden, pages=24, portions=portions)
    m = attention(heads, kv_heads, dim, vdim, 0.25, 0.3, None, (10000.0, 16))
    at = torch.arange(n)

    def run(to, r):
        names = {k: to(v) for k, v in plain_names(params).items()}
        return plain.differential_attention(to(x), names, "p.", m, 1e-5, at, r=r).float()

    want = compare(got, run, dtype)
    near = dict(m, mask={"size": 130, "keep_first": 0})
    cut = plain.differential_attention(x.float(), plain_names(params), "p.", near, 1e-5, at)
    assert (cut - want).abs().amax(-1)[prompt:].max() > 0.05


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("masks", [((12, 3), (20, 5)), ((20, 5), (6, 0)), (None, (9, 2)), ((8, 1), None)],
                         ids=["reader-wider", "reader-narrower", "writer-sees-all", "reader-sees-all"])
def test_a_layer_that_reads_another_layer_s_keys_and_values(dtype, masks):
    """The writer projects, turns and stores keys and values; the reader, with queries, mask,
    lambda and gate of its own and no key or value tensors, reads the same pages in the same
    step.  The cache keeps what the wider of the two masks needs."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import LayerCache

    hidden, heads, kv_heads, dim, vdim, page, pages = 64, 4, 2, 16, 24, 16, 8
    own, other = masks
    if own is None or other is None:
        kept = (None, 0)
    else:
        kept = (max(own[0], other[0]), max(own[1], other[1]))
    rot = (10000.0, 8)
    writer = two_map_attention(hidden, heads, kv_heads, dim, vdim, 0.2, 0.25, own, rot,
                               cache_window=kept[0], cache_keep_first=kept[1])
    reader = two_map_attention(hidden, heads, kv_heads, dim, vdim, 0.3, 0.4, other, rot, own_kv=False)
    assert not any(n.startswith(("k.", "v.")) for n in reader.param_specs())
    pw = bind_random(writer, dtype, scale=0.25, seed=41)
    pr = bind_random(reader, dtype, scale=0.25, seed=51)
    sharpen(writer, pw, dtype, ["q.weight"], 4.0)
    sharpen(reader, pr, dtype, ["q.weight"], 4.0)
    for part in (writer, reader):
        part.prepare(pages * page, DEV)
    spec = writer.cache_spec()
    manager = CacheManager({0: spec}, pages, page, 2)
    k = torch.zeros(pages, spec.kv_heads, page, spec.head_dim, dtype=dtype, device=DEV)
    v = torch.zeros(pages, spec.kv_heads, spec.v_dim, page, dtype=dtype, device=DEV)
    xw, xr = rnd(60, hidden, seed=42).to(dtype), rnd(60, hidden, seed=52).to(dtype)
    out_w, out_r = [], []
    portions = ((0, 21), (21, 2), (23, 17)) + tuple((i, 1) for i in range(40, 60))
    for start, count in portions:
        if not manager.holds("s"):
            manager.admit("s", [], count)
        manager.grow("s", start, start + count)
        step = build_step([SeqChunk("s", [0] * count, start, [])], manager, 10, 4096, DEV)
        for part, x, cache, out in ((writer, xw, LayerCache(k, v, 0, page, True), out_w),
                                    (reader, xr, LayerCache(k, v, 0, page, False), out_r)):
            acc = torch.zeros(count, hidden, device=DEV)
            settle(acc, part.forward(x[start:start + count].to(DEV).contiguous(), step, cache, None, acc))
            out.append(acc.cpu())
    at = torch.arange(60)
    mw = attention(heads, kv_heads, dim, vdim, 0.2, 0.25, own, rot)
    mr = attention(heads, kv_heads, dim, vdim, 0.3, 0.4, other, rot)

    def run_writer(to, r):
        names = {k: to(v) for k, v in plain_names(pw).items()}
        return plain.differential_attention(to(xw), names, "p.", mw, 1e-5, at, r=r).float()

    def run_reader(to, r):
        kv = plain.attention_keys_values(to(xw), {k: to(v) for k, v in plain_names(pw).items()},
                                         "p.", mw, at, r)
        names = {k: to(v) for k, v in plain_names(pr).items()}
        return plain.differential_attention(to(xr), names, "p.", mr, 1e-5, at, kv=kv, r=r).float()

    compare(torch.cat(out_w), run_writer, dtype)
    compare(torch.cat(out_r), run_reader, dtype)


def retention_part(hidden, heads, dim, vdim, decay, rot):
    from mercury_amd.parts import NoPosition, Retention, RotaryPosition

    position = RotaryPosition(dim, rot[0], rotary_dim=rot[1]) if rot and rot[1] else NoPosition()
    return Retention(hidden, heads, dim, vdim, decay, position, eps=1e-5, names=RET_NAMES)


RETENTION_SIZES = {
    "small-partly-turned": (64, 2, 16, 24, (0.9, 0.96875), (5000.0, 8)),
    "odd": (100, 3, 10, 14, (0.75, 0.9375, 0.998), (100000.0, 10)),
    "never-decays-or-forgets-at-once": (64, 3, 8, 8, (1.0, 0.0, 0.99), None),
    "sized": (128, 2, 64, 128, (0.96875, 0.99609375), (1e6, 32)),
    "one-head-forty-rows-columns-past-128": (64, 1, 40, 130, (0.97,), (700.0, 40)),
    "seventy-two-rows": (64, 2, 72, 16, (0.95, 0.999), (700.0, 2)),
    "two-hundred-rows": (48, 1, 200, 33, (0.9,), None),
}


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("sizes", RETENTION_SIZES.values(), ids=RETENTION_SIZES.keys())
def test_retention_alone_carries_its_state(dtype, sizes):
    """The state carried over portions of 21, 2, 9, 1, 1 and 6 tokens, from a slot that held
    something else before."""
    hidden, heads, dim, vdim, decay, rot = sizes
    part = retention_part(hidden, heads, dim, vdim, decay, rot)
    params = bind_random(part, dtype, scale=0.3, seed=7)
    x = rnd(40, hidden, seed=32).to(dtype)
    got = run_mixer_in_portions(part, x, dtype, hidden)
    m = retention(heads, dim, vdim, decay, rot)
    at = torch.arange(40)
    want = plain.retention(x.float(), plain_names(params), "p.", m, 1e-5, at)
    rounded = plain.retention(x.float(), plain_names(params), "p.", m, 1e-5, at, plain.to_bf16)
    close(got, want, dtype, rounded)


@pytest.mark.parametrize("dtype", BOTH)
def test_retention_over_long_portions_and_odd_cuts(dtype):
    """Portions of 300, 1, 129, 128 and 2 tokens (the kernel stages 16 tokens at a time: cuts
    at, before and after such an edge), against the recurrence in float64."""
    hidden, heads, dim, vdim, decay, rot = 64, 2, 16, 24, (0.984375, 0.99951171875), (1e6, 16)
    part = retention_part(hidden, heads, dim, vdim, decay, rot)
    params = bind_random(part, dtype, scale=0.3, seed=19)
    x = rnd(560, hidden, seed=34).to(dtype)
    portions = ((0, 300), (300, 1), (301, 129), (430, 128), (558, 2))
    got = run_mixer_in_portions(part, x, dtype, hidden, pages=40, portions=portions)
    m = retention(heads, dim, vdim, decay, rot)
    at = torch.arange(560)
    want = plain.retention(x.double(), {k: v.double() for k, v in plain_names(params).items()},
                           "p.", m, 1e-5, at).float()
    rounded = plain.retention(x.float(), plain_names(params), "p.", m, 1e-5, at, plain.to_bf16)
    close(got, want, dtype, rounded)
    # a slow head remembers the first tokens to the end: without them the last rows differ
    late = plain.retention(x[200:].float(), plain_names(params), "p.", m, 1e-5, at[200:])
    assert (late[-20:] - want[-20:]).abs().max() > 1e-2


@pytest.mark.parametrize("dtype", BOTH)
def test_retention_decoding_for_long_beside_another_sequence(dtype):
    """300 steps token by token, a second sequence of 120 tokens beside the first in the same
    state tensor: no drift from the plain recurrence, nothing leaks between the slots."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import CacheSpec

    hidden = 64
    part = retention_part(hidden, 3, 16, 24, (0.9, 0.99, 1.0), (10000.0, 8))
    params = bind_random(part, dtype, scale=0.3, seed=11)
    part.prepare(640, DEV)
    xs = {"a": rnd(300, hidden, seed=1).to(dtype), "b": rnd(120, hidden, seed=2).to(dtype)}
    manager = CacheManager({0: CacheSpec(1, 8)}, 40, 16, 2, True)
    state = torch.full((2, *part.state_spec().shape), 5.0, device=DEV)
    out, done = {"a": [], "b": []}, {"a": 0, "b": 0}
    while done["a"] < 300:
        chunks = []
        for key in ("a", "b"):
            if done[key] >= len(xs[key]):
                continue
            if not manager.holds(key):
                manager.admit(key, [], 1)
            manager.grow(key, done[key], done[key] + 1)
            chunks.append(SeqChunk(key, [0], done[key], []))
        step = build_step(chunks, manager, 10, 4096, DEV)
        if step.fresh_slots:
            state[step.fresh_slots] = 0
        x = torch.stack([xs[c.key][done[c.key]] for c in chunks]).to(DEV)
        acc = torch.zeros(len(chunks), hidden, device=DEV)
        settle(acc, part.forward(x, step, None, state, acc))
        for row, c in enumerate(chunks):
            out[c.key].append(acc[row].cpu())
            done[c.key] += 1
    m = retention(3, 16, 24, (0.9, 0.99, 1.0), (10000.0, 8))
    for key in ("a", "b"):
        at = torch.arange(len(xs[key]))
        want = plain.retention(xs[key].float(), plain_names(params), "p.", m, 1e-5, at)
        rounded = plain.retention(xs[key].float(), plain_names(params), "p.", m, 1e-5, at, plain.to_bf16)
        close(torch.stack(out[key]), want, dtype, rounded)


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("ff,scaled", [(96, True), (0, True), (80, False)],
                         ids=["both-sublayers", "no-feed-forward", "no-stored-scale"])
def test_norms_around_each_sublayer_and_the_stored_scale(dtype, ff, scaled):
    """s += ls1 * n1b(mixer(n1(s))); s += ls2 * n2b(ff(n2(s))) around a retention and a tanh-gelu
    gated projection, over portions, the stream in float32."""
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import CacheSpec, GatedMLP, PrePostNormBlock, RMSNorm

    hidden, eps = 72, 1e-5
    names = {"mixer": "mix.", "ffn": "mlp.", "norm_mixer": "norm1.", "norm_ffn": "norm2.",
             "post_mixer": "norm1b.", "post_ffn": "norm2b.", "scale_mixer": "ls1", "scale_ffn": "ls2"}
    mixer = retention_part(hidden, 2, 16, 24, (0.9, 0.97), (10000.0, 8))
    norm = lambda: RMSNorm(hidden, eps)
    ffn = GatedMLP(hidden, ff, "gelu_tanh", names=FF_NAMES) if ff else None
    block = PrePostNormBlock(mixer, ffn, norm(), norm() if ffn else None, norm(), norm() if ffn else None,
                             names, layer_scale=scaled)
    params = bind_random(block, dtype, scale=0.3, seed=61)
    block.prepare(64, DEV)
    manager = CacheManager({0: CacheSpec(1, 8)}, 8, 16, 2, True)
    state = torch.full((2, *mixer.state_spec().shape), 2.0, device=DEV)
    x = rnd(30, hidden, seed=62)
    out = []
    for start, count in ((0, 19), (19, 2), (21, 8), (29, 1)):
        if not manager.holds("s"):
            manager.admit("s", [], count)
        manager.grow("s", start, start + count)
        step = build_step([SeqChunk("s", [0] * count, start, [])], manager, 10, 4096, DEV)
        if step.fresh_slots:
            state[step.fresh_slots] = 0
        h = x[start:start + count].to(DEV).contiguous()
        settle(h, block.forward(h, step, None, state, dtype))
        out.append(h.cpu())

    def plain_block(r):
        w = plain_names(params)
        one = torch.ones(hidden)
        s = x.clone()
        y = plain.retention(r(plain.rms_norm(s, w["p.norm1"], eps)), w, "p.mix.",
                            retention(2, 16, 24, (0.9, 0.97), (10000.0, 8)), eps, torch.arange(30), r)
        s = s + (w["p.ls1"] if scaled else one) * plain.rms_norm(y, w["p.norm1b"], eps)
        if ff:
            y = plain.gated(r(plain.rms_norm(s, w["p.norm2"], eps)), w, "p.mlp.", plain.gelu_tanh, r)
            s = s + (w["p.ls2"] if scaled else one) * plain.rms_norm(y, w["p.norm2b"], eps)
        return s

    close(torch.cat(out), plain_block(plain.same), dtype, plain_block(plain.to_bf16))


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("sizes", [(64, 6, 2, 32, 48), (100, 5, 3, 18, 22), (128, 4, 1, 40, 0),
                                   (64, 3, 3, 24, 8), (64, 16, 3, 48, 80)],
                         ids=["two-of-six-shared", "odd-three-of-five", "one-of-four-none-shared",
                              "all-of-three", "three-of-sixteen"])
@pytest.mark.parametrize("rows", [7, 70])
def test_routed_experts_beside_a_gated_shared_expert(dtype, sizes, rows):
    """The chosen experts' weights are the softmax over the chosen logits alone; the shared
    expert's output is multiplied by one sigmoid a token.  Tokens whose routing is a close call
    are compared in float32 only."""
    from mercury_amd.parts import GatedMLP, RoutedExperts

    hidden, experts, top, ff, shared_ff = sizes
    shared = GatedMLP(hidden, shared_ff, "silu", names=FF_NAMES) if shared_ff else None
    part = RoutedExperts(hidden, experts, top, ff, scale=1.0, renormalize=True, activation="silu",
                         shared=shared, shared_gated=shared is not None)
    params = bind_random(part, dtype, scale=0.25, seed=5)
    x = rnd(rows, hidden, seed=9).to(dtype)
    acc = rnd(rows, hidden, seed=8)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(DEV), None, acc_d))
    mlp = moe(experts, top, ff, shared_ff)
    w = plain_names(params)
    want = acc + plain.routed_experts(x.float(), w, "p.", mlp)
    rounded = acc + plain.routed_experts(x.float(), w, "p.", mlp, plain.to_bf16)
    got, full = acc_d.cpu(), want
    if dtype == torch.bfloat16 and top < experts:
        ranked = (x.float() @ w["p.router"].T).sort(-1, descending=True).values
        clear = (ranked[:, top - 1] - ranked[:, top]) > 0.02 * ranked.abs().amax(-1)
        assert clear.float().mean() > 0.4
        got, want, rounded = got[clear], want[clear], rounded[clear]
    close(got, want, dtype, rounded)
    if shared is not None:
        # the gate matters: without it the result is another
        off = dict(w)
        off["p.shared.sg"] = torch.zeros_like(off["p.shared.sg"])
        assert (acc + plain.routed_experts(x.float(), off, "p.", mlp) - full).abs().max() > 1e-3


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("rows", [3, 37, 300])
def test_tanh_gelu_gated_feed_forward(dtype, rows):
    from mercury_amd.parts import GatedMLP

    part = GatedMLP(72, 136, "gelu_tanh", names=FF_NAMES)
    params = bind_random(part, dtype, scale=0.5, seed=17)
    x = rnd(rows, 72, seed=9).to(dtype) * 2
    acc = rnd(rows, 72, seed=8)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(DEV), None, acc_d))
    w = plain_names(params)
    want = acc + plain.gated(x.float(), w, "p.", plain.gelu_tanh)
    rounded = acc + plain.gated(x.float(), w, "p.", plain.gelu_tanh, plain.to_bf16)
    close(acc_d.cpu(), want, dtype, rounded)
    # the gate's arguments reach where the tanh form and silu part ways
    assert (acc + plain.gated(x.float(), w, "p.", plain.silu) - want).abs().max() > 0.05


# ---------------------------------------------------------------------------- whole models


CLOSE_CALL = 0.03
_PICKED: dict = {}


def routing_gaps(cfg, weights, tokens):
    """[T]: the least routing gap of the position over the routed layers (1 without any)."""
    gaps = []
    plain.forward(cfg, weights, tokens, gaps=gaps)
    return torch.stack(gaps).min(0).values if gaps else torch.ones(len(tokens))


def decisive_tokens(cfg, weights, count, seed):
    """Random tokens, drawn again wherever a routed layer's choice is a close call (the last
    chosen logit within CLOSE_CALL of the first one left out, relative to the largest): such a
    token may go to another expert once its input is rounded to bfloat16, and what it then
    writes into caches and states reaches every later position.  A position depends on no later
    one, so the first close call is redrawn until there is none."""
    key = (repr(cfg), float(weights["embed"].double().sum()), count, seed)
    if key in _PICKED:
        return _PICKED[key]
    tokens = helpers.random_tokens(cfg["vocab"], count, seed=seed)
    spare = iter(helpers.random_tokens(cfg["vocab"], 40 * count + 400, seed=seed + 7919))
    while True:
        close_calls = (routing_gaps(cfg, weights, tokens) <= CLOSE_CALL).nonzero()
        if not len(close_calls):
            _PICKED[key] = tokens
            return tokens
        tokens[int(close_calls[0])] = next(spare)


class Plain:
    """The plain implementation under the names the schedules call."""

    to_bf16 = staticmethod(plain.to_bf16)
    read_config = staticmethod(plain.read_config)
    read_weights = staticmethod(plain.read_weights)

    @staticmethod
    def forward(cfg, weights, tokens, r=plain.same):
        return plain.forward(cfg, weights, tokens, r)

    pick_tokens = staticmethod(decisive_tokens)


MODELS = [("small", 16), ("odd", 16), ("small", 64), ("sized", 32)]


@pytest.fixture(scope="module", params=MODELS, ids=[f"{n}-page{p}" for n, p in MODELS])
def model(request):
    name, page = request.param
    return schedules.Case(name, folder_for(name), page, Plain)


def entry(key, tokens):
    return schedules.entry(key, tokens)


@pytest.mark.parametrize("name", ["small", "odd"])
def test_residual_stream_after_every_layer(name):
    """The stream after every layer (float32), so that a wrong layer names itself: the engine
    gets a configuration of the first layers, an identity head and a unit last norm, and its
    logits are the normed stream."""
    import copy
    import json
    import tempfile
    from pathlib import Path

    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import save_file

    folder = folder_for(name)
    cfg = plain.read_config(folder)
    width = cfg["width"]
    stored = plain.read_weights(folder, torch.bfloat16)
    tokens = [t % width for t in helpers.random_tokens(cfg["vocab"], 53, seed=4)]
    exact = plain.read_weights(folder, torch.float64)
    exact["embed"] = exact["embed"][:width]
    _, streams = plain.forward(cfg, exact, tokens, return_layers=True)
    for depth in range(1, len(cfg["layers"]) + 1):
        cut = copy.deepcopy(cfg)
        cut["layers"] = cut["layers"][:depth]
        cut["vocab"] = width
        part = {k: v for k, v in stored.items() if any(k.startswith(f"l{i}.") for i in range(depth))}
        part["embed"] = stored["embed"][:width].contiguous()
        part["final.norm"] = torch.ones(width, dtype=torch.bfloat16)
        part["head"] = torch.eye(width, dtype=torch.bfloat16)
        where = Path(tempfile.mkdtemp(prefix="mercury_videdra_cut_"))
        (where / "config.json").write_text(json.dumps(cut))
        save_file(part, where / "model.safetensors", metadata={"format": "pt"})
        want = plain.rms_norm(streams[depth - 1], None, cfg["norm"]["eps"]).float()
        s = ReplaySession(where, "float32", 64)
        got = torch.cat([s.step([entry("r", tokens[:31])], []), s.step([entry("r", tokens[31:])], ["r"])])
        torch.testing.assert_close(got, want, atol=3e-5, rtol=3e-5, msg=lambda m: f"after layer {depth - 1}: {m}")


DTYPES = ["float32", "bfloat16"]


@pytest.mark.parametrize("dtype", DTYPES)
def test_each_request_alone_and_whole(model, dtype):
    schedules.whole(model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_prompt_then_the_last_tokens_one_by_one(model, dtype):
    """Tails of 32 and of 70 tokens: the longer passes every window of the configurations over
    decoded tokens."""
    schedules.decoded_tail(model, dtype)
    schedules.decoded_tail(model, dtype, keys=("a", "b"), tail=70)


@pytest.mark.parametrize("dtype", DTYPES)
def test_portions_of_changing_size_down_to_two_tokens(model, dtype):
    schedules.portions(model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_decoding_from_the_first_token(model, dtype):
    schedules.from_the_first_token(model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_unequal_requests_mixed_in_a_pool_that_is_used_again(model, dtype):
    schedules.mixed(model, dtype)


@pytest.mark.parametrize("dtype", DTYPES)
def test_a_batch_of_unequal_requests_equals_each_alone(model, dtype):
    """Four requests in one step (a prompt of 150 beside one of 5), then one more token of each
    in one step: the same logits, to rounding, as each request in a session of its own."""
    keys = ["a", "f", "c", "e"]
    together = model.session(dtype, 512)
    first = together.step([entry(k, model.reqs[k][:-1]) for k in keys], [])
    last = together.step([entry(k, model.reqs[k][-1:]) for k in keys], keys)
    at = 0
    for row, key in enumerate(keys):
        n = len(model.reqs[key]) - 1
        alone = model.session(dtype, 192)
        one = torch.cat([alone.step([entry(key, model.reqs[key][:-1])], []),
                         alone.step([entry(key, model.reqs[key][-1:])], [key])])
        both = torch.cat([first[at:at + n], last[row:row + 1]])
        at += n
        model.check(both, key, dtype, "batched")
        if dtype == "float32":
            assert (both - one).abs().max() <= 2e-5 * max(1.0, float(one.abs().max())), f"{key} depends on its neighbours"
        else:
            # the products of a step of many rows and of one of few are summed in other orders
            schedules.check_positions(both, one, model.cost[key], f"{key} beside its neighbours")
    assert together.manager.leaked_pages() == 0


@pytest.mark.parametrize("dtype", DTYPES)
def test_sharpened_attention_and_slow_decays_over_a_long_request(dtype):
    """Queries scaled so that a map sits on a few keys, a prompt of 700 whole and then decoded
    on past page borders, against the plain implementation in float64.  The start of the
    sequence reaches the end, through the layer that sees every token and through the states:
    other first tokens change the last logits."""
    from mercury_amd.engine.replay import ReplaySession

    folder = folder_for("small", sharpen=4.0)
    cfg = plain.read_config(folder)
    w64, w32 = plain.read_weights(folder, torch.float64), plain.read_weights(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 740, seed=77)
    want = plain.forward(cfg, w64, tokens).float()
    f32 = plain.forward(cfg, w32, tokens)
    moved = tokens[:]
    moved[:300] = helpers.random_tokens(cfg["vocab"], 300, seed=78)
    assert (plain.forward(cfg, w32, moved)[-40:] - f32[-40:]).abs().max() > 0.05
    cost = float((plain.forward(cfg, w32, tokens, plain.to_bf16) - want).abs().max())
    s = ReplaySession(folder, dtype, 768, page_size=16)
    rows = [s.step([entry("r", tokens[:700])], [])]
    for i in range(700, 740):
        rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 739 else []))
    got = torch.cat(rows)
    if dtype == "float32":
        slack = float((f32 - want).abs().max())      # what float32 costs the plain implementation
        bound = 2e-5 * max(1.0, float(want.abs().max())) + 2e-5 * want.abs() + 1.5 * slack
        assert ((got - want).abs() <= bound).all(), f"worst {(got - want).abs().max():.3e}, plain's own {slack:.3e}"
    else:
        schedules.check(got, want, dtype, "sharpened", cost)
    assert s.manager.leaked_pages() == 0


def check_float32(got, want, own, what):
    """float32 tolerances relative to the size of the logits, plus three times what float32
    costs the plain implementation at the position (`own` [T, 1]): where a position is badly
    conditioned (a head's output that nearly cancels is divided by its own size), the last
    bits of float32 show there too."""
    bound = 2e-5 * max(1.0, float(want.abs().max())) + 2e-5 * want.abs() + 3.0 * own
    bad = ((got - want).abs() > bound).any(-1)
    assert not bad.any(), (f"{what}: first wrong token {int(bad.nonzero()[0])} of {got.shape[0]}, "
                           f"worst {(got - want).abs().max():.3e}")


def draw_config(seed: int) -> dict:
    """A configuration whose sizes, counts, constants and order of layers are drawn: widths
    that are and are not multiples of 8, one to many heads in one to as many groups, maps of
    sizes the matrix cores take and others, values narrower and wider than a map, windows from
    one token to none, kept tokens from none to more than the window, readers of earlier
    layers, decays from a half to 1 (a head that forgets at once puts out a value's direction
    with a sign, which no rounding leaves alone), every kind of feed-forward or none."""
    import random

    r = random.Random(seed)
    width = r.choice([48, 50, 64, 72, 100, 128, 136])
    layers, writers = [], []
    for i in range(r.randint(1, 5)):
        if r.random() < 0.6:
            source = r.choice(writers) if writers and r.random() < 0.4 else None
            if source is None:
                kv = r.choice([1, 2, 3])
                heads = kv * r.choice([1, 2, 4])
                dim = r.choice([8, 10, 16, 32, 64])
                vdim = r.choice([dim, 2 * dim, 12, 24, 40])
                turned = r.choice([0, 2, dim // 2 - (dim // 2) % 2, dim])
                rot = (r.uniform(50, 1e6), turned) if turned else None
            else:
                old = layers[source]["mixer"]
                heads, kv, dim, vdim = old["heads"], old["kv_heads"], old["dim"], old["vdim"]
                rot = (old["rot"]["base"], old["rot"]["dims"]) if "rot" in old else None
            mask = None if r.random() < 0.25 else (r.choice([1, 5, 16, 31, 64, 100]), r.choice([0, 1, 4, 17, 40]))
            mixer = attention(heads, kv, dim, vdim, r.uniform(0.1, 0.4), r.uniform(0.05, 0.7), mask, rot, source)
            if source is None:
                writers.append(i)
            kind = "attention"
        else:
            heads, dim = r.choice([1, 2, 3, 5]), r.choice([8, 10, 16, 32, 64])
            turned = r.choice([0, 2, dim])
            decay = [r.choice([0.5, 0.9, 0.96875, 0.99, 0.999, 1.0]) for _ in range(heads)]
            mixer = retention(heads, dim, r.choice([8, 14, 32, 64, 130]), decay,
                              (r.uniform(50, 1e6), turned) if turned else None)
            kind = "retention"
        which = r.random()
        if which < 0.15:
            mlp = None
        elif which < 0.5:
            mlp = dense(r.choice([24, 40, 90]))
        else:
            experts = r.choice([2, 3, 6, 16])
            mlp = moe(experts, r.randint(1, min(experts, 4)), r.choice([16, 18, 40]), r.choice([0, 22, 48]))
        layers.append(layer(kind, mixer, mlp))
    return {"architecture": "Videdra", "vocab": r.choice([97, 256, 301]), "width": width,
            "norm": {"eps": r.choice([1e-6, 1e-5, 1e-3])}, "layers": layers}


@pytest.mark.parametrize("seed", range(24))
def test_drawn_configurations(seed):
    """Whole, then a portion that ends inside a page, a portion of two tokens and decoding, in
    both dtypes, for configurations nobody chose."""
    from mercury_amd.engine.replay import ReplaySession

    cfg = draw_config(seed)
    folder = write_folder(cfg, std=0.1, seed=100 + seed)
    weights = plain.read_weights(folder)
    tokens = decisive_tokens(cfg, weights, 171, seed)
    want = plain.forward(cfg, plain.read_weights(folder, torch.float64), tokens).float()
    own = (plain.forward(cfg, weights, tokens) - want).abs().amax(-1, keepdim=True)
    rounded = schedules.rounding_cost(Plain, cfg, weights, tokens, want)
    for dtype in DTYPES:
        s = ReplaySession(folder, dtype, 256, max_live=2)
        whole = s.step([entry("w", tokens)], ["w"])
        rows = [s.step([entry("r", tokens[:137])], []), s.step([entry("r", tokens[137:139])], [])]
        for i in range(139, 171):
            rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 170 else []))
        for got, how in ((whole, "whole"), (torch.cat(rows), "cut")):
            what = f"drawn {seed} {how} {cfg}"
            if dtype == "float32":
                check_float32(got, want, own, what)
            else:
                schedules.check_positions(got, want, rounded, what)
        assert s.manager.leaked_pages() == 0


# ------------------------------------------------ generation through the engine's entry point


@pytest.mark.parametrize("name", ["small", "odd"])
def test_greedy_generation_through_the_engine(name):
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = folder_for(name)
    cfg, weights = plain.read_config(folder), plain.read_weights(folder)
    prompts = [helpers.random_tokens(cfg["vocab"], n, seed=40 + n) for n in (3, 19, 41)]
    want = [plain.greedy_generate(cfg, weights, p, 12) for p in prompts]
    engine = Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=24,
                                 block_size=16, max_model_len=128, prefill_budget=16))
    got = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=12)
    assert got == want
    assert engine.leaked_blocks() == 0
    # bfloat16: the tokens are the plain implementation's, or so close to its choice that the
    # format's own error can have swapped them
    engine = Engine(EngineConfig(model=str(folder), device=DEV, dtype="bfloat16", num_blocks=24,
                                 block_size=16, max_model_len=128))
    out = engine.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=12)
    # (a generated sequence is nobody's choice: where a routed layer's choice is a close call
    # the engine's rounding may turn it and none of the plain runs'; one token of all may be
    # further from the plain implementation's choice)
    far = []
    for prompt, tokens in zip(prompts, out):
        logits = plain.forward(cfg, weights, prompt + tokens)
        runs = [plain.forward(cfg, weights, prompt + tokens, (lambda t, c=c: plain.to_bf16(t * c) / c))
                for c in schedules.SCALES]
        cost = torch.stack([(run - logits).abs().amax(-1) for run in runs]).max(0).values
        cost = torch.maximum(cost, cost.median())
        for i, token in enumerate(tokens):
            at = len(prompt) - 1 + i
            row = logits[at]
            if row.max() - row[token] > 3 * cost[at]:
                far.append((tokens, i, float(row.max() - row[token]), float(cost[at])))
    assert len(far) <= 1, far


def test_preemption_and_sampling_with_state_and_windows():
    """A pool so small that requests are preempted and start over (state slot and pages given
    back, taken again, the slot cleared): the greedy tokens stay the plain implementation's.
    Sampled tokens (temperature, nucleus) do not depend on what else is in the batch."""
    from mercury_amd import Engine, EngineConfig, SamplingParams

    folder = folder_for("small")
    cfg, weights = plain.read_config(folder), plain.read_weights(folder)
    prompts = [helpers.random_tokens(cfg["vocab"], 60, seed=70 + i) for i in range(4)]
    tight = Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=14,
                                block_size=16, max_model_len=128, max_running=4,
                                debug_invariants=True))
    got = tight.generate(prompts, SamplingParams(ignore_eos=True), max_tokens=24)
    assert tight.sched.stats["preemptions"] > 0
    assert got == [plain.greedy_generate(cfg, weights, p, 24) for p in prompts]
    assert tight.leaked_blocks() == 0

    def fresh():
        return Engine(EngineConfig(model=str(folder), device=DEV, dtype="float32", num_blocks=48,
                                   block_size=16, max_model_len=128, seed=9))

    params = SamplingParams(temperature=0.9, top_p=0.8, ignore_eos=True)
    together = fresh().generate(prompts[:3], params, max_tokens=10)
    alone = fresh().generate(prompts[:1], params, max_tokens=10)
    assert together[0] == alone[0] and len(set(together[0])) > 1


def test_command_line_and_trace_replay(tmp_path):
    """`random-weights` and `generate` on the command line for this architecture, and the
    replay program over a trace of three steps."""
    import json
    import subprocess
    import sys

    import numpy as np

    from tests.videdra_cases import ODD

    config = tmp_path / "config.json"
    config.write_text(json.dumps(ODD))
    out = subprocess.run([sys.executable, "-m", "mercury_amd", "random-weights", "--config",
                          str(config), "--out", str(tmp_path / "m"), "--seed", "5", "--std", "0.08"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert out.returncode == 0, out.stderr
    prompt = [(i * 7) % ODD["vocab"] for i in range(20)]
    run = subprocess.run([sys.executable, "-m", "mercury_amd", "generate", "--model",
                          str(tmp_path / "m"), "--prompt-ids", ",".join(map(str, prompt)),
                          "--prompt-ids", "1 2 3", "--max-tokens", "5", "--dtype", "float32",
                          "--num-blocks", "32", "--max-model-len", "256", "--ignore-eos"],
                         capture_output=True, text=True, cwd=helpers.ROOT)
    assert run.returncode == 0, run.stderr
    lines = [json.loads(line) for line in run.stdout.strip().splitlines()]
    cfg, weights = plain.read_config(tmp_path / "m"), plain.read_weights(tmp_path / "m")
    assert lines[0] == {"prompt_index": 0, "tokens": plain.greedy_generate(cfg, weights, prompt, 5)}
    assert lines[1]["tokens"] == plain.greedy_generate(cfg, weights, [1, 2, 3], 5)

    steps = [{"step": 0, "entries": [{"id": "x", "tokens": prompt[:13], "want": [12]}], "end": []},
             {"step": 1, "entries": [{"id": "x", "tokens": prompt[13:15], "want": []},
                                     {"id": "y", "tokens": [1, 2, 3], "want": [0, 2]}], "end": ["y"]},
             {"step": 2, "entries": [{"id": "x", "tokens": prompt[15:], "want": [4, 0]}], "end": ["x"]}]
    run = subprocess.run([str(helpers.ROOT / "bin" / "trace_run"), "--model", str(tmp_path / "m"),
                          "--dtype", "float32", "--out", str(tmp_path / "o"), "--max-tokens", "128"],
                         input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                         text=True, cwd=helpers.ROOT)
    assert run.returncode == 0, run.stderr
    assert [l for l in run.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    x, y = plain.forward(cfg, weights, prompt), plain.forward(cfg, weights, [1, 2, 3])
    read = lambda i: torch.from_numpy(np.fromfile(tmp_path / "o" / f"{i}.f32", dtype="<f4").reshape(-1, ODD["vocab"]).copy())
    tol = dict(atol=3e-5, rtol=3e-5)
    torch.testing.assert_close(read(0), x[12:13], **tol)
    torch.testing.assert_close(read(1), y[[0, 2]], **tol)
    torch.testing.assert_close(read(2), x[[19, 15]], **tol)


def test_the_benchmark_s_layer_sizes(tmp_path):
    """The layer sizes the benchmark runs (maps of 64 over values of 128, retention heads of
    64 x 128, experts beside a shared one), cut down in width and count so that the plain
    implementation is quick: whole, a portion and decoding in both dtypes."""
    from mercury_amd.engine.replay import ReplaySession

    folder = folder_for("sized")
    cfg = plain.read_config(folder)
    weights = plain.read_weights(folder)
    tokens = decisive_tokens(cfg, weights, 300, 5)
    want = plain.forward(cfg, plain.read_weights(folder, torch.float64), tokens).float()
    own = (plain.forward(cfg, weights, tokens) - want).abs().amax(-1, keepdim=True)
    rounded = schedules.rounding_cost(Plain, cfg, weights, tokens, want)
    for dtype in DTYPES:
        s = ReplaySession(folder, dtype, 320, page_size=64)
        rows = [s.step([entry("r", tokens[:200])], []), s.step([entry("r", tokens[200:270])], [])]
        for i in range(270, 300):
            rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 299 else []))
        if dtype == "float32":
            check_float32(torch.cat(rows), want, own, "sized")
        else:
            schedules.check_positions(torch.cat(rows), want, rounded, "sized")
