"""The Mogilorn design on the GPU against the plain implementation: every mechanism alone (the
gated attention with a norm per head and slowed frequencies, values mixed across layers, the
matrix memory with its carried state, the windowed latent attention with sinks, sublayers that
read the stream itself, the tanh-gelu feed-forward), window edges and far keys made to show,
then whole models replayed whole, with a decoded tail, in portions down to two tokens, from the
first token on, mixed in a pool so small that pages and slots are used again, configurations
nobody chose, and greedy generation through the engine's entry point, its scheduler and the
command line."""

from __future__ import annotations

import copy
import json
import random
import subprocess
import sys
import tempfile
from pathlib import Path

import numpy as np
import pytest
import torch

from tests import helpers, replay_schedules as schedules
from tests.mogilorn_cases import (CASES, SCALING, attention, folder_for, latent, layer, memory,
                                  model as model_config, write_folder)
from tests.plain import mogilorn_plain as plain
from tests.test_gpu_larozen import bind_random, rnd, run_mixer_in_portions, settle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
BOTH = [torch.float32, torch.bfloat16]
DTYPES = ["float32", "bfloat16"]
ATT_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "q_norm": "q.norm", "k_norm": "k.norm",
             "gate": "g", "v_mix": "vmix"}
MEM_NAMES = {"q": "q", "k": "k", "v": "v", "gate": "g", "o": "o", "input": "i", "forget": "f",
             "norm": "norm"}
LAT_NAMES = {"q": "q", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv", "o": "o",
             "sink": "sink", "gate": "g"}
BF16_SLACK = 2.0


def plain_names(params, prefix="p."):
    """The part's local names ('q.norm.weight', 'q.bias', 'vmix') as the plain implementation
    calls them ('p.q.norm', 'p.q.b', 'p.vmix')."""
    out = {}
    for n, t in params.items():
        if n.endswith(".weight"):
            n = n[:-len(".weight")]
        elif n.endswith(".bias"):
            n = n[:-len(".bias")] + ".b"
        out[prefix + n] = t
    return out


def compare(got, run, dtype, slack=1.0):
    """`run(to, r)` is the plain result with inputs and weights cast by `to` and roundings `r`;
    the truth is its float64 run.  float32: float32 tolerances relative to the size of the
    outputs, plus three times what float32 costs the plain implementation.  bfloat16:
    BF16_SLACK times what the format costs the plain run."""
    want = run(torch.Tensor.double, plain.same).float()
    assert got.shape == want.shape and torch.isfinite(got).all()
    worst = float((got - want).abs().max())
    if dtype == torch.float32:
        own = float((run(torch.Tensor.float, plain.same) - want).abs().max())
        bound = 2e-5 * max(1.0, float(want.abs().max())) + 3.0 * own
    else:
        bound = BF16_SLACK * float((run(torch.Tensor.float, plain.to_bf16) - want).abs().max()) + 1e-3
    assert worst <= slack * bound, f"off by {worst:.3e}, allowed {slack * bound:.3e}"
    return want


def rebind(part, params, dtype, change):
    """Changes the part's tensors (`change(params)`, float32 on the host) and binds again."""
    change(params)
    for n in params:
        params[n] = params[n].to(dtype).float()
    part.bind({n: t.to(dtype).to(DEV) for n, t in params.items()}, dtype, DEV)


# ------------------------------------------------------------------- mechanisms, one by one


def gated_attention(hidden, m):
    from mercury_amd.parts import Attention, NoPosition, RotaryPosition

    rot = m.get("rot")
    s = rot.get("scaling") if rot else None
    position = (RotaryPosition(m["dim"], rot["base"], rotary_dim=rot["dims"], interleaved=True,
                               scaling=(s["factor"], s["low"], s["high"], s["original"]) if s else None)
                if rot else NoPosition())
    return Attention(hidden, m["heads"], m["kv_heads"], m["dim"], position, qkv_bias=True, o_bias=True,
                     scale=m["scale"], names=ATT_NAMES, score_cap=m.get("softcap") or None,
                     value_dim=m["vdim"], qk_norm="head", norm_eps=1e-5, out_gate=True)


ATTENTION_SIZES = {
    "grouped-narrow-values": (64, attention(4, 2, 16, 8, 0.25, softcap=12.0, rot=(10000.0, 8), scaling=SCALING)),
    "one-group-odd": (100, attention(3, 1, 10, 12, 0.3, rot=(300.0, 10))),
    "own-kv-heads-no-turn-no-cap": (72, attention(3, 3, 6, 6, 0.4)),
    "one-head-wide-values": (64, attention(1, 1, 8, 24, 0.35, softcap=3.0, rot=(100.0, 2))),
    "equal-widths-64": (128, attention(4, 2, 64, 64, 0.125, softcap=30.0, rot=(10000.0, 64), scaling=SCALING)),
    "equal-widths-128": (256, attention(2, 1, 128, 128, 0.09, softcap=20.0, rot=(10000.0, 128))),
    "equal-widths-64-no-bound": (128, attention(4, 2, 64, 64, 0.125, rot=(10000.0, 32))),
    "equal-widths-32": (64, attention(4, 4, 32, 32, 0.18, softcap=10.0, rot=(1000.0, 32), scaling=SCALING)),
    "equal-widths-96": (96, attention(2, 1, 96, 96, 0.1, softcap=25.0, rot=(10000.0, 48))),
    "equal-widths-80-no-bound": (80, attention(2, 2, 80, 80, 0.11)),
}


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("sizes", ATTENTION_SIZES.values(), ids=ATTENTION_SIZES.keys())
def test_gated_attention_alone(dtype, sizes):
    """Projections with biases, a norm per head with one weight for all heads, interleaved pairs
    over a head's first dims with slowed frequencies, the bounded score, the gate per column:
    over portions of 21, 2, 9, 1, 1 and 6 tokens from a cache of its own."""
    hidden, m = sizes
    part = gated_attention(hidden, m)
    params = bind_random(part, dtype, scale=0.15, seed=3)
    x = rnd(40, hidden, seed=5).to(dtype).float()
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden)
    positions = torch.arange(40)

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return plain.attention(to(x), w, "p.", m, 1e-5, positions, None, r)

    want = compare(got, run, dtype)
    # the gate, the norms' weight and the bound are not idle
    w = plain_names(params)
    ungated = dict(w, **{"p.g": torch.zeros_like(w["p.g"])})
    assert (plain.attention(x, ungated, "p.", m, 1e-5, positions) - want).abs().max() > 0.01
    plainly = dict(w, **{"p.q.norm": torch.ones_like(w["p.q.norm"])})
    assert (plain.attention(x, plainly, "p.", m, 1e-5, positions) - want).abs().max() > 1e-3


def test_slowed_frequencies_are_the_formula_s():
    """The angle table against the rule written out pair by pair: short wavelengths untouched,
    long ones slowed by the factor, the band between blended; and a table without scaling."""
    from mercury_amd.parts import RotaryPosition

    for dims, base, s in ((32, 10000.0, SCALING), (64, 500000.0, {"factor": 8.0, "low": 1.0, "high": 4.0, "original": 8192}),
                          (8, 100.0, {"factor": 2.0, "low": 0.5, "high": 3.0, "original": 20})):
        part = RotaryPosition(dims, base, interleaved=True,
                              scaling=(s["factor"], s["low"], s["high"], s["original"]))
        want = torch.tensor(plain.frequencies({"base": base, "dims": dims, "scaling": s}), dtype=torch.float64)
        torch.testing.assert_close(part.frequencies(), want, rtol=1e-12, atol=0)
        kinds = {("same" if a == b else "slow" if abs(a - b / s["factor"]) < 1e-15 * b else "mixed")
                 for a, b in zip(want.tolist(), plain.frequencies({"base": base, "dims": dims}))}
        assert {"same", "slow"} <= kinds
        part.prepare(50, DEV)
        angle = torch.arange(50, dtype=torch.float64)[:, None] * want[None, :]
        torch.testing.assert_close(part.cos.cpu().double(), angle.cos(), atol=1e-7, rtol=0)


MEMORY_SIZES = {
    "two-workgroups-a-head": (64, memory(2, 16, 40, gate_cap=9.0)),
    "odd": (100, memory(3, 10, 14)),
    "one-head": (72, memory(1, 24, 30, gate_cap=4.0)),
    "columns-28": (64, memory(2, 8, 28, gate_cap=15.0)),
    "columns-29": (64, memory(2, 8, 29, gate_cap=15.0)),
    "rows-72": (96, memory(2, 72, 16, gate_cap=15.0)),
    "rows-200": (64, memory(1, 200, 8)),
    "sized": (128, memory(2, 64, 128, gate_cap=15.0)),
}


def matrix_memory(hidden, m):
    from mercury_amd.parts import MatrixMemory

    return MatrixMemory(hidden, m["heads"], m["dim"], m["vdim"], gate_cap=m.get("gate_cap") or None,
                        eps=1e-5, names=MEM_NAMES)


def slow_and_loud(params):
    """Half of the heads forget slowly and every other head takes a lot in: the state then holds
    many tokens, and its running maximum moves."""
    params["f.bias"][::2] += 5.0
    params["i.bias"][1::2] += 2.0
    params["i.weight"] *= 4.0


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("sizes", MEMORY_SIZES.values(), ids=MEMORY_SIZES.keys())
def test_matrix_memory_alone_carries_its_state(dtype, sizes):
    """S, n and the running maximum carried over portions of 21, 2, 9, 1, 1 and 6 tokens in a
    slot that held something else before."""
    hidden, m = sizes
    part = matrix_memory(hidden, m)
    params = bind_random(part, dtype, scale=0.2, seed=11)
    rebind(part, params, dtype, slow_and_loud)
    assert part.state_spec().shape == (part.state_floats(),)
    x = rnd(40, hidden, seed=6).to(dtype).float()
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden)

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return plain.matrix_memory(to(x), w, "p.", m, 1e-5, r)

    want = compare(got, run, dtype, slack=1.5)
    # the state reaches from the first portion into the last: another first portion, another end
    other = x.clone()
    other[:21] = rnd(21, hidden, seed=66)
    w = plain_names(params)
    assert (plain.matrix_memory(other, w, "p.", m, 1e-5)[-1] - want[-1]).abs().max() > 1e-3


def test_the_memory_s_state_size_is_the_kernel_library_s():
    from mercury_amd.hostcore import core
    from mercury_amd.kernels import lib

    lib.load("core")
    for heads, dim, vdim in ((2, 16, 40), (3, 10, 14), (1, 256, 28), (4, 64, 128), (2, 8, 57)):
        part = matrix_memory(64, memory(heads, dim, vdim))
        assert part.state_floats() == core.mlstm_state_floats(heads, dim, vdim)


@pytest.mark.parametrize("dtype", BOTH)
def test_matrix_memory_long_portions_and_long_decoding(dtype):
    """Portions of 300, 1, 129, 128 and 2 tokens (more than 128 tokens of a sequence run in
    chunks side by side whose start states are carried), then 200 tokens one by one, gates that
    let the running maximum rise and fall."""
    hidden, m = 64, memory(2, 16, 40, gate_cap=9.0)
    part = matrix_memory(hidden, m)
    params = bind_random(part, dtype, scale=0.2, seed=21)
    rebind(part, params, dtype, slow_and_loud)
    total = 760
    x = rnd(total, hidden, seed=7).to(dtype).float()
    cuts = [(0, 300), (300, 1), (301, 129), (430, 128), (558, 2)] + [(560 + i, 1) for i in range(200)]
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden, pages=50, portions=cuts)

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return plain.matrix_memory(to(x), w, "p.", m, 1e-5, r)

    compare(got, run, dtype, slack=1.5)


def test_the_running_maximum_changes_nothing_but_the_floor():
    """The plain recurrence against the same memory written without a running maximum, in
    float64: S_t = sum_j exp(i_j + sum_(j<s<=t) f_s) k_j v_j^T and the denominator
    max(|n.q|, 1) + 1e-6 exp(m_t), all times exp(-m_t)."""
    m = memory(2, 6, 5, gate_cap=6.0)
    g = torch.Generator().manual_seed(3)
    w = {"p." + n: torch.randn(*shape, generator=g, dtype=torch.float64) * 0.5 for n, shape in
         (("q", (12, 16)), ("k", (12, 16)), ("v", (10, 16)), ("g", (10, 16)), ("o", (16, 10)),
          ("i", (2, 16)), ("i.b", (2,)), ("f", (2, 16)), ("f.b", (2,)), ("norm", (10,)))}
    x = torch.randn(9, 16, generator=g, dtype=torch.float64)
    got = plain.matrix_memory(x, w, "p.", m, 1e-6)
    cap = m["gate_cap"]
    q = (x @ w["p.q"].T).view(9, 2, 6) * 6 ** -0.5
    k, v = (x @ w["p.k"].T).view(9, 2, 6), (x @ w["p.v"].T).view(9, 2, 5)
    a = cap * torch.tanh((x @ w["p.i"].T + w["p.i.b"]) / cap)
    f = torch.nn.functional.logsigmoid(cap * torch.tanh((x @ w["p.f"].T + w["p.f.b"]) / cap))
    out = torch.zeros(9, 2, 5, dtype=torch.float64)
    for t in range(9):
        for h in range(2):
            weights = torch.stack([torch.exp(a[j, h] + f[j + 1:t + 1, h].sum()) for j in range(t + 1)])
            top = max(float(f[:t + 1, h].sum()), max(float(a[j, h] + f[j + 1:t + 1, h].sum()) for j in range(t + 1)))
            S = torch.einsum("j,jd,jv->dv", weights, k[:t + 1, h], v[:t + 1, h])
            n = torch.einsum("j,jd->d", weights, k[:t + 1, h])
            below = max(abs(float(n @ q[t, h])), 1.0) + 1e-6 * float(np.exp(top))
            out[t, h] = (S.T @ q[t, h]) / below
    o = plain.rms(out, 1e-6).reshape(9, 10) * w["p.norm"] * torch.sigmoid(x @ w["p.g"].T)
    torch.testing.assert_close(got, o @ w["p.o"].T, rtol=1e-9, atol=1e-11)


def windowed_latent(hidden, m):
    from mercury_amd.parts import LatentAttention, NoPosition, RotaryPosition

    rot = m.get("rot")
    position = (RotaryPosition(m["rot_dim"], rot["base"], rotary_dim=rot.get("dims", m["rot_dim"]),
                               interleaved=True) if rot and m["rot_dim"] else NoPosition())
    window = (m.get("mask") or {}).get("size")
    return LatentAttention(hidden, m["heads"], m["dim"], m["rot_dim"], m["vdim"], 0, m["kv_rank"],
                           position, 1e-5, scale=m["scale"], window=window, names=LAT_NAMES,
                           sinks=True, out_gate=True)


LATENT_SIZES = {
    "window-24": (64, latent(4, 8, 16, 24, 32, 0.2, window=24, rot=(5000.0, 8))),
    "sees-all-odd": (100, latent(3, 10, 6, 14, 20, 0.3, rot=(300.0, 6))),
    "nothing-turns-window-7": (72, latent(2, 6, 0, 10, 12, 0.35, window=7)),
    "window-1": (64, latent(2, 8, 8, 8, 16, 0.3, window=1, rot=(100.0, 8))),
    "sized": (128, latent(4, 32, 32, 32, 96, 0.125, window=20, rot=(50000.0, 32))),
}


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("sizes", LATENT_SIZES.values(), ids=LATENT_SIZES.keys())
def test_windowed_latent_attention_alone(dtype, sizes):
    """Queries straight from the input, the latent's norm, the shared turned key part, the
    window, the sink and the gate, against keys and values written out head by head."""
    hidden, m = sizes
    part = windowed_latent(hidden, m)
    params = bind_random(part, dtype, scale=0.2, seed=31)
    rebind(part, params, dtype, lambda p: p["sink.weight"].add_(1.0))
    x = rnd(40, hidden, seed=8).to(dtype).float()
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden)
    positions = torch.arange(40)

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return plain.latent_attention(to(x), w, "p.", m, 1e-5, positions, r)

    want = compare(got, run, dtype)
    w = plain_names(params)
    sunk = dict(w, **{"p.sink": w["p.sink"] - 30.0})
    assert (plain.latent_attention(x, sunk, "p.", m, 1e-5, positions) - want).abs().max() > 1e-3


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("window", [1, 2, 5, 16, 17, 33])
def test_the_edge_of_the_window_shows(dtype, window):
    """Queries scaled so that a head sits on one or two keys: a window one token wider or
    narrower gives another result, in the prompt's portions and in 38 tokens decoded one by
    one, across page borders (pages of 16)."""
    hidden = 64
    m = latent(4, 8, 8, 16, 24, 0.5, window=window, rot=(1000.0, 8))
    part = windowed_latent(hidden, m)
    params = bind_random(part, dtype, scale=0.25, seed=41)
    rebind(part, params, dtype, lambda p: (p["q.weight"].mul_(6.0), p["sink.weight"].sub_(3.0)))
    total = 90
    x = rnd(total, hidden, seed=9).to(dtype).float()
    cuts = [(0, 30), (30, 2), (32, 20)] + [(52 + i, 1) for i in range(38)]
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden, pages=8, portions=cuts)
    positions = torch.arange(total)

    def run_with(size):
        def run(to, r):
            w = {n: to(t) for n, t in plain_names(params).items()}
            return plain.latent_attention(to(x), w, "p.", dict(m, mask={"size": size}), 1e-5, positions, r)
        return run

    want = compare(got, run_with(window), dtype, slack=2.0)
    for other in (window + 1, window - 1):
        if other < 1:
            continue
        shifted = run_with(other)(torch.Tensor.double, plain.same).float()
        gap = (shifted - want).abs().amax(-1)
        mine = (got - want).abs().amax(-1)
        for part_of, rows in (("prompt", slice(0, 52)), ("decoded", slice(52, total))):
            assert gap[rows].max() > 5 * mine[rows].max() + 1e-3, (
                f"a window of {other} instead of {window} does not show in the {part_of} tokens")


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("window", [0, 300])
def test_decoding_over_many_latents_splits_them_over_wavefronts(dtype, window):
    """A prompt of 700 tokens, then 40 decoded one by one: a decoding step's keys (all 700 and
    more, or the 300 of the window) are walked in parts that a second kernel merges, sinks
    included; sharpened queries put weight on keys hundreds of tokens back."""
    hidden = 64
    m = latent(4, 8, 8, 16, 24, 0.5, window=window, rot=(1000.0, 8))
    part = windowed_latent(hidden, m)
    params = bind_random(part, dtype, scale=0.25, seed=43)
    rebind(part, params, dtype, lambda p: (p["q.weight"].mul_(5.0), p["sink.weight"].add_(1.0)))
    total = 740
    x = rnd(total, hidden, seed=15).to(dtype).float()
    cuts = [(0, 700)] + [(700 + i, 1) for i in range(40)]
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden, pages=48, portions=cuts)
    positions = torch.arange(total)

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return plain.latent_attention(to(x), w, "p.", m, 1e-5, positions, r)

    want = compare(got, run, dtype, slack=2.0)
    w = plain_names(params)
    nearer = dict(m, mask={"size": 200})
    assert (plain.latent_attention(x, w, "p.", nearer, 1e-5, positions)[-40:] - want[-40:]).abs().max() > 0.01


@pytest.mark.parametrize("dtype", BOTH)
def test_keys_far_back_and_at_page_borders(dtype):
    """The gated attention with its score bounded loosely and queries scaled up: the softmax
    sits on single keys hundreds of tokens back; 600 tokens whole, then decoded across page
    borders."""
    hidden, m = 64, attention(4, 2, 16, 8, 0.5, softcap=40.0, rot=(10000.0, 8), scaling=SCALING)
    part = gated_attention(hidden, m)
    params = bind_random(part, dtype, scale=0.25, seed=51)
    rebind(part, params, dtype, lambda p: p["q.weight"].mul_(8.0))
    total = 640
    x = rnd(total, hidden, seed=10).to(dtype).float()
    cuts = [(0, 600)] + [(600 + i, 1) for i in range(40)]
    got = run_mixer_in_portions(part, x.to(dtype), dtype, hidden, pages=41, portions=cuts)
    positions = torch.arange(total)

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return plain.attention(to(x), w, "p.", m, 1e-5, positions, None, r)

    want = compare(got, run, dtype)
    # far keys carry weight: without the first 300 tokens the last rows are others
    w = plain_names(params)
    late = plain.attention(x[300:], w, "p.", m, 1e-5, positions[300:])
    assert (late[-40:] - want[-40:]).abs().max() > 0.01


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("ff", [96, 0])
def test_sublayers_read_the_stream_and_their_outputs_are_normed(dtype, ff):
    """s += rms(mixer(s)) (1 + w1); s += rms(ff(s)) (1 + w2) with no norm before a sublayer: the
    layer alone over a stream that is far from normed."""
    from mercury_amd.parts import NoNorm, PrePostNormBlock, RMSNorm, UnaryMLP

    hidden, m = 64, memory(2, 16, 24, gate_cap=9.0)
    ffn = UnaryMLP(hidden, ff, "gelu_tanh", names={"up": "up", "down": "down"}) if ff else None
    post = lambda: RMSNorm(hidden, 1e-5, one_plus=True)
    names = {"mixer": "mix.", "ffn": "mlp.", "norm_mixer": "a.", "norm_ffn": "b.",
             "post_mixer": "norm1.", "post_ffn": "norm2."}
    block = PrePostNormBlock(matrix_memory(hidden, m), ffn, NoNorm(hidden), NoNorm(hidden) if ff else None,
                             post(), post() if ff else None, names, layer_scale=False)
    params = bind_random(block, dtype, scale=0.2, seed=61)
    stream = rnd(33, hidden, seed=12) * 3.0
    from mercury_amd.cache import CacheManager
    from mercury_amd.engine.batch import SeqChunk, build_step
    from mercury_amd.parts import CacheSpec

    manager = CacheManager({0: CacheSpec(1, 8)}, 8, 16, 2, True)
    state = torch.zeros(2, block.mixer.state_floats(), device=DEV)
    manager.admit("s", [], 33)
    manager.grow("s", 0, 33)
    step = build_step([SeqChunk("s", [0] * 33, 0, [])], manager, 10, 4096, DEV)
    h = stream.clone().to(DEV)
    settle(h, block.forward(h, step, None, state, dtype, None))

    def run(to, r):
        w = {"l0." + (n[:-7] if n.endswith(".weight") else n[:-5] + ".b" if n.endswith(".bias") else n): to(t)
             for n, t in params.items()}
        s = to(stream)
        s = s + plain.normed(plain.matrix_memory(s, w, "l0.mix.", m, 1e-5, r), w["l0.norm1"], 1e-5)
        if ff:
            s = s + plain.normed(plain.feed_forward(s, w, "l0.mlp.", r), w["l0.norm2"], 1e-5)
        return s

    compare(h.cpu(), run, dtype, slack=1.5)


@pytest.mark.parametrize("dtype", BOTH)
@pytest.mark.parametrize("rows", [3, 37, 300])
def test_tanh_gelu_feed_forward(dtype, rows):
    from mercury_amd.parts import UnaryMLP

    part = UnaryMLP(72, 136, "gelu_tanh", names={"up": "up", "down": "down"})
    params = bind_random(part, dtype, scale=0.2, seed=71)
    x = rnd(rows, 72, seed=13).to(dtype).float() * 2
    acc = rnd(rows, 72, seed=14)
    acc_d = acc.clone().to(DEV)
    settle(acc_d, part.forward(x.to(dtype).to(DEV), None, acc_d))

    def run(to, r):
        w = {n: to(t) for n, t in plain_names(params).items()}
        return to(acc) + plain.feed_forward(to(x), w, "p.", r)

    want = compare(acc_d.cpu(), run, dtype)
    relu = lambda z: torch.relu(z) ** 2
    w = plain_names(params)
    assert (acc + relu(x @ w["p.up"].T) @ w["p.down"].T - want).abs().max() > 0.05


# ---------------------------------------------------------------------------- whole models


_PICKED: dict = {}


def well_conditioned_tokens(cfg, weights, count, seed):
    """Random tokens, drawn again wherever float32 arithmetic alone moves the plain
    implementation's logits by a quarter of what the float32 comparisons allow: a memory that
    holds one or two terms whose sum nearly cancels before it is divided by its own size makes a
    rounding error large, in anybody's arithmetic.  A position depends on no later one, so the
    first such position is redrawn until there is none."""
    key = (repr(cfg), float(weights["embed"].double().sum()), count, seed)
    if key in _PICKED:
        return _PICKED[key]
    exact = {n: t.double() if t.is_floating_point() else t for n, t in weights.items()}
    single = {n: t.float() if t.is_floating_point() else t for n, t in weights.items()}
    tokens = helpers.random_tokens(cfg["vocab"], count, seed=seed)
    spare = iter(helpers.random_tokens(cfg["vocab"], 40 * count + 400, seed=seed + 7919))
    while True:
        want = plain.forward(cfg, exact, tokens).float()
        own = (plain.forward(cfg, single, tokens) - want).abs().amax(-1)
        touchy = (own > 0.25 * 2e-5 * max(1.0, float(want.abs().max()))).nonzero()
        if not len(touchy):
            _PICKED[key] = tokens
            return tokens
        tokens[int(touchy[0])] = next(spare)


class Plain:
    """The plain implementation under the names the schedules call."""

    pick_tokens = staticmethod(well_conditioned_tokens)

    to_bf16 = staticmethod(plain.to_bf16)
    read_config = staticmethod(plain.read_config)
    read_weights = staticmethod(plain.read_weights)

    @staticmethod
    def forward(cfg, weights, tokens, r=plain.same):
        return plain.forward(cfg, weights, tokens, r)


MODELS = [("small", 16), ("odd", 16), ("blended", 32), ("small", 64), ("sized", 32)]


@pytest.fixture(scope="module", params=MODELS, ids=[f"{n}-page{p}" for n, p in MODELS])
def model(request):
    name, page = request.param
    return schedules.Case(name, folder_for(name), page, Plain)


def entry(key, tokens):
    return schedules.entry(key, tokens)


@pytest.mark.parametrize("name", ["small", "odd", "blended"])
def test_residual_stream_after_every_layer(name):
    """The stream after every layer (float32), so that a wrong layer names itself: the engine
    gets a configuration of the first layers with an embedding (which is the head) of unit rows
    and a final norm of weight one, and its logits are the normed stream."""
    from mercury_amd.engine.replay import ReplaySession
    from mercury_amd.weights import save_file

    folder = folder_for(name)
    cfg = plain.read_config(folder)
    width = cfg["width"]
    stored = plain.read_weights(folder, torch.bfloat16)
    tokens = [t % width for t in helpers.random_tokens(cfg["vocab"], 53, seed=4)]
    exact = plain.read_weights(folder, torch.float64)
    exact["embed"] = torch.eye(width, dtype=torch.float64)
    _, streams = plain.forward(cfg, exact, tokens, return_layers=True)
    for depth in range(1, len(cfg["layers"]) + 1):
        cut = copy.deepcopy(cfg)
        cut["layers"] = cut["layers"][:depth]
        cut["vocab"] = width
        part = {k: v for k, v in stored.items() if any(k.startswith(f"l{i}.") for i in range(depth))}
        part["embed"] = torch.eye(width, dtype=torch.bfloat16)
        part["final.norm"] = torch.zeros(width, dtype=torch.bfloat16)
        where = Path(tempfile.mkdtemp(prefix="mercury_mogilorn_cut_"))
        (where / "config.json").write_text(json.dumps(cut))
        save_file(part, where / "model.safetensors", metadata={"format": "pt"})
        want = plain.rms(streams[depth - 1], cfg["norm"]["eps"]).float()
        s = ReplaySession(where, "float32", 64)
        got = torch.cat([s.step([entry("r", tokens[:31])], []), s.step([entry("r", tokens[31:])], ["r"])])
        torch.testing.assert_close(got, want, atol=3e-5, rtol=3e-5, msg=lambda m: f"after layer {depth - 1}: {m}")


def test_mixed_values_are_not_idle():
    """The plain implementation with every mixing number at zero gives other logits: what the
    schedules below compare with depends on the blend."""
    for name in ("small", "blended"):
        folder = folder_for(name)
        cfg, w = plain.read_config(folder), plain.read_weights(folder)
        tokens = helpers.random_tokens(cfg["vocab"], 30, seed=2)
        unmixed = {n: (torch.zeros_like(t) if n.endswith(".vmix") else t) for n, t in w.items()}
        assert (plain.forward(cfg, w, tokens) - plain.forward(cfg, unmixed, tokens)).abs().max() > 0.02


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
            schedules.check_positions(both, one, model.cost[key], f"{key} beside its neighbours")
    assert together.manager.leaked_pages() == 0


def check_float32(got, want, own, what):
    """float32 tolerances relative to the size of the logits, plus three times what float32
    costs the plain implementation at the position."""
    assert got.shape == want.shape and torch.isfinite(got).all(), what
    bound = 2e-5 * max(1.0, float(want.abs().max())) + 2e-5 * want.abs() + 3.0 * own
    bad = ((got - want).abs() > bound).any(-1)
    assert not bad.any(), f"{what}: first wrong token {int(bad.nonzero()[0])}, {int(bad.sum())} wrong"


@pytest.mark.parametrize("dtype", DTYPES)
def test_sharpened_queries_and_slow_memories_over_a_long_request(dtype):
    """Queries scaled so that a softmax sits on a few keys, a prompt of 700 whole and then 40
    tokens decoded past page borders, against the plain implementation in float64.  The start
    of the sequence reaches the end: other first tokens change the last logits."""
    from mercury_amd.engine.replay import ReplaySession

    folder = folder_for("small", sharpen=4.0)
    cfg, weights = plain.read_config(folder), plain.read_weights(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 740, seed=77)
    want = plain.forward(cfg, plain.read_weights(folder, torch.float64), tokens).float()
    own = (plain.forward(cfg, weights, tokens) - want).abs().amax(-1, keepdim=True)
    s = ReplaySession(folder, dtype, 768)
    rows = [s.step([entry("r", tokens[:700])], [])]
    for i in range(700, 740):
        rows.append(s.step([entry("r", tokens[i:i + 1])], ["r"] if i == 739 else []))
    got = torch.cat(rows)
    if dtype == "float32":
        check_float32(got, want, own, "long")
    else:
        schedules.check_positions(got, want, schedules.rounding_cost(Plain, cfg, weights, tokens, want), "long")
    other = helpers.random_tokens(cfg["vocab"], 200, seed=78) + tokens[200:]
    assert (plain.forward(cfg, weights, other)[-40:] - want[-40:]).abs().max() > 0.01


def draw_config(seed: int) -> dict:
    """A configuration nobody chose: layer kinds in any order, sizes that are and are not
    multiples of 8, mixing layers or none, windows, absent feed-forwards."""
    r = random.Random(seed)
    width = r.choice([40, 64, 72, 100])
    mixed_shape = (r.choice([1, 2, 3]), r.choice([6, 8, 12]))
    layers = []
    for _ in range(r.randint(2, 5)):
        kind = r.choice(["attention", "attention", "mlstm", "latent_attention"])
        if kind == "attention":
            mixes = r.random() < 0.6
            kv, vdim = mixed_shape if mixes else (r.choice([1, 2]), r.choice([4, 10, 16]))
            dim = r.choice([6, 8, 16, 20])
            dims = r.choice([0, 2, dim - dim % 2, dim // 2 - (dim // 2) % 2])
            mixer = attention(kv * r.choice([1, 2, 3]), kv, dim, vdim, r.choice([0.2, 0.35]),
                              softcap=r.choice([0.0, 4.0, 30.0]), v_mix=mixes,
                              rot=(r.choice([100.0, 10000.0]), dims) if dims else None,
                              scaling=r.choice([None, SCALING]) if dims else None)
        elif kind == "mlstm":
            mixer = memory(r.choice([1, 2, 3]), r.choice([4, 8, 10, 24]), r.choice([6, 28, 30, 40]),
                           gate_cap=r.choice([0.0, 5.0, 15.0]))
        else:
            rot_dim = r.choice([0, 4, 6, 8])
            mixer = latent(r.choice([1, 2, 4]), r.choice([4, 6, 8]), rot_dim, r.choice([6, 8, 12]),
                           r.choice([8, 12, 20]), r.choice([0.25, 0.4]), window=r.choice([0, 1, 9, 40]),
                           rot=(r.choice([100.0, 50000.0]), rot_dim) if rot_dim and r.random() < 0.8 else None)
        layers.append(layer(kind, mixer, r.choice([0, 30, 64])))
    return model_config(r.choice([97, 256, 301]), width, r.choice([1e-6, 1e-5, 1e-3]),
                        r.choice([1.0, 4.0, 11.0]), layers)


@pytest.mark.parametrize("seed", range(16))
def test_drawn_configurations(seed):
    """Whole, then a portion that ends inside a page, a portion of two tokens and decoding, in
    both dtypes, for configurations nobody chose."""
    from mercury_amd.engine.replay import ReplaySession

    cfg = draw_config(seed)
    folder = write_folder(cfg, std=0.1, seed=100 + seed)
    weights = plain.read_weights(folder)
    tokens = helpers.random_tokens(cfg["vocab"], 171, seed=seed)
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
    from tests.mogilorn_cases import ODD

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
