"""The Mogilorn configuration and builder on the CPU: what `config.json` says is what the
model is made of, what it cannot mean is refused, and the plain implementation's mechanisms
hold the properties that define them."""

from __future__ import annotations

import copy
import math

import pytest
import torch

from mercury_amd.config import ConfigError
from mercury_amd.config.registry import build_model, resolve
from tests.mogilorn_cases import BLENDED, CASES, ODD, SCALING, SMALL
from tests.plain import mogilorn_plain as plain


def test_every_size_and_constant_comes_from_the_configuration():
    cfg, _ = resolve(SMALL)
    assert (cfg.vocab, cfg.width, cfg.norm_eps, cfg.embedding_scale) == (300, 64, 1e-5, 6.0)
    a = cfg.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.scale, a.softcap, a.v_mix, a.rot_base, a.rot_dims) == \
        (4, 2, 16, 8, 0.25, 12.0, True, 10000.0, 8)
    assert a.rot_scaling == (4.0, 1.0, 4.0, 64.0)
    m = cfg.layers[1].mixer
    assert (m.heads, m.dim, m.vdim, m.gate_cap) == (2, 16, 40, 9.0)
    la = cfg.layers[2].mixer
    assert (la.heads, la.dim, la.rot_dim, la.vdim, la.kv_rank, la.window, la.rot_base, la.rot_dims) == \
        (4, 8, 16, 24, 32, 24, 5000.0, 8)
    assert cfg.layers[3].ff == 0 and cfg.layers[0].ff == 96
    assert cfg.mixing_layers() == [0, 3, 4]
    assert resolve(cfg.to_dict())[0] == cfg
    odd, _ = resolve(ODD)
    assert odd.layers[1].mixer.softcap == 0.0 and odd.layers[2].mixer.rot_dims == 0
    assert odd.layers[3].mixer.gate_cap == 0.0 and odd.layers[0].mixer.window == 0
    assert odd.layers[4].mixer.rot_dim == 0 and odd.embedding_scale == 1.0


@pytest.mark.parametrize("name", sorted(CASES))
def test_the_builder_declares_the_stored_tensors(name):
    raw = CASES[name]
    model = build_model(raw)
    specs = model.param_specs()
    width = raw["width"]
    assert specs["embed"].shape == (raw["vocab"], width) and "head" not in specs
    assert specs["final.norm"].shape == (width,)
    for i, entry in enumerate(raw["layers"]):
        m, p = entry["mixer"], f"l{i}."
        assert specs[p + "norm1"].shape == (width,)
        assert ((p + "norm2") in specs) == (entry["mlp"] is not None) == ((p + "mlp.up") in specs)
        if entry["type"] == "attention":
            assert specs[p + "mix.q"].shape == (m["heads"] * m["dim"], width)
            assert specs[p + "mix.k.b"].shape == (m["kv_heads"] * m["dim"],)
            assert specs[p + "mix.v"].shape == (m["kv_heads"] * m["vdim"], width)
            assert specs[p + "mix.q.norm"].shape == (m["dim"],) == specs[p + "mix.k.norm"].shape
            assert specs[p + "mix.g"].shape == (m["heads"] * m["vdim"], width)
            assert specs[p + "mix.o"].shape == (width, m["heads"] * m["vdim"])
            assert specs[p + "mix.o.b"].shape == (width,)
            assert specs[p + "mix.vmix"].shape == () and specs[p + "mix.vmix"].optional != m["v_mix"]
        elif entry["type"] == "mlstm":
            assert specs[p + "mix.q"].shape == (m["heads"] * m["dim"], width)
            assert specs[p + "mix.v"].shape == (m["heads"] * m["vdim"], width) == specs[p + "mix.g"].shape
            assert specs[p + "mix.i"].shape == (m["heads"], width) and specs[p + "mix.f.b"].shape == (m["heads"],)
            assert specs[p + "mix.norm"].shape == (m["heads"] * m["vdim"],)
        else:
            assert specs[p + "mix.q"].shape == (m["heads"] * (m["dim"] + m["rot_dim"]), width)
            assert specs[p + "mix.dkv"].shape == (m["kv_rank"] + m["rot_dim"], width)
            assert specs[p + "mix.dkv.norm"].shape == (m["kv_rank"],)
            assert specs[p + "mix.uk"].shape == (m["heads"] * m["dim"], m["kv_rank"])
            assert specs[p + "mix.uv"].shape == (m["heads"] * m["vdim"], m["kv_rank"])
            assert specs[p + "mix.sink"].shape == (m["heads"],)
            assert specs[p + "mix.g"].shape == (m["heads"] * m["vdim"], width)


def test_caches_states_and_who_mixes_with_whom():
    model = build_model(SMALL)
    slots = {slot: spec.as_tuple() for slot, spec in model.cache_slots.items()}
    assert slots[0][:3] == (2, 16, 8) and slots[0][4] == 0
    assert slots[2][0] == 1 and slots[2][4] == 24          # one shared head inside its window
    assert 1 not in slots
    assert model.layers[1].mixer.state_spec().shape == (2 * (16 * 40 + 2 * 17),)
    assert [model.layers[i].mixer.v_mix for i in (0, 3, 4)] == ["leave", "blend", "blend"]
    odd = build_model(ODD)
    # one mixing layer alone has nobody to mix with; a layer that does not mix may or may not
    # store a number
    assert odd.layers[1].mixer.v_mix is None and odd.layers[1].mixer.v_mix_stored == "yes"
    assert odd.layers[2].mixer.v_mix_stored == "maybe"
    blended = build_model(BLENDED)
    assert [layer.mixer.v_mix for layer in blended.layers if hasattr(layer.mixer, "v_mix")] == \
        ["leave", None, "blend", "blend"]
    assert model.tied_head and model.embedding_part.scale == 6.0


def bad(path, value):
    raw = copy.deepcopy(SMALL)
    at = raw
    for key in path[:-1]:
        at = at[key]
    if value is None:
        at.pop(path[-1])
    else:
        at[path[-1]] = value
    return raw


@pytest.mark.parametrize("raw", [
    bad(("layers", 0, "type"), "convolution"),
    bad(("layers", 0, "mixer", "kv_heads"), 3),
    bad(("layers", 0, "mixer", "rot", "dims"), 7),
    bad(("layers", 0, "mixer", "rot", "dims"), 18),
    bad(("layers", 0, "mixer", "rot", "scaling", "high"), 0.5),
    bad(("layers", 0, "mixer", "rot", "scaling", "factor"), None),
    bad(("layers", 0, "mixer", "scale"), None),
    bad(("layers", 1, "mixer", "heads"), 0),
    bad(("layers", 1, "mixer", "gate_cap"), -1.0),
    bad(("layers", 2, "mixer", "kv_rank"), None),
    bad(("layers", 2, "mixer", "mask", "size"), -4),
    bad(("layers", 2, "mixer", "rot", "dims"), 18),
    bad(("layers", 3, "mixer", "vdim"), 12),
    bad(("layers", 0, "mlp", "kind"), "moe"),
    bad(("layers", 0, "mlp", "ff"), 0),
    bad(("norm",), {}),
    bad(("width",), 0),
], ids=lambda raw: "")
def test_what_a_configuration_cannot_mean_is_refused(raw):
    with pytest.raises(ConfigError):
        resolve(raw)


# ------------------------------------------------- pins of the plain implementation's reading


def test_plain_frequencies_slow_long_wavelengths_only():
    rot = {"base": 10000.0, "dims": 32, "scaling": SCALING}
    plainly = plain.frequencies({"base": 10000.0, "dims": 32})
    scaled = plain.frequencies(rot)
    assert plainly[0] == 1.0 and plainly[1] == 10000.0 ** (-2 / 32)
    for f, g in zip(plainly, scaled):
        wavelength = 2 * math.pi / f
        if wavelength < SCALING["original"] / SCALING["high"]:
            assert g == f
        elif wavelength > SCALING["original"] / SCALING["low"]:
            assert g == f / SCALING["factor"]
        else:
            assert f / SCALING["factor"] <= g <= f
    assert scaled[0] == plainly[0] and scaled[-1] == plainly[-1] / 4.0
    assert any(f / 4.0 < g < f for f, g in zip(plainly, scaled))


def test_plain_turn_pairs_neighbours_and_leaves_the_rest():
    x = torch.arange(12, dtype=torch.float64).reshape(1, 1, 12) + 1
    out = plain.turn(x.expand(3, 1, 12).clone(), torch.tensor([0, 1, 5]), {"base": 100.0, "dims": 4})
    assert torch.equal(out[0], x[0]) and torch.equal(out[:, :, 4:], x.expand(3, 1, 12)[:, :, 4:])
    a = 5 * 100.0 ** (-2 / 4)
    assert out[2, 0, 2] == pytest.approx(3 * math.cos(a) - 4 * math.sin(a))
    assert out[2, 0, 3] == pytest.approx(4 * math.cos(a) + 3 * math.sin(a))
    # a shift of all positions leaves the products of turned queries and keys alone
    q, k = torch.randn(6, 2, 8, dtype=torch.float64), torch.randn(6, 2, 8, dtype=torch.float64)
    rot, at = {"base": 50.0, "dims": 6}, torch.arange(6)
    near = torch.einsum("ihd,jhd->hij", plain.turn(q, at, rot), plain.turn(k, at, rot))
    far = torch.einsum("ihd,jhd->hij", plain.turn(q, at + 37, rot), plain.turn(k, at + 37, rot))
    torch.testing.assert_close(near, far)


def test_plain_window_and_sink():
    seen = plain.visible(torch.arange(6), 3)
    assert seen[4].tolist() == [False, False, True, True, True, False]
    assert plain.visible(torch.arange(6), 0)[4].tolist() == [True] * 5 + [False]
    g = torch.Generator().manual_seed(1)
    q, k, v = (torch.randn(7, 2, 4, generator=g, dtype=torch.float64) for _ in range(3))
    at = torch.arange(7)
    # a sink is a key of score sink_h (unscaled) whose value is zero
    sink = torch.tensor([0.7, -1.2], dtype=torch.float64)
    got = plain.softmax_attention(q, k, v, at, 0.5, window=4, sink=sink)
    for h in range(2):
        for i in range(7):
            lo = max(0, i - 3)
            s = torch.cat([(q[i, h] @ k[lo:i + 1, h].T) * 0.5, sink[h:h + 1]])
            p = torch.softmax(s, -1)
            torch.testing.assert_close(got[i, h], p[:-1] @ v[lo:i + 1, h])
    # without a sink and a window: the library's attention
    want = torch.nn.functional.scaled_dot_product_attention(
        q.transpose(0, 1), k.transpose(0, 1), v.transpose(0, 1), is_causal=True, scale=0.5).transpose(0, 1)
    torch.testing.assert_close(plain.softmax_attention(q, k, v, at, 0.5), want)
    capped = plain.softmax_attention(q * 9, k, v, at, 0.5, softcap=2.0)
    assert (capped - plain.softmax_attention(q * 9, k, v, at, 0.5)).abs().max() > 0.05


def test_plain_rows_of_a_prefix_are_rows_of_the_whole():
    from tests.mogilorn_cases import folder_for

    folder = folder_for("odd")
    cfg, w = plain.read_config(folder), plain.read_weights(folder, torch.float64)
    tokens = [(7 * i + 3) % cfg["vocab"] for i in range(30)]
    whole = plain.forward(cfg, w, tokens)
    torch.testing.assert_close(plain.forward(cfg, w, tokens[:11]), whole[:11])
    # the memory's state carried by hand equals the whole run
    s = torch.randn(20, cfg["width"], dtype=torch.float64)
    m = cfg["layers"][3]["mixer"]
    all_at_once = plain.matrix_memory(s, w, "l3.mix.", m, 1e-6)
    first, state = plain.matrix_memory(s[:8], w, "l3.mix.", m, 1e-6, return_state=True)
    second = plain.matrix_memory(s[8:], w, "l3.mix.", m, 1e-6, state=state)
    torch.testing.assert_close(torch.cat([first, second]), all_at_once)
