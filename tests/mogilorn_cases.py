"""Small Mogilorn configurations for the tests, and their model folders with random weights.

SMALL: multiples of 8 (the matrix-core projections run in bfloat16); three attention layers
whose values are mixed (the second and third blend the first's), with values narrower than
keys, a partly turned head with slowed frequencies and a bounded score; a matrix memory whose
columns need two workgroups a head; a latent attention in a window of 24 whose turned part is
wider than what turns; a layer without a feed-forward.
ODD: sizes that are no multiple of 8 (the float32-arithmetic kernels run in either dtype); one
key/value head under three query heads, heads turned whole and unscaled, no bound on the score;
one mixing layer alone (nobody to mix with); a matrix memory with unbounded gates; a latent
attention that sees every earlier token and turns nothing; an attention that does not mix
between two that do.
SIZED: widths of a real layer: heads of 128 over values of 128, a memory of 64 x 128, a latent
of 256 with a turned part of 64.
"""

from __future__ import annotations

import tempfile
from pathlib import Path

import torch

SCALING = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}


def attention(heads, kv_heads, dim, vdim, scale, softcap=0.0, v_mix=False, rot=None, scaling=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
           "v_mix": v_mix}
    if softcap:
        out["softcap"] = softcap
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
        if scaling:
            out["rot"]["scaling"] = dict(scaling)
    return out


def memory(heads, dim, vdim, gate_cap=0.0):
    out = {"heads": heads, "dim": dim, "vdim": vdim}
    if gate_cap:
        out["gate_cap"] = gate_cap
    return out


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, window=0, rot=None):
    out = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
           "scale": scale}
    if window:
        out["mask"] = {"size": window}
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    return out


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


def model(vocab, width, eps, scale, layers):
    return {"architecture": "Mogilorn", "vocab": vocab, "width": width, "norm": {"eps": eps},
            "embedding": {"scale": scale}, "layers": layers}


SMALL = model(300, 64, 1e-5, 6.0, [
    layer("attention", attention(4, 2, 16, 8, 0.25, softcap=12.0, v_mix=True, rot=(10000.0, 8),
                                 scaling=SCALING), 96),
    layer("mlstm", memory(2, 16, 40, gate_cap=9.0), 80),
    layer("latent_attention", latent(4, 8, 16, 24, 32, 0.2, window=24, rot=(5000.0, 8)), 72),
    layer("attention", attention(4, 2, 16, 8, 0.25, softcap=12.0, v_mix=True, rot=(10000.0, 8),
                                 scaling=SCALING), None),
    layer("attention", attention(2, 2, 32, 8, 0.18, softcap=20.0, v_mix=True, rot=(300.0, 32)), 64),
])

ODD = model(211, 100, 3e-6, 1.0, [
    layer("latent_attention", latent(3, 10, 6, 14, 20, 0.3), 70),
    layer("attention", attention(3, 1, 10, 12, 0.3, v_mix=True, rot=(300.0, 10)), 50),
    layer("attention", attention(3, 3, 6, 6, 0.4, softcap=7.0), None),
    layer("mlstm", memory(3, 10, 14), 30),
    layer("latent_attention", latent(2, 6, 0, 10, 12, 0.35, window=7), 50),
])

BLENDED = model(157, 72, 1e-6, 3.0, [
    layer("attention", attention(6, 3, 12, 10, 0.3, v_mix=True, rot=(1000.0, 12)), 40),
    layer("attention", attention(3, 3, 12, 10, 0.3), 40),
    layer("attention", attention(3, 3, 20, 10, 0.2, softcap=5.0, v_mix=True, rot=(1000.0, 4)), None),
    layer("mlstm", memory(1, 24, 30, gate_cap=4.0), None),
    layer("attention", attention(6, 3, 12, 10, 0.3, v_mix=True), 40),
])

SIZED = model(1201, 512, 1e-6, 8.0, [
    layer("attention", attention(4, 2, 128, 128, 0.09, softcap=30.0, v_mix=True, rot=(10000.0, 128),
                                 scaling={"factor": 8.0, "low": 1.0, "high": 4.0, "original": 256}), 1024),
    layer("mlstm", memory(4, 64, 128, gate_cap=15.0), 512),
    layer("latent_attention", latent(8, 64, 64, 64, 256, 0.09, window=100, rot=(10000.0, 64)), 512),
    layer("attention", attention(4, 2, 128, 128, 0.09, softcap=30.0, v_mix=True, rot=(10000.0, 128)), 512),
])

CASES = {"small": SMALL, "odd": ODD, "blended": BLENDED, "sized": SIZED}
_FOLDERS: dict = {}


def make_it_show(config: dict, tensors: dict, sharpen: float = 1.0) -> None:
    """Random weights hide some of the design: a mixing number near zero, a memory that forgets
    within a token or two, sinks near zero.  Give the mixing layers a number far from zero, half
    of every memory's heads a slow decay, every other sink a weight of its own, and (with
    `sharpen`) larger queries so that a softmax sits on few keys."""
    for i, entry in enumerate(config["layers"]):
        p, kind = f"l{i}.mix.", entry["type"]
        cast = lambda name, t: t.to(tensors[name].dtype)
        if kind == "attention" and p + "vmix" in tensors:
            tensors[p + "vmix"] = cast(p + "vmix", torch.tensor(0.25 + 0.125 * (i % 3)))
        if kind == "mlstm":
            bias = tensors[p + "f.b"].float()
            bias[::2] += 5.0
            tensors[p + "f.b"] = cast(p + "f.b", bias)
        if kind == "latent_attention":
            sink = tensors[p + "sink"].float()
            sink[::2] += 1.5
            tensors[p + "sink"] = cast(p + "sink", sink)
        if sharpen != 1.0 and kind != "mlstm":
            tensors[p + "q"] = cast(p + "q", tensors[p + "q"].float() * sharpen)


def folder_for(name: str, std: float = 0.08, seed: int = 13, sharpen: float = 1.0) -> Path:
    """A model folder of configuration `name` with random bfloat16 weights, edited by
    `make_it_show`."""
    return write_folder(CASES[name], std, seed, sharpen, key=name)


def write_folder(config: dict, std: float = 0.08, seed: int = 13, sharpen: float = 1.0,
                 key=None, edit=None) -> Path:
    """`edit(tensors)` may change the tensors (a dict name -> tensor) once more before they are
    written."""
    from mercury_amd.weights import save_file, write_random_model
    from mercury_amd.weights.safetensors_io import SafetensorsFile

    key = (key or repr(config), std, seed, sharpen, None if edit is None else id(edit))
    if key not in _FOLDERS:
        folder = Path(tempfile.mkdtemp(prefix="mercury_mogilorn_"))
        write_random_model(folder, config, seed=seed, std=std, dtype=torch.bfloat16)
        path = folder / "model.safetensors"
        source = SafetensorsFile(path)
        tensors = {n: source.tensor(n).clone() for n in source.names()}
        source.close()
        make_it_show(config, tensors, sharpen)
        if edit is not None:
            edit(tensors)
        save_file(tensors, path, metadata={"format": "pt"})
        _FOLDERS[key] = folder
    return _FOLDERS[key]
