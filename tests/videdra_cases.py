"""Small Videdra configurations for the tests, and their model folders with random weights.

SMALL: multiples of 8 (the matrix-core projections run in bfloat16); a retention layer first
(partly turned heads, routed experts beside a shared one); an attention whose values are
neither as wide as a map nor as a key row, in a window of 24 that keeps 3 tokens; a layer that
reads that layer's keys and values through a wider window that keeps more, without a
feed-forward; an attention that sees every earlier token, unturned, over experts of which a
token takes one and no shared one; a retention last whose heads do not turn, one of which
never decays.
ODD: sizes that are no multiple of 8 (the float32-arithmetic kernels run in either dtype); one
key/value head under three query heads, heads turned whole, a window of 7 that keeps 2, all
five experts' top three; a reader two layers after its writer with a retention between.
SIZED: widths of a real layer: maps of 64, values of 128, retention heads of 64 x 128.
"""

from __future__ import annotations

import tempfile
from pathlib import Path

import torch


def attention(heads, kv_heads, dim, vdim, scale, diff, mask=None, rot=None, kv_from=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
           "diff": diff}
    if mask:
        out["mask"] = {"size": mask[0], "keep_first": mask[1]}
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    if kv_from is not None:
        out["kv_from"] = kv_from
    return out


def retention(heads, dim, vdim, decay, rot=None):
    out = {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    return out


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff, shared=0):
    out = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        out["shared"] = {"ff": shared}
    return out


def layer(kind, mixer, mlp):
    return {"type": kind, "mixer": mixer, "mlp": mlp}


SMALL = {
    "architecture": "Videdra", "vocab": 300, "width": 64, "norm": {"eps": 1e-5},
    "layers": [
        layer("retention", retention(2, 16, 24, (0.9, 0.96875), rot=(5000.0, 8)), moe(6, 2, 32, shared=48)),
        layer("attention", attention(4, 2, 16, 24, 0.2, 0.25, mask=(24, 3), rot=(10000.0, 8)), dense(96)),
        layer("attention", attention(4, 2, 16, 24, 0.3, 0.4, mask=(40, 5), rot=(10000.0, 8), kv_from=1), None),
        layer("attention", attention(2, 2, 8, 16, 0.35, 0.1), moe(4, 1, 40)),
        layer("retention", retention(3, 8, 8, (1.0, 0.5, 0.99)), dense(80)),
    ],
}

ODD = {
    "architecture": "Videdra", "vocab": 211, "width": 100, "norm": {"eps": 3e-6},
    "layers": [
        layer("attention", attention(3, 1, 10, 12, 0.3, 0.35, mask=(7, 2), rot=(300.0, 10)), moe(5, 3, 18, shared=22)),
        layer("retention", retention(3, 10, 14, (0.75, 0.9375, 0.998), rot=(100000.0, 10)), dense(70)),
        layer("attention", attention(3, 1, 10, 12, 0.25, 0.2, mask=(7, 2), rot=(300.0, 10), kv_from=0), dense(50)),
    ],
}

SIZED = {
    "architecture": "Videdra", "vocab": 1201, "width": 512, "norm": {"eps": 1e-6},
    "layers": [
        layer("attention", attention(8, 2, 64, 128, 0.125, 0.3, mask=(64, 4), rot=(10000.0, 64)), dense(1024)),
        layer("retention", retention(4, 64, 128, (0.96875, 0.984375, 0.9921875, 0.99609375), rot=(1e6, 32)),
              moe(8, 2, 256, shared=512)),
        layer("attention", attention(8, 2, 64, 128, 0.125, 0.3, mask=(100, 0), rot=(10000.0, 64), kv_from=0),
              moe(8, 2, 256, shared=512)),
    ],
}

CASES = {"small": SMALL, "odd": ODD, "sized": SIZED}
_FOLDERS: dict = {}


def folder_for(name: str, std: float = 0.08, seed: int = 13, sharpen: float = 1.0) -> Path:
    """A model folder of configuration `name` with random bfloat16 weights.  `sharpen` scales
    the query projections of the attentions, so that a map sits on few keys."""
    return write_folder(CASES[name], std, seed, sharpen, key=name)


def write_folder(config: dict, std: float = 0.08, seed: int = 13, sharpen: float = 1.0,
                 key=None, edit=None) -> Path:
    """`edit(tensors)` may change the drawn tensors (a dict name -> tensor) before they are
    written."""
    from mercury_amd.weights import save_file, write_random_model
    from mercury_amd.weights.safetensors_io import SafetensorsFile

    key = (key or repr(config), std, seed, sharpen, None if edit is None else id(edit))
    if key not in _FOLDERS:
        folder = Path(tempfile.mkdtemp(prefix="mercury_videdra_"))
        write_random_model(folder, config, seed=seed, std=std, dtype=torch.bfloat16)
        if sharpen != 1.0 or edit is not None:
            path = folder / "model.safetensors"
            source = SafetensorsFile(path)
            tensors = {n: source.tensor(n).clone() for n in source.names()}
            source.close()
            for i, entry in enumerate(config["layers"]):
                if entry["type"] == "attention" and sharpen != 1.0:
                    n = f"l{i}.mix.q"
                    tensors[n] = (tensors[n].float() * sharpen).to(tensors[n].dtype)
            if edit is not None:
                edit(tensors)
            save_file(tensors, path, metadata={"format": "pt"})
        _FOLDERS[key] = folder
    return _FOLDERS[key]
