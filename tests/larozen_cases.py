"""Small Larozen configurations for the tests, and their model folders with random weights.

SMALL: multiples of 8 (the matrix-core projections run in bfloat16); a loop over the two
middle layers, three times; a parallel layer first and last; a layer without a feed-forward;
heads partly turned, a bounded score; a sink attention whose values are wider than its keys
and whose query temperature changes every 8 positions; a convolution over 4 tokens.
ODD: sizes that are no multiple of 8 (the float32-arithmetic kernels run in either dtype), no
loop, heads turned whole and an unbounded score, one key/value head, no query temperature, a
state of 9 rows in 3 groups, a convolution over 2 tokens, 3 norm groups.
SIZED: widths of a real layer; a loop over the first layer alone, twice; state-space heads of
64 columns (two workgroups a head) with 128 rows of state.
"""

from __future__ import annotations

import tempfile
from pathlib import Path

import torch


def attention(heads, kv_heads, dim, scale, rot=None, softcap=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale}
    if rot:
        out["rot"] = {"base": rot[0], "dims": rot[1]}
    if softcap:
        out["softcap"] = softcap
    return out


def side_by_side(left, right):
    return {"left": dict(left), "right": dict(right)}


def sink_attention(heads, kv_heads, dim, vdim, scale, q_temp=None):
    out = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp:
        out["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return out


def state_space(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv,
            "norm_groups": norm_groups}


def layer(kind, mixer, ff):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


_A_SMALL = attention(4, 2, 32, 0.2, rot=(5000.0, 16), softcap=20.0)
_P_SMALL = side_by_side(sink_attention(4, 4, 16, 24, 0.3, q_temp=(0.7, 8)),
                        state_space(4, 16, 24, 1, 4, 1))
SMALL = {
    "architecture": "Larozen", "vocab": 300, "width": 64, "norm": {"eps": 1e-5},
    "layers": [layer("parallel", _P_SMALL, 96), layer("attention", _A_SMALL, 80),
               layer("attention", _A_SMALL, 0), layer("parallel", _P_SMALL, 96)],
    "loop": {"start": 1, "stop": 3, "times": 3},
}

ODD = {
    "architecture": "Larozen", "vocab": 211, "width": 100, "norm": {"eps": 3e-6},
    "layers": [layer("attention", attention(3, 1, 12, 0.35, rot=(300.0, 12)), 70),
               layer("parallel", side_by_side(sink_attention(2, 1, 10, 10, 0.4),
                                              state_space(3, 10, 9, 3, 2, 3)), 50)],
}

SIZED = {
    "architecture": "Larozen", "vocab": 1201, "width": 512, "norm": {"eps": 1e-6},
    "layers": [layer("attention", attention(8, 2, 64, 0.125, rot=(10000.0, 64), softcap=50.0), 1024),
               layer("parallel", side_by_side(sink_attention(8, 2, 64, 64, 0.125, q_temp=(0.3, 32)),
                                              state_space(16, 64, 128, 2, 4, 4)), 1024)],
    "loop": {"start": 0, "stop": 1, "times": 2},
}

CASES = {"small": SMALL, "odd": ODD, "sized": SIZED}
_FOLDERS: dict = {}


def folder_for(name: str, std: float = 0.08, seed: int = 13, sharpen: float = 1.0,
               sink: float | None = None) -> Path:
    """A model folder of configuration `name` with random bfloat16 weights.  `sharpen` scales
    the query projections, so that the attention sits on few keys; `sink` sets every sink."""
    return write_folder(CASES[name], std, seed, sharpen, sink, key=name)


def write_folder(config: dict, std: float = 0.08, seed: int = 13, sharpen: float = 1.0,
                 sink: float | None = None, key=None) -> Path:
    from mercury_amd.weights import save_file, write_random_model
    from mercury_amd.weights.safetensors_io import SafetensorsFile

    key = (key or repr(config), std, seed, sharpen, sink)
    if key not in _FOLDERS:
        folder = Path(tempfile.mkdtemp(prefix="mercury_larozen_"))
        write_random_model(folder, config, seed=seed, std=std, dtype=torch.bfloat16)
        if sharpen != 1.0 or sink is not None:
            path = folder / "model.safetensors"
            source = SafetensorsFile(path)
            tensors = {n: source.tensor(n).clone() for n in source.names()}
            source.close()
            for n in tensors:
                if n.endswith(".q") and sharpen != 1.0:
                    tensors[n] = (tensors[n].float() * sharpen).to(tensors[n].dtype)
                if n.endswith(".sink") and sink is not None:
                    tensors[n] = torch.full_like(tensors[n], sink)
            save_file(tensors, path, metadata={"format": "pt"})
        _FOLDERS[key] = folder
    return _FOLDERS[key]
