"""Small Talolorn configurations for the tests, and their model folders with random weights.

SMALL: multiples of 8 everywhere (the matrix-core kernels run in bfloat16), three heads, a
dense layer, routed experts, a layer that runs another's tensors, a layer without a
feed-forward.  ODD: sizes that are no multiple of 8 (the float32-arithmetic kernels run in
either dtype), one head, a rotated part only partly turned, every expert chosen, residual
factor and embedding scale of 1, the layers in another order.  SIZED: widths of a real layer,
sixteen heads (a decoded token fills one tile of the matrix-core attention).
"""

from __future__ import annotations

import tempfile
from pathlib import Path

import torch


def _mixer(heads, dim, rot_dim, vdim, q_rank, kv_rank, scale, base, dims):
    return {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank,
            "kv_rank": kv_rank, "scale": scale, "rot": {"base": base, "dims": dims}}


def _layer(mixer, mlp, **extra):
    return {"type": "latent_attention", "mixer": dict(mixer), "mlp": mlp and dict(mlp), **extra}


def _dense(ff, limit):
    return {"kind": "dense", "ff": ff, "limit": limit}


def _moe(experts, top, scale, ff, limit):
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit},
            "router": {"experts": experts, "top": top, "scale": scale}}


_M_SMALL = _mixer(3, 16, 8, 24, 40, 48, 0.21, 5000.0, 8)
SMALL = {
    "architecture": "Talolorn", "vocab": 300, "width": 64, "embedding": {"scale": 4.0},
    "norm": {"eps": 1e-5}, "residual_mult": 0.5,
    "layers": [_layer(_M_SMALL, _dense(96, 2.0)), _layer(_M_SMALL, _moe(6, 2, 1.5, 40, 1.0)),
               _layer(_M_SMALL, _moe(6, 2, 1.5, 40, 1.0), weights_of=1), _layer(_M_SMALL, None)],
}

_M_ODD = _mixer(1, 12, 6, 10, 20, 36, 0.4, 300.0, 4)
ODD = {
    "architecture": "Talolorn", "vocab": 211, "width": 100, "embedding": {"scale": 1.0},
    "norm": {"eps": 3e-6}, "residual_mult": 1.0,
    "layers": [_layer(_M_ODD, _moe(4, 4, 1.0, 50, 0.75)), _layer(_M_ODD, _dense(70, 1.5)),
               _layer(_M_ODD, _moe(4, 4, 1.0, 50, 0.75), weights_of=0)],
}

_M_SIZED = _mixer(16, 64, 32, 64, 192, 256, 0.1, 10000.0, 32)
SIZED = {
    "architecture": "Talolorn", "vocab": 1201, "width": 512, "embedding": {"scale": 8.0},
    "norm": {"eps": 1e-6}, "residual_mult": 0.8,
    "layers": [_layer(_M_SIZED, _dense(1024, 3.0)), _layer(_M_SIZED, _moe(8, 2, 2.0, 256, 3.0))],
}

CASES = {"small": SMALL, "odd": ODD, "sized": SIZED}
_FOLDERS: dict = {}


def folder_for(name: str, std: float = 0.08, seed: int = 11, sharpen: float = 1.0) -> Path:
    """A model folder of configuration `name` with random bfloat16 weights.  `sharpen` scales
    the query and key latents' up-projections, so that the attention sits on few keys."""
    from mercury_amd.weights import save_file, write_random_model
    from mercury_amd.weights.safetensors_io import SafetensorsFile

    key = (name, std, seed, sharpen)
    if key not in _FOLDERS:
        folder = Path(tempfile.mkdtemp(prefix=f"mercury_talolorn_{name}_"))
        write_random_model(folder, CASES[name], seed=seed, std=std, dtype=torch.bfloat16)
        if sharpen != 1.0:
            path = folder / "model.safetensors"
            source = SafetensorsFile(path)
            tensors = {n: source.tensor(n).clone() for n in source.names()}
            source.close()
            for n in tensors:
                if n.endswith(".mix.uq") or n.endswith(".mix.uk"):
                    tensors[n] = (tensors[n].float() * sharpen).to(tensors[n].dtype)
            save_file(tensors, path, metadata={"format": "pt"})
        _FOLDERS[key] = folder
    return _FOLDERS[key]
