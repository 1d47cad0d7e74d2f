"""Reading and writing the golden fixtures: one ``.npz`` per case, inputs and expected outputs.

numpy has no bfloat16 or float8: such tensors are stored as their bit patterns (uint16 / uint8)
under a key that carries the type (``name__bf16``, ``name__f8e4m3``) and come back as torch
tensors of the original dtype.  Python scalars (window, scale, eps ...) are 0-d arrays.
"""
import os

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def path(name):
    return os.path.join(HERE, name + ".npz")


def save(name, **items):
    arrays = {}
    for key, val in items.items():
        if isinstance(val, torch.Tensor):
            val = val.detach().contiguous()
            if val.dtype == torch.bfloat16:
                arrays[key + "__bf16"] = val.view(torch.int16).numpy().view(np.uint16)
            elif val.dtype == torch.float8_e4m3fn:
                arrays[key + "__f8e4m3"] = val.view(torch.uint8).numpy()
            else:
                arrays[key] = val.numpy()
        else:
            arrays[key] = np.asarray(val)
    np.savez_compressed(path(name), **arrays)


def load(name):
    out = {}
    with np.load(path(name), allow_pickle=False) as z:
        for key in z.files:
            a = z[key]
            if key.endswith("__bf16"):
                out[key[:-6]] = torch.from_numpy(a.view(np.int16).copy()).view(torch.bfloat16)
            elif key.endswith("__f8e4m3"):
                out[key[:-8]] = torch.from_numpy(a.copy()).view(torch.float8_e4m3fn)
            elif a.ndim == 0:
                out[key] = a.item()
            else:
                out[key] = torch.from_numpy(a.copy())
    return out
