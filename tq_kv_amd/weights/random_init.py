"""Random weights from a configuration and a seed.

Not in the reference.  Every tensor has a random stream of its own, seeded by the
seed and the tensor's name, so a tensor's values do not depend on which other
tensors exist or in which order they are made.  Distributions by the tensor's
`init`: "normal" N(0, std), "one_plus_normal" 1 + N(0, std), "zeros".
"""
import hashlib
import json
import os

import torch

from .safetensors_io import write_file


def _tensor_seed(seed, name):
    digest = hashlib.sha256(("%d:%s" % (seed, name)).encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little") & ((1 << 63) - 1)


def random_tensor(name, spec, seed, dtype, device="cpu"):
    if spec.dtype == "int32":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    gen = torch.Generator(device=device)
    gen.manual_seed(_tensor_seed(seed, name))
    t = torch.randn(spec.shape, generator=gen, dtype=torch.float32, device=device) * spec.std
    if spec.init == "one_plus_normal":
        t = t + 1.0
    elif spec.init != "normal":
        raise ValueError("unknown init '%s' for tensor %s" % (spec.init, name))
    return t.to(dtype)


def random_tensors(wanted, seed, dtype, device="cpu"):
    """name -> tensor for every wanted name.  The stream of a tensor depends on the device
    kind it is made on (CPU and GPU generators differ)."""
    return {name: random_tensor(name, spec, seed, dtype, device) for name, spec in wanted.items()}


def write_model_folder(folder, config_dict, wanted, seed, dtype=torch.bfloat16):
    """Write config.json and model.safetensors of a model with random weights."""
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w", encoding="utf-8") as f:
        json.dump(config_dict, f, indent=2)
    write_file(os.path.join(folder, "model.safetensors"),
               ((name, random_tensor(name, spec, seed, dtype)) for name, spec in wanted.items()),
               metadata={"format": "pt", "seed": seed})
    return folder
