"""Random weights from a configuration and a seed: the same bits on the host and on the GPU.

Not in the reference.  Element i of a tensor is a function of (seed, tensor name, i)
alone: a 64-bit key from the seed and the name, a counter-based 64-bit hash of key
and index, and from its bits one standard normal value by Box and Muller's
transform.  A tensor's values therefore depend neither on which other tensors exist
nor on the order or the device they are made on.

So that the host (numpy) and the GPU (csrc/random_init.hip) give the same bits, the
transform is built from operations that IEEE arithmetic fixes exactly and from nothing
else: integer operations, float32 multiplications and additions each rounded on its
own (no fused multiply-add), and polynomials of those for the logarithm, the cosine
and the reciprocal square root.  Both sides follow the recipe below line by line.

    x    = mix(key + (i + 1) * GOLDEN)                      (64-bit, wrapping)
    u1   = ((x >> 40) + 1) / 2^24                  in (0, 1]
    ln u1 = e * LN2 + t * Q(t),  u1 = m * 2^e,  m in [sqrt(1/2), sqrt(2)),  t = m - 1
    r    = sqrt(-2 ln u1)  by three Newton steps for 1/sqrt from an integer first guess
    low 32 bits: quadrant (2 bits) and 23 bits of angle inside it, taken from the middle
                 of a cell so that the angle is never 0 or pi/2; odd quadrants mirror the
                 angle, so one cosine polynomial C(angle^2) serves
    z    = +-r * C,  value = z * std  (+ 1 for "one_plus_normal")

Distributions by the tensor's `init`: "normal" N(0, std), "one_plus_normal" 1 + N(0, std),
"zeros".  The largest |z| is sqrt(2 * 24 * ln 2) = 5.77.
"""
import hashlib
import json
import os

import numpy as np
import torch

from .safetensors_io import write_file

GOLDEN = 0x9E3779B97F4A7C15
MIX_A, MIX_B = 0xBF58476D1CE4E5B9, 0x94D049BB133111EB
LN2 = np.float32(0.6931471805599453)
HALF_PI = np.float32(1.5707963267948966)
SQRT2 = np.float32(1.4142135)
# ln(1 + t) = t * Q(t) on [sqrt(1/2) - 1, sqrt(2) - 1], lowest power first (error 4e-8)
LOG_Q = [1.0, -0.5, 0.33333301544189453, -0.2500002384185791, 0.2000257670879364, -0.16668042540550232,
         0.14212606847286224, -0.1239922046661377, 0.11923925578594208, -0.11727229505777359, 0.06740232557058334]
# cos(a) = C(a^2) on [0, pi/2], lowest power first (error 2e-7)
COS_C = [1.0, -0.5, 0.0416666679084301, -0.0013888884568586946, 2.4801040126476437e-05, -2.752467764821631e-07,
         1.990758891068367e-09]
HOST_CHUNK = 1 << 22      # elements made at a time on the host


def tensor_key(seed, name):
    """The 64-bit key of a tensor's stream."""
    digest = hashlib.sha256(("%d:%s" % (seed, name)).encode("utf-8")).digest()
    return int.from_bytes(digest[:8], "little")


def _horner(coef, x):
    acc = np.full(x.shape, np.float32(coef[-1]), dtype=np.float32)
    for c in coef[-2::-1]:
        acc = acc * x                      # rounded
        acc = acc + np.float32(c)          # rounded again: never a fused multiply-add
    return acc


def standard_normal_host(key, begin, count):
    """z for the elements begin .. begin + count - 1 of the stream `key`: float32 numpy array."""
    with np.errstate(over="ignore"):
        i = np.arange(begin + 1, begin + count + 1, dtype=np.uint64)
        x = np.uint64(key) + i * np.uint64(GOLDEN)
        x ^= x >> np.uint64(30)
        x *= np.uint64(MIX_A)
        x ^= x >> np.uint64(27)
        x *= np.uint64(MIX_B)
        x ^= x >> np.uint64(31)
    hi = (x >> np.uint64(32)).astype(np.uint32)
    lo = (x & np.uint64(0xFFFFFFFF)).astype(np.uint32)
    # ln u1
    n = (hi >> np.uint32(8)).astype(np.int32) + np.int32(1)              # 1 .. 2^24
    bits = n.astype(np.float32).view(np.int32)
    e = (bits >> 23) - np.int32(151)                                      # u1 = m * 2^e, m in [1, 2)
    m = ((bits & np.int32(0x7FFFFF)) | np.int32(0x3F800000)).view(np.float32)
    big = m > SQRT2
    m = np.where(big, m * np.float32(0.5), m)
    e = e + big.astype(np.int32)
    t = m - np.float32(1.0)
    ln_u = e.astype(np.float32) * LN2 + t * _horner(LOG_Q, t)
    # r = sqrt(-2 ln u1) = v * (1 / sqrt(v))
    v = ln_u * np.float32(-2.0)
    y = (np.int32(0x5F3759DF) - (v.view(np.int32) >> 1)).view(np.float32)
    hv = v * np.float32(0.5)
    for _ in range(3):
        y = y * (np.float32(1.5) - hv * (y * y))
    r = v * y
    # cosine of the angle
    quadrant = lo >> np.uint32(30)
    f = ((lo >> np.uint32(7)) & np.uint32(0x7FFFFF)).astype(np.int32)
    f = np.where((quadrant & np.uint32(1)) != 0, np.int32(0x7FFFFF) - f, f)
    a = ((2 * f + 1).astype(np.float32) * np.float32(2.0 ** -24)) * HALF_PI
    c = _horner(COS_C, a * a)
    z = r * c
    return np.where((quadrant == 1) | (quadrant == 2), -z, z).astype(np.float32)


def _fill_host(key, numel, std, plus_one, dtype):
    out = torch.empty((numel,), dtype=dtype)
    for begin in range(0, numel, HOST_CHUNK):
        count = min(HOST_CHUNK, numel - begin)
        val = standard_normal_host(key, begin, count) * np.float32(std)
        if plus_one:
            val = np.float32(1.0) + val
        out[begin:begin + count] = torch.from_numpy(val).to(dtype)       # bfloat16: round to nearest even
    return out


def random_tensor(name, spec, seed, dtype, device="cpu"):
    device = torch.device(device)
    if spec.dtype == "int32":
        return torch.zeros(spec.shape, dtype=torch.int32, device=device)
    if spec.init == "zeros":
        return torch.zeros(spec.shape, dtype=dtype, device=device)
    if spec.init not in ("normal", "one_plus_normal"):
        raise ValueError("unknown init '%s' for tensor %s" % (spec.init, name))
    if dtype not in (torch.float32, torch.bfloat16):
        raise ValueError("random weights are made in float32 or bfloat16, not %s" % dtype)
    key = tensor_key(seed, name)
    plus_one = spec.init == "one_plus_normal"
    numel = 1
    for s in spec.shape:
        numel *= int(s)
    if device.type == "cuda":
        from .. import kernels as K
        out = torch.empty(tuple(spec.shape), dtype=dtype, device=device)
        return K.random_normal(out, key, spec.std, plus_one)
    return _fill_host(key, numel, spec.std, plus_one, dtype).reshape(tuple(spec.shape))


def random_tensors(wanted, seed, dtype, device="cpu"):
    """name -> tensor for every wanted name; the same values wherever they are made."""
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
