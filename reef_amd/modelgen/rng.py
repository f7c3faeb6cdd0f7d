"""Seeded synthetic tensors: SplitMix64 -> Box-Muller (fp64) -> fp32.

Deterministic across machines and independent of numpy's generators, so the
240 MB of ResNet-152 weights never need to be stored: any host regenerates the
same bits from (base seed, tensor name).
"""
import numpy as np

BASE_SEED = 0x5EEF
_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_C1 = np.uint64(0xBF58476D1CE4E5B9)
_C2 = np.uint64(0x94D049BB133111EB)


def fnv1a(name):
    h = 0xCBF29CE484222325
    for b in name.encode("ascii"):
        h ^= b
        h = (h * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def splitmix64(seed, n):
    """n successive SplitMix64 outputs for `seed` (uint64 array)."""
    with np.errstate(over="ignore"):
        idx = np.arange(1, n + 1, dtype=np.uint64)
        z = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) + idx * _GAMMA
        z = (z ^ (z >> np.uint64(30))) * _C1
        z = (z ^ (z >> np.uint64(27))) * _C2
        z = z ^ (z >> np.uint64(31))
    return z


def uniform(seed, n):
    """n doubles in (0, 1)."""
    z = splitmix64(seed, n)
    return ((z >> np.uint64(11)).astype(np.float64) + 0.5) * (1.0 / 9007199254740992.0)


def normal(seed, n):
    m = (n + 1) // 2
    u = uniform(seed, 2 * m)
    r = np.sqrt(-2.0 * np.log(u[:m]))
    t = 2.0 * np.pi * u[m:]
    out = np.concatenate([r * np.cos(t), r * np.sin(t)])[:n]
    return out


def tensor_seed(name, base=BASE_SEED):
    return base ^ fnv1a(name)


def normal_f32(name, n, std, base=BASE_SEED):
    return (normal(tensor_seed(name, base), n) * std).astype(np.float32)


def uniform_f32(name, n, base=BASE_SEED):
    return uniform(tensor_seed(name, base), n).astype(np.float32)


def randint(name, n, high, base=BASE_SEED):
    z = splitmix64(tensor_seed(name, base), n)
    return (z % np.uint64(high)).astype(np.int64)
