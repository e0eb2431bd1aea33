"""Seeded synthetic tensors for the benchmark configurations.

One counter-based generator, so any element of any tensor can be produced
independently and the same bits feed the GPU path and the CPU checker:

    state = seed + (index + 1) * 0x9E3779B97F4A7C15            (mod 2**64)
    u64   = splitmix64 finaliser of state
    U(a,b) = a + (b - a) * ((u64 >> 40) + 0.5) / 2**24          (float64, rounded to float32 once)
    N(0,s) = s * sqrt(-2 ln u1) * cos(2 pi u2), u1/u2 = U(0,1) at indices 2i, 2i+1

Tensor t of benchmark configuration c uses seed 1000*c + t (t = 0 for the
input, then weights and biases in the lowered function's constant order).
"""
import numpy as np

_GOLD = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _splitmix64(seed, idx):
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (idx + np.uint64(1)) * _GOLD
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        z = z ^ (z >> np.uint64(31))
    return z


def _unit(seed, idx):
    """U(0,1) in float64 with 24 random bits, never 0 or 1."""
    return ((_splitmix64(seed, idx) >> np.uint64(40)).astype(np.float64) + 0.5) / 16777216.0


def uniform(shape, seed, lo=-1.0, hi=1.0):
    n = int(np.prod(shape))
    idx = np.arange(n, dtype=np.uint64)
    v = lo + (hi - lo) * _unit(seed, idx)
    return v.astype(np.float32).reshape(shape)


def normal(shape, seed, sigma=1.0):
    n = int(np.prod(shape))
    idx = np.arange(n, dtype=np.uint64)
    u1 = _unit(seed, idx * np.uint64(2))
    u2 = _unit(seed, idx * np.uint64(2) + np.uint64(1))
    v = sigma * np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)
    return v.astype(np.float32).reshape(shape)


def kaiming(shape, seed):
    """N(0, sqrt(2 / fan_in)), fan_in = product of all dims but the first."""
    fan_in = int(np.prod(shape[1:]))
    return normal(shape, seed, float(np.sqrt(2.0 / fan_in)))


# ResNet-18 constants in the lowered function's parameter order (depth-first
# argument order of the Relay graph): conv1, then per BasicBlock conv1, conv2
# and, for the first block of stages 2-4, the 1x1/2 downsample AFTER conv2.
def resnet18_const_shapes():
    shapes = [(64, 3, 7, 7), (64,)]
    cin = 64
    for stage, ch in enumerate((64, 128, 256, 512)):
        for blk in range(2):
            first = blk == 0 and stage > 0
            shapes += [(ch, cin if blk == 0 else ch, 3, 3), (ch,), (ch, ch, 3, 3), (ch,)]
            if first:
                shapes += [(ch, cin, 1, 1), (ch,)]
        cin = ch
    shapes += [(1000, 512), (1000,)]
    return shapes


def resnet18_consts(config):
    """Kaiming-normal weights, U(-0.1, 0.1) biases (folded batch-norm shifts)."""
    out = []
    for t, shp in enumerate(resnet18_const_shapes(), start=1):
        seed = 1000 * config + t
        out.append(kaiming(shp, seed) if len(shp) > 1 else uniform(shp, seed, -0.1, 0.1))
    return out


def resnet18_input(config, batch, hw=224):
    return normal((batch, 3, hw, hw), 1000 * config, 1.0)
