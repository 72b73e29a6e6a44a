"""Counter-based generator for synthetic inputs: splitmix64 stream -> U[0,1) -> Box-Muller.
Same functions as csrc/host/rng.h (integer stream and uniforms are bit-identical; normals go
through libm/numpy transcendental functions and may differ in the last f32 bit)."""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z):
    z = (z ^ (z >> np.uint64(30))) * _M1
    z = (z ^ (z >> np.uint64(27))) * _M2
    return z ^ (z >> np.uint64(31))


def u64(seed, n, start=0):
    """Outputs start .. start+n of splitmix64 started from `seed`."""
    with np.errstate(over="ignore"):
        i = np.arange(start + 1, start + n + 1, dtype=np.uint64)
        return _mix(np.uint64(seed) + i * _GOLDEN)


def u01(seed, n, start=0):
    return (u64(seed, n, start) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def uniform_pm1(seed, n):
    """U(-1, 1) as f32."""
    return (2.0 * u01(seed, n) - 1.0).astype(np.float32)


def normal(seed, n, std=1.0):
    """N(0, std^2) as f32: outputs 2p, 2p+1 of the stream feed Box-Muller pair p."""
    pairs = (n + 1) // 2
    u = u01(seed, 2 * pairs)
    u1, u2 = u[0::2], u[1::2]
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    a = 6.283185307179586476925286766559 * u2
    out = np.empty(2 * pairs, dtype=np.float64)
    out[0::2] = r * np.cos(a)
    out[1::2] = r * np.sin(a)
    return (out[:n] * std).astype(np.float32)


def token_ids(seed, n, vocab):
    """Uniform ids in [0, vocab)."""
    return (u64(seed, n) % np.uint64(vocab)).astype(np.int32)


def bf16_round(x):
    """Round-to-nearest-even f32 -> bf16 -> f32 (half::bf16::from_f32)."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return ((u + r) & np.uint32(0xFFFF0000)).view(np.float32)


def to_bf16_bits(x):
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    r = np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))
    return ((u + r) >> np.uint32(16)).astype(np.uint16)


def from_bf16_bits(b):
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)
