"""Counter-based uniform numbers for sampling: one draw per (seed, sequence key, step), so a
sequence's draws do not depend on what else is in its batch.  The reference seeds one
generator per request (`StdRng::seed_from_u64(seed)`, src/main.rs:538 of yusiwen/minfer);
the generator itself is a library detail there and is not reproduced.

The host folds seed and key into one 64-bit stream id per sequence (`stream`); the device
(`uniform01` in csrc/sampling.hip) hashes that id with the step.  The seed is therefore data
that the kernels read, not an argument baked into a captured decode step."""
from __future__ import annotations

_M = 0xFFFFFFFFFFFFFFFF


def mix64(z: int) -> int:
    z = (z + 0x9E3779B97F4A7C15) & _M
    z = ((z ^ (z >> 30)) * 0xBF58476D1CE4E5B9) & _M
    z = ((z ^ (z >> 27)) * 0x94D049BB133111EB) & _M
    return z ^ (z >> 31)


def stream(seed: int, key: int) -> int:
    """The stream id of sequence `key` under `seed`, as an unsigned 64-bit integer."""
    return mix64((seed & _M) ^ mix64(key & _M))


def stream_i64(seed: int, key: int) -> int:
    """The same id as the signed 64-bit value that an int64 tensor holds."""
    s = stream(seed, key)
    return s - (1 << 64) if s >= (1 << 63) else s


def uniform(seed: int, key: int, step: int) -> float:
    """In [0, 1), 24 bits, exactly representable in float32."""
    h = mix64(stream(seed, key) ^ (step & _M))
    return (h >> 40) / 16777216.0
