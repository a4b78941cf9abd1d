"""Seeded synthetic inputs that are bit-reproducible on any machine.

The reference fills its buffers with glibc ``rand()`` (src/utils.c:20-29), which
is not portable.  Here every value comes from a counter-based SplitMix64 stream
evaluated with exact 64-bit integer arithmetic in numpy, so the same (seed,
index) gives the same float everywhere:

* ``ternary``  -- i.i.d. uniform over {-1, 0, +1}  (rand()%3 - 1 in the reference)
* ``binary``   -- i.i.d. uniform over {-1, +1}     (2*(rand()%2) - 1)
* ``normal``   -- N(0,1) built as an Irwin-Hall sum of twelve 16-bit uniforms,
  (sum - 393210) / 65536: an exact integer construction (mean 0, variance 1,
  support +-6) with no libm call, so thresholding it is reproducible.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def splitmix64(seed, n, offset=0):
    """n 64-bit outputs of SplitMix64 started at `seed`, counters offset..offset+n-1."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = np.uint64(seed) + idx * _GOLDEN
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _chunks(n, step=1 << 22):
    for start in range(0, n, step):
        yield start, min(step, n - start)


def ternary(seed, shape):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    for s, c in _chunks(n):
        out[s:s + c] = (splitmix64(seed, c, s) >> np.uint64(11)) % np.uint64(3)
    out -= 1.0
    return out.reshape(shape)


def binary(seed, shape):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    for s, c in _chunks(n):
        out[s:s + c] = (splitmix64(seed, c, s) >> np.uint64(17)) & np.uint64(1)
    out = out * 2.0 - 1.0
    return out.astype(np.float32).reshape(shape)


def normal(seed, shape):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    mask = np.uint64(0xFFFF)
    for s, c in _chunks(n, 1 << 20):
        acc = np.zeros(c, dtype=np.int64)
        for k in range(3):
            z = splitmix64(seed + 0x1000003 * (k + 1), c, s)
            for sh in (0, 16, 32, 48):
                acc += ((z >> np.uint64(sh)) & mask).astype(np.int64)
        out[s:s + c] = (acc - 393210).astype(np.float32) / np.float32(65536.0)
    return out.reshape(shape)
