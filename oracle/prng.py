"""Counter-based PRNG used for temperature sampling (test infrastructure only).

Reference: tunix/generate/sampler.py:562 (``jax.random.fold_in(seed,
decoding_step)``), :128 and :144 (``jax.random.categorical``), :938-941
(``PRNGKey(0)`` default).  JAX is a third-party dependency that is not
installed here (jax>=0.6.0, pyproject.toml:31); its published algorithm is
restated: threefry2x32 (Salmon et al., Random123, 20 rounds), the
"partitionable" bit generation that is the default from jax 0.5 on
(bits[i] = x0 ^ x1 of threefry(key, (hi32(i), lo32(i))) over the row-major
linear index i), ``uniform`` = mantissa fill, ``gumbel`` = -log(-log(u)).
The block function is pinned by the Random123 known-answer vectors; the key and
counter word order by the key pair JAX's documentation prints for
split(PRNGKey(0)); random_bits and the mantissa fill by the documented value of
normal(key(42)).  fold_in's counter words, gumbel's clamping at the smallest
normal float and categorical's use of them have no published value to check
against: for these the wiring is parity unpinned.
"""
import numpy as np

_ROT = ((13, 15, 26, 6), (17, 29, 16, 24))
_M32 = np.uint64(0xFFFFFFFF)


def _rotl(x, r):
  return ((x << np.uint32(r)) | (x >> np.uint32(32 - r))).astype(np.uint32)


def threefry2x32(k0, k1, c0, c1):
  """Threefry-2x32, 20 rounds.  All arguments uint32 (scalars or arrays)."""
  with np.errstate(over='ignore'):
    k0 = np.asarray(k0, np.uint32)
    k1 = np.asarray(k1, np.uint32)
    ks = (k0, k1, (k0 ^ k1 ^ np.uint32(0x1BD11BDA)).astype(np.uint32))
    x0 = (np.asarray(c0, np.uint32) + ks[0]).astype(np.uint32)
    x1 = (np.asarray(c1, np.uint32) + ks[1]).astype(np.uint32)
    for g in range(5):
      for r in _ROT[g % 2]:
        x0 = (x0 + x1).astype(np.uint32)
        x1 = _rotl(x1, r)
        x1 = (x1 ^ x0).astype(np.uint32)
      x0 = (x0 + ks[(g + 1) % 3]).astype(np.uint32)
      x1 = (x1 + ks[(g + 2) % 3] + np.uint32(g + 1)).astype(np.uint32)
  return x0, x1


def prng_key(seed):
  """jax.random.PRNGKey(int) -> (hi32, lo32) with 64-bit types disabled, the reference's
  configuration: the seed becomes an int32 array (low 32 bits, two's complement), whose logical
  shift by 32 is 0, so the high key word is 0 for every int, negative ones included."""
  return np.uint32(0), np.uint32(int(seed) & 0xFFFFFFFF)


def fold_in(key, data):
  """jax.random.fold_in: threefry(key, (0, data)) -> new key."""
  x0, x1 = threefry2x32(key[0], key[1], np.uint32(0), np.uint32(int(data) & 0xFFFFFFFF))
  return np.uint32(x0), np.uint32(x1)


def random_bits(key, shape):
  n = int(np.prod(shape))
  idx = np.arange(n, dtype=np.uint64)
  hi = (idx >> np.uint64(32)).astype(np.uint32)
  lo = (idx & _M32).astype(np.uint32)
  x0, x1 = threefry2x32(key[0], key[1], hi, lo)
  return (x0 ^ x1).reshape(shape)


def uniform_from_bits(bits):
  """jax.random.uniform(minval=tiny, maxval=1) applied to raw 32-bit words."""
  tiny = np.float32(np.finfo(np.float32).tiny)
  f = ((bits >> np.uint32(9)) | np.uint32(0x3F800000)).view(np.float32) - np.float32(1.0)
  return np.maximum(tiny, f * (np.float32(1.0) - tiny) + tiny).astype(np.float32)


def gumbel(key, shape):
  u = uniform_from_bits(random_bits(key, shape))
  return (-np.log(-np.log(u))).astype(np.float32)


def categorical(key, logits):
  """argmax(logits + gumbel) along the last axis (first index on ties)."""
  logits = np.asarray(logits, np.float32)
  return np.argmax(logits + gumbel(key, logits.shape), axis=-1).astype(np.int32)
