"""Dropout masks as pure functions of a key and an element index (TEST ORACLE, numpy).

The reference applies ``nn.Dropout`` at four places of an encoder layer (DeepSpeedExamples/pipeline_parallelism/
transformer.py: attention probabilities :125-126, the two ``SublayerConnection`` outputs :98-103, the feed-forward's
hidden activation :154-158) and reseeds torch's generator per layer and micro-batch so that a forward can be repeated
(deepspeed/runtime/pipe/module.py:538-545).  Which elements torch's generator drops is not part of the reference
(it depends on the device kernel's launch shape): **parity unpinned** for the mask bits themselves.  What is
fixed, and restated here, is the arithmetic -- kept elements are scaled by 1 / (1 - p), dropped ones are zero, an
element is kept with probability 1 - p -- and, for this build, the decision function the HIP kernels evaluate
(a 32-bit xorshift-multiply finalizer over (index / 2, key), sixteen of its bits per element), restated with numpy integer arithmetic and
pinned against the library's own host-side evaluation of it (tests/test_dropout.py)."""
import numpy as np

M64 = (1 << 64) - 1

# the four dropout sites of an encoder layer
SITE_ATTENTION, SITE_SUBLAYER0, SITE_FFN, SITE_SUBLAYER1 = 0, 1, 2, 3


def key(base_seed, step, micro_batch, layer_idx, site):
    """(k0, k1): splitmix64 chained over what identifies one mask."""
    z = 0x9E3779B97F4A7C15
    for v in (base_seed, step, micro_batch, layer_idx, site):
        z = (z + (int(v) & M64) * 0xBF58476D1CE4E5B9 + 0x9E3779B97F4A7C15) & M64
        z ^= z >> 30
        z = (z * 0xBF58476D1CE4E5B9) & M64
        z ^= z >> 27
        z = (z * 0x94D049BB133111EB) & M64
        z ^= z >> 31
    return z & 0xFFFFFFFF, z >> 32


def _mix32(x):
    x = x.astype(np.uint64)
    x ^= x >> np.uint64(16)
    x = (x * np.uint64(0x7FEB352D)) & np.uint64(0xFFFFFFFF)
    x ^= x >> np.uint64(15)
    x = (x * np.uint64(0x846CA68B)) & np.uint64(0xFFFFFFFF)
    x ^= x >> np.uint64(16)
    return x


def threshold(p):
    """16-bit threshold: an element is kept when its 16 hash bits are >= round(p * 65536) (at least 1 for p > 0)."""
    if p <= 0:
        return 0
    t = float(np.float32(p)) * 65536.0
    return 65535 if t >= 65535.0 else 1 if t < 1.0 else int(t + 0.5)


def pair_bits(k, pair):
    """The 32 hash bits shared by elements 2 * pair and 2 * pair + 1."""
    pair = np.asarray(pair, dtype=np.uint64)
    lo, hi = pair & np.uint64(0xFFFFFFFF), pair >> np.uint64(32)
    rot = ((hi << np.uint64(16)) | (hi >> np.uint64(16))) & np.uint64(0xFFFFFFFF)
    return _mix32(((lo ^ np.uint64(k[0])) + (np.uint64(k[1]) ^ rot)) & np.uint64(0xFFFFFFFF))


def keep(p, k, index):
    """Boolean array: element ``index`` (array of non-negative ints) is kept under probability-to-drop ``p``: the low
    16 bits of its pair's hash decide an even element, the high 16 bits an odd one."""
    idx = np.asarray(index, dtype=np.uint64)
    x = pair_bits(k, idx >> np.uint64(1))
    bits = np.where((idx & np.uint64(1)) == 1, x >> np.uint64(16), x & np.uint64(0xFFFF))
    return bits >= np.uint64(threshold(p))


def mask(p, k, shape):
    """0/1 float64 mask of a contiguous tensor of ``shape`` (element index = row-major position)."""
    n = int(np.prod(shape))
    return keep(p, k, np.arange(n, dtype=np.uint64)).reshape(shape).astype(np.float64)
