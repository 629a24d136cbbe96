"""Seeded synthetic inputs for the five benchmark configurations.

The generator is counter based (splitmix64 over an index range), so a buffer depends
only on (seed, stream, length), never on a library's RNG version.  Normals come from
Box-Muller in fp64 and are rounded / cast afterwards.

l-ten's quantized path takes both operands as uint8 with uint8 zero points
(l-ten/math_fns.cpp:1311): an "int8 weight w with zero point 0" is handed over as the
byte w XOR 0x80 (= w + 128) with zero point 128.
"""
import hashlib

import numpy as np

_M64 = np.uint64(0xFFFFFFFFFFFFFFFF)


def splitmix64(index, seed):
    """splitmix64 output for counters `index` (uint64 array) under `seed`."""
    with np.errstate(over="ignore"):
        z = (index.astype(np.uint64) + np.uint64(seed)) * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def _bits(n, seed, stream):
    idx = np.arange(n, dtype=np.uint64)
    s = (int(seed) * 0x100000001B3 + int(stream) * 0x9E3779B1 + 0x1234567) & 0xFFFFFFFFFFFFFFFF
    return splitmix64(idx, s)


def uniform_u8(n, seed, stream=0):
    """n bytes uniform over 0..255."""
    return (_bits(n, seed, stream) >> np.uint64(56)).astype(np.uint8)


def uniform_f64(n, seed, stream=0):
    """n doubles uniform in [0, 1) with 53 random bits."""
    return (_bits(n, seed, stream) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def normal_f64(n, seed, stream=0):
    """n standard normals (Box-Muller on two uniform streams)."""
    u1 = uniform_f64(n, seed, stream * 2 + 101)
    u2 = uniform_f64(n, seed, stream * 2 + 102)
    u1 = np.maximum(u1, 2.0 ** -53)
    return np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)


def uniform_int(n, lo, hi, seed, stream=0):
    """n integers uniform over lo..hi inclusive."""
    span = np.uint64(hi - lo + 1)
    return ((_bits(n, seed, stream) >> np.uint64(16)) % span).astype(np.int64) + lo


def int8_weights_as_u8(n, std, seed, stream=0):
    """clip(round(N(0,std)), -127, 127) stored as the byte w XOR 0x80 (zero point 128)."""
    w = np.clip(np.rint(normal_f64(n, seed, stream) * std), -127, 127).astype(np.int16)
    return (w + 128).astype(np.uint8)


def digest(*arrays):
    h = hashlib.sha256()
    for a in arrays:
        h.update(np.ascontiguousarray(a).tobytes())
    return h.hexdigest()[:16]


# ---------------------------------------------------------------------------- configs

def int8_fc(M, N, K, zp_a, scale_a, scale_b, scale_c, zp_c, seed):
    """uint8 activations X[M,K], weights W[N,K] (int8 N(0,40) as u8, zero point 128)."""
    X = uniform_u8(M * K, seed, 1).reshape(M, K)
    W = int8_weights_as_u8(N * K, 40.0, seed, 2).reshape(N, K)
    scales = np.array([scale_a, scale_b, scale_c], dtype=np.float32)
    zps = np.array([zp_a, 128, zp_c], dtype=np.uint8)
    return X, W, scales, zps


def cfg1(seed=1):
    """64x784 u8 (zero point 0, scale 1/255) x 512x784 int8 (scale 0.01) -> u8 (scale 0.05, zero point 128)."""
    return int8_fc(64, 512, 784, 0, 1.0 / 255.0, 0.01, 0.05, 128, seed)


def cfg3(seed=3, size=4096):
    """Square int8 FC, activations zero point 128.  Scales: accumulator std is about
    sqrt(K)*74*40 = 1.9e5 at K=4096; multiplier 4e-4 puts outputs at 128 + N(0,76), so
    most land in 0..255 and roughly one in ten wraps."""
    return int8_fc(size, size, size, 128, 0.02, 0.02, 1.0, 128, seed)


def cfg4(M, seed=4, K=8192, N=8192):
    """Skinny weight streaming int8 FC, M in {1,4,16}; multiplier 2.8e-4 (about 128 + N(0,75))."""
    return int8_fc(M, N, K, 128, 0.02, 0.014, 1.0, 128, seed)


# (scales, zero points) of the int8 configurations without generating their operands
def cfg1_params():
    return np.array([1.0 / 255.0, 0.01, 0.05], np.float32), np.array([0, 128, 128], np.uint8)


def cfg3_params():
    return np.array([0.02, 0.02, 1.0], np.float32), np.array([128, 128, 128], np.uint8)


def cfg4_params():
    return np.array([0.02, 0.014, 1.0], np.float32), np.array([128, 128, 128], np.uint8)


def cfg2(seed=2, batch=128, sizes=(784, 1024, 1024, 10)):
    """fp32 MLP: X uniform [0,1), W_l and b_l ~ N(0,0.05), labels uniform 0..9."""
    X = uniform_f64(batch * sizes[0], seed, 1).astype(np.float32).reshape(batch, sizes[0])
    Ws, bs = [], []
    for l in range(len(sizes) - 1):
        Ws.append((normal_f64(sizes[l + 1] * sizes[l], seed, 10 + l) * 0.05).astype(np.float32)
                  .reshape(sizes[l + 1], sizes[l]))
        bs.append((normal_f64(sizes[l + 1], seed, 20 + l) * 0.05).astype(np.float32))
    labels = uniform_int(batch, 0, sizes[-1] - 1, seed, 30)
    return X, Ws, bs, labels


def cfg5(seed=5, N=32, H=128, W=128, channels=(1, 32, 64)):
    """fp32 NCHW conv stack input N(0,1); 3x3 Kaiming-normal weights (std = sqrt(2/fan_in));
    upstream gradients for the weight gradient ~ N(0,1)."""
    x = normal_f64(N * channels[0] * H * W, seed, 1).astype(np.float32).reshape(N, channels[0], H, W)
    ws, dys = [], []
    for l in range(len(channels) - 1):
        fan_in = channels[l] * 9
        ws.append((normal_f64(channels[l + 1] * fan_in, seed, 10 + l) * np.sqrt(2.0 / fan_in)).astype(np.float32)
                  .reshape(channels[l + 1], channels[l], 3, 3))
        dys.append((N, channels[l + 1], H, W))
    return x, ws, dys


def cfg5_dy(shape, seed=5, layer=0):
    n = int(np.prod(shape))
    return normal_f64(n, seed, 40 + layer).astype(np.float32).reshape(shape)
