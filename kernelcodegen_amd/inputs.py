"""Deterministic, counter-based input generator shared by tests and bench.

Element i of tensor `tensor_id` under `seed` is a pure function of
(seed, tensor_id, i), so any slice of a tensor can be regenerated anywhere:

    x  = seed ^ (tensor_id << 56) ^ i                     (64-bit)
    z  = splitmix64 finaliser of (x + 0x9E3779B97F4A7C15)
    u1 = z >> 40            (top 24 bits)      u2 = (z >> 16) & 0xFFFFFF
    uniform[-1,1) = u1 / 2^23 - 1                          (exact in fp32)
    normal(0,1)   = sqrt(-2 ln((u1+1)/2^24)) * cos(2 pi u2/2^24)   in fp64,
                    rounded once to fp32
    bf16          = round-to-nearest-even of the fp32 value

The reference has no input generator (its harness is not in its tree); the
distributions are those BASELINE.json's configs name.
"""
import numpy as np

_GOLDEN = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)
_CHUNK = 1 << 22


def _mix(x):
    with np.errstate(over="ignore"):
        x = x + _GOLDEN
        z = (x ^ (x >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def _bits(seed, tensor_id, start, count):
    idx = np.arange(start, start + count, dtype=np.uint64)
    base = np.uint64(seed & 0xFFFFFFFFFFFFFFFF) ^ (np.uint64(tensor_id) << np.uint64(56))
    return _mix(base ^ idx)


def _fill(shape, seed, tensor_id, kind, std):
    n = int(np.prod(shape))
    out = np.empty(n, dtype=np.float32)
    for s in range(0, n, _CHUNK):
        c = min(_CHUNK, n - s)
        z = _bits(seed, tensor_id, s, c)
        u1 = (z >> np.uint64(40)).astype(np.float64)
        if kind == "uniform":
            out[s:s + c] = (u1 / 8388608.0 - 1.0).astype(np.float32)
        else:
            u2 = ((z >> np.uint64(16)) & np.uint64(0xFFFFFF)).astype(np.float64)
            r = np.sqrt(-2.0 * np.log((u1 + 1.0) / 16777216.0))
            v = r * np.cos((2.0 * np.pi / 16777216.0) * u2)
            if std != 1.0:
                v = v * std
            out[s:s + c] = v.astype(np.float32)
    return out.reshape(shape)


def uniform(shape, seed, tensor_id):
    """fp32 i.i.d. uniform on [-1, 1)."""
    return _fill(shape, seed, tensor_id, "uniform", 1.0)


def normal(shape, seed, tensor_id, std=1.0):
    """fp32 i.i.d. normal(0, std^2)."""
    return _fill(shape, seed, tensor_id, "normal", float(std))


def to_bf16_bits(x):
    """Round fp32 to bf16 (nearest even); returns uint16 bit patterns."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32)
    nan = (u & np.uint32(0x7FFFFFFF)) > np.uint32(0x7F800000)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    r = ((u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)).astype(np.uint16)
    r[nan] = ((u[nan] >> np.uint32(16)) | np.uint32(0x40)).astype(np.uint16)
    return r


def bf16_bits_to_f32(b):
    """Widen bf16 bit patterns (uint16) exactly to fp32."""
    return (np.ascontiguousarray(b, dtype=np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


# The five workloads of BASELINE.json's `configs`, by position.
SEED_BASE = 0xC0DE0000


def config_inputs(cfg):
    """Host tensors for workload `cfg` (0..4): dict with the operands and attributes."""
    seed = SEED_BASE + cfg
    if cfg == 0:
        return dict(kind="gemm", A=uniform((4096, 1024), seed, 0), B=uniform((1024, 2048), seed, 1), relu=True)
    if cfg == 1:
        return dict(kind="gemm", A=normal((4096, 4096), seed, 0), B=normal((4096, 4096), seed, 1), relu=True)
    if cfg == 2:
        return dict(kind="gemm", A=normal((32768, 768), seed, 0), B=normal((768, 768), seed, 1, std=0.02), relu=False)
    if cfg == 3:
        shp = (1, 32, 2048, 128)
        return dict(kind="fmha", dtype="f32", causal=False, scale=128 ** -0.5,
                    Q=normal(shp, seed, 0), K=normal(shp, seed, 1), V=normal(shp, seed, 2))
    if cfg == 4:
        shp = (4, 32, 4096, 128)
        return dict(kind="fmha", dtype="bf16", causal=True, scale=128 ** -0.5,
                    Q=to_bf16_bits(normal(shp, seed, 0)), K=to_bf16_bits(normal(shp, seed, 1)),
                    V=to_bf16_bits(normal(shp, seed, 2)))
    raise ValueError("cfg must be 0..4")
