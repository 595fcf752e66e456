"""Deterministic synthetic tensors for the quantized-matmul / MoE configurations.

One counter-based generator (splitmix64 -> uniform / Box-Muller normal) seeded per tensor, so a
tensor's bytes depend only on (config, tensor id, shape) and never on generation order. All f16
fields are RNE conversions of the drawn magnitudes; block layouts follow the GGUF encodings the
engine decodes (Q4_K 144 B / 256 weights, Q6_K 210 B / 256, Q8_0 34 B / 32).
"""
import numpy as np

BASE_SEED = 0x746F6B73


def tensor_seed(config, tensor_id):
    return (BASE_SEED ^ (config << 16) ^ tensor_id) & 0xFFFFFFFFFFFFFFFF


def splitmix64(seed, n, offset=0):
    """n 64-bit outputs of the splitmix64 sequence starting at counter `offset`."""
    with np.errstate(over="ignore"):
        idx = np.arange(offset + 1, offset + n + 1, dtype=np.uint64)
        z = np.uint64(seed) + idx * np.uint64(0x9E3779B97F4A7C15)
        z = (z ^ (z >> np.uint64(30))) * np.uint64(0xBF58476D1CE4E5B9)
        z = (z ^ (z >> np.uint64(27))) * np.uint64(0x94D049BB133111EB)
        return z ^ (z >> np.uint64(31))


def uniform_bytes(seed, n):
    words = splitmix64(seed, (n + 7) // 8)
    return words.view(np.uint8)[:n].copy()


def uniform01(seed, n, offset=0):
    return (splitmix64(seed, n, offset) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def normal(seed, n, sigma=1.0):
    """Box-Muller over consecutive pairs of uniforms; float64."""
    m = (n + 1) // 2
    u1 = uniform01(seed, m)
    u2 = uniform01(seed ^ 0x5851F42D4C957F2D, m)
    r = np.sqrt(-2.0 * np.log(1.0 - u1))
    out = np.empty(2 * m, dtype=np.float64)
    out[0::2] = r * np.cos(2 * np.pi * u2)
    out[1::2] = r * np.sin(2 * np.pi * u2)
    return out[:n] * sigma


def f16_bits(x):
    return np.asarray(x, dtype=np.float64).astype(np.float16).view(np.uint16)


def activations_f32(seed, shape):
    return normal(seed, int(np.prod(shape))).astype(np.float32).reshape(shape)


def round_bf16(a):
    """RNE float32 -> bf16 -> float32 (finite inputs)."""
    a = np.ascontiguousarray(a, dtype=np.float32)
    bits = a.view(np.uint32).astype(np.uint64)
    r = (((bits + 0x7FFF + ((bits >> 16) & 1)) >> 16) << 16).astype(np.uint32)
    return r.view(np.float32).reshape(a.shape)


def bf16_bits(a):
    return (round_bf16(a).view(np.uint32) >> 16).astype(np.uint16)


def pack_scales12(sc, mn):
    """[n,8] 6-bit scales and mins -> [n,12] GGUF Q4_K/Q5_K scale bytes."""
    sc = sc.astype(np.uint8)
    mn = mn.astype(np.uint8)
    s = np.zeros((sc.shape[0], 12), dtype=np.uint8)
    s[:, 0:4] = (sc[:, 0:4] & 63) | ((sc[:, 4:8] >> 4) << 6)
    s[:, 4:8] = (mn[:, 0:4] & 63) | ((mn[:, 4:8] >> 4) << 6)
    s[:, 8:12] = (sc[:, 4:8] & 15) | ((mn[:, 4:8] & 15) << 4)
    return s


def q4k_blocks(seed, nblocks, sigma=0.02):
    """[nblocks,144] Q4_K super-blocks: uniform nibbles, uniform 6-bit scales/mins, d,dmin = f16(|N(0,sigma)|)."""
    out = np.empty((nblocks, 144), dtype=np.uint8)
    dm = np.abs(normal(seed ^ 0x11, 2 * nblocks, sigma)).reshape(nblocks, 2)
    out[:, 0:4] = f16_bits(dm).view(np.uint8).reshape(nblocks, 4)
    sm = uniform_bytes(seed ^ 0x22, 16 * nblocks).reshape(nblocks, 16) & 63
    out[:, 4:16] = pack_scales12(sm[:, 0:8], sm[:, 8:16])
    out[:, 16:144] = uniform_bytes(seed ^ 0x33, 128 * nblocks).reshape(nblocks, 128)
    return out


def q6k_blocks(seed, nblocks, sigma=0.02):
    """[nblocks,210] Q6_K blocks: uniform 6-bit codes, uniform int8 sub-scales, d = f16(|N(0,sigma)|)."""
    out = np.empty((nblocks, 210), dtype=np.uint8)
    out[:, 0:192] = uniform_bytes(seed ^ 0x44, 192 * nblocks).reshape(nblocks, 192)
    out[:, 192:208] = uniform_bytes(seed ^ 0x55, 16 * nblocks).reshape(nblocks, 16)
    out[:, 208:210] = f16_bits(np.abs(normal(seed ^ 0x66, nblocks, sigma))).view(np.uint8).reshape(nblocks, 2)
    return out


def q8_0_blocks(seed, nblocks, sigma=0.01):
    """[nblocks,34] Q8_0 blocks: int8 uniform in [-127,127], d = f16(|N(0,sigma)|)."""
    out = np.empty((nblocks, 34), dtype=np.uint8)
    out[:, 0:2] = f16_bits(np.abs(normal(seed ^ 0x77, nblocks, sigma))).view(np.uint8).reshape(nblocks, 2)
    u = splitmix64(seed ^ 0x88, 32 * nblocks)
    q = ((u >> np.uint64(32)) % np.uint64(255)).astype(np.int64) - 127
    out[:, 2:34] = q.astype(np.int8).view(np.uint8).reshape(nblocks, 32)
    return out


def q5_1_blocks(seed, nblocks, sigma=0.02):
    out = uniform_bytes(seed ^ 0x99, 24 * nblocks).reshape(nblocks, 24).copy()
    dm = normal(seed ^ 0xAA, 2 * nblocks, sigma).reshape(nblocks, 2)
    out[:, 0:4] = f16_bits(dm).view(np.uint8).reshape(nblocks, 4)
    return out


def q5k_blocks(seed, nblocks, sigma=0.02):
    out = np.empty((nblocks, 176), dtype=np.uint8)
    q4 = q4k_blocks(seed, nblocks, sigma)
    out[:, 0:16] = q4[:, 0:16]
    out[:, 16:48] = uniform_bytes(seed ^ 0xBB, 32 * nblocks).reshape(nblocks, 32)
    out[:, 48:176] = q4[:, 16:144]
    return out


BLOCKS = {7: (q5_1_blocks, 32, 24), 8: (q8_0_blocks, 32, 34), 12: (q4k_blocks, 256, 144),
          13: (q5k_blocks, 256, 176), 14: (q6k_blocks, 256, 210)}


def matrix(encoding, seed, rows, columns):
    """Row-major block-quantised matrix bytes [rows * columns/epb * bytes_per_block]."""
    gen, epb, _ = BLOCKS[encoding]
    assert columns % epb == 0
    return gen(seed, rows * (columns // epb)).reshape(-1)


# The rank bias ln(rank^-1.1) at full strength sends almost every token to the same ten experts (per-expert
# loads up to T = 2048, two thirds of the experts empty). Scaled by 0.25 the realised loads for T = 2048,
# top-10 of 512 are min 7 / median 27 / max 444 with every expert non-empty: the ragged 0..~400 profile the
# grouped-GEMM configuration describes, and the worst case for weight traffic.
ZIPF_BIAS_SCALE = 0.25


def zipf_router_logits(seed, tokens, experts, s=1.1, scale=1.0):
    """N(0,1) logits plus scale*ln(rank^-s) under a fixed random expert ranking (Zipf-like expert loads)."""
    rank = np.argsort(uniform01(seed ^ 0xCC, experts)).argsort() + 1
    bias = -s * np.log(rank.astype(np.float64)) * scale
    return (normal(seed, tokens * experts).reshape(tokens, experts) + bias).astype(np.float32)
