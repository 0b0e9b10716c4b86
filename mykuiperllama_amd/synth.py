"""Seeded synthetic inputs for the AWQ GEMV path.

One counter-based generator (SplitMix64) written out here, so that every consumer
(tests, benchmark, smoke check, any later session) sees the same tensors for the same
(base seed, shape name, tensor name) triple regardless of numpy / torch versions.

Distributions (the benchmark configurations fix them):
  codes q, zero points z ... iid uniform on {0..15}  (packed words are uniform 32-bit)
  scales ................... fp16(RNE) of U(0.001, 0.02)
  activations .............. bf16(RNE) of N(0, 1), Box-Muller on the same generator
"""
import numpy as np

BASE_SEED = 20251125
GROUP = 128

_GAMMA = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)

# (K, N) per projection; the names are the ones the benchmark configurations use.
QWEN3_0P6B = {"q_proj": (1024, 2048)}
QWEN3_8B = {
    "q_proj": (4096, 4096),
    "k_proj": (4096, 1024),
    "v_proj": (4096, 1024),
    "o_proj": (4096, 4096),
    "gate_proj": (4096, 12288),
    "up_proj": (4096, 12288),
    "down_proj": (12288, 4096),
}
QWEN3_32B = {
    "q_proj": (5120, 8192),
    "k_proj": (5120, 1024),
    "v_proj": (5120, 1024),
    "o_proj": (8192, 5120),
    "gate_proj": (5120, 25600),
    "up_proj": (5120, 25600),
    "down_proj": (25600, 5120),
}


def awq_gemv_bytes(M, K, N, group=GROUP):
    """Algorithmic bytes of one fused dequant+GEMV: every operand byte touched once."""
    return K * N // 2 + (K // group) * N * 2 + (K // group) * N // 2 + 2 * M * K + 2 * M * N


def bf16_gemv_bytes(M, K, N):
    return 2 * K * N + 2 * M * (K + N)


def _fnv1a64(text):
    h = 0xCBF29CE484222325
    for b in text.encode("utf-8"):
        h ^= b
        h = (h * 0x100000001B3) & 0xFFFFFFFFFFFFFFFF
    return h


def tensor_seed(shape_name, tensor_name, base_seed=BASE_SEED):
    return (_fnv1a64(f"{shape_name}/{tensor_name}") ^ (base_seed * 0x9E3779B97F4A7C15)) \
        & 0xFFFFFFFFFFFFFFFF


def splitmix64(seed, n):
    """n outputs of SplitMix64 started at `seed` (output i mixes seed + (i+1)*gamma)."""
    with np.errstate(over="ignore"):
        z = np.uint64(seed) + (np.arange(1, n + 1, dtype=np.uint64) * _GAMMA)
        z = (z ^ (z >> np.uint64(30))) * _M1
        z = (z ^ (z >> np.uint64(27))) * _M2
        return z ^ (z >> np.uint64(31))


def uniform01(seed, n):
    """float64 in [0, 1) from the top 53 bits."""
    return (splitmix64(seed, n) >> np.uint64(11)).astype(np.float64) * (1.0 / 9007199254740992.0)


def normal(seed, n):
    """N(0,1) by Box-Muller; element 2i is the cosine branch, 2i+1 the sine branch."""
    half = (n + 1) // 2
    u = uniform01(seed, 2 * half)
    u1 = 1.0 - u[:half]  # (0, 1]
    u2 = u[half:]
    r = np.sqrt(-2.0 * np.log(u1))
    out = np.empty(2 * half, np.float64)
    out[0::2] = r * np.cos(2.0 * np.pi * u2)
    out[1::2] = r * np.sin(2.0 * np.pi * u2)
    return out[:n]


def f32_to_bf16_bits(a):
    """Round-to-nearest-even fp32 -> bf16 bit patterns (uint16); inputs must be finite."""
    u = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    u = u + np.uint64(0x7FFF) + ((u >> np.uint64(16)) & np.uint64(1))
    return (u >> np.uint64(16)).astype(np.uint16)


def bf16_bits_to_f32(a):
    return (np.ascontiguousarray(a, np.uint16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_f16_bits(a):
    return np.ascontiguousarray(a, np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(a):
    return np.ascontiguousarray(a, np.uint16).view(np.float16).astype(np.float32)


def random_words(seed, n):
    """Uniform 32-bit words: eight iid uniform int4 codes each."""
    return (splitmix64(seed, n) & np.uint64(0xFFFFFFFF)).astype(np.uint32).view(np.int32)


def make_awq_problem(name, M, K, N, group=GROUP, base_seed=BASE_SEED):
    """Seeded tensors of one AWQ GEMV as numpy arrays (16-bit floats as uint16 bit patterns)."""
    if K % group or N % 8:
        raise ValueError("K must be a multiple of the group size and N of 8")
    G = K // group
    qweight = random_words(tensor_seed(name, "qweight", base_seed), K * (N // 8)).reshape(K, N // 8)
    qzeros = random_words(tensor_seed(name, "qzeros", base_seed), G * (N // 8)).reshape(G, N // 8)
    s = 0.001 + 0.019 * uniform01(tensor_seed(name, "scales", base_seed), G * N)
    scales = f32_to_f16_bits(s.astype(np.float32)).reshape(G, N)
    x = f32_to_bf16_bits(normal(tensor_seed(name, "x", base_seed), M * K).astype(np.float32))
    return {"name": name, "M": M, "K": K, "N": N, "group": group,
            "x": x.reshape(M, K), "qweight": qweight, "scales": scales, "qzeros": qzeros}


def make_bf16_problem(name, M, K, N, std=0.02, base_seed=BASE_SEED):
    """Seeded tensors of one BF16 GEMV: W is bf16 [N, K] ~ N(0, std), x bf16 [M, K] ~ N(0, 1)."""
    w = f32_to_bf16_bits((std * normal(tensor_seed(name, "w_bf16", base_seed), N * K))
                         .astype(np.float32)).reshape(N, K)
    x = f32_to_bf16_bits(normal(tensor_seed(name, "x", base_seed), M * K).astype(np.float32))
    return {"name": name, "M": M, "K": K, "N": N, "x": x.reshape(M, K), "w": w}
