"""The deterministic inputs the reference's own benchmarks build (not arithmetic of the path):

* Qwen3.8 synthetic affine-Q4 matrices and activation (qwen38_m3.m:64-87,567-580): xorshift32
  code bytes, scale = 0.0035 + 0.00025 * (draw & 7), bias = -7.5 * scale + 0.0002 * (group % 5 - 2)
  as fp16; x_i = fp16(0.75 * sinf(0.013 i) + 0.20 * cosf(0.031 i)).
* MiniMax H3 closed-form GEMM (minimax_h3_m3_gemm.m:14-19,75-104; initialisers
  minimax_h3_attention.metal:190-209): K = 5376, N = 14336; code byte i: block = i >> 5,
  low = (5 i + 3 block + 3) & 15, high = (7 i + 11 block + 11) & 15; metadata of block b:
  phase = b % 7, scale = fp16(0.0175 + 0.0017 phase), bias = fp16(-0.1875 + 0.0078125 phase);
  input element i (flat over rows): ((13 i + 17) % 17 - 8) * 0.0625.
"""
import numpy as np

QWEN38_SEEDS = {"gate": 0x36A110C, "up": 0x27B4C51, "down": 0x36D027B}
H3_K, H3_N = 5376, 14336


def qwen38_weights(oracle, seed, N, K):
    """(quants uint8 [N*K/2], meta uint16 [N*(K/64)*2] of fp16 {scale, bias} pairs)."""
    groups = N * (K // 64)
    quants = np.empty(groups * 32, dtype=np.uint8)
    meta = np.empty(groups * 2, dtype=np.uint16)
    oracle.lib().orc_recipe_qwen38_weights(seed, groups, quants.ctypes.data, meta.ctypes.data)
    return quants, meta


def qwen38_weights_numpy(seed, groups):
    """The same recipe step by step in numpy integers (slow: for pinning the first groups)."""
    state = seed & 0xFFFFFFFF
    quants = np.empty(groups * 32, dtype=np.uint8)
    meta = np.empty(groups * 2, dtype=np.uint16)

    def step(s):
        s ^= (s << 13) & 0xFFFFFFFF
        s ^= s >> 17
        s ^= (s << 5) & 0xFFFFFFFF
        return s

    for g in range(groups):
        for byte in range(32):
            state = step(state)
            quants[g * 32 + byte] = state & 0xFF
        state = step(state)
        scale = np.float32(0.0035) + np.float32(0.00025) * np.float32(state & 7)
        bias = np.float32(-7.5) * scale + np.float32(0.0002) * np.float32((g % 5) - 2)
        meta[2 * g] = np.float16(scale).view(np.uint16)
        meta[2 * g + 1] = np.float16(bias).view(np.uint16)
    return quants, meta


def qwen38_activation(M, K):
    """Rows of the bench's activation formula, the index running on over the rows: fp16 [M][K]."""
    i = np.arange(M * K, dtype=np.float32)
    x = np.float32(0.75) * np.sin(np.float32(0.013) * i) + np.float32(0.20) * np.cos(np.float32(0.031) * i)
    return x.astype(np.float16).reshape(M, K)


def h3_weights(N=H3_N, K=H3_K):
    groups = K // 64
    index = np.arange(N * K // 2, dtype=np.uint32)
    block = index >> np.uint32(5)
    low = (index * np.uint32(5) + block * np.uint32(3) + np.uint32(3)) & np.uint32(15)
    high = (index * np.uint32(7) + block * np.uint32(11) + np.uint32(11)) & np.uint32(15)
    quants = (low | (high << np.uint32(4))).astype(np.uint8)
    phase = (np.arange(N * groups) % 7).astype(np.float32)
    scale = (np.float32(0.0175) + phase * np.float32(0.0017)).astype(np.float16)
    bias = (np.float32(-0.1875) + phase * np.float32(0.0078125)).astype(np.float16)
    meta = np.empty(N * groups * 2, dtype=np.uint16)
    meta[0::2], meta[1::2] = scale.view(np.uint16), bias.view(np.uint16)
    return quants, meta


def h3_input(M, K=H3_K):
    """fp32 [M][K]; every value is a multiple of 1/16 in [-0.5, 0.5]: exact in fp16 and bf16."""
    i = np.arange(M * K, dtype=np.uint32)
    return ((((i * np.uint32(13) + np.uint32(17)) % np.uint32(17)).astype(np.int32) - 8)
            * np.float32(0.0625)).astype(np.float32).reshape(M, K)
