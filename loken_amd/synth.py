"""Seeded synthetic GGUF blocks and activations, shared by tests and the benchmark.

A counter-based generator: value ``i`` of tensor ``stream`` under ``seed`` is
``mix(mix(seed * G + stream) + (i + 1) * G)`` with the splitmix64 finalizer ``mix`` and
``G = 0x9E3779B97F4A7C15``; no state is carried, so any slice can be produced on its own and
the same call gives the same bytes on every machine.

  * bytes: the little-endian bytes of consecutive 64-bit outputs;
  * uniform ints in ``[0, r)``: ``u64 % r``;
  * normals: Box-Muller in f64 from the two 32-bit halves of one output,
    ``sqrt(-2 ln((hi + 1) / 2^32)) * cos(2 pi lo / 2^32)``, cast to f32.

Block field distributions (configs of the quantized-matmul benchmark):
  Q4_K  qs bytes uniform (each nibble 0..15), the sixteen 6-bit fields uniform 0..63,
        d = f16(|N(0,1)| * 1e-3), dmin = f16(|N(0,1)| * 5e-4)
  Q6_K  ql, qh bytes uniform, scales int8 uniform in [-64, 63], d = f16(|N(0,1)| * 1e-3)
  Q8_0  qs uniform in [-127, 127], d = f16(|N(0,1)| * 1e-3)
"""
from __future__ import annotations

import numpy as np

GGML_Q4_0, GGML_Q4_1, GGML_Q5_0, GGML_Q5_1 = 2, 3, 6, 7
GGML_IQ4_NL, GGML_MXFP4 = 20, 39
GGML_Q2_K, GGML_Q3_K = 10, 11
GGML_IQ4_XS = 23
GGML_IQ2_XXS, GGML_IQ3_XXS, GGML_IQ3_S, GGML_IQ2_S, GGML_Q2_0 = 16, 18, 21, 22, 42   # the codebook expert formats
GGML_Q8_0, GGML_Q8_1, GGML_Q4_K, GGML_Q5_K, GGML_Q6_K = 8, 9, 12, 13, 14
BLOCK_LEN = {GGML_IQ2_XXS: 256, GGML_IQ3_XXS: 256, GGML_IQ3_S: 256, GGML_IQ2_S: 256, GGML_Q2_0: 64, GGML_IQ4_XS: 256, GGML_Q2_K: 256, GGML_Q3_K: 256, GGML_IQ4_NL: 32, GGML_MXFP4: 32, GGML_Q4_0: 32, GGML_Q4_1: 32, GGML_Q5_0: 32, GGML_Q5_1: 32, GGML_Q8_0: 32, GGML_Q8_1: 32, GGML_Q4_K: 256, GGML_Q5_K: 256, GGML_Q6_K: 256}
BLOCK_BYTES = {GGML_IQ2_XXS: 66, GGML_IQ3_XXS: 98, GGML_IQ3_S: 110, GGML_IQ2_S: 82, GGML_Q2_0: 18, GGML_IQ4_XS: 136, GGML_Q2_K: 84, GGML_Q3_K: 110, GGML_IQ4_NL: 18, GGML_MXFP4: 17, GGML_Q4_0: 18, GGML_Q4_1: 20, GGML_Q5_0: 22, GGML_Q5_1: 24, GGML_Q8_0: 34, GGML_Q8_1: 36, GGML_Q4_K: 144, GGML_Q5_K: 176, GGML_Q6_K: 210}

_G = np.uint64(0x9E3779B97F4A7C15)
_M1 = np.uint64(0xBF58476D1CE4E5B9)
_M2 = np.uint64(0x94D049BB133111EB)


def _mix(z: np.ndarray) -> np.ndarray:
    z = z.copy()
    z ^= z >> np.uint64(30)
    z *= _M1
    z ^= z >> np.uint64(27)
    z *= _M2
    z ^= z >> np.uint64(31)
    return z


def u64(seed: int, stream: int, count: int, start: int = 0) -> np.ndarray:
    """``count`` 64-bit outputs of (seed, stream), from index ``start``."""
    with np.errstate(over="ignore"):
        base = _mix(np.array([np.uint64(seed) * _G + np.uint64(stream)], dtype=np.uint64))[0]
        idx = np.arange(start + 1, start + 1 + count, dtype=np.uint64)
        return _mix(idx * _G + base)


def rand_bytes(seed: int, stream: int, count: int) -> np.ndarray:
    return u64(seed, stream, (count + 7) // 8).view(np.uint8)[:count].copy()


def rand_ints(seed: int, stream: int, count: int, r: int) -> np.ndarray:
    return (u64(seed, stream, count) % np.uint64(r)).astype(np.int64)


def normal(seed: int, stream: int, count: int) -> np.ndarray:
    v = u64(seed, stream, count)
    hi = (v >> np.uint64(32)).astype(np.float64)
    lo = (v & np.uint64(0xFFFFFFFF)).astype(np.float64)
    u1 = (hi + 1.0) / 4294967296.0
    u2 = lo / 4294967296.0
    return (np.sqrt(-2.0 * np.log(u1)) * np.cos(2.0 * np.pi * u2)).astype(np.float32)


def pack_scales_mins(scales: np.ndarray, mins: np.ndarray) -> np.ndarray:
    """``[..., 8]`` six-bit scales and mins -> ``[..., 12]`` packed bytes (K-quant layout)."""
    sc = scales.astype(np.uint8)
    mn = mins.astype(np.uint8)
    out = np.zeros(sc.shape[:-1] + (12,), np.uint8)
    out[..., 0:4] = (sc[..., 0:4] & 0x3F) | ((sc[..., 4:8] >> 4) << 6)
    out[..., 4:8] = (mn[..., 0:4] & 0x3F) | ((mn[..., 4:8] >> 4) << 6)
    out[..., 8:12] = (sc[..., 4:8] & 0x0F) | ((mn[..., 4:8] & 0x0F) << 4)
    return out


def _f16_bytes(values: np.ndarray) -> np.ndarray:
    return values.astype(np.float16).view(np.uint8).reshape(values.shape + (2,))


def q4k_blocks(n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """``[n_blocks, 144]`` random Q4_K super-blocks."""
    s = stream * 8
    out = np.empty((n_blocks, 144), np.uint8)
    out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 0, n_blocks)) * np.float32(1e-3))
    out[:, 2:4] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(5e-4))
    fields = rand_ints(seed, s + 2, n_blocks * 16, 64).reshape(n_blocks, 16)
    out[:, 4:16] = pack_scales_mins(fields[:, :8], fields[:, 8:])
    out[:, 16:144] = rand_bytes(seed, s + 3, n_blocks * 128).reshape(n_blocks, 128)
    return out


def q5k_blocks(n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """``[n_blocks, 176]`` random Q5_K super-blocks: the Q4_K fields plus 32 bytes of fifth bits."""
    s = stream * 8
    out = np.empty((n_blocks, 176), np.uint8)
    out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 0, n_blocks)) * np.float32(1e-3))
    out[:, 2:4] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(5e-4))
    fields = rand_ints(seed, s + 2, n_blocks * 16, 64).reshape(n_blocks, 16)
    out[:, 4:16] = pack_scales_mins(fields[:, :8], fields[:, 8:])
    out[:, 16:48] = rand_bytes(seed, s + 4, n_blocks * 32).reshape(n_blocks, 32)
    out[:, 48:176] = rand_bytes(seed, s + 3, n_blocks * 128).reshape(n_blocks, 128)
    return out


def q6k_blocks(n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """``[n_blocks, 210]`` random Q6_K super-blocks."""
    s = stream * 8
    out = np.empty((n_blocks, 210), np.uint8)
    out[:, 0:192] = rand_bytes(seed, s + 0, n_blocks * 192).reshape(n_blocks, 192)
    sc = (rand_ints(seed, s + 1, n_blocks * 16, 128) - 64).astype(np.int8)
    out[:, 192:208] = sc.view(np.uint8).reshape(n_blocks, 16)
    out[:, 208:210] = _f16_bytes(np.abs(normal(seed, s + 2, n_blocks)) * np.float32(1e-3))
    return out


def q80_blocks(n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """``[n_blocks, 34]`` random Q8_0 blocks."""
    s = stream * 8
    out = np.empty((n_blocks, 34), np.uint8)
    out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 0, n_blocks)) * np.float32(1e-3))
    q = (rand_ints(seed, s + 1, n_blocks * 32, 255) - 127).astype(np.int8)
    out[:, 2:34] = q.view(np.uint8).reshape(n_blocks, 32)
    return out


def lowbit_blocks(dtype: int, n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """Random Q2_K (84 bytes: scales, codes, d, dmin) or Q3_K (110 bytes: high bits, codes, scales, d) blocks."""
    s = stream * 8
    nbytes = BLOCK_BYTES[dtype]
    out = rand_bytes(seed, s + 0, n_blocks * nbytes).reshape(n_blocks, nbytes).copy()
    if dtype == GGML_IQ4_XS:   # d leads the block; everything else is codes and scale bits
        out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(2e-5))
        return out
    out[:, nbytes - 2:] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(1e-3))
    if dtype == GGML_Q2_K:
        out[:, 80:82] = _f16_bytes(np.abs(normal(seed, s + 2, n_blocks)) * np.float32(2e-3))   # d; dmin is the tail
    return out


def legacy_blocks(dtype: int, n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """Random blocks of the 32-value nibble formats: f16 d (and m), uniform code bytes and fifth bits."""
    s = stream * 8
    nbytes = BLOCK_BYTES[dtype]
    out = rand_bytes(seed, s + 0, n_blocks * nbytes).reshape(n_blocks, nbytes).copy()
    out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(2e-3))
    if dtype in (GGML_Q4_1, GGML_Q5_1):
        out[:, 2:4] = _f16_bytes(normal(seed, s + 2, n_blocks) * np.float32(1e-2))
    if dtype == GGML_IQ4_NL:
        out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(2e-4))
    if dtype == GGML_MXFP4:   # the scale is one E8M0 byte: 0.5 * 2^(e - 127), here 2^-12 .. 2^-5
        out[:, 1:2] = out[:, 2:3]   # (byte 1 is a code byte again)
        out[:, 0] = 116 + rand_ints(seed, s + 3, n_blocks, 8)
    return out


def codebook_blocks(dtype: int, n_blocks: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """Random blocks of the codebook formats (IQ2_XXS, IQ3_XXS, IQ3_S, IQ2_S, Q2_0): an f16 d sized so that
    the weights come out around 1e-2, every other byte uniform (each is a code, a sign pattern or scale bits)."""
    s = stream * 8
    nbytes = BLOCK_BYTES[dtype]
    out = rand_bytes(seed, s + 0, n_blocks * nbytes).reshape(n_blocks, nbytes).copy()
    scale = {GGML_IQ2_XXS: 1e-4, GGML_IQ2_S: 1e-4, GGML_IQ3_XXS: 5e-5, GGML_IQ3_S: 5e-5, GGML_Q2_0: 1e-2}[dtype]
    out[:, 0:2] = _f16_bytes(np.abs(normal(seed, s + 1, n_blocks)) * np.float32(scale))
    return out


_MAKERS = {**{t: (lambda n, seed=0, stream=0, t=t: codebook_blocks(t, n, seed, stream))
              for t in (GGML_IQ2_XXS, GGML_IQ3_XXS, GGML_IQ3_S, GGML_IQ2_S, GGML_Q2_0)},
           GGML_IQ4_XS: lambda n, seed=0, stream=0: lowbit_blocks(GGML_IQ4_XS, n, seed, stream),
           GGML_Q2_K: lambda n, seed=0, stream=0: lowbit_blocks(GGML_Q2_K, n, seed, stream),
           GGML_Q3_K: lambda n, seed=0, stream=0: lowbit_blocks(GGML_Q3_K, n, seed, stream),
           GGML_IQ4_NL: lambda n, seed=0, stream=0: legacy_blocks(GGML_IQ4_NL, n, seed, stream),
           GGML_MXFP4: lambda n, seed=0, stream=0: legacy_blocks(GGML_MXFP4, n, seed, stream),
           GGML_Q4_0: lambda n, seed=0, stream=0: legacy_blocks(GGML_Q4_0, n, seed, stream),
           GGML_Q4_1: lambda n, seed=0, stream=0: legacy_blocks(GGML_Q4_1, n, seed, stream),
           GGML_Q5_0: lambda n, seed=0, stream=0: legacy_blocks(GGML_Q5_0, n, seed, stream),
           GGML_Q5_1: lambda n, seed=0, stream=0: legacy_blocks(GGML_Q5_1, n, seed, stream),
           GGML_Q4_K: q4k_blocks, GGML_Q5_K: q5k_blocks, GGML_Q6_K: q6k_blocks, GGML_Q8_0: q80_blocks}


def weight(dtype: int, n: int, k: int, seed: int = 0, stream: int = 0) -> np.ndarray:
    """Row-major ``[n, k / block_len, block_bytes]`` weight blob of ``dtype``."""
    nb = k // BLOCK_LEN[dtype]
    assert nb * BLOCK_LEN[dtype] == k, "k must be whole blocks"
    return _MAKERS[dtype](n * nb, seed, stream).reshape(n, nb, BLOCK_BYTES[dtype])


def activation(rows: int, k: int, seed: int = 0, stream: int = 1000) -> np.ndarray:
    """``[rows, k]`` f32 drawn from N(0, 1)."""
    return normal(seed, stream, rows * k).reshape(rows, k)


def weight_bytes(dtype: int, n: int, k: int) -> int:
    """Algorithmic weight bytes of one matmul: n * (k / block_len) * block_bytes."""
    return n * (k // BLOCK_LEN[dtype]) * BLOCK_BYTES[dtype]
