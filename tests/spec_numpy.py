"""Independent numpy restatement of the packed layout and of w = (q - z) * s.

Written from the layout definition alone (not from oracle/kx_oracle.c), so that the C oracle
and this file can check each other:
  word (r, j) of a packed tensor holds, in nibble i (bits 4i..4i+3), the code of column
  8*j + ORDER[i] with ORDER = (0, 2, 4, 6, 1, 3, 5, 7).
"""
import numpy as np

ORDER = (0, 2, 4, 6, 1, 3, 5, 7)


def unpack(words):
    """int32 [R, C/8] -> uint8 [R, C]."""
    w = np.ascontiguousarray(words).view(np.uint32)
    R, J = w.shape
    out = np.zeros((R, J * 8), np.uint8)
    for i, col in enumerate(ORDER):
        out[:, col::8] = ((w >> np.uint32(4 * i)) & np.uint32(0xF)).astype(np.uint8)
    return out


def pack(codes):
    """uint8 [R, C] -> int32 [R, C/8]."""
    c = np.ascontiguousarray(codes, np.uint8)
    R, C = c.shape
    w = np.zeros((R, C // 8), np.uint32)
    for i, col in enumerate(ORDER):
        w |= c[:, col::8].astype(np.uint32) << np.uint32(4 * i)
    return w.view(np.int32)


def f16_bits_to_f64(bits):
    return np.ascontiguousarray(bits, np.uint16).view(np.float16).astype(np.float64)


def bf16_bits_to_f64(bits):
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << np.uint32(16)) \
        .view(np.float32).astype(np.float64)


def dequant_f64(qweight, scales_bits, qzeros, group):
    """Exact (unrounded) dequantised weights as float64 [K, N]."""
    q = unpack(qweight).astype(np.float64)
    z = np.repeat(unpack(qzeros).astype(np.float64), group, axis=0)
    s = np.repeat(f16_bits_to_f64(scales_bits), group, axis=0)
    return (q - z) * s


def gemv_awq_f64(x_bits, qweight, scales_bits, qzeros, group):
    return bf16_bits_to_f64(x_bits) @ dequant_f64(qweight, scales_bits, qzeros, group)
