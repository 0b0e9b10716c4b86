"""Shared test plumbing: numpy bit patterns <-> torch device tensors, error metrics."""
import numpy as np


def to_dev_bf16(bits, torch):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.bfloat16).cuda()


def to_dev_f16(bits, torch):
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).view(torch.float16).cuda()


def to_dev_i32(a, torch):
    return torch.from_numpy(np.ascontiguousarray(a, np.int32)).cuda()


def bf16_bits(t, torch):
    """torch bf16 tensor (any device) -> numpy uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def bf16_to_f64(bits):
    return (np.ascontiguousarray(bits, np.uint16).astype(np.uint32) << np.uint32(16)) \
        .view(np.float32).astype(np.float64)


def rel_l2(a, b):
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    den = np.sqrt((b * b).sum())
    return float(np.sqrt(((a - b) ** 2).sum()) / den) if den > 0 else float(np.abs(a - b).max())


def bf16_ulp_of(v):
    """Spacing of bf16 numbers at magnitude v (v > 0)."""
    e = np.floor(np.log2(v))
    return float(2.0 ** (e - 7))
