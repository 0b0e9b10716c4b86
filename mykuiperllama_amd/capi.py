"""ctypes binding of the C ABI in include/kx_hip.h.

Device memory comes from torch tensors (plumbing only): the binding passes `tensor.data_ptr()`
and torch's current HIP stream.  There is no fallback: if libkx_hip.so is missing, loading
raises, and every entry point turns a non-zero return code into an exception.
"""
import ctypes
import os

from .build import KX_LIB

_P = ctypes.c_void_p
_I32 = ctypes.c_int32
_I64 = ctypes.c_int64
_SZ = ctypes.c_size_t

ABI_VERSION = 3  # KX_ABI_VERSION of the include/kx_hip.h this file mirrors

# name -> (restype, argtypes); mirrors include/kx_hip.h declaration by declaration
SIGNATURES = {
    "kx_abi_version": (ctypes.c_int, []),
    "kx_error_string": (ctypes.c_char_p, [ctypes.c_int]),
    "kx_gemv_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "kx_workspace_init": (ctypes.c_int, [_P, _SZ, _P]),
    "kx_gemv_awq_bf16": (ctypes.c_int, [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _P, _SZ, _P]),
    "kx_gemv_awq_static_scratch_bytes": (_SZ, []),
    "kx_gemv_awq_bf16_static": (ctypes.c_int, [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _P]),
    "kx_gemv_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _I32, _I32, _P, _SZ, _P]),
    "kx_gemv_awq_swiglu_bf16": (ctypes.c_int, [_P, _P, _I32, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _P, _SZ, _P]),
    "kx_gemv_awq_addnorm_bf16": (ctypes.c_int, [_P, _P, _P, ctypes.c_float, _P, _P, _P, _P, _P, _I32, _I32,
                                                _I32, _I32, _P, _SZ, _P]),
    "kx_gemv_awq_qkv_rope_bf16": (ctypes.c_int, [_P, _P, _P, ctypes.c_float, _P, _P, _P, _P, _P, _P, _P, _P, _P,
                                                 _I32, _I32, _I32, _P, _I32, ctypes.c_float, ctypes.c_float, _I32,
                                                 _I32, _P, _SZ, _P]),
    "kx_gemv_awq_chain_bf16": (ctypes.c_int, [_P, _P, _P, _P, _I32, _I32, _I32, _P, _SZ, _P]),
    "kx_awq_unpack_u8": (ctypes.c_int, [_P, _P, _I64, _I64, _P]),
    "kx_rmsnorm_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _I32, ctypes.c_float, _P]),
    "kx_add_rmsnorm_bf16": (ctypes.c_int, [_P, _P, _P, _P, _I32, _I32, ctypes.c_float, _P]),
    "kx_qk_norm_rope_bf16": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _I32, _I32, _I32, _P, _I32, ctypes.c_float,
                                            ctypes.c_float, _P]),
    "kx_attn_decode_workspace_bytes": (_SZ, [_I32, _I32, _I32]),
    "kx_attn_decode_bf16": (ctypes.c_int, [_P, _P, _P, _P, _I32, _I32, _I32, _P, _I32, _P, _SZ, _P]),
    "kx_attn_decode_partial_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _I32, _I32, _P, _I32, _P, _SZ, _P]),
    "kx_gemv_awq_attn_merge_bf16": (ctypes.c_int, [_P, _SZ, _I32, _I32, _I32, _I32, _P, _P, _P, _P, _I32, _I32, _P,
                                                   _SZ, _P]),
    "kx_swiglu_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _P]),
    "kx_add_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _P]),
    "kx_embedding_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _I32, _P]),
    "kx_argmax_bf16": (ctypes.c_int, [_P, _I32, _P, _P]),
    "kx_qk_norm_rope_batch_bf16": (ctypes.c_int, [_P, _P, _P, _P, _P, _P, _SZ, _I32, _I32, _I32, _P, _I32,
                                                  ctypes.c_float, ctypes.c_float, _I32, _P]),
    "kx_attn_decode_batch_bf16": (ctypes.c_int, [_P, _P, _P, _SZ, _P, _I32, _I32, _I32, _P, _I32, _P, _SZ, _I32, _P]),
    "kx_embedding_rows_bf16": (ctypes.c_int, [_P, _P, _P, _I32, _I32, _I32, _P]),
    "kx_argmax_rows_bf16": (ctypes.c_int, [_P, _I32, _I32, _P, _I32, _P]),
    "kx_awq_dequant_bf16": (ctypes.c_int, [_P, _P, _P, _P, _I32, _I32, _I32, _P]),
}


# entry points outside the drop-in boundary (csrc/kx_internal.h): tests and the benchmark only
INTERNAL_SIGNATURES = {
    "kx_gemv_awq_bf16_policy": (ctypes.c_int, [_P, _P, _P, _P, _P, _I32, _I32, _I32, _I32, _P, _SZ, _P, _I32]),
}


class ChainDesc(ctypes.Structure):
    """Mirror of kx_chain_desc (include/kx_hip.h), field for field."""
    _fields_ = [
        ("in_kind", _I32), ("out_kind", _I32),
        ("x", _P),
        ("gate", _P), ("up", _P),
        ("attn_workspace", _P), ("attn_workspace_bytes", _SZ),
        ("n_q_heads", _I32), ("n_kv_heads", _I32), ("max_positions", _I32),
        ("norm_parts", _I32), ("norm_row", _P), ("norm_sumsq", _P), ("norm_gain", _P), ("norm_eps", ctypes.c_float),
        ("rope_theta", ctypes.c_float), ("qk_eps", ctypes.c_float),
        ("rope_n_q_heads", _I32), ("rope_n_kv_heads", _I32), ("cache_positions", _I32),
        ("y", _P),
        ("residual_in", _P), ("residual_out", _P), ("sumsq_out", _P),
        ("q_gain", _P), ("k_gain", _P), ("q_out", _P), ("k_cache", _P), ("v_cache", _P), ("pos", _P),
        ("rows", _I32), ("act_ld", _I32), ("cache_stride", _SZ),
    ]


IN_ROW, IN_SWIGLU, IN_ATTN, IN_NORM = 0, 1, 2, 3
OUT_ROW, OUT_RESIDUAL, OUT_QKV_ROPE = 0, 1, 2


class KxError(RuntimeError):
    def __init__(self, code, text):
        super().__init__(f"kx call failed with code {code}: {text}")
        self.code = code


_lib = None


def load(path=None):
    """Load libkx_hip.so; raises if it has not been built.  `path` names another build of the library (the
    benchmark's --lib, for profiling builds); it only has an effect on the first call."""
    global _lib
    if _lib is not None:
        return _lib
    lib_path = path or KX_LIB
    # torch ships its own HIP runtime; it has to be in the process first so that this library
    # binds to the same copy (two runtimes in one process do not share a device context).
    import torch  # noqa: F401
    if not os.path.exists(lib_path):
        raise RuntimeError(
            f"{lib_path} is missing: the HIP library has not been built "
            "(python -m mykuiperllama_amd.build). There is no CPU fallback for this path.")
    lib = ctypes.CDLL(lib_path)
    for name, (res, args) in list(SIGNATURES.items()) + list(INTERNAL_SIGNATURES.items()):
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    built_as = lib.kx_abi_version()
    if built_as != ABI_VERSION:
        raise RuntimeError(f"{lib_path} was built as ABI version {built_as}, this binding mirrors version "
                           f"{ABI_VERSION} of include/kx_hip.h (ChainDesc would not match kx_chain_desc)")
    _lib = lib
    return lib


_probe = None


def _load_probe():
    global _probe
    if _probe is None:
        import torch  # noqa: F401
        from .build import PROBE_LIB
        if not os.path.exists(PROBE_LIB):
            raise RuntimeError(f"{PROBE_LIB} is missing (python -m mykuiperllama_amd.build)")
        _probe = ctypes.CDLL(PROBE_LIB)
        _probe.kx_probe_stream_read.restype = ctypes.c_int
        _probe.kx_probe_stream_read.argtypes = [_P, _SZ, _P, _SZ, _P, _SZ, _P, _P]
        _probe.kx_probe_empty_launch.restype = ctypes.c_int
        _probe.kx_probe_empty_launch.argtypes = [_I32, _P, _P]
    return _probe


def probe_empty_launch(blocks):
    """Measurement only: a launch of `blocks` workgroups of 512 threads that do nothing (libkx_probe.so)."""
    rc = _load_probe().kx_probe_empty_launch(blocks, None, _stream())
    if rc != 0:
        raise RuntimeError(f"kx_probe_empty_launch failed with HIP error {rc}")


def probe_stream_read(buffers, sink=None):
    """Measurement only: read up to three device tensors once with plain 16-byte loads (libkx_probe.so)."""
    _load_probe()
    args = []
    for i in range(3):
        t = buffers[i] if i < len(buffers) else None
        args += [_ptr(t), 0 if t is None else t.numel() * t.element_size()]
    rc = _probe.kx_probe_stream_read(*args, _ptr(sink), _stream())
    if rc != 0:
        raise RuntimeError(f"kx_probe_stream_read failed with HIP error {rc}")


def _check(code):
    if code != 0:
        raise KxError(code, load().kx_error_string(code).decode())


def _stream():
    import torch
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return None if t is None else t.data_ptr()


def workspace_bytes(M, K, N):
    return int(load().kx_gemv_workspace_bytes(M, K, N))


def make_workspace(M, K, N, device="cuda"):
    """Allocate and initialise a workspace large enough for a GEMV of this shape."""
    import torch
    nbytes = workspace_bytes(M, K, N)  # the zeroed area of every workspace plus the shape's partial sums
    if nbytes == 0:
        raise ValueError(f"no GEMV takes M={M}, K={K}, N={N}")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=device)
    _check(load().kx_workspace_init(ws.data_ptr(), nbytes, _stream()))
    return ws


def gemv_awq_bf16(x, qweight, scales, qzeros, y, group_size, workspace):
    """x bf16 [M,K], qweight int32 [K,N/8], scales fp16 [K/G,N], qzeros int32 [K/G,N/8], y bf16 [M,N]."""
    M, K = x.shape
    N = y.shape[-1]
    if _policy != 0:
        _check(load().kx_gemv_awq_bf16_policy(_ptr(x), _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(y),
                                              M, K, N, group_size, _ptr(workspace),
                                              0 if workspace is None else workspace.numel(), _stream(), _policy))
        return
    _check(load().kx_gemv_awq_bf16(_ptr(x), _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(y),
                                   M, K, N, group_size, _ptr(workspace),
                                   0 if workspace is None else workspace.numel(), _stream()))


def gemv_awq_bf16_static(x, qweight, scales, qzeros, y, group_size):
    """gemv_awq_bf16 on the library's static scratch array: no workspace, no allocation."""
    M, K = x.shape
    N = y.shape[-1]
    _check(load().kx_gemv_awq_bf16_static(_ptr(x), _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(y),
                                          M, K, N, group_size, _stream()))


def gemv_awq_swiglu_bf16(gate, up, qweight, scales, qzeros, y, group_size, workspace):
    """y = (bf16(bf16(silu(gate)) * up)) W; gate and up are bf16 [M,K] views that share a row stride."""
    M, K = gate.shape
    N = y.shape[-1]
    if gate.stride(0) != up.stride(0) or gate.stride(1) != 1 or up.stride(1) != 1:
        raise ValueError("gate and up must be row views with one common row stride")
    _check(load().kx_gemv_awq_swiglu_bf16(_ptr(gate), _ptr(up), gate.stride(0), _ptr(qweight), _ptr(scales),
                                          _ptr(qzeros), _ptr(y), M, K, N, group_size, _ptr(workspace),
                                          0 if workspace is None else workspace.numel(), _stream()))


def gemv_awq_addnorm_bf16(residual, delta, gain, eps, residual_out, qweight, scales, qzeros, y, group_size,
                          workspace):
    """r = bf16(residual + delta) (delta may be None), y = (gain * bf16(r * rsqrt(mean r^2 + eps))) W;
    r goes to residual_out (may be None, must not be residual or delta)."""
    M, K = residual.shape
    N = y.shape[-1]
    _check(load().kx_gemv_awq_addnorm_bf16(_ptr(residual), _ptr(delta), _ptr(gain), eps, _ptr(residual_out),
                                           _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(y), M, K, N,
                                           group_size, _ptr(workspace),
                                           0 if workspace is None else workspace.numel(), _stream()))


def gemv_awq_qkv_rope_bf16(residual, delta, gain, eps, residual_out, qweight, scales, qzeros, q_gain, k_gain,
                           q_out, k_cache, v_cache, n_q, n_kv, pos, rope_theta, qk_eps, group_size, workspace):
    """add + RMSNorm, fused q|k|v projection, per-head norm + rotation + cache append; one row.
    k_cache / v_cache: bf16 [positions, n_kv, 128]; the first dimension is the capacity the kernel guards."""
    K = residual.shape[-1]
    _check(load().kx_gemv_awq_qkv_rope_bf16(_ptr(residual), _ptr(delta), _ptr(gain), eps, _ptr(residual_out),
                                            _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(q_gain), _ptr(k_gain),
                                            _ptr(q_out), _ptr(k_cache), _ptr(v_cache), n_q, n_kv, 128, _ptr(pos),
                                            _cache_positions(k_cache, v_cache), rope_theta, qk_eps, K, group_size,
                                            _ptr(workspace),
                                            0 if workspace is None else workspace.numel(), _stream()))


_policy = 0


def set_awq_kernel_policy(policy):
    """Test and benchmark plumbing: which kernel gemv_awq_bf16 of THIS module asks for from now on.
    0 = the product entry point (the library chooses by shape); 1 = vector-ALU kernel, 2 = one-shot MFMA
    kernel, each through the internal entry point kx_gemv_awq_bf16_policy.
    The library itself keeps no such state."""
    global _policy
    if policy not in (0, 1, 2):
        raise ValueError("policy must be 0, 1 or 2")
    _policy = policy


def gemv_bf16(x, w, y, workspace=None):
    """x bf16 [M,K], w bf16 [N,K], y bf16 [M,N]."""
    M, K = x.shape
    N = w.shape[0]
    _check(load().kx_gemv_bf16(_ptr(x), _ptr(w), _ptr(y), M, K, N, _ptr(workspace),
                               0 if workspace is None else workspace.numel(), _stream()))


def awq_unpack_u8(words, codes):
    rows, wcols = words.shape
    _check(load().kx_awq_unpack_u8(_ptr(words), _ptr(codes), rows, wcols * 8, _stream()))


def awq_dequant_bf16(qweight, scales, qzeros, w, group_size):
    K, wcols = qweight.shape
    _check(load().kx_awq_dequant_bf16(_ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(w), K,
                                      wcols * 8, group_size, _stream()))


# ---------------------------------------------------------------- decode-step operators
def rmsnorm_bf16(x, gain, y, eps):
    rows = x.numel() // x.shape[-1]
    _check(load().kx_rmsnorm_bf16(_ptr(x), _ptr(gain), _ptr(y), rows, x.shape[-1], eps, _stream()))


def add_rmsnorm_bf16(x_inout, delta, gain, y, eps):
    rows = x_inout.numel() // x_inout.shape[-1]
    _check(load().kx_add_rmsnorm_bf16(_ptr(x_inout), _ptr(delta), _ptr(gain), _ptr(y), rows, x_inout.shape[-1],
                                      eps, _stream()))


def _cache_positions(k_cache, v_cache):
    """Rows of a KV cache pair laid out [positions, n_kv, 128] (the capacity the append is guarded by)."""
    if k_cache is None or v_cache is None:
        return 1  # the call fails on the null pointer
    return min(k_cache.shape[0], v_cache.shape[0])


def qk_norm_rope_bf16(qkv, q_gain, k_gain, q_out, k_cache, v_cache, n_q, n_kv, pos, theta, eps):
    _check(load().kx_qk_norm_rope_bf16(_ptr(qkv), _ptr(q_gain), _ptr(k_gain), _ptr(q_out), _ptr(k_cache),
                                       _ptr(v_cache), n_q, n_kv, 128, _ptr(pos), _cache_positions(k_cache, v_cache),
                                       theta, eps, _stream()))


def attn_decode_workspace(n_q, max_positions, device="cuda"):
    import torch
    nbytes = int(load().kx_attn_decode_workspace_bytes(n_q, 128, max_positions))
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def attn_decode_bf16(q, k_cache, v_cache, out, n_q, n_kv, pos, max_positions, workspace):
    _check(load().kx_attn_decode_bf16(_ptr(q), _ptr(k_cache), _ptr(v_cache), _ptr(out), n_q, n_kv, 128, _ptr(pos),
                                      max_positions, _ptr(workspace), workspace.numel(), _stream()))


def attn_decode_partial_bf16(q, k_cache, v_cache, n_q, n_kv, pos, max_positions, workspace):
    """First attention stage only; the per-chunk results stay in `workspace`."""
    _check(load().kx_attn_decode_partial_bf16(_ptr(q), _ptr(k_cache), _ptr(v_cache), n_q, n_kv, 128, _ptr(pos),
                                              max_positions, _ptr(workspace), workspace.numel(), _stream()))


def gemv_awq_attn_merge_bf16(attn_workspace, n_q, n_kv, max_positions, qweight, scales, qzeros, y, group_size,
                             workspace):
    """y = (attention output merged from `attn_workspace`) W, one row."""
    _check(load().kx_gemv_awq_attn_merge_bf16(_ptr(attn_workspace), attn_workspace.numel(), n_q, n_kv, 128,
                                              max_positions, _ptr(qweight), _ptr(scales), _ptr(qzeros), _ptr(y),
                                              y.shape[-1], group_size, _ptr(workspace),
                                              0 if workspace is None else workspace.numel(), _stream()))


def gemv_awq_chain_bf16(desc, qweight, scales, qzeros, K, N, group_size, workspace):
    """One link of a decoder layer's chain: see kx_chain_desc.  `desc` maps field names to tensors,
    None or scalars; tensors are passed by address."""
    d = ChainDesc()
    if "cache_positions" not in desc and desc.get("k_cache") is not None and desc.get("v_cache") is not None:
        d.cache_positions = _cache_positions(desc["k_cache"], desc["v_cache"])
    for name, value in desc.items():
        setattr(d, name, value.data_ptr() if hasattr(value, "data_ptr") else value)
    _check(load().kx_gemv_awq_chain_bf16(ctypes.byref(d), _ptr(qweight), _ptr(scales), _ptr(qzeros), K, N, group_size,
                                         _ptr(workspace), 0 if workspace is None else workspace.numel(), _stream()))


FUSED_MERGE_MAX_POSITIONS = 80 * 128  # the o projection merges at most 80 chunks (of 128 positions past 5120)


def swiglu_bf16(gate, up, out):
    _check(load().kx_swiglu_bf16(_ptr(gate), _ptr(up), _ptr(out), out.numel(), _stream()))


def add_bf16(a, b, out):
    _check(load().kx_add_bf16(_ptr(a), _ptr(b), _ptr(out), out.numel(), _stream()))


def embedding_bf16(table, token, out):
    _check(load().kx_embedding_bf16(_ptr(table), _ptr(token), _ptr(out), table.shape[0], table.shape[1], _stream()))


def qk_norm_rope_batch_bf16(qkv, q_gain, k_gain, q_out, k_cache, v_cache, n_q, n_kv, pos, theta, eps):
    """Batched form: qkv [B, (n_q + 2 n_kv) * 128], caches [B, positions, n_kv, 128] (any stride between
    sequences), pos int32 [B]."""
    B = qkv.shape[0]
    if k_cache.stride(0) != v_cache.stride(0):
        raise ValueError("the K and V caches must share the stride between sequences")
    _check(load().kx_qk_norm_rope_batch_bf16(_ptr(qkv), _ptr(q_gain), _ptr(k_gain), _ptr(q_out), _ptr(k_cache),
                                             _ptr(v_cache), k_cache.stride(0), n_q, n_kv, 128, _ptr(pos),
                                             min(k_cache.shape[1], v_cache.shape[1]), theta, eps, B, _stream()))


def attn_decode_batch_workspace(batch, n_q, max_positions, device="cuda"):
    import torch
    nbytes = int(load().kx_attn_decode_workspace_bytes(n_q, 128, max_positions))
    return torch.empty(batch * nbytes, dtype=torch.uint8, device=device)


def attn_decode_batch_bf16(q, k_cache, v_cache, out, n_q, n_kv, pos, max_positions, workspace):
    B = q.shape[0]
    if k_cache.stride(0) != v_cache.stride(0):
        raise ValueError("the K and V caches must share the stride between sequences")
    _check(load().kx_attn_decode_batch_bf16(_ptr(q), _ptr(k_cache), _ptr(v_cache), k_cache.stride(0), _ptr(out), n_q,
                                            n_kv, 128, _ptr(pos), max_positions, _ptr(workspace),
                                            workspace.numel(), B, _stream()))


def embedding_rows_bf16(table, tokens, out):
    _check(load().kx_embedding_rows_bf16(_ptr(table), _ptr(tokens), _ptr(out), table.shape[0], table.shape[1],
                                         tokens.numel(), _stream()))


def argmax_rows_bf16(x, out_index):
    rows, n = x.shape
    _check(load().kx_argmax_rows_bf16(_ptr(x), n, x.stride(0), _ptr(out_index), rows, _stream()))


def argmax_bf16(x, out_index):
    _check(load().kx_argmax_bf16(_ptr(x), x.numel(), _ptr(out_index), _stream()))
