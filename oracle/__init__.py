"""ctypes front end of the CPU oracle (oracle/maxfp8_oracle.c).

TEST INFRASTRUCTURE ONLY.  Importable from tests/, ``__graft_entry__.smoke()``
and the ``cpu_baseline`` leg of ``bench.py``; the product package never imports
it.  Arrays are numpy: bf16 travels as ``uint16`` bit patterns, e4m3fn as
``uint8`` bytes.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libmaxfp8_oracle.so")

BF16, F16, F32 = 0, 1, 2

_lib = None


def build(force: bool = False) -> str:
    """Compile the oracle with gcc (seconds).  Returns the path of the .so."""
    src = os.path.join(_HERE, "maxfp8_oracle.c")
    if force or not os.path.exists(_SO) or os.path.getmtime(_SO) < os.path.getmtime(src):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libmaxfp8_oracle.so"],
                              stdout=subprocess.DEVNULL)
    return _SO


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        build()
        L = ctypes.CDLL(_SO)
        L.orc_e4m3fn_to_f32.restype = ctypes.c_float
        L.orc_e4m3fn_to_f32.argtypes = [ctypes.c_uint8]
        L.orc_f32_to_e4m3fn.restype = ctypes.c_uint8
        L.orc_f32_to_e4m3fn.argtypes = [ctypes.c_float]
        L.orc_f32_to_e4m3fn_array.restype = None
        L.orc_f32_to_e4m3fn_array.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64]
        L.orc_dynamic_scale.restype = None
        L.orc_dynamic_scale.argtypes = [ctypes.c_float, ctypes.c_float, ctypes.c_int,
                                        ctypes.POINTER(ctypes.c_float),
                                        ctypes.POINTER(ctypes.c_float)]
        i64, vp, ci, cf = ctypes.c_int64, ctypes.c_void_p, ctypes.c_int, ctypes.c_float
        L.orc_quantize_dynamic_scaled_fp8.restype = ci
        L.orc_quantize_dynamic_scaled_fp8.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64,
                                                      i64, ci, ci, cf, ci]
        L.orc_matmul_blockwise.restype = ci
        L.orc_matmul_blockwise.argtypes = [vp, vp, vp, vp, vp] + [i64] * 11 + [ci, ci, ci]
        L.orc_matmul_rowwise.restype = ci
        L.orc_matmul_rowwise.argtypes = [vp, vp, vp, vp, vp] + [i64] * 8 + [ci, ci, ci]
        L.orc_grouped_matmul.restype = ci
        L.orc_grouped_matmul.argtypes = [vp] * 7 + [i64] * 7 + [ci, ci, ci]
        L.orc_rms_norm_fused_quantize.restype = ci
        L.orc_rms_norm_fused_quantize.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, ci, ci, cf, cf, cf, ci]
        L.orc_quantize_static.restype = ci
        L.orc_quantize_static.argtypes = [vp, vp, i64, i64, ci, cf]
        L.orc_moe_create_indices.restype = ci
        L.orc_moe_create_indices.argtypes = [vp] * 6 + [i64, i64]
        L.orc_fused_silu.restype = ci
        L.orc_fused_silu.argtypes = [vp, vp, vp, i64, i64, i64, i64, i64, ci, ci]
        L.orc_max_threads.restype = ci
        _lib = L
    return _lib


def _p(a: np.ndarray) -> ctypes.c_void_p:
    return ctypes.c_void_p(a.ctypes.data)


def default_threads() -> int:
    try:
        return max(1, len(os.sched_getaffinity(0)))
    except AttributeError:  # pragma: no cover
        return os.cpu_count() or 1


# ---- codec -----------------------------------------------------------------

def e4m3fn_decode_table() -> np.ndarray:
    L = lib()
    return np.array([L.orc_e4m3fn_to_f32(i) for i in range(256)], dtype=np.float32)


def e4m3fn_decode(b: np.ndarray) -> np.ndarray:
    return e4m3fn_decode_table()[np.asarray(b, dtype=np.uint8)]


def e4m3fn_encode(x: np.ndarray) -> np.ndarray:
    """Encode f32 values (round to nearest even, saturating, NaN -> 0x7f)."""
    x = np.ascontiguousarray(x, dtype=np.float32)
    out = np.empty(x.shape, dtype=np.uint8)
    lib().orc_f32_to_e4m3fn_array(_p(out), _p(x), x.size)
    return out


def dynamic_scale(amax: float, scale_ub: float = 1200.0, scales_dtype: int = F32):
    s, r = ctypes.c_float(), ctypes.c_float()
    lib().orc_dynamic_scale(amax, scale_ub, scales_dtype, ctypes.byref(s), ctypes.byref(r))
    return np.float32(s.value), np.float32(r.value)


# ---- operators ---------------------------------------------------------------

def quantize_dynamic_scaled_fp8(x: np.ndarray, group_size: int, *, in_dtype: int = BF16,
                                scales_dtype: int = F32, scale_ub: float = 1200.0,
                                scales_ld: int | None = None, threads: int = 1):
    """x: [M, K] (uint16 bits for bf16/f16, float32 for f32).  Returns
    (q uint8 [M, K], scales [K/G, scales_ld]); unwritten scale columns hold NaN
    bit patterns (f32) / 0xFFFF (bf16) so a test can see they stay untouched."""
    if scales_dtype not in (F32, BF16):
        raise ValueError("the oracle's quantisers write f32 or bf16 scales")
    x = np.ascontiguousarray(x)
    M, K = x.shape
    G = K if group_size == -1 else group_size
    ld = M if scales_ld is None else scales_ld
    q = np.zeros((M, K), dtype=np.uint8)
    if scales_dtype == F32:
        sc = np.full((K // G, ld), np.nan, dtype=np.float32)
    else:
        sc = np.full((K // G, ld), 0xFFFF, dtype=np.uint16)
    rc = lib().orc_quantize_dynamic_scaled_fp8(_p(q), _p(sc), _p(x), M, K, K, K, G, ld,
                                               in_dtype, scales_dtype, scale_ub, threads)
    if rc:
        raise ValueError(f"oracle quantize failed: {rc}")
    return q, sc


def round_to_dtype(v: float, dtype: int) -> float:
    """v rounded to bf16 / f16 / f32 and widened back (how an op parameter of the input's dtype arrives)."""
    if dtype == BF16:
        import torch
        return float(torch.tensor(v, dtype=torch.float32).to(torch.bfloat16).float())
    if dtype == F16:
        return float(np.float32(np.float16(v)))
    return float(np.float32(v))


def rms_norm_fused_quantize(x: np.ndarray, gamma: np.ndarray, epsilon: float, weight_offset: float = 0.0, *,
                            in_dtype: int = BF16, scales_dtype: int = F32, scale_ub: float = 1200.0,
                            threads: int = 1):
    """x: [rows, K], gamma: [K] (uint16 bits for bf16/f16, float32 for f32).  epsilon and
    weight_offset are rounded to the input dtype first, as the op registration does
    (builtin_kernels/quantization.mojo:205-213).  Returns (q uint8 [rows, K], scales [1, rows])."""
    if scales_dtype not in (F32, BF16):
        raise ValueError("the oracle's quantisers write f32 or bf16 scales")
    x = np.ascontiguousarray(x)
    gamma = np.ascontiguousarray(gamma)
    rows, K = x.shape
    q = np.zeros((rows, K), dtype=np.uint8)
    sc = np.zeros((1, rows), dtype=np.float32 if scales_dtype == F32 else np.uint16)
    rc = lib().orc_rms_norm_fused_quantize(_p(q), _p(sc), _p(x), _p(gamma), rows, K, K, K, in_dtype, scales_dtype,
                                           round_to_dtype(epsilon, in_dtype), round_to_dtype(weight_offset, in_dtype),
                                           scale_ub, threads)
    if rc:
        raise ValueError(f"oracle rms_norm_fused_quantize failed: {rc}")
    return q, sc


def quantize_static(x: np.ndarray, scale: float, *, in_dtype: int = BF16) -> np.ndarray:
    """x: [M, K] (uint16 bits for bf16/f16, float32 for f32) -> e4m3fn bytes of clamp(x * (1 / scale))."""
    x = np.ascontiguousarray(x)
    q = np.zeros(x.shape, dtype=np.uint8)
    lib().orc_quantize_static(_p(q), _p(x), x.shape[0], x.shape[1], in_dtype, scale)
    return q


def quantize_tensor_dynamic(x: np.ndarray, *, in_dtype: int = BF16, scales_dtype: int = F32, scale_ub: float = 1200.0,
                            threads: int = 1):
    """Per-tensor dynamic quantisation (fp8_quantization.mojo:209-360, 596-775): the whole [M, K] tensor is
    one group of quantize_dynamic_scaled_fp8.  Returns (q uint8 [M, K], scales [1, M], all equal)."""
    x = np.ascontiguousarray(x)
    M, K = x.shape
    q, sc = quantize_dynamic_scaled_fp8(x.reshape(1, M * K), M * K, in_dtype=in_dtype, scales_dtype=scales_dtype,
                                        scale_ub=scale_ub, threads=threads)
    return q.reshape(M, K), np.repeat(sc[:1, :1], M, axis=1)


def grouped_matmul_rowwise(a: np.ndarray, b: np.ndarray, a_scales: np.ndarray, b_scales: np.ndarray,
                           offsets: np.ndarray, expert_ids: np.ndarray, num_active: int, *, c_dtype: int = F32,
                           threads: int = 1, fill: float = np.nan) -> np.ndarray:
    """grouped_matmul_rowwise_scaled_fp8_kernel (max/kernels/src/linalg/grouped_matmul.mojo:1440-1541): slot z
    multiplies its rows by expert expert_ids[z] with matmul_rowwise's arithmetic; expert -1 gives zeros; rows
    past the last active slot keep `fill`.  a [T, K], b [E, N, K] bytes; a_scales [T, 1], b_scales [E, N, 1]."""
    T = a.shape[0]
    E, N, _ = b.shape
    c = np.full((T, N), fill, dtype=np.float32) if c_dtype == F32 else np.full((T, N), 0xFFFF, dtype=np.uint16)
    for z in range(num_active):
        lo, hi = int(offsets[z]), int(offsets[z + 1])
        if hi <= lo:
            continue
        e = int(expert_ids[z])
        if e < 0:
            c[lo:hi] = 0
            continue
        c[lo:hi] = matmul_rowwise(a[lo:hi], b[e], np.asarray(a_scales, np.float32).reshape(1, -1)[:, lo:hi],
                                  np.asarray(b_scales, np.float32)[e].reshape(-1, 1), c_dtype=c_dtype, threads=threads)
    return c


def bf16_round(x: np.ndarray) -> np.ndarray:
    """float32 array rounded to bf16 (nearest even; NaN kept) and widened back."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    r = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
    nan = (u & 0x7FFFFFFF) > 0x7F800000
    r = np.where(nan, u | 0x400000, r)
    return (r & 0xFFFFFFFF).astype(np.uint32).view(np.float32).reshape(np.shape(x))


def bf16_bits_of(x: np.ndarray) -> np.ndarray:
    """float32 array whose values are bf16-representable -> uint16 bit patterns."""
    return (np.ascontiguousarray(x, dtype=np.float32).view(np.uint32) >> 16).astype(np.uint16)


def fused_qkv_matmul(a: np.ndarray, w: np.ndarray, input_scale: np.ndarray, weight_scale: np.ndarray, gmnk,
                     row_offsets: np.ndarray, cache_lengths: np.ndarray, lookup_table: np.ndarray,
                     kv_blocks: np.ndarray, layer_idx: int, q_dim: int, *, bias: np.ndarray | None = None,
                     threads: int = 1) -> np.ndarray:
    """The fused QKV matmul of kv_cache_ragged.mojo:1122-1307 (and, with q_dim = 0, the K-cache
    matmul of :3025-3224).  a [T, K], w [N, K] e4m3fn bytes; kv_blocks uint16 (bf16 bits)
    [blocks, kv_dim, layers, page, heads, head_dim], UPDATED IN PLACE; bias uint16 [N] or None.
    Returns the Q part, uint16 [T, q_dim].  Rounding steps as in the reference's epilogue: the matmul
    result arrives as bf16; per tensor (-1,-1,-1) / per channel (1,1,-1) it is multiplied in bf16 by
    the bf16 product of the two bf16-rounded scales; the bias is added in bf16."""
    T, K = a.shape
    N = w.shape[0]
    gmnk = tuple(gmnk)
    if gmnk in ((-1, -1, -1), (1, 1, -1)):
        raw = matmul_rowwise(a, w, np.ones((1, 1), np.float32), np.ones((1, 1), np.float32), tensor_scales=True,
                             threads=threads)
        sa = bf16_round(np.asarray(input_scale, dtype=np.float32).reshape(-1))
        sb = bf16_round(np.asarray(weight_scale, dtype=np.float32).reshape(-1))
        if gmnk[0] == -1:
            sc = np.full((T, N), bf16_round(sa[:1] * sb[:1])[0], dtype=np.float32)
        else:
            sc = bf16_round(sa[:T, None] * sb[None, :N])
        val = bf16_round(bf16_round(raw) * sc)
    else:
        bits = matmul_blockwise(a, w, input_scale, weight_scale, gmnk=gmnk, c_dtype=BF16, threads=threads)
        val = (bits.astype(np.uint32) << 16).view(np.float32)
    if bias is not None:
        val = bf16_round(val + (np.asarray(bias, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)[None, :])
    out_bits = bf16_bits_of(val)
    heads, head_dim = kv_blocks.shape[4], kv_blocks.shape[5]
    page = kv_blocks.shape[3]
    k_dim = heads * head_dim
    has_v = N - q_dim == 2 * k_dim
    assert N - q_dim == k_dim or (has_v and kv_blocks.shape[1] == 2)
    ro = np.asarray(row_offsets, dtype=np.int64)
    for t in range(T):
        b = int(np.searchsorted(ro, t, side="right")) - 1   # the last sequence whose first row is <= t
        tok = t - int(ro[b]) + int(cache_lengths[b])
        blk = int(lookup_table[b, tok // page])
        kv_blocks[blk, 0, layer_idx, tok % page] = out_bits[t, q_dim:q_dim + k_dim].reshape(heads, head_dim)
        if has_v:
            kv_blocks[blk, 1, layer_idx, tok % page] = out_bits[t, q_dim + k_dim:].reshape(heads, head_dim)
    return np.ascontiguousarray(out_bits[:, :q_dim])


def moe_create_indices(topk_ids: np.ndarray, num_experts: int):
    """topk_ids: int32 [n].  Returns (token_expert_order, expert_start_indices, restore_token_order,
    expert_ids, expert_usage_stats) in the canonical order (slot z = expert z, stable)."""
    ids = np.ascontiguousarray(topk_ids, dtype=np.int32)
    n = ids.shape[0]
    order = np.zeros(n, dtype=np.uint32)
    start = np.zeros(num_experts + 1, dtype=np.uint32)
    restore = np.zeros(n, dtype=np.uint32)
    eids = np.zeros(num_experts, dtype=np.int32)
    stats = np.zeros(2, dtype=np.uint32)
    lib().orc_moe_create_indices(_p(order), _p(start), _p(restore), _p(eids), _p(stats), _p(ids), n, num_experts)
    return order, start, restore, eids, stats


def fused_silu(x: np.ndarray, rows: int, *, quantize: bool = False, scales_ld: int | None = None, threads: int = 1):
    """x: bf16 bits [max_rows, 2*I].  Rows >= `rows` are left at zero (scales at NaN).  Returns the bf16
    bits [max_rows, I], or (e4m3fn bytes [max_rows, I], f32 scales [I/128, scales_ld]) when quantize."""
    x = np.ascontiguousarray(x, dtype=np.uint16)
    max_rows, two_i = x.shape
    inter = two_i // 2
    if not quantize:
        out = np.zeros((max_rows, inter), dtype=np.uint16)
        lib().orc_fused_silu(_p(out), None, _p(x), rows, inter, two_i, inter, 0, 0, threads)
        return out
    ld = max_rows if scales_ld is None else scales_ld
    out = np.zeros((max_rows, inter), dtype=np.uint8)
    sc = np.full((inter // 128, ld), np.nan, dtype=np.float32)
    lib().orc_fused_silu(_p(out), _p(sc), _p(x), rows, inter, two_i, inter, ld, 1, threads)
    return out, sc


def matmul_blockwise(a: np.ndarray, b: np.ndarray, a_scales: np.ndarray, b_scales: np.ndarray,
                     *, gmnk=(1, 128, 128), c_dtype: int = F32, mode: int = 0,
                     threads: int = 1) -> np.ndarray:
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    a_scales = np.ascontiguousarray(a_scales, dtype=np.float32)
    b_scales = np.ascontiguousarray(b_scales, dtype=np.float32)
    M, K = a.shape
    N = b.shape[0]
    c = np.zeros((M, N), dtype=np.float32 if c_dtype == F32 else np.uint16)
    rc = lib().orc_matmul_blockwise(_p(c), _p(a), _p(b), _p(a_scales), _p(b_scales),
                                    M, N, K, K, K, N, gmnk[0], gmnk[1], gmnk[2],
                                    a_scales.shape[1], b_scales.shape[1], c_dtype, mode, threads)
    if rc:
        raise ValueError(f"oracle blockwise matmul failed: {rc}")
    return c


def matmul_rowwise(a: np.ndarray, b: np.ndarray, a_scales: np.ndarray, b_scales: np.ndarray,
                   *, c_dtype: int = F32, tensor_scales: bool = False,
                   threads: int = 1, scales_dtype: int = F32) -> np.ndarray:
    """a_scales [1, M] (or [1,1]), b_scales [N, 1] (or [1,1]): float32 arrays, or with
    scales_dtype BF16 / F16 uint16 bit patterns / float16 values that the oracle widens."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    sdt = {F32: np.float32, BF16: np.uint16, F16: np.float16}[scales_dtype]
    a_scales = np.ascontiguousarray(a_scales, dtype=sdt)
    b_scales = np.ascontiguousarray(b_scales, dtype=sdt)
    M, K = a.shape
    N = b.shape[0]
    c = np.zeros((M, N), dtype=np.float32 if c_dtype == F32 else np.uint16)
    st = 0 if tensor_scales else 1
    rc = lib().orc_matmul_rowwise(_p(c), _p(a), _p(b), _p(a_scales), _p(b_scales),
                                  M, N, K, K, K, N, st, st, c_dtype, scales_dtype, threads)
    if rc:
        raise ValueError(f"oracle rowwise matmul failed: {rc}")
    return c


def grouped_matmul(a: np.ndarray, b: np.ndarray, a_scales: np.ndarray, b_scales: np.ndarray,
                   offsets: np.ndarray, expert_ids: np.ndarray, max_tokens: int,
                   num_active: int, *, c_dtype: int = F32, mode: int = 0, threads: int = 1,
                   fill: float = np.nan) -> np.ndarray:
    """Rows no active slot owns keep `fill` (f32 output) so a test can see that
    they are not written."""
    a = np.ascontiguousarray(a, dtype=np.uint8)
    b = np.ascontiguousarray(b, dtype=np.uint8)
    a_scales = np.ascontiguousarray(a_scales, dtype=np.float32)
    b_scales = np.ascontiguousarray(b_scales, dtype=np.float32)
    offsets = np.ascontiguousarray(offsets, dtype=np.uint32)
    expert_ids = np.ascontiguousarray(expert_ids, dtype=np.int32)
    T, K = a.shape
    E, N, _ = b.shape
    if c_dtype == F32:
        c = np.full((T, N), fill, dtype=np.float32)
    else:
        c = np.full((T, N), 0x7FC0, dtype=np.uint16)
    rc = lib().orc_grouped_matmul(_p(c), _p(a), _p(b), _p(a_scales), _p(b_scales),
                                  _p(offsets), _p(expert_ids), T, N, K, E, max_tokens,
                                  num_active, a_scales.shape[1], c_dtype, mode, threads)
    if rc:
        raise ValueError(f"oracle grouped matmul failed: {rc}")
    return c


def bf16_bits_to_f32(u: np.ndarray) -> np.ndarray:
    return (np.asarray(u, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)
