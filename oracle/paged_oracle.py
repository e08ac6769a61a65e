"""numpy front end to the CPU oracle (oracle/paged_oracle.c) -- TEST INFRASTRUCTURE ONLY.

Only tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg import this
module; the shipped package never does.  Every function here is a thin ctypes
call; see paged_oracle.h for the reference file:line each one restates.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libpaged_oracle.so")
_REF_LIB_PATH = os.path.join(_HERE, "_ref", "libref_attention_cpu.so")
REF_ALLOC_DRIVER = os.path.join(_HERE, "_ref", "ref_alloc_driver")

_u16p = C.POINTER(C.c_uint16)
_u32p = C.POINTER(C.c_uint32)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_sz = C.c_size_t


def build(force: bool = False) -> None:
    """Compile libpaged_oracle.so (and oracle/_ref when the reference checkout exists)."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "all"])
    if os.path.isdir("/root/reference") and (force or not os.path.exists(_REF_LIB_PATH)
                                             or not os.path.exists(REF_ALLOC_DRIVER)):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "_ref"])


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        L.oracle_fp16_to_float.restype = C.c_float
        L.oracle_fp16_to_float.argtypes = [C.c_uint16]
        L.oracle_float_to_fp16_ref.restype = C.c_uint16
        L.oracle_float_to_fp16_ref.argtypes = [C.c_float]
        L.oracle_float_to_fp16_rne.restype = C.c_uint16
        L.oracle_float_to_fp16_rne.argtypes = [C.c_float]
        L.oracle_fp16_to_float_n.restype = None
        L.oracle_fp16_to_float_n.argtypes = [_u16p, _f32p, _sz]
        L.oracle_float_to_fp16_ref_n.restype = None
        L.oracle_float_to_fp16_ref_n.argtypes = [_f32p, _u16p, _sz]
        L.oracle_float_to_fp16_rne_n.restype = None
        L.oracle_float_to_fp16_rne_n.argtypes = [_f32p, _u16p, _sz]
        L.oracle_scatter_kv_paged_batched_f16.restype = C.c_int
        L.oracle_scatter_kv_paged_batched_f16.argtypes = [_u16p, _u32p, _u32p, _sz, _sz, _sz, _sz, _u16p]
        L.oracle_scatter_kv_paged.restype = C.c_int
        L.oracle_scatter_kv_paged.argtypes = [C.c_void_p, _u32p, _sz, _sz, _sz, _sz, _sz, _sz,
                                              C.c_void_p, _sz]
        L.oracle_qkv_split_rope_cast.restype = C.c_int
        L.oracle_qkv_split_rope_cast.argtypes = [_f32p, _f32p, _f32p, _f32p, _u16p, _u16p, C.c_void_p,
                                                 C.c_void_p] + [_sz] * 9
        L.oracle_rotary_coefficients.restype = _sz
        L.oracle_rotary_coefficients.argtypes = [_sz, _sz, C.c_float, C.c_float, _f32p, _f32p]
        L.oracle_rms_norm_batched.restype = C.c_int
        L.oracle_rms_norm_batched.argtypes = [_f32p, C.c_void_p, _sz, C.c_float, _sz, _sz, _f32p]
        L.oracle_add.restype = C.c_int
        L.oracle_add.argtypes = [_f32p, _f32p, _f32p, _sz]
        L.oracle_silu_mul.restype = C.c_int
        L.oracle_silu_mul.argtypes = [_f32p, _f32p, _f32p, _sz]
        L.oracle_gate_up_split_silu_mul.restype = C.c_int
        L.oracle_gate_up_split_silu_mul.argtypes = [_f32p, _f32p, _f32p, _f32p, _sz, _sz, _sz]
        L.oracle_matmul_q4_0_batched.restype = C.c_int
        L.oracle_matmul_q4_0_batched.argtypes = [C.c_void_p, _f32p, _sz, _sz, _sz, _sz, _f32p, C.c_int]
        L.oracle_quantize_row_q4_0.restype = None
        L.oracle_quantize_row_q4_0.argtypes = [_f32p, _sz, C.c_void_p]
        L.oracle_matmul_q6_k_batched.restype = C.c_int
        L.oracle_matmul_q6_k_batched.argtypes = [C.c_void_p, _f32p, _sz, _sz, _sz, _sz, _f32p, C.c_int]
        L.oracle_quantize_row_q6_k.restype = None
        L.oracle_quantize_row_q6_k.argtypes = [_f32p, _sz, C.c_void_p]
        L.oracle_dequantize_row_q6_k.restype = None
        L.oracle_dequantize_row_q6_k.argtypes = [C.c_void_p, _sz, _f32p]
        L.oracle_gather_kv_pages.restype = C.c_int
        L.oracle_gather_kv_pages.argtypes = [C.c_void_p, _u32p, _sz, _sz, _sz, _sz, _sz,
                                             C.c_void_p, _sz]
        attn = [_f32p, _u16p, _u16p, _f32p, _u32p, _sz, _u32p, _u32p, _u32p,
                _sz, _sz, _sz, _sz, _sz, C.c_int]
        L.oracle_paged_attention_executor.restype = C.c_int
        L.oracle_paged_attention_executor.argtypes = attn + [C.c_int]
        L.oracle_paged_attention_flashref.restype = C.c_int
        L.oracle_paged_attention_flashref.argtypes = attn
        L.oracle_paged_attention_prefill.restype = C.c_int
        L.oracle_paged_attention_prefill.argtypes = [_u16p, _u16p, _u16p, _f32p, _u32p, _sz, _u32p,
                                                     _u32p, _u32p, _sz, _sz, _sz, _sz, _sz, _sz,
                                                     C.c_int]
        L.oracle_metrics.restype = None
        L.oracle_metrics.argtypes = [_f32p, _f32p, _sz, _f64p, _f64p, _f64p, _f64p]
        L.oracle_cosine.restype = C.c_double
        L.oracle_cosine.argtypes = [_f32p, _f32p, _sz]
        L.oracle_pool_new.restype = C.c_void_p
        L.oracle_pool_new.argtypes = [C.c_uint32]
        L.oracle_pool_free.restype = None
        L.oracle_pool_free.argtypes = [C.c_void_p]
        L.oracle_pool_allocate.restype = C.c_int
        L.oracle_pool_allocate.argtypes = [C.c_void_p, _u32p]
        L.oracle_pool_allocate_n.restype = C.c_int
        L.oracle_pool_allocate_n.argtypes = [C.c_void_p, _sz, _u32p]
        L.oracle_pool_release.restype = None
        L.oracle_pool_release.argtypes = [C.c_void_p, C.c_uint32]
        L.oracle_pool_in_use.restype = _sz
        L.oracle_pool_in_use.argtypes = [C.c_void_p]
        L.oracle_pool_free_count.restype = _sz
        L.oracle_pool_free_count.argtypes = [C.c_void_p]
        L.oracle_req_total_tokens.restype = _sz
        L.oracle_req_total_tokens.argtypes = [C.c_void_p]
        for name in ("oracle_req_reserve",):
            getattr(L, name).restype = C.c_int
            getattr(L, name).argtypes = [C.c_void_p, C.c_void_p, _sz]
        L.oracle_req_extend_one_token.restype = C.c_int
        L.oracle_req_extend_one_token.argtypes = [C.c_void_p, C.c_void_p, _u32p, _u32p]
        L.oracle_req_locate.restype = C.c_int
        L.oracle_req_locate.argtypes = [C.c_void_p, _sz, _u32p, _u32p]
        L.oracle_req_release_all.restype = None
        L.oracle_req_release_all.argtypes = [C.c_void_p, C.c_void_p]
        _lib = L
    return _lib


def _p(a: np.ndarray, typ):
    return a.ctypes.data_as(typ)


def _c(a, dtype) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=dtype)


# ---------------------------------------------------------------- fp16

def fp16_to_float(h) -> np.ndarray:
    h = _c(h, np.uint16).ravel()
    out = np.empty(h.size, np.float32)
    lib().oracle_fp16_to_float_n(_p(h, _u16p), _p(out, _f32p), h.size)
    return out


def float_to_fp16_ref(v) -> np.ndarray:
    v = _c(v, np.float32).ravel()
    out = np.empty(v.size, np.uint16)
    lib().oracle_float_to_fp16_ref_n(_p(v, _f32p), _p(out, _u16p), v.size)
    return out


def float_to_fp16_rne(v) -> np.ndarray:
    v = _c(v, np.float32).ravel()
    out = np.empty(v.size, np.uint16)
    lib().oracle_float_to_fp16_rne_n(_p(v, _f32p), _p(out, _u16p), v.size)
    return out


# ------------------------------------------------------ scatter / gather

def scatter_kv_paged_batched_f16(page_storage: np.ndarray, page_ids, slots_in_page,
                                 page_size_tokens: int, n_kv_heads: int, head_dim: int,
                                 batch: int, src: np.ndarray) -> bool:
    """In place on page_storage (uint16 view of the fp16 pool)."""
    assert page_storage.dtype == np.uint16 and page_storage.flags.c_contiguous
    pid = _c(page_ids, np.uint32)
    sl = _c(slots_in_page, np.uint32)
    s = _c(src, np.uint16)
    return bool(lib().oracle_scatter_kv_paged_batched_f16(
        _p(page_storage, _u16p), _p(pid, _u32p), _p(sl, _u32p), page_size_tokens, n_kv_heads,
        head_dim, batch, _p(s, _u16p)))


def scatter_kv_paged(page_storage: np.ndarray, page_table, page_size_tokens: int, n_kv_heads: int,
                     head_dim: int, tokens: int, start_slot: int, src: np.ndarray,
                     dtype_bytes: int) -> bool:
    assert page_storage.flags.c_contiguous
    pt = _c(page_table, np.uint32)
    s = np.ascontiguousarray(src)
    return bool(lib().oracle_scatter_kv_paged(
        page_storage.ctypes.data, _p(pt, _u32p), pt.size, page_size_tokens, n_kv_heads, head_dim,
        tokens, start_slot, s.ctypes.data, dtype_bytes))


def gather_kv_pages(page_storage: np.ndarray, page_table, page_size_tokens: int, n_kv_heads: int,
                    head_dim: int, num_tokens: int, dst: np.ndarray, dtype_bytes: int) -> bool:
    assert dst.flags.c_contiguous
    ps = np.ascontiguousarray(page_storage)
    pt = _c(page_table, np.uint32)
    return bool(lib().oracle_gather_kv_pages(
        ps.ctypes.data, _p(pt, _u32p), pt.size, page_size_tokens, n_kv_heads, head_dim,
        num_tokens, dst.ctypes.data, dtype_bytes))


# ------------------------------------------------- qkv split + RoPE + cast

def rotary_coefficients(position: int, rotary_dim: int, freq_base: float = 10000.0,
                        freq_scale: float = 1.0):
    """(cos, sin), each rotary_dim // 2 floats (quantization.cpp:795-823)."""
    pairs = rotary_dim // 2
    cos = np.zeros(max(pairs, 1), np.float32)
    sin = np.zeros(max(pairs, 1), np.float32)
    n = lib().oracle_rotary_coefficients(position, rotary_dim, freq_base, freq_scale,
                                         _p(cos, _f32p), _p(sin, _f32p))
    return cos[:n], sin[:n]


def qkv_split_rope_cast(qkv, cos, sin, batch, num_heads, kv_heads, head_dim, qkv_rows, q_rows, k_rows,
                        v_rows, rotary_dim):
    """Returns (q, k, v, k_f16, v_f16) or None on the argument errors."""
    qkv = _c(qkv, np.float32)
    q = np.zeros((batch, q_rows), np.float32)
    k = np.zeros((batch, k_rows), np.float32)
    v = np.zeros((batch, v_rows), np.float32)
    k16 = np.zeros((batch, k_rows), np.uint16)
    v16 = np.zeros((batch, v_rows), np.uint16)
    cosp = sinp = None
    if cos is not None:
        cos = _c(cos, np.float32)
        sin = _c(sin, np.float32)
        cosp, sinp = cos.ctypes.data, sin.ctypes.data
    ok = lib().oracle_qkv_split_rope_cast(_p(qkv, _f32p), _p(q, _f32p), _p(k, _f32p), _p(v, _f32p),
                                          _p(k16, _u16p), _p(v16, _u16p), cosp, sinp, batch, num_heads,
                                          kv_heads, head_dim, qkv_rows, q_rows, k_rows, v_rows, rotary_dim)
    return (q, k, v, k16, v16) if ok else None


# ------------------------------------------------ walker layer operators

def rms_norm_batched(x, weight, epsilon, batch, length):
    x = _c(x, np.float32)
    w = None if weight is None else _c(weight, np.float32)
    out = np.zeros((batch, length), np.float32)
    ok = lib().oracle_rms_norm_batched(_p(x, _f32p), None if w is None else w.ctypes.data,
                                       0 if w is None else w.size, epsilon, batch, length, _p(out, _f32p))
    return out if ok else None


def add(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    out = np.zeros(a.shape, np.float32)
    return out if lib().oracle_add(_p(a, _f32p), _p(b, _f32p), _p(out, _f32p), a.size) else None


def silu_mul(gate, up):
    g, u = _c(gate, np.float32), _c(up, np.float32)
    out = np.zeros(g.shape, np.float32)
    return out if lib().oracle_silu_mul(_p(g, _f32p), _p(u, _f32p), _p(out, _f32p), g.size) else None


def gate_up_split_silu_mul(gate_up, batch, ffn_inner, gate_up_rows):
    """Returns (gate, up, out) or None."""
    gu = _c(gate_up, np.float32)
    gate = np.zeros((batch, ffn_inner), np.float32)
    up = np.zeros((batch, ffn_inner), np.float32)
    out = np.zeros((batch, ffn_inner), np.float32)
    ok = lib().oracle_gate_up_split_silu_mul(_p(gu, _f32p), _p(gate, _f32p), _p(up, _f32p), _p(out, _f32p),
                                             batch, ffn_inner, gate_up_rows)
    return (gate, up, out) if ok else None


def q4_0_row_bytes(cols: int) -> int:
    return (cols + 31) // 32 * 18


def quantize_q4_0(w) -> np.ndarray:
    """Rows of floats -> Q4_0 rows (uint8 [rows][q4_0_row_bytes(cols)]), quantizeRowQ4_0."""
    w = _c(w, np.float32)
    rows, cols = w.shape
    out = np.zeros((rows, q4_0_row_bytes(cols)), np.uint8)
    L = lib()
    for r in range(rows):
        L.oracle_quantize_row_q4_0(_p(w[r], _f32p), cols, out[r].ctypes.data)
    return out


def matmul_q4_0_batched(weights, x, batch, rows, cols, row_stride=None, n_threads=8):
    wq = _c(weights, np.uint8)
    x = _c(x, np.float32)
    out = np.zeros((batch, rows), np.float32)
    ok = lib().oracle_matmul_q4_0_batched(wq.ctypes.data, _p(x, _f32p), batch, rows, cols,
                                          row_stride or q4_0_row_bytes(cols), _p(out, _f32p), n_threads)
    return out if ok else None


def q6_k_row_bytes(cols: int) -> int:
    return (cols + 255) // 256 * 210


def quantize_q6_k(w) -> np.ndarray:
    """Rows of floats -> Q6_K rows (uint8 [rows][q6_k_row_bytes(cols)]), quantizeRowQ6_K."""
    w = _c(w, np.float32)
    rows, cols = w.shape
    out = np.zeros((rows, q6_k_row_bytes(cols)), np.uint8)
    L = lib()
    for r in range(rows):
        L.oracle_quantize_row_q6_k(_p(w[r], _f32p), cols, out[r].ctypes.data)
    return out


def dequantize_q6_k(weights, cols) -> np.ndarray:
    wq = _c(weights, np.uint8)
    out = np.zeros((wq.shape[0], cols), np.float32)
    L = lib()
    for r in range(wq.shape[0]):
        L.oracle_dequantize_row_q6_k(wq[r].ctypes.data, cols, _p(out[r], _f32p))
    return out


def matmul_q6_k_batched(weights, x, batch, rows, cols, row_stride=None, n_threads=8):
    wq = _c(weights, np.uint8)
    x = _c(x, np.float32)
    out = np.zeros((batch, rows), np.float32)
    ok = lib().oracle_matmul_q6_k_batched(wq.ctypes.data, _p(x, _f32p), batch, rows, cols,
                                          row_stride or q6_k_row_bytes(cols), _p(out, _f32p), n_threads)
    return out if ok else None


# ------------------------------------------------------------ attention

def _attn_args(q, k_pages, v_pages, pt_flat, pt_off, seq_lens, q_pos, batch, num_heads, head_dim):
    q = _c(q, np.float32)
    k = _c(k_pages, np.uint16)
    v = _c(v_pages, np.uint16)
    flat = _c(pt_flat, np.uint32)
    if flat.size == 0:
        flat = np.zeros(1, np.uint32)
        n_flat = 0
    else:
        n_flat = flat.size
    off = _c(pt_off, np.uint32)
    sl = _c(seq_lens, np.uint32)
    qp = _c(q_pos, np.uint32)
    out = np.zeros(batch * num_heads * head_dim, np.float32)
    return q, k, v, flat, n_flat, off, sl, qp, out


def paged_attention_executor(q, k_pages, v_pages, pt_flat, pt_off, seq_lens, q_pos, batch,
                             num_heads, kv_heads, head_dim, page_size_tokens, apply_causal,
                             n_threads: int = 1):
    """Executor-CPU ordering (attention_cpu.cpp:437-470) over paged fp16 K/V.  None on bad args."""
    q, k, v, flat, n_flat, off, sl, qp, out = _attn_args(
        q, k_pages, v_pages, pt_flat, pt_off, seq_lens, q_pos, batch, num_heads, head_dim)
    ok = lib().oracle_paged_attention_executor(
        _p(q, _f32p), _p(k, _u16p), _p(v, _u16p), _p(out, _f32p), _p(flat, _u32p), n_flat,
        _p(off, _u32p), _p(sl, _u32p), _p(qp, _u32p), batch, num_heads, kv_heads, head_dim,
        page_size_tokens, int(bool(apply_causal)), n_threads)
    return out.reshape(batch, num_heads, head_dim) if ok else None


def paged_attention_flashref(q, k_pages, v_pages, pt_flat, pt_off, seq_lens, q_pos, batch,
                             num_heads, kv_heads, head_dim, page_size_tokens, apply_causal):
    """tests/test_paged_flash.cpp:17-91 ordering.  None on bad args."""
    q, k, v, flat, n_flat, off, sl, qp, out = _attn_args(
        q, k_pages, v_pages, pt_flat, pt_off, seq_lens, q_pos, batch, num_heads, head_dim)
    ok = lib().oracle_paged_attention_flashref(
        _p(q, _f32p), _p(k, _u16p), _p(v, _u16p), _p(out, _f32p), _p(flat, _u32p), n_flat,
        _p(off, _u32p), _p(sl, _u32p), _p(qp, _u32p), batch, num_heads, kv_heads, head_dim,
        page_size_tokens, int(bool(apply_causal)))
    return out.reshape(batch, num_heads, head_dim) if ok else None


def paged_attention_prefill(q_f16, k_pages, v_pages, pt_flat, pt_off, seq_lens, q_start, batch,
                            chunk, num_heads, kv_heads, head_dim, page_size_tokens,
                            n_threads: int = 1):
    qh = _c(q_f16, np.uint16)
    k = _c(k_pages, np.uint16)
    v = _c(v_pages, np.uint16)
    flat = _c(pt_flat, np.uint32)
    off = _c(pt_off, np.uint32)
    sl = _c(seq_lens, np.uint32)
    qs = _c(q_start, np.uint32)
    out = np.zeros(batch * chunk * num_heads * head_dim, np.float32)
    ok = lib().oracle_paged_attention_prefill(
        _p(qh, _u16p), _p(k, _u16p), _p(v, _u16p), _p(out, _f32p), _p(flat, _u32p), flat.size,
        _p(off, _u32p), _p(sl, _u32p), _p(qs, _u32p), batch, chunk, num_heads, kv_heads, head_dim,
        page_size_tokens, n_threads)
    return out.reshape(batch, chunk, num_heads, head_dim) if ok else None


def metrics(a, b) -> dict:
    """max_abs / mean_abs / rms / cosine as parity_harness.cpp:214-255 computes them."""
    a = _c(a, np.float32).ravel()
    b = _c(b, np.float32).ravel()
    assert a.size == b.size
    mx, me, rms, cos = C.c_double(), C.c_double(), C.c_double(), C.c_double()
    lib().oracle_metrics(_p(a, _f32p), _p(b, _f32p), a.size, C.byref(mx), C.byref(me),
                         C.byref(rms), C.byref(cos))
    return {"max_abs": mx.value, "mean_abs": me.value, "rms": rms.value, "cosine": cos.value}


def cosine(a, b) -> float:
    a = _c(a, np.float32).ravel()
    b = _c(b, np.float32).ravel()
    return float(lib().oracle_cosine(_p(a, _f32p), _p(b, _f32p), a.size))


def per_head_report(got, want, head_dim: int) -> dict:
    """Worst per-(request, head) cosine and max-abs: the acceptance rubric
    (cosine >= 0.9999 and max_abs <= 2e-3 for every head)."""
    g = _c(got, np.float32).reshape(-1, head_dim)
    w = _c(want, np.float32).reshape(-1, head_dim)
    assert g.shape == w.shape
    worst_cos, worst_abs = 1.0, 0.0
    for i in range(g.shape[0]):
        if not (np.any(g[i]) or np.any(w[i])):
            continue  # both all-zero (empty sequence): identical
        worst_cos = min(worst_cos, cosine(g[i], w[i]))
        worst_abs = max(worst_abs, float(np.max(np.abs(g[i].astype(np.float64) - w[i]))))
    return {"min_cosine": worst_cos, "max_abs": worst_abs}


# ------------------------------------------------------------ allocator

class PagePool:
    """oracle_pool_* (paged_kv.cpp:10-42)."""

    def __init__(self, capacity: int):
        self._h = lib().oracle_pool_new(capacity)
        self.capacity = capacity

    def __del__(self):
        if getattr(self, "_h", None):
            lib().oracle_pool_free(self._h)
            self._h = None

    def allocate(self):
        out = C.c_uint32()
        return out.value if lib().oracle_pool_allocate(self._h, C.byref(out)) else None

    def allocate_n(self, n: int):
        buf = (C.c_uint32 * max(n, 1))()
        if not lib().oracle_pool_allocate_n(self._h, n, buf):
            return None
        return [int(buf[i]) for i in range(n)]

    def release(self, page_id: int) -> None:
        lib().oracle_pool_release(self._h, page_id)

    def pages_in_use(self) -> int:
        return int(lib().oracle_pool_in_use(self._h))

    def pages_free(self) -> int:
        return int(lib().oracle_pool_free_count(self._h))


class _ReqStruct(C.Structure):
    _fields_ = [("page_size_tokens", C.c_uint32), ("page_table", _u32p), ("page_table_cap", _sz),
                ("n_pages", _sz), ("tokens_in_last_page", C.c_uint32)]


class RequestKVState:
    """oracle_req_* (paged_kv.hpp:65-97, paged_kv.cpp:44-81)."""

    def __init__(self, page_size_tokens: int = 64, max_pages: int = 4096):
        self._buf = (C.c_uint32 * max_pages)()
        self._st = _ReqStruct(page_size_tokens, C.cast(self._buf, _u32p), max_pages, 0, 0)

    @property
    def page_table(self):
        return [int(self._buf[i]) for i in range(self._st.n_pages)]

    @property
    def tokens_in_last_page(self) -> int:
        return int(self._st.tokens_in_last_page)

    def total_tokens(self) -> int:
        return int(lib().oracle_req_total_tokens(C.byref(self._st)))

    def reserve(self, pool: PagePool, target_tokens: int) -> bool:
        return bool(lib().oracle_req_reserve(C.byref(self._st), pool._h, target_tokens))

    def extend_one_token(self, pool: PagePool):
        pid, slot = C.c_uint32(), C.c_uint32()
        ok = lib().oracle_req_extend_one_token(C.byref(self._st), pool._h, C.byref(pid), C.byref(slot))
        return (pid.value, slot.value) if ok else None

    def locate(self, pos: int):
        pid, slot = C.c_uint32(), C.c_uint32()
        ok = lib().oracle_req_locate(C.byref(self._st), pos, C.byref(pid), C.byref(slot))
        return (pid.value, slot.value) if ok else None

    def release_all(self, pool: PagePool) -> None:
        lib().oracle_req_release_all(C.byref(self._st), pool._h)


# ------------------------------------------------- the real reference

_ref = None


def ref_lib():
    """oracle/_ref/libref_attention_cpu.so: the reference's own RunAttentionCPU and fp16
    helpers.  None when it has not been built (no reference checkout on this machine)."""
    global _ref
    if _ref is None:
        if not os.path.exists(_REF_LIB_PATH):
            return None
        R = C.CDLL(_REF_LIB_PATH)
        R.ref_fp16_to_float.restype = C.c_float
        R.ref_fp16_to_float.argtypes = [C.c_uint16]
        R.ref_float_to_fp16.restype = C.c_uint16
        R.ref_float_to_fp16.argtypes = [C.c_float]
        R.ref_fp16_to_float_n.restype = None
        R.ref_fp16_to_float_n.argtypes = [_u16p, _f32p, _sz]
        R.ref_float_to_fp16_n.restype = None
        R.ref_float_to_fp16_n.argtypes = [_f32p, _u16p, _sz]
        R.ref_apply_rotary.restype = None
        R.ref_apply_rotary.argtypes = [_f32p, _f32p, _f32p, _sz, _sz, _sz]
        R.ref_rotary_coefficients.restype = _sz
        R.ref_rotary_coefficients.argtypes = [_sz, _sz, C.c_float, C.c_float, _f32p, _f32p]
        R.ref_quantize_row_q4_0.restype = _sz
        R.ref_quantize_row_q4_0.argtypes = [_f32p, _sz, C.c_void_p, _sz]
        R.ref_dot_q4_0.restype = C.c_float
        R.ref_dot_q4_0.argtypes = [C.c_void_p, _sz, _f32p]
        R.ref_dequantize_row_q4_0.restype = None
        R.ref_dequantize_row_q4_0.argtypes = [C.c_void_p, _sz, _f32p]
        R.ref_quantize_row_q6_k.restype = _sz
        R.ref_quantize_row_q6_k.argtypes = [_f32p, _sz, C.c_void_p, _sz]
        R.ref_dot_q6_k.restype = C.c_float
        R.ref_dot_q6_k.argtypes = [C.c_void_p, _sz, _f32p]
        R.ref_dequantize_row_q6_k.restype = None
        R.ref_dequantize_row_q6_k.argtypes = [C.c_void_p, _sz, _f32p]
        R.ref_run_attention_cpu.restype = C.c_int
        R.ref_run_attention_cpu.argtypes = [_f32p, _u16p, _u16p, _sz, _sz, _sz, _sz, _sz, _f32p,
                                            _f32p, _f32p]
        _ref = R
    return _ref


def ref_fp16_to_float(h) -> np.ndarray:
    h = _c(h, np.uint16).ravel()
    out = np.empty(h.size, np.float32)
    ref_lib().ref_fp16_to_float_n(_p(h, _u16p), _p(out, _f32p), h.size)
    return out


def ref_float_to_fp16(v) -> np.ndarray:
    v = _c(v, np.float32).ravel()
    out = np.empty(v.size, np.uint16)
    ref_lib().ref_float_to_fp16_n(_p(v, _f32p), _p(out, _u16p), v.size)
    return out


def ref_apply_rotary(vec, cos, sin, head_dim, rotary_dim) -> np.ndarray:
    """The reference's applyRotaryEmbedding on one head vector (returns a rotated copy)."""
    x = np.array(vec, np.float32).ravel().copy()
    cos, sin = _c(cos, np.float32), _c(sin, np.float32)
    ref_lib().ref_apply_rotary(_p(x, _f32p), _p(cos, _f32p), _p(sin, _f32p), cos.size, head_dim, rotary_dim)
    return x


def ref_rotary_coefficients(position, rotary_dim, freq_base, freq_scale):
    pairs = max(rotary_dim // 2, 1)
    cos, sin = np.zeros(pairs, np.float32), np.zeros(pairs, np.float32)
    n = ref_lib().ref_rotary_coefficients(position, rotary_dim, freq_base, freq_scale,
                                          _p(cos, _f32p), _p(sin, _f32p))
    return cos[:n], sin[:n]


def ref_run_attention_cpu(q, k_cache, v_cache, heads, kv_heads, head_dim, ctx_len, position,
                          k_new, v_new):
    R = ref_lib()
    assert R is not None
    q = _c(q, np.float32)
    kc = _c(k_cache, np.uint16)
    vc = _c(v_cache, np.uint16)
    kn = _c(k_new, np.float32)
    vn = _c(v_new, np.float32)
    out = np.zeros(heads * head_dim, np.float32)
    ok = R.ref_run_attention_cpu(_p(q, _f32p), _p(kc, _u16p), _p(vc, _u16p), heads, kv_heads,
                                 head_dim, ctx_len, position, _p(kn, _f32p), _p(vn, _f32p),
                                 _p(out, _f32p))
    return out.reshape(heads, head_dim) if ok else None
