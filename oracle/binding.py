"""ctypes binding of the CPU oracle (``libhipml_oracle.so``).

Test infrastructure only.  Every wrapper takes and returns numpy arrays and
maps one-to-one onto a C function in ``hipml_oracle.h``; the arithmetic lives
in C so that a 32K-row decode finishes in well under a second.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhipml_oracle.so")

Q8, Q4, BLOCK = 0, 1, 32


def build(force: bool = False) -> str:
    """Compile the oracle with the Makefile beside it; returns the .so path."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.run(["make", "-C", _HERE] + (["-B"] if force else []), check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _declare(_lib)
    return _lib


_f32p = C.POINTER(C.c_float)
_u8p = C.POINTER(C.c_uint8)
_i32p = C.POINTER(C.c_int32)
_szp = C.POINTER(C.c_size_t)


class _Rng(C.Structure):
    _fields_ = [("state", C.c_uint64)]


def _declare(l: C.CDLL) -> None:
    sz, f32, i = C.c_size_t, C.c_float, C.c_int
    sig = {
        "orc_block_bytes": (sz, [i]),
        "orc_row_bytes": (sz, [i, sz]),
        "orc_token_bytes": (sz, [i, sz, sz, sz]),
        "orc_f16_to_f32": (f32, [C.c_uint16]),
        "orc_f32_to_f16": (C.c_uint16, [f32]),
        "orc_quantize_block": (None, [i, _f32p, _u8p]),
        "orc_quantize": (None, [i, _f32p, sz, _u8p]),
        "orc_block_f32": (None, [i, _u8p, _f32p]),
        "orc_dequantize": (None, [i, _u8p, sz, _f32p]),
        "orc_synthetic_blocks": (None, [i, sz, C.c_uint64, _u8p]),
        "orc_rng_new": (None, [C.POINTER(_Rng), C.c_uint64]),
        "orc_rng_next_u64": (C.c_uint64, [C.POINTER(_Rng)]),
        "orc_rng_uniform": (f32, [C.POINTER(_Rng)]),
        "orc_rng_normal": (f32, [C.POINTER(_Rng)]),
        "orc_rng_fill_normal": (None, [C.POINTER(_Rng), _f32p, sz, f32]),
        "orc_rng_fill_uniform": (None, [C.POINTER(_Rng), _f32p, sz]),
        "orc_sigmoid_f32": (None, [_f32p, _f32p, sz]),
        "orc_rope_neox_f32": (None, [_f32p, _f32p, sz, sz, sz, f32]),
        "orc_rope_multi_f32": (None, [_f32p, _f32p, sz, sz, sz, _szp, _szp, f32]),
        "orc_q_gate_f32": (None, [_f32p, _f32p, _f32p, sz]),
        "orc_rmsnorm_f32": (None, [_f32p, _f32p, _f32p, sz, f32]),
        "orc_head_rmsnorm_f32": (None, [_f32p, _f32p, _f32p, sz, sz, f32]),
        "orc_rmsnorm_tree_f32": (None, [_f32p, _f32p, _f32p, sz, f32]),
        "orc_qg_split_f32": (None, [_f32p, _f32p, _f32p, sz, sz]),
        "orc_kv_append_f32": (None, [_f32p, _f32p, _f32p, _f32p, sz, sz]),
        "orc_attn_causal_f32": (None, [_f32p, _f32p, _f32p, sz, sz, sz, sz, f32, _f32p]),
        "orc_attn_decode_f32": (None, [_f32p, _f32p, _f32p, sz, sz, sz, sz, f32, _f32p]),
        "orc_attn_decode_kv": (None, [_f32p, _u8p, _u8p, sz, sz, sz, sz, sz, f32, i, _f32p]),
        "orc_attn_core_token_f32": (None, [_f32p, _f32p, _f32p, _f32p, _f32p, _f32p, sz, sz, sz,
                                           sz, sz, _szp, sz, f32, _f32p]),
        "orc_attn_chunk_kv": (None, [_f32p, _u8p, _u8p, sz, sz, sz, sz, sz, sz, f32, i, _i32p, sz,
                                     i, _f32p]),
        "orc_dequant_q8_0": (None, [_u8p, _f32p]),
        "orc_gemv_q8_0": (None, [_u8p, _f32p, sz, sz, _f32p]),
        "orc_gemm_q8_0": (None, [_u8p, _f32p, sz, sz, sz, i, _f32p]),
        "orc_random_q8_0_bytes": (None, [C.POINTER(_Rng), sz, _u8p]),
        "orc_compare": (i, [_f32p, _f32p, sz, f32, f32, _f32p, _f32p]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(l, name)
        fn.restype = res
        fn.argtypes = args


def _f(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32)


def _b(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.uint8)


def _pf(a: np.ndarray):
    return a.ctypes.data_as(_f32p)


def _pb(a: np.ndarray):
    return a.ctypes.data_as(_u8p)


def _sz4(v):
    return (C.c_size_t * 4)(*[int(x) for x in v])


# ---- formats ---------------------------------------------------------------

def block_bytes(dtype: int) -> int:
    return lib().orc_block_bytes(dtype)


def row_bytes(dtype: int, head_dim: int) -> int:
    return lib().orc_row_bytes(dtype, head_dim)


def token_bytes(dtype: int, n_kv: int, head_dim: int, n_layers: int) -> int:
    return lib().orc_token_bytes(dtype, n_kv, head_dim, n_layers)


def f16_to_f32(h: int) -> np.float32:
    return np.float32(lib().orc_f16_to_f32(h))


def f32_to_f16(v) -> int:
    return lib().orc_f32_to_f16(C.c_float(float(np.float32(v))))


def f32_bits_to_f16(bits: int) -> int:
    """f32 given as its bit pattern (keeps NaN payloads intact)."""
    return lib().orc_f32_to_f16(C.c_float.from_buffer_copy(np.uint32(bits).tobytes()))


def quantize(dtype: int, values) -> np.ndarray:
    v = _f(values).ravel()
    assert v.size % BLOCK == 0, "values must be a multiple of 32"
    out = np.empty(v.size // BLOCK * block_bytes(dtype), dtype=np.uint8)
    lib().orc_quantize(dtype, _pf(v), v.size, _pb(out))
    return out


def dequantize(dtype: int, data) -> np.ndarray:
    b = _b(data).ravel()
    bb = block_bytes(dtype)
    assert b.size % bb == 0, "truncated block"
    out = np.empty(b.size // bb * BLOCK, dtype=np.float32)
    lib().orc_dequantize(dtype, _pb(b), b.size, _pf(out))
    return out


def synthetic_blocks(dtype: int, n_blocks: int, seed: int) -> np.ndarray:
    out = np.empty(n_blocks * block_bytes(dtype), dtype=np.uint8)
    lib().orc_synthetic_blocks(dtype, n_blocks, seed, _pb(out))
    return out


# ---- RNG -------------------------------------------------------------------

class Rng:
    """xorshift64* + Box-Muller, the reference's deterministic generator."""

    def __init__(self, seed: int):
        self._r = _Rng()
        lib().orc_rng_new(C.byref(self._r), seed)

    def next_u64(self) -> int:
        return lib().orc_rng_next_u64(C.byref(self._r))

    def uniform(self) -> np.float32:
        return np.float32(lib().orc_rng_uniform(C.byref(self._r)))

    def normal(self) -> np.float32:
        return np.float32(lib().orc_rng_normal(C.byref(self._r)))

    def normal_array(self, shape, std: float = 1.0) -> np.ndarray:
        out = np.empty(shape, dtype=np.float32)
        lib().orc_rng_fill_normal(C.byref(self._r), _pf(out), out.size, std)
        return out

    def uniform_array(self, shape) -> np.ndarray:
        out = np.empty(shape, dtype=np.float32)
        lib().orc_rng_fill_uniform(C.byref(self._r), _pf(out), out.size)
        return out


# ---- ops -------------------------------------------------------------------

def sigmoid(x) -> np.ndarray:
    x = _f(x)
    out = np.empty_like(x)
    lib().orc_sigmoid_f32(_pf(x), _pf(out), x.size)
    return out


def q_gate(q, gate) -> np.ndarray:
    q, gate = _f(q), _f(gate)
    out = np.empty_like(q)
    lib().orc_q_gate_f32(_pf(q), _pf(gate), _pf(out), q.size)
    return out


def rmsnorm(x, w, eps) -> np.ndarray:
    x, w = _f(x), _f(w)
    y = np.empty_like(x)
    lib().orc_rmsnorm_f32(_pf(x), _pf(w), _pf(y), x.size, eps)
    return y


def head_rmsnorm(x, w, n_heads, head_dim, eps, tree=False) -> np.ndarray:
    """Per-head RMS norm; `tree` sums the squares in the order of the reference's GPU kernels."""
    x, w = _f(x), _f(w)
    y = np.empty_like(x)
    if not tree:
        lib().orc_head_rmsnorm_f32(_pf(x), _pf(w), _pf(y), n_heads, head_dim, eps)
        return y
    xr, yr = x.reshape(n_heads, head_dim), y.reshape(n_heads, head_dim)
    for h in range(n_heads):
        row = np.ascontiguousarray(xr[h])
        out = np.empty_like(row)
        lib().orc_rmsnorm_tree_f32(_pf(row), _pf(w), _pf(out), head_dim, eps)
        yr[h] = out
    return y


def qg_split(qg, n_heads, head_dim):
    qg = _f(qg)
    q = np.empty(n_heads * head_dim, dtype=np.float32)
    gate = np.empty(n_heads * head_dim, dtype=np.float32)
    lib().orc_qg_split_f32(_pf(qg), _pf(q), _pf(gate), n_heads, head_dim)
    return q, gate


def attn_front(qg, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, sections, pos, theta, eps,
               tree=True):
    """q|gate split, per-head RMS norm of q and k, M-RoPE of both: the reference's decode front
    end (attn_front_f32.hip:34-135 = qg_split + head_rmsnorm x2 + mrope x2).  Returns q, gate, k."""
    q, gate = qg_split(qg, n_heads, head_dim)
    q = head_rmsnorm(q, q_norm, n_heads, head_dim, eps, tree)
    kk = head_rmsnorm(k, k_norm, n_kv, head_dim, eps, tree)
    q = rope_multi(q, n_heads, head_dim, n_rot, sections, pos, theta)
    kk = rope_multi(kk, n_kv, head_dim, n_rot, sections, pos, theta)
    return q.ravel(), gate.ravel(), kk.ravel()


def rope_neox(x, n_heads, head_dim, pos, theta) -> np.ndarray:
    x = _f(x)
    y = np.empty_like(x)
    lib().orc_rope_neox_f32(_pf(x), _pf(y), n_heads, head_dim, pos, theta)
    return y


def rope_multi(x, n_heads, head_dim, n_rot, sections, pos, theta) -> np.ndarray:
    x = _f(x)
    y = np.empty_like(x)
    lib().orc_rope_multi_f32(_pf(x), _pf(y), n_heads, head_dim, n_rot, _sz4(sections), _sz4(pos),
                             theta)
    return y


def kv_append(k_cache, v_cache, k, v, off, width) -> None:
    """In place on the two (contiguous float32) caches."""
    assert k_cache.dtype == np.float32 and k_cache.flags.c_contiguous
    assert v_cache.dtype == np.float32 and v_cache.flags.c_contiguous
    k, v = _f(k), _f(v)
    lib().orc_kv_append_f32(_pf(k_cache), _pf(v_cache), _pf(k), _pf(v), off, width)


def attn_causal(q, k_cache, v_cache, n_heads, n_kv, head_dim, seq, scale) -> np.ndarray:
    q, k_cache, v_cache = _f(q), _f(k_cache), _f(v_cache)
    out = np.empty(n_heads * head_dim, dtype=np.float32)
    lib().orc_attn_causal_f32(_pf(q), _pf(k_cache), _pf(v_cache), n_heads, n_kv, head_dim, seq,
                              scale, _pf(out))
    return out


def attn_decode_f32(q, k, v, n_heads, n_kv, head_dim, seq, scale) -> np.ndarray:
    q, k, v = _f(q), _f(k), _f(v)
    out = np.empty(n_heads * head_dim, dtype=np.float32)
    lib().orc_attn_decode_f32(_pf(q), _pf(k), _pf(v), n_heads, n_kv, head_dim, seq, scale,
                              _pf(out))
    return out


def attn_decode_kv(q, k, v, n_heads, n_kv, head_dim, seq, scale, dtype=Q8, stride=None):
    q, k, v = _f(q), _b(k), _b(v)
    stride = seq if stride is None else stride
    need = n_kv * stride * row_bytes(dtype, head_dim)
    assert k.size >= need and v.size >= need, "cache smaller than n_kv*stride*row_bytes"
    out = np.empty(n_heads * head_dim, dtype=np.float32)
    lib().orc_attn_decode_kv(_pf(q), _pb(k), _pb(v), n_heads, n_kv, head_dim, seq, stride, scale,
                             dtype, _pf(out))
    return out


def attn_core_token(q, k, v, gate, k_cache, v_cache, n_heads, n_kv, head_dim, n_rot, sections,
                    pos, theta):
    """rope -> append -> causal attention -> gate for one token (caches updated in place).
    Returns (out, q_roped, k_roped)."""
    q, k, v, gate = _f(q).copy(), _f(k).copy(), _f(v), _f(gate)
    n_ctx = k_cache.size // (n_kv * head_dim)
    out = np.empty(n_heads * head_dim, dtype=np.float32)
    lib().orc_attn_core_token_f32(_pf(q), _pf(k), _pf(v), _pf(gate), _pf(k_cache), _pf(v_cache),
                                  n_ctx, n_heads, n_kv, head_dim, n_rot, _sz4(sections), pos,
                                  theta, _pf(out))
    return out, q, k


def attn_chunk_kv(q, k, v, n_heads, n_kv, head_dim, pos0, tokens, stride, scale, dtype=Q8,
                  rows=None, n_threads=1) -> np.ndarray:
    q, k, v = _f(q), _b(k), _b(v)
    if rows is None:
        rp, n_rows = None, tokens
    else:
        rows = np.ascontiguousarray(rows, dtype=np.int32)
        rp, n_rows = rows.ctypes.data_as(_i32p), rows.size
    out = np.empty((n_rows, n_heads, head_dim), dtype=np.float32)
    lib().orc_attn_chunk_kv(_pf(q), _pb(k), _pb(v), n_heads, n_kv, head_dim, pos0, tokens, stride,
                            scale, dtype, rp, n_rows, n_threads, _pf(out))
    return out


# ---- Q8_0 weight matrices ---------------------------------------------------------

def dequant_q8_0(block) -> np.ndarray:
    block = _b(block)
    assert block.size == 34
    out = np.empty(32, dtype=np.float32)
    lib().orc_dequant_q8_0(_pb(block), _pf(out))
    return out


def gemv_q8_0(w, x, m, k) -> np.ndarray:
    w, x = _b(w), _f(x)
    assert w.size == m * (k // 32) * 34 and x.size == k
    y = np.empty(m, dtype=np.float32)
    lib().orc_gemv_q8_0(_pb(w), _pf(x), m, k, _pf(y))
    return y


def gemm_q8_0(w, x, tokens, m, k, n_threads=1) -> np.ndarray:
    """y[tokens][m]; n_threads > 1 spreads weight rows over OpenMP threads (each output is still the
    scalar in-order sum)."""
    w, x = _b(w), _f(x)
    assert w.size == m * (k // 32) * 34 and x.size == tokens * k
    y = np.empty((tokens, m), dtype=np.float32)
    lib().orc_gemm_q8_0(_pb(w), _pf(x), tokens, m, k, n_threads, _pf(y))
    return y


def random_q8_0_bytes(rng: "Rng", nblocks: int) -> np.ndarray:
    out = np.empty(nblocks * 34, dtype=np.uint8)
    lib().orc_random_q8_0_bytes(C.byref(rng._r), nblocks, _pb(out))
    return out


def compare(expected, actual, abs_tol, rel_tol):
    """(ok, max_abs, max_rel) with the reference's OR rule."""
    e, a = _f(expected).ravel(), _f(actual).ravel()
    assert e.size == a.size, "length mismatch"
    ma, mr = C.c_float(), C.c_float()
    ok = lib().orc_compare(_pf(e), _pf(a), e.size, abs_tol, rel_tol, C.byref(ma), C.byref(mr))
    return bool(ok), float(ma.value), float(mr.value)
