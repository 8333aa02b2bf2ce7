"""Host-side mirror of the reference's attention launchers over libhipml_attn.so.

Function names and argument order follow the reference's Rust launchers
(`launch_kv::launch_ptrs`, `launch_cols_ptrs`, `Launcher::kv_encode*`,
`attn_decode_batch`, `AttnLayer::chunk_attention_q8_split`, ...); tensors are
torch CUDA(HIP) tensors used purely as device memory.  Every call goes through
the C ABI declared in include/hipml_attn.h and raises :class:`HipmlError` with
the library's message on a non-zero return, like the reference's `Err(String)`.

There is no CPU fallback: if the shared library is missing this module raises.
"""
from __future__ import annotations

import ctypes as C
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
# HIPML_ATTN_LIB selects another build of the same library (e.g. an experimental variant).
LIB_PATH = os.environ.get("HIPML_ATTN_LIB") or os.path.join(_HERE, "libhipml_attn.so")

ROW_BYTES = 272      # one head_dim-256 row of q8_0: 8 blocks x 34 bytes
BLOCK_BYTES = 34
HEAD_DIM = 256

EXPORTS = [
    "hipml_attn_init", "hipml_attn_last_error", "hipml_attn_version",
    "hipml_attn_decode_splits", "hipml_attn_batch_splits", "hipml_attn_chunk_splits",
    "hipml_attn_chunk_slices",
    "hipml_rope_table_bytes", "hipml_rope_table_fill_host", "hipml_rope_set_table",
    "hipml_mrope_f32", "hipml_mrope_rows_f32", "hipml_rope_chunk_f32",
    "hipml_kv_encode", "hipml_kv_encode_bulk", "hipml_kv_encode_rows",
    "hipml_attn_decode_kv", "hipml_attn_decode_kv_cols", "hipml_attn_decode_rows",
    "hipml_attn_decode_batch", "hipml_attn_decode_batch_cols",
    "hipml_attn_decode_kv_gate", "hipml_attn_decode_batch_cols_gate",
    "hipml_attn_chunk_q8_split", "hipml_attn_chunk_q8_split_gate", "hipml_q_gate_f32",
    "hipml_attn_front_f32", "hipml_attn_chunk_front_f32",
    "hipml_gemv_q8_0_rows", "hipml_gemm_q8_0_f16", "hipml_attn_output_chunk_q8_0",
    "hipml_kv_rows_copy", "hipml_rope_encode_chunk_f32",
    "hipml_attn_front_encode_f32", "hipml_attn_chunk_front_encode_f32",
    "hipml_attn_chunk_q8_split_gate_f16", "hipml_attn_chunk_rope_q8",
    "hipml_kv_f16_bytes",
    "hipml_kv_f16_rows",
    "hipml_attn_chunk_kv_f16",
    "hipml_attn_front_rows_f32", "hipml_attn_front_rows_encode_f32",
    "hipml_attn_decode_kv_noalloc", "hipml_rope_allow_device_angles",
    "hipml_attn_decode_one_launch",
    "hipml_bench_stream_read", "hipml_bench_mfma_f16",
    "hipml_kv_f16_attach", "hipml_kv_f16_detach",
]


class HipmlError(RuntimeError):
    """A launcher refused its arguments or the HIP runtime refused the launch."""

    def __init__(self, code: int, message: str):
        super().__init__(f"{message} (status {code})")
        self.code = code
        self.message = message


_lib = None


def lib() -> C.CDLL:
    """Load libhipml_attn.so; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m hipml_amd.build` "
                "(there is no CPU fallback)")
        l = C.CDLL(LIB_PATH)
        vp, i, f, sz = C.c_void_p, C.c_int, C.c_float, C.c_size_t
        sig = {
            "hipml_attn_init": (i, [i]),
            "hipml_attn_last_error": (C.c_char_p, []),
            "hipml_attn_version": (C.c_char_p, []),
            "hipml_attn_decode_splits": (i, [i, i]),
            "hipml_attn_batch_splits": (i, [i, i, i]),
            "hipml_attn_chunk_splits": (i, [i, i, i]),
            "hipml_attn_chunk_slices": (i, [i, i, i]),
            "hipml_rope_table_bytes": (sz, [i, i]),
            "hipml_rope_table_fill_host": (i, [vp, f, i, i]),
            "hipml_rope_set_table": (i, [vp, f, i, i]),
            "hipml_mrope_f32": (i, [vp, vp, vp, i, i, i, i, i, i, i, vp, f]),
            "hipml_mrope_rows_f32": (i, [vp, vp, vp, i, i, i, i, i, i, i, vp, i, f]),
            "hipml_rope_chunk_f32": (i, [vp, vp, vp, i, i, i, i, f, i, i]),
            "hipml_kv_encode": (i, [vp, vp, i, vp, vp, vp, vp, i, i, i]),
            "hipml_kv_encode_bulk": (i, [vp, i, vp, vp, vp, vp, i, i, i, i, i, i]),
            "hipml_kv_encode_rows": (i, [vp, i, vp, vp, vp, vp, i, i, i, vp, sz, i]),
            "hipml_attn_decode_kv": (i, [vp, vp, i, vp, vp, vp, vp, vp, vp, i, i, i, i, f, i, sz,
                                         sz]),
            "hipml_attn_decode_kv_cols": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, i,
                                              i, sz, sz, sz]),
            "hipml_attn_decode_rows": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, i, sz,
                                           sz, sz, sz, i]),
            "hipml_attn_decode_batch": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, i,
                                            sz, sz, sz, sz, i, i]),
            "hipml_attn_decode_batch_cols": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f,
                                                 i, sz, sz, sz, sz, i, vp]),
            "hipml_attn_decode_kv_gate": (i, [vp, vp, i, vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, i,
                                              sz, sz]),
            "hipml_attn_decode_kv_noalloc": (i, [vp, vp, i, vp, vp, vp, vp, i, i, i, i, f, i, sz, sz]),
            "hipml_rope_allow_device_angles": (i, [i]),
            "hipml_attn_decode_one_launch": (i, [i]),
            "hipml_kv_f16_attach": (i, [vp, i, vp, vp, vp, i, i, i, i]),
            "hipml_kv_f16_detach": (i, [vp]),
            "hipml_bench_stream_read": (i, [vp, vp, vp, sz, i, vp]),
            "hipml_bench_mfma_f16": (i, [vp, i, i, vp, vp]),
            "hipml_attn_decode_batch_cols_gate": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, vp, i, i, i,
                                                      i, f, i, sz, sz, sz, sz, i, vp]),
            "hipml_attn_chunk_q8_split": (i, [vp, vp, vp, vp, vp, i, i, i, i, i, i, i, vp, vp, i]),
            "hipml_attn_chunk_q8_split_gate": (i, [vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, vp, vp, i]),
            "hipml_attn_chunk_q8_split_gate_f16": (i, [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, vp, vp, i]),
            # stream, q, kc, vc, gate, out, out16, n_head, n_kv, head_dim, n_rot, theta, pos0, tokens, dtype, stride, acc, ml, splits
            "hipml_attn_chunk_rope_q8": (i, [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, i, i, i, i, vp, vp, i]),
            "hipml_kv_f16_bytes": (sz, [i, i]),
            "hipml_kv_f16_rows": (i, [vp, i, vp, vp, vp, i, i, i, i, i]),
            "hipml_attn_chunk_kv_f16": (i, [vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, vp, vp, i]),
            "hipml_q_gate_f32": (i, [vp, vp, vp, vp, sz]),
            "hipml_attn_front_f32": (i, [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, i, i, i, i, vp, f, f]),
            "hipml_attn_chunk_front_f32": (i, [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, f, i, i]),
            "hipml_attn_front_encode_f32": (i, [vp, vp, i, vp, vp, vp, vp, vp, vp, vp, vp, vp,
                                                i, i, i, i, i, i, i, i, f, f, i]),
            "hipml_attn_chunk_front_encode_f32": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, vp, vp,
                                                      i, i, i, i, f, f, i, i, i]),
            "hipml_attn_front_rows_f32": (i, [vp, vp, vp, vp, vp, vp, vp, i, i, i, i, f, f, vp, i]),
            "hipml_attn_front_rows_encode_f32": (i, [vp, i, vp, vp, vp, vp, vp, vp, vp, vp, vp,
                                                     i, i, i, i, f, f, i, vp, sz, i]),
            "hipml_kv_rows_copy": (i, [vp, i, vp, vp, vp, vp, i, i, i, i, i]),
            "hipml_rope_encode_chunk_f32": (i, [vp, vp, vp, vp, vp, vp, i, i, i, i, f, i, i, i, i]),
            "hipml_gemv_q8_0_rows": (i, [vp, vp, vp, vp, i, i, i]),
            "hipml_gemm_q8_0_f16": (i, [vp, vp, vp, vp, i, i, i]),
            "hipml_attn_output_chunk_q8_0": (i, [vp, vp, vp, vp, vp, i, i, i, vp]),
        }
        for name, (res, args) in sig.items():
            fn = getattr(l, name)
            fn.restype = res
            fn.argtypes = args
        _lib = l
    return _lib


def _check(rc: int) -> None:
    if rc != 0:
        raise HipmlError(rc, lib().hipml_attn_last_error().decode())


def _p(t) -> int:
    """Device (or host) address of a tensor; None -> NULL."""
    return 0 if t is None else t.data_ptr()


def _stream(stream=None) -> int:
    s = stream if stream is not None else torch.cuda.current_stream()
    return s.cuda_stream


def init(device: int = 0) -> None:
    _check(lib().hipml_attn_init(device))


def version() -> str:
    return lib().hipml_attn_version().decode()


# ---- split policies ----------------------------------------------------------------

def decode_splits(seq: int, n_kv: int = 4) -> int:
    return lib().hipml_attn_decode_splits(seq, n_kv)


def batch_splits(stride: int, n_kv: int, slots: int) -> int:
    return lib().hipml_attn_batch_splits(stride, n_kv, slots)


def chunk_splits(pos0: int, tokens: int, n_kv: int = 4) -> int:
    """0 = keys cut inside the workgroups (no scratch), 1 = single pass, n >= 2 = n key slices with scratch."""
    return lib().hipml_attn_chunk_splits(pos0, tokens, n_kv)


def chunk_slices(pos0: int, tokens: int, n_kv: int = 4) -> int:
    """The slice count (>= 1) of the sliced kernel, also where `chunk_splits` prefers the other one."""
    return lib().hipml_attn_chunk_slices(pos0, tokens, n_kv)


# ---- RoPE ----------------------------------------------------------------------------

_rope_tables = {}


def rope_table(theta: float, n_rot: int, max_pos: int, device="cuda") -> torch.Tensor:
    """Build the host cos/sin table, upload it and register it with the library.
    The device tensor is kept alive here (the library does not own it)."""
    key = (float(theta), int(n_rot), int(max_pos), str(device))
    if key not in _rope_tables:
        host = torch.empty((max_pos, n_rot // 2, 2), dtype=torch.float32)
        _check(lib().hipml_rope_table_fill_host(host.data_ptr(), theta, n_rot, max_pos))
        _rope_tables[key] = host.to(device)
    tab = _rope_tables[key]
    _check(lib().hipml_rope_set_table(tab.data_ptr(), theta, n_rot, max_pos))
    return tab


def rope_clear_table() -> None:
    _check(lib().hipml_rope_set_table(0, 0.0, 0, 0))


def rope_allow_device_angles(allow: bool) -> None:
    """Opt in to (or out of) device-computed angles for positions outside the registered table."""
    _check(lib().hipml_rope_allow_device_angles(1 if allow else 0))


def mrope(x, y, n_heads, head_dim, n_rot, sections, pos, theta, stream=None):
    """`mrope_f32`: pos is a device int32[4]."""
    s0, s1, s2, s3 = sections
    _check(lib().hipml_mrope_f32(_stream(stream), _p(x), _p(y), n_heads, head_dim, n_rot, s0, s1,
                                 s2, s3, _p(pos), theta))


def mrope_rows(x, y, n_heads, head_dim, n_rot, sections, pos, rows, theta, stream=None):
    """`mrope_b`: pos is a device int32[rows][2] of (pos, seq)."""
    s0, s1, s2, s3 = sections
    _check(lib().hipml_mrope_rows_f32(_stream(stream), _p(x), _p(y), n_heads, head_dim, n_rot, s0,
                                      s1, s2, s3, _p(pos), rows, theta))


def rope_chunk(q, k, n_head, n_kv, head_dim, n_rot, theta, pos0, tokens, stream=None):
    _check(lib().hipml_rope_chunk_f32(_stream(stream), _p(q), _p(k), n_head, n_kv, head_dim, n_rot,
                                      theta, pos0, tokens))


# ---- attention front end ---------------------------------------------------------------

def attn_front(qg, q, gate, k, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, sections, pos, theta,
               eps, stream=None):
    """`AttnLayer::front`: q|gate split, head RMS norm of q and k, M-RoPE of both (one token);
    `pos` is the device int32[4] of M-RoPE position ids (step buffer + 4)."""
    s0, s1, s2, s3 = sections
    _check(lib().hipml_attn_front_f32(_stream(stream), _p(qg), _p(q), _p(gate), _p(k), _p(q_norm),
                                      _p(k_norm), n_heads, n_kv, head_dim, n_rot, s0, s1, s2, s3,
                                      _p(pos), theta, eps))


def chunk_front(qg, k, q, gate, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta, eps, pos0,
                tokens, stream=None):
    """`AttnLayer::chunk_front`: the same over `tokens` rows at text positions pos0.."""
    _check(lib().hipml_attn_chunk_front_f32(_stream(stream), _p(qg), _p(k), _p(q), _p(gate),
                                            _p(q_norm), _p(k_norm), n_heads, n_kv, head_dim, n_rot,
                                            theta, eps, pos0, tokens))


def attn_front_encode(step, dtype, qg, q, gate, k, v, q_norm, k_norm, k_cache, v_cache, n_heads, n_kv,
                      head_dim, n_rot, sections, theta, eps, stride, stream=None):
    """`attn_front` and `kv_encode` of the same token in one launch (same bits): the row goes to
    position step[0], the M-RoPE ids are step[4..7]."""
    s0, s1, s2, s3 = sections
    _check(lib().hipml_attn_front_encode_f32(_stream(stream), _p(step), dtype, _p(qg), _p(q), _p(gate),
                                             _p(k), _p(v), _p(q_norm), _p(k_norm), _p(k_cache),
                                             _p(v_cache), n_heads, n_kv, head_dim, n_rot, s0, s1, s2, s3,
                                             theta, eps, stride))


def chunk_front_encode(dtype, qg, k, v, q, gate, q_norm, k_norm, k_cache, v_cache, n_heads, n_kv,
                       head_dim, n_rot, theta, eps, pos0, tokens, stride, stream=None):
    """`chunk_front` and `kv_encode_bulk(start=pos0, src0=0, rows=tokens)` in one launch (same bits)."""
    _check(lib().hipml_attn_chunk_front_encode_f32(_stream(stream), dtype, _p(qg), _p(k), _p(v), _p(q),
                                                   _p(gate), _p(q_norm), _p(k_norm), _p(k_cache),
                                                   _p(v_cache), n_heads, n_kv, head_dim, n_rot, theta,
                                                   eps, pos0, tokens, stride))


def front_rows(qg, k, q, gate, q_norm, k_norm, n_heads, n_kv, head_dim, n_rot, theta, eps, pos, rows,
               stream=None):
    """`AttnLayer::split_rope_rows`: the front end over one row per sequence, row r at text position
    pos[r][0] (`pos` = device int32 [rows][2])."""
    _check(lib().hipml_attn_front_rows_f32(_stream(stream), _p(qg), _p(k), _p(q), _p(gate), _p(q_norm),
                                           _p(k_norm), n_heads, n_kv, head_dim, n_rot, theta, eps,
                                           _p(pos), rows))


def front_rows_encode(dtype, qg, k, v, q, gate, q_norm, k_norm, k_cache, v_cache, n_heads, n_kv, head_dim,
                      n_rot, theta, eps, stride, pos, slot_bytes, slots, stream=None):
    """`front_rows` and `kv_encode_rows` of the same step in one launch (same bits)."""
    _check(lib().hipml_attn_front_rows_encode_f32(_stream(stream), dtype, _p(qg), _p(k), _p(v), _p(q),
                                                  _p(gate), _p(q_norm), _p(k_norm), _p(k_cache),
                                                  _p(v_cache), n_heads, n_kv, head_dim, n_rot, theta, eps,
                                                  stride, _p(pos), slot_bytes, slots))


# ---- KV append ------------------------------------------------------------------------

def kv_encode(step, dtype, k_in, v_in, k_cache, v_cache, n_kv, head_dim, stride, stream=None):
    _check(lib().hipml_kv_encode(_stream(stream), _p(step), dtype, _p(k_in), _p(v_in), _p(k_cache),
                                 _p(v_cache), n_kv, head_dim, stride))


def kv_encode_bulk(dtype, k_f32, v_f32, k_cache, v_cache, n_kv, head_dim, stride, start, src0,
                   rows, stream=None):
    _check(lib().hipml_kv_encode_bulk(_stream(stream), dtype, _p(k_f32), _p(v_f32), _p(k_cache),
                                      _p(v_cache), n_kv, head_dim, stride, start, src0, rows))


def kv_encode_rows(dtype, k_f32, v_f32, k_cache, v_cache, n_kv, head_dim, stride, pos, slot_bytes,
                   slots, stream=None):
    _check(lib().hipml_kv_encode_rows(_stream(stream), dtype, _p(k_f32), _p(v_f32), _p(k_cache),
                                      _p(v_cache), n_kv, head_dim, stride, _p(pos), slot_bytes,
                                      slots))


def rope_encode_chunk(q, k, v, k_cache, v_cache, n_head, n_kv, head_dim, n_rot, theta, pos0, tokens,
                      dtype, stride, stream=None):
    """`rope_chunk` + `kv_encode_bulk(start=pos0, src0=0, rows=tokens)` in one launch."""
    _check(lib().hipml_rope_encode_chunk_f32(_stream(stream), _p(q), _p(k), _p(v), _p(k_cache),
                                             _p(v_cache), n_head, n_kv, head_dim, n_rot, theta, pos0,
                                             tokens, dtype, stride))


def kv_rows_copy(dtype, k_src, v_src, k_dst, v_dst, n_kv, head_dim, src_stride, dst_stride, rows,
                 stream=None):
    """Prefix snapshot / restore of cache rows (`GpuEngine::prefix_capture` / `prefix_restore`)."""
    _check(lib().hipml_kv_rows_copy(_stream(stream), dtype, _p(k_src), _p(v_src), _p(k_dst), _p(v_dst),
                                    n_kv, head_dim, src_stride, dst_stride, rows))


# ---- decode -------------------------------------------------------------------------------

def attn_decode_kv(step, dtype, q, k, v, part_acc, part_ml, out, n_heads, n_kv, head_dim, stride,
                   scale, splits, k_off=0, v_off=0, stream=None):
    """`launch_kv::launch_ptrs`."""
    _check(lib().hipml_attn_decode_kv(_stream(stream), _p(step), dtype, _p(q), _p(k), _p(v),
                                      _p(part_acc), _p(part_ml), _p(out), n_heads, n_kv, head_dim,
                                      stride, scale, splits, k_off, v_off))


def attn_decode_kv_cols(dtype, pos, q, k, v, part_acc, part_ml, out, n_heads, n_kv, head_dim,
                        stride, scale, splits, cols, acc_slot, ml_slot, q_slot, stream=None):
    """`launch_kv::launch_cols_ptrs`."""
    _check(lib().hipml_attn_decode_kv_cols(_stream(stream), dtype, _p(pos), _p(q), _p(k), _p(v),
                                           _p(part_acc), _p(part_ml), _p(out), n_heads, n_kv,
                                           head_dim, stride, scale, splits, cols, acc_slot,
                                           ml_slot, q_slot))


def attn_decode_rows(dtype, pos, q, k_cache, v_cache, part_acc, part_ml, out, n_heads, n_kv,
                     head_dim, stride, scale, splits, kv_slot_bytes, acc_slot, ml_slot, q_slot,
                     slots, stream=None):
    """`Launcher::attn_decode_rows_ptr`."""
    _check(lib().hipml_attn_decode_rows(_stream(stream), dtype, _p(pos), _p(q), _p(k_cache),
                                        _p(v_cache), _p(part_acc), _p(part_ml), _p(out), n_heads,
                                        n_kv, head_dim, stride, scale, splits, kv_slot_bytes,
                                        acc_slot, ml_slot, q_slot, slots))


def attn_decode_batch(dtype, pos, q, k_cache, v_cache, part_acc, part_ml, out, n_heads, n_kv,
                      head_dim, stride, scale, splits, kv_slot_bytes, acc_slot, ml_slot, q_slot,
                      slots, live_seq=0, stream=None):
    """`Launcher::attn_decode_batch`."""
    _check(lib().hipml_attn_decode_batch(_stream(stream), dtype, _p(pos), _p(q), _p(k_cache),
                                         _p(v_cache), _p(part_acc), _p(part_ml), _p(out), n_heads,
                                         n_kv, head_dim, stride, scale, splits, kv_slot_bytes,
                                         acc_slot, ml_slot, q_slot, slots, live_seq))


def attn_decode_batch_cols(dtype, pos, q, k_cache, v_cache, part_acc, part_ml, out, n_heads, n_kv,
                           head_dim, stride, scale, splits, kv_slot_bytes, acc_slot, ml_slot,
                           q_slot, cols_per_slot, stream=None):
    """Plain and MTP-verify slots in one launch; cols_per_slot is a host sequence."""
    arr = (C.c_int32 * len(cols_per_slot))(*[int(c) for c in cols_per_slot])
    _check(lib().hipml_attn_decode_batch_cols(
        _stream(stream), dtype, _p(pos), _p(q), _p(k_cache), _p(v_cache), _p(part_acc),
        _p(part_ml), _p(out), n_heads, n_kv, head_dim, stride, scale, splits, kv_slot_bytes,
        acc_slot, ml_slot, q_slot, len(cols_per_slot), C.addressof(arr)))


def attn_decode_kv_gate(step, dtype, q, k, v, part_acc, part_ml, out, gate, n_heads, n_kv, head_dim,
                        stride, scale, splits, k_off=0, v_off=0, stream=None):
    """`launch_kv::launch_ptrs` followed by `AttnLayer::q_gate_only`, in the merge kernel."""
    _check(lib().hipml_attn_decode_kv_gate(_stream(stream), _p(step), dtype, _p(q), _p(k), _p(v),
                                           _p(part_acc), _p(part_ml), _p(out), _p(gate), n_heads,
                                           n_kv, head_dim, stride, scale, splits, k_off, v_off))


def attn_decode_kv_noalloc(step, dtype, q, k, v, out, n_heads, n_kv, head_dim, stride, scale, splits,
                           k_off=0, v_off=0, stream=None):
    """`attn_decode_kv` with the split partials in the library's built-in array: allocates nothing,
    n_heads * splits <= 4096, calls on one GPU must not overlap."""
    _check(lib().hipml_attn_decode_kv_noalloc(_stream(stream), _p(step), dtype, _p(q), _p(k), _p(v),
                                              _p(out), n_heads, n_kv, head_dim, stride, scale, splits,
                                              k_off, v_off))


def kv_f16_attach(dtype, k_cache, v_cache, kv_f16, n_kv, head_dim, stride, rows=0, stream=None):
    """Register kv_f16 as the f16 shadow of (k_cache, v_cache): the library keeps it current through its own
    append entry points and the chunk attention over the cache reads it.  Detach before freeing either."""
    _check(lib().hipml_kv_f16_attach(_stream(stream), dtype, _p(k_cache), _p(v_cache), _p(kv_f16), n_kv, head_dim,
                                     stride, rows))


def kv_f16_detach(k_cache):
    _check(lib().hipml_kv_f16_detach(_p(k_cache)))


def bench_stream_read(a, b, bytes_each, mode, sink, stream=None):
    """Measurement only: one launch that reads `bytes_each` bytes of each of a and b in the decode kernel's pattern."""
    _check(lib().hipml_bench_stream_read(_stream(stream), _p(a), _p(b), bytes_each, mode, _p(sink)))


def bench_mfma_f16(workgroups, iters, sink, clocks=None, stream=None):
    """Measurement only: workgroups x 4 waves x iters x 8 independent 32x32x16 f16 MFMAs."""
    _check(lib().hipml_bench_mfma_f16(_stream(stream), workgroups, iters, _p(sink), _p(clocks)))


def decode_one_launch(on: int = -1) -> int:
    """Process-wide: 1 = a single sequence over q8_0 merges its key splits inside the one launch, 0 (the
    default) = in a second launch; a negative value only reads the mode.  Returns the mode before the call."""
    return int(lib().hipml_attn_decode_one_launch(int(on)))


def attn_decode_batch_cols_gate(dtype, pos, q, k_cache, v_cache, part_acc, part_ml, out, gate,
                                n_heads, n_kv, head_dim, stride, scale, splits, kv_slot_bytes,
                                acc_slot, ml_slot, q_slot, cols_per_slot, stream=None):
    """`attn_decode_batch_cols` with the gate half of `output_rows` applied in the merge kernel."""
    arr = (C.c_int32 * len(cols_per_slot))(*[int(c) for c in cols_per_slot])
    _check(lib().hipml_attn_decode_batch_cols_gate(
        _stream(stream), dtype, _p(pos), _p(q), _p(k_cache), _p(v_cache), _p(part_acc),
        _p(part_ml), _p(out), _p(gate), n_heads, n_kv, head_dim, stride, scale, splits,
        kv_slot_bytes, acc_slot, ml_slot, q_slot, len(cols_per_slot), C.addressof(arr)))


# ---- chunk prefill ---------------------------------------------------------------------------

def chunk_attention_q8_split(q, kc, vc, out, n_head, n_kv, head_dim, pos0, tokens, dtype, stride,
                             part_acc, part_ml, splits, stream=None):
    """`AttnLayer::chunk_attention_q8_split` (dtype 1 = q8_0)."""
    _check(lib().hipml_attn_chunk_q8_split(_stream(stream), _p(q), _p(kc), _p(vc), _p(out), n_head,
                                           n_kv, head_dim, pos0, tokens, dtype, stride,
                                           _p(part_acc), _p(part_ml), splits))


def chunk_attention_q8_split_gate(q, kc, vc, gate, out, n_head, n_kv, head_dim, pos0, tokens, dtype,
                                  stride, part_acc, part_ml, splits, stream=None):
    """`chunk_attention_q8_split` followed by `q_gate_only`, as one call (same bits)."""
    _check(lib().hipml_attn_chunk_q8_split_gate(_stream(stream), _p(q), _p(kc), _p(vc), _p(gate),
                                                _p(out), n_head, n_kv, head_dim, pos0, tokens, dtype,
                                                stride, _p(part_acc), _p(part_ml), splits))


def chunk_attention_q8_split_gate_f16(q, kc, vc, gate, out, out16, n_head, n_kv, head_dim, pos0, tokens,
                                      dtype, stride, part_acc, part_ml, splits, stream=None):
    """The gated chunk attention with its rows delivered as f16 in `out16` (what the output projection
    reads); `out` is working memory."""
    _check(lib().hipml_attn_chunk_q8_split_gate_f16(_stream(stream), _p(q), _p(kc), _p(vc), _p(gate),
                                                    _p(out), _p(out16), n_head, n_kv, head_dim, pos0,
                                                    tokens, dtype, stride, _p(part_acc), _p(part_ml),
                                                    splits))


def chunk_attention_rope_q8(q, kc, vc, gate, out, out16, n_head, n_kv, head_dim, n_rot, theta, pos0, tokens,
                            dtype, stride, part_acc, part_ml, splits, stream=None):
    """RoPE of the (unrotated) query rows and the chunk attention in one call; gate and out16 may be None.
    splits == 0: rotated inside the attention kernel, q untouched; otherwise q is rotated in place first."""
    _check(lib().hipml_attn_chunk_rope_q8(_stream(stream), _p(q), _p(kc), _p(vc), _p(gate), _p(out), _p(out16),
                                          n_head, n_kv, head_dim, n_rot, theta, pos0, tokens, dtype, stride,
                                          _p(part_acc), _p(part_ml), splits))


def kv_f16_bytes(stride: int, n_kv: int) -> int:
    """Bytes of the f16 copy of a layer cache of `stride` rows per KV head."""
    return int(lib().hipml_kv_f16_bytes(stride, n_kv))


def kv_f16_alloc(stride: int, n_kv: int, device="cuda"):
    return torch.empty(kv_f16_bytes(stride, n_kv), dtype=torch.uint8, device=device)


def kv_f16_rows(dtype, k_cache, v_cache, kv_f16, n_kv, head_dim, stride, start, rows, stream=None):
    """Bring the tiles of the f16 copy that hold cache rows [start, start + rows) up to date."""
    _check(lib().hipml_kv_f16_rows(_stream(stream), dtype, _p(k_cache), _p(v_cache), _p(kv_f16), n_kv,
                                   head_dim, stride, start, rows))


def chunk_attention_kv_f16(q, kv_f16, gate, out, out16, n_head, n_kv, head_dim, pos0, tokens, stride,
                           part_acc, part_ml, splits, stream=None):
    """Chunk attention over the f16 copy of the cache; gate and out16 may be None."""
    _check(lib().hipml_attn_chunk_kv_f16(_stream(stream), _p(q), _p(kv_f16), _p(gate), _p(out), _p(out16),
                                         n_head, n_kv, head_dim, pos0, tokens, stride, _p(part_acc),
                                         _p(part_ml), splits))


def chunk_scratch(tokens: int, n_head: int, splits: int, device="cuda"):
    """Split-K scratch sized as the reference's prefill path sizes it."""
    qslots = (tokens + 31) // 32 * 32
    acc = torch.empty((splits, qslots, n_head, HEAD_DIM), dtype=torch.float32, device=device)
    ml = torch.empty((splits, qslots, n_head, 2), dtype=torch.float32, device=device)
    return acc, ml


# ---- gate -----------------------------------------------------------------------------------------

def q_gate(x, gate, y, n=None, stream=None):
    n = x.numel() if n is None else n
    _check(lib().hipml_q_gate_f32(_stream(stream), _p(x), _p(gate), _p(y), n))


# ---- projections over Q8_0 weights ------------------------------------------------------------------

def gemv_q8_0_rows(w, x, y, m, k, rows, stream=None):
    """`AttnLayer::gemv` / `gemv_rows` / `gemv_batched` over a Q8_0 weight matrix: y[rows][m]."""
    _check(lib().hipml_gemv_q8_0_rows(_stream(stream), _p(w), _p(x), _p(y), m, k, rows))


def gemm_q8_0_f16(w, x, y, m, k, tokens, stream=None):
    """`AttnLayer::apply_output_chunk`'s tiled GEMM (after the gate) over a Q8_0 weight matrix:
    y[tokens][m], f16 operands."""
    _check(lib().hipml_gemm_q8_0_f16(_stream(stream), _p(w), _p(x), _p(y), m, k, tokens))


def output_chunk_q8_0(wo, attn_out, gate, y, m, k, tokens, x16, stream=None):
    """`AttnLayer::apply_output_chunk`: y = W_o (attn_out * sigmoid(gate)); gate may be None; x16 is
    scratch of tokens*k f16.  attn_out None: x16 already holds the rows as f16."""
    _check(lib().hipml_attn_output_chunk_q8_0(_stream(stream), _p(wo), _p(attn_out),
                                              _p(gate) if gate is not None else None, _p(y), m, k,
                                              tokens, _p(x16)))


# ---- cache owner ------------------------------------------------------------------------------------

class DeepKv:
    """One layer's quantized cache plus its decode scratch: the role of the reference's
    `DeepKv` (crates/hipml-model/src/gpu/deep_kv.rs:11-83).  K and V are separate
    uint8 tensors of [n_kv][stride][row bytes]: 272 for q8_0 (dtype 0), 144 for q4_0 (dtype 1)."""

    def __init__(self, n_heads=24, n_kv=4, head_dim=HEAD_DIM, stride=4096, max_cols=1,
                 device="cuda", dtype=0):
        assert head_dim == HEAD_DIM
        assert dtype in (0, 1), "KvDtype id: 0 = q8_0, 1 = q4_0"
        self.dtype = dtype
        self.row_bytes = ROW_BYTES if dtype == 0 else head_dim // 32 * 18
        self.n_heads, self.n_kv, self.head_dim, self.seq = n_heads, n_kv, head_dim, stride
        self.k = torch.zeros((n_kv, stride, self.row_bytes), dtype=torch.uint8, device=device)
        self.v = torch.zeros((n_kv, stride, self.row_bytes), dtype=torch.uint8, device=device)
        self.max_splits = max(decode_splits(stride, n_kv), 1)
        self.max_cols = max_cols
        self.part_acc = torch.empty((max_cols, n_heads, self.max_splits, head_dim),
                                    dtype=torch.float32, device=device)
        self.part_ml = torch.empty((max_cols, n_heads, self.max_splits, 2), dtype=torch.float32,
                                   device=device)
        self.f16 = None  # the optional f16 copy of the rows (enable_f16_copy, attach_f16)
        self._attached = False

    def enable_f16_copy(self, live: int = 0, stream=None):
        """Keep an f16 copy of this cache for chunk prefill over long prefixes (chunk_attention_kv_f16
        reads it); `live` rows are converted now, later appends are followed by sync_f16."""
        if self.f16 is None:
            self.f16 = kv_f16_alloc(self.seq, self.n_kv, self.k.device)
        self.sync_f16(0, live, stream)

    def attach_f16(self, live: int = 0, stream=None):
        """Hand the f16 copy to the library (hipml_kv_f16_attach): appends through the library keep it current
        and `chunk_attention_q8_split*` over this cache reads it; no sync_f16 calls are needed."""
        if self.f16 is None:
            self.f16 = kv_f16_alloc(self.seq, self.n_kv, self.k.device)
        kv_f16_attach(self.dtype, self.k, self.v, self.f16, self.n_kv, self.head_dim, self.seq, live, stream)
        self._attached = True

    def detach_f16(self):
        if self._attached:
            self._attached = False
            kv_f16_detach(self.k)

    def __del__(self):
        try:
            self.detach_f16()
        except Exception:  # (interpreter shutdown: the library may be gone)
            pass

    def sync_f16(self, start: int, rows: int, stream=None):
        """After rows [start, start + rows) were appended (or restored): bring the copy up to date."""
        if self.f16 is not None and rows > 0:
            kv_f16_rows(self.dtype, self.k, self.v, self.f16, self.n_kv, self.head_dim, self.seq, start, rows,
                        stream)

    def splits(self, seq: int) -> int:
        return min(decode_splits(seq, self.n_kv), self.max_splits)

    def bytes(self) -> int:
        return 2 * self.n_kv * self.seq * self.row_bytes

    def snapshot(self, pos: int, stream=None):
        """Rows [0, pos) of every head, packed [n_kv][pos][row bytes] (K, V): the quantized half of a
        prefix snapshot (crates/hipml-model/src/gpu/prefix.rs:214-239)."""
        k = torch.empty((self.n_kv, pos, self.row_bytes), dtype=torch.uint8, device=self.k.device)
        v = torch.empty_like(k)
        if pos > 0:
            kv_rows_copy(self.dtype, self.k, self.v, k, v, self.n_kv, self.head_dim, self.seq, pos, pos,
                         stream)
        return k, v

    def restore(self, k, v, stream=None):
        """Write a packed snapshot back as rows [0, pos) of this cache; rows past pos keep their bytes
        (they are never read: the live length says so)."""
        pos = k.shape[1]
        assert pos <= self.seq and k.shape == v.shape == (self.n_kv, pos, self.row_bytes)
        if pos > 0:
            kv_rows_copy(self.dtype, k, v, self.k, self.v, self.n_kv, self.head_dim, pos, self.seq, pos,
                         stream)
            self.sync_f16(0, pos, stream)


class BatchKv:
    """One layer's quantized caches of `slots` sequences plus the batched decode scratch: the role of
    the reference's `BatchKv` (crates/hipml-model/src/gpu/batch/kv.rs:11-75).  The caches are
    contiguous across slots -- slot b starts `b * slot_bytes` into K (and V), each slot laid out
    [n_kv][stride][row bytes] -- so the batched append and attention address a slot by its index."""

    def __init__(self, slots, n_heads=24, n_kv=4, head_dim=HEAD_DIM, stride=4096, max_rows=None,
                 device="cuda", dtype=0):
        assert head_dim == HEAD_DIM
        assert dtype in (0, 1), "KvDtype id: 0 = q8_0, 1 = q4_0"
        self.dtype, self.slots = dtype, slots
        self.row_bytes = ROW_BYTES if dtype == 0 else head_dim // 32 * 18
        self.n_heads, self.n_kv, self.head_dim, self.seq = n_heads, n_kv, head_dim, stride
        self.slot_bytes = n_kv * stride * self.row_bytes
        self.k = torch.zeros((slots, n_kv, stride, self.row_bytes), dtype=torch.uint8, device=device)
        self.v = torch.zeros_like(self.k)
        self.splits = batch_splits(stride, n_kv, slots)
        # one scratch slot per query row: a verify group brings several rows per sequence
        self.max_rows = max_rows or slots
        self.acc_slot = n_heads * self.splits * head_dim
        self.ml_slot = n_heads * self.splits * 2
        self.part_acc = torch.empty((self.max_rows, self.acc_slot), dtype=torch.float32, device=device)
        self.part_ml = torch.empty((self.max_rows, self.ml_slot), dtype=torch.float32, device=device)

    def bytes(self) -> int:
        return 2 * self.slots * self.slot_bytes

    def append(self, k_f32, v_f32, pos, rows, stream=None):
        """Quantize and append one K/V row per entry of `pos` (device int32 [rows][2] = (position,
        live length), row i belonging to slot i): `Launcher::kv_encode_rows_ptr`."""
        kv_encode_rows(self.dtype, k_f32, v_f32, self.k, self.v, self.n_kv, self.head_dim, self.seq, pos,
                       self.slot_bytes, rows, stream)

    def front_append(self, qg, k, v, q, gate, q_norm, k_norm, n_rot, theta, eps, pos, stream=None):
        """The step in front of `decode`: q|gate split, head norms and RoPE of one row per slot at its
        own position, and the append of its K/V row, in one launch."""
        front_rows_encode(self.dtype, qg, k, v, q, gate, q_norm, k_norm, self.k, self.v, self.n_heads,
                          self.n_kv, self.head_dim, n_rot, theta, eps, self.seq, pos, self.slot_bytes,
                          self.slots, stream)

    def decode(self, pos, q, out, scale, cols_per_slot=None, gate=None, stream=None):
        """Batched decode over every slot: one query row per slot (`Launcher::attn_decode_batch`), or
        `cols_per_slot[b]` rows for slot b -- verify groups beside plain slots in one launch -- with
        the output gate applied in the merge when `gate` is given.  `pos` is device int32 [rows][2]."""
        q_slot = self.n_heads * self.head_dim
        if cols_per_slot is None and gate is None:
            attn_decode_batch(self.dtype, pos, q, self.k, self.v, self.part_acc, self.part_ml, out,
                              self.n_heads, self.n_kv, self.head_dim, self.seq, scale, self.splits,
                              self.slot_bytes, self.acc_slot, self.ml_slot, q_slot, self.slots, 0, stream)
            return
        cols = list(cols_per_slot) if cols_per_slot is not None else [1] * self.slots
        assert len(cols) == self.slots and sum(cols) <= self.max_rows
        if gate is None:
            attn_decode_batch_cols(self.dtype, pos, q, self.k, self.v, self.part_acc, self.part_ml, out,
                                   self.n_heads, self.n_kv, self.head_dim, self.seq, scale, self.splits,
                                   self.slot_bytes, self.acc_slot, self.ml_slot, q_slot, cols, stream)
        else:
            attn_decode_batch_cols_gate(self.dtype, pos, q, self.k, self.v, self.part_acc, self.part_ml,
                                        out, gate, self.n_heads, self.n_kv, self.head_dim, self.seq, scale,
                                        self.splits, self.slot_bytes, self.acc_slot, self.ml_slot, q_slot,
                                        cols, stream)
