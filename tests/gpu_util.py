"""Shared helpers for the GPU parity tests: seeded inputs from the oracle's RNG,
cache construction, comparison with the reference's OR rule."""
import numpy as np
import torch

from oracle import binding as orc
from hipml_amd import attn

N_HEADS, N_KV, HD, N_ROT, THETA = 24, 4, 256, 64, 1e7
SECTIONS = (11, 11, 10, 0)
SCALE = 0.0625
ROW = 272


def dev(a, dtype=None):
    t = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()


def host(t):
    return t.detach().cpu().numpy()


def quantized_cache(kf, vf, stride=None):
    """kf, vf: float32 [n_kv][seq][hd] -> uint8 [n_kv][stride][272] (padding rows = 0xA5 junk)."""
    n_kv, seq, hd = kf.shape
    stride = seq if stride is None else stride
    kb = np.full((n_kv, stride, ROW), 0xA5, dtype=np.uint8)
    vb = np.full((n_kv, stride, ROW), 0x5A, dtype=np.uint8)
    kb[:, :seq] = orc.quantize(0, kf).reshape(n_kv, seq, ROW)
    vb[:, :seq] = orc.quantize(0, vf).reshape(n_kv, seq, ROW)
    return kb, vb


def decode_scratch(n_heads, splits, rows=1):
    acc = torch.full((rows, n_heads, splits, HD), float("nan"), dtype=torch.float32, device="cuda")
    ml = torch.full((rows, n_heads, splits, 2), float("nan"), dtype=torch.float32, device="cuda")
    return acc, ml


def step_buffer(pos, seq):
    return torch.tensor([pos, seq, 0, 0, pos, pos, pos, pos], dtype=torch.int32, device="cuda")


def run_decode(q, kb, vb, n_heads, n_kv, seq, stride, scale, splits):
    acc, ml = decode_scratch(n_heads, splits)
    out = torch.full((n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv(step_buffer(seq - 1, seq), 0, dev(q), dev(kb), dev(vb), acc, ml, out,
                        n_heads, n_kv, HD, stride, scale, splits)
    torch.cuda.synchronize()
    return host(out).ravel()


def report(name, want, got, abs_tol, rel_tol):
    ok, ma, mr = orc.compare(want, got, abs_tol, rel_tol)
    print(f"[parity] {name}: max_abs {ma:.3e} max_rel {mr:.3e} (tol {abs_tol:g}/{rel_tol:g})",
          flush=True)
    return ok, ma, mr
