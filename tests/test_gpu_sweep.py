"""Seeded sweeps over geometry: head groupings other than the model's, ragged depths and strides,
every split count, both cache formats, chunk shapes around the tile edges, projection shapes around
the row and k tiles -- each case against the oracle on the same inputs.  The cases are drawn from
the oracle's own generator, so the sweep is the same on every run."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import HD, SCALE, dev, host  # noqa: E402

KERNEL_CLASS = (1e-3, 5e-3)   # decode over q8_0 (see test_gpu_decode.py)
Q4_CLASS = (2e-3, 1e-2)       # the parity gate; q4_0 decode sits well inside it
CHUNK_GATE = (2e-3, 1e-2)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def draw(r, lo, hi):
    return lo + int(float(r.uniform()) * (hi - lo + 1)) % (hi - lo + 1)


def decode_cases(n):
    r = orc.Rng(0x5EE9_0001)
    cases = []
    for i in range(n):
        n_kv = (1, 2, 4)[draw(r, 0, 2)]
        group = draw(r, 1, 8)
        cols = draw(r, 1, 4)
        pos0 = draw(r, 0, 2600) if i % 5 else draw(r, 0, 40)
        stride = pos0 + cols + draw(r, 0, 300)
        splits = draw(r, 1, 48)
        cases.append((i, n_kv, group, cols, pos0, stride, splits, i % 3 == 2))
    return cases


@pytest.mark.parametrize("i,n_kv,group,cols,pos0,stride,splits,q4", decode_cases(36))
def test_decode_sweep(i, n_kv, group, cols, pos0, stride, splits, q4):
    n_heads = n_kv * group
    dtype = 1 if q4 else 0
    row = 144 if q4 else 272
    r = orc.Rng(0xD5EE_0000 + i)
    live = pos0 + cols
    q = r.normal_array((cols, n_heads, HD))
    kf = r.normal_array((n_kv, live, HD))
    vf = r.normal_array((n_kv, live, HD))
    kb = np.full((n_kv, stride, row), 0xA5, dtype=np.uint8)
    vb = np.full((n_kv, stride, row), 0x5A, dtype=np.uint8)
    kb[:, :live] = orc.quantize(dtype, kf).reshape(n_kv, live, row)
    vb[:, :live] = orc.quantize(dtype, vf).reshape(n_kv, live, row)
    acc = torch.full((cols, n_heads, splits, HD), float("nan"), device="cuda")
    ml = torch.full((cols, n_heads, splits, 2), float("nan"), device="cuda")
    out = torch.full((cols, n_heads, HD), float("nan"), device="cuda")
    pos = torch.tensor([[pos0 + c, pos0 + c + 1] for c in range(cols)], dtype=torch.int32, device="cuda")
    attn.attn_decode_kv_cols(dtype, pos, dev(q), dev(kb), dev(vb), acc, ml, out, n_heads, n_kv, HD, stride,
                             SCALE, splits, cols, n_heads * splits * HD, n_heads * splits * 2, n_heads * HD)
    torch.cuda.synchronize()
    got = host(out)
    for c in range(cols):
        want = orc.attn_decode_kv(q[c], kb, vb, n_heads, n_kv, HD, pos0 + c + 1, SCALE, stride=stride,
                                  dtype=dtype)
        ok, ma, mr = orc.compare(want, got[c].ravel(), *(Q4_CLASS if q4 else KERNEL_CLASS))
        assert ok, f"case {i}: kv {n_kv} group {group} col {c}/{cols} pos0 {pos0} stride {stride} " \
                   f"splits {splits} q4 {q4}: max_abs {ma:.3e} max_rel {mr:.3e}"


def chunk_cases(n):
    r = orc.Rng(0x5EE9_0002)
    cases = []
    for i in range(n):
        n_kv = (1, 2, 4)[draw(r, 0, 2)]
        group = (1, 2, 3, 6, 8)[draw(r, 0, 4)]
        tok = (1, 31, 32, 33, 63, 64, 65, 100, 129)[draw(r, 0, 8)]
        pos0 = (0, 1, 31, 63, 64, 200, 777)[draw(r, 0, 6)]
        pad = draw(r, 0, 40)
        splits = (1, 2, 3, 5, 8)[draw(r, 0, 4)]
        cases.append((i, n_kv, group, tok, pos0, pad, splits, i % 4 == 3))
    return cases


@pytest.mark.parametrize("i,n_kv,group,tok,pos0,pad,splits,q4", chunk_cases(24))
def test_chunk_sweep(i, n_kv, group, tok, pos0, pad, splits, q4):
    n_heads = n_kv * group
    dtype = 1 if q4 else 0
    row = 144 if q4 else 272
    stride = pos0 + tok + pad
    r = orc.Rng(0xC5EE_0000 + i)
    q = r.normal_array((tok, n_heads, HD))
    k = r.normal_array((stride, n_kv, HD))
    v = r.normal_array((stride, n_kv, HD))
    kb = orc.quantize(dtype, k.transpose(1, 0, 2)).reshape(n_kv, stride, row)
    vb = orc.quantize(dtype, v.transpose(1, 0, 2)).reshape(n_kv, stride, row)
    out = torch.full((tok, n_heads, HD), float("nan"), device="cuda")
    acc = ml = None
    if splits >= 2:
        acc, ml = attn.chunk_scratch(tok, n_heads, splits)
        acc.fill_(float("nan"))
        ml.fill_(float("nan"))
    attn.chunk_attention_q8_split(dev(q), dev(kb), dev(vb), out, n_heads, n_kv, HD, pos0, tok, 1 + dtype,
                                  stride, acc, ml, splits)
    torch.cuda.synchronize()
    want = orc.attn_chunk_kv(q, kb, vb, n_heads, n_kv, HD, pos0, tok, stride, SCALE, dtype=dtype, n_threads=8)
    ok, ma, mr = orc.compare(want, host(out), *CHUNK_GATE)
    assert ok, f"case {i}: kv {n_kv} group {group} tok {tok} pos0 {pos0} pad {pad} splits {splits} q4 {q4}: " \
               f"max_abs {ma:.3e} max_rel {mr:.3e}"
    # the same chunk over the f16 copy of the cache, brought up to date in two calls
    copy = attn.kv_f16_alloc(stride, n_kv)
    copy.fill_(0xFF)
    first = (pos0 + tok) // 2
    attn.kv_f16_rows(dtype, dev(kb), dev(vb), copy, n_kv, HD, stride, 0, first)
    attn.kv_f16_rows(dtype, dev(kb), dev(vb), copy, n_kv, HD, stride, first, pos0 + tok - first)
    out.fill_(float("nan"))
    if splits >= 2:
        acc.fill_(float("nan"))
        ml.fill_(float("nan"))
    attn.chunk_attention_kv_f16(dev(q), copy, None, out, None, n_heads, n_kv, HD, pos0, tok, stride, acc, ml, splits)
    torch.cuda.synchronize()
    ok, ma, mr = orc.compare(want, host(out), *CHUNK_GATE)
    assert ok, f"case {i} over the f16 copy: max_abs {ma:.3e} max_rel {mr:.3e}"
    # and with the keys cut inside the workgroups (splits = 0: no scratch)
    out.fill_(float("nan"))
    attn.chunk_attention_q8_split(dev(q), dev(kb), dev(vb), out, n_heads, n_kv, HD, pos0, tok, 1 + dtype,
                                  stride, None, None, 0)
    torch.cuda.synchronize()
    ok, ma, mr = orc.compare(want, host(out), *CHUNK_GATE)
    assert ok, f"case {i} with in-workgroup slices: max_abs {ma:.3e} max_rel {mr:.3e}"


def batch_cases(n):
    r = orc.Rng(0x5EE9_0004)
    cases = []
    for i in range(n):
        slots = (1, 2, 3, 5, 8, 16, 24, 40)[draw(r, 0, 7)]
        cols = [(1, 1, 1, 2, 3, 4)[draw(r, 0, 5)] for _ in range(slots)]
        deep = draw(r, 0, 3) == 0
        depths = [draw(r, 0, 2500 if deep else 300) for _ in range(slots)]
        if slots > 1:
            depths[draw(r, 0, slots - 1)] = 0  # a slot whose only keys are its own rows
        stride = max(d + c for d, c in zip(depths, cols)) + draw(r, 0, 100)
        splits = (1, 2, 5, 8, 32)[draw(r, 0, 4)]
        cases.append((i, depths, cols, stride, splits))
    return cases


@pytest.mark.parametrize("i,depths,cols,stride,splits", batch_cases(16))
def test_batch_sweep(i, depths, cols, stride, splits):
    # plain and verify slots mixed in one launch: work items of 6 to 16 columns, worker launches (few
    # items) and plain grids (many), slots at depth 0, depths around tile and split edges
    from test_gpu_configs import _batch
    worst = _batch(depths, cols, stride, 0xBA7C_0000 + i, splits)
    print(f"[parity] batch sweep {i}: {len(depths)} slots, {sum(cols)} rows, stride {stride}, splits {splits}: "
          f"worst max_abs {worst:.3e}", flush=True)


def proj_cases(n):
    r = orc.Rng(0x5EE9_0003)
    return [(i, draw(r, 1, 300), 64 * draw(r, 1, 40), draw(r, 1, 9)) for i in range(n)]


@pytest.mark.parametrize("i,m,k,rows", proj_cases(20))
def test_projection_sweep(i, m, k, rows):
    r = orc.Rng(0x95EE_0000 + i)
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array((rows, k))
    want = orc.gemm_q8_0(w, x, rows, m, k)
    y = torch.full((rows, m), float("nan"), device="cuda")
    attn.gemv_q8_0_rows(dev(w), dev(x), y, m, k, rows)
    z = torch.full((rows, m), float("nan"), device="cuda")
    attn.gemm_q8_0_f16(dev(w), dev(x), z, m, k, rows)
    torch.cuda.synchronize()
    ok, ma, mr = orc.compare(want, host(y), 1e-4, 1e-3)
    assert ok, f"rows kernel {m}x{k} t={rows}: max_abs {ma:.3e} max_rel {mr:.3e}"
    ok, ma, mr = orc.compare(want, host(z), 1e-2, 1e-1)
    assert ok, f"chunk kernel {m}x{k} t={rows}: max_abs {ma:.3e} max_rel {mr:.3e}"
