"""Attention front end (q|gate split, per-head RMS norm, M-RoPE) on the GPU against the oracle.
Bit-exact against the oracle's restatement of the reference's GPU summation order
(crates/hipml-kernels/kernels/attn_front_f32.hip:79-103: one square per thread, 256-wide halving
tree); the reference's CPU definition (ops.rs:181-187, index-order sum) differs from that only in
the rounding of the sum and is reported to 1e-5."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, N_ROT, THETA, SECTIONS, dev, host, report  # noqa: E402

EPS = 1e-6


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)
    attn.rope_table(THETA, N_ROT, 131072)
    yield


def front_inputs(seed, rows):
    r = orc.Rng(seed)
    qg = r.normal_array((rows, N_HEADS, 2 * HD), 2.0)
    k = r.normal_array((rows, N_KV, HD), 0.7)
    qw = (1.0 + 0.1 * r.normal_array((HD,))).astype(np.float32)
    kw = (1.0 + 0.1 * r.normal_array((HD,))).astype(np.float32)
    qg[0, 0, :HD] = 0.0           # an all-zero head: scale = 1/sqrt(eps), values stay 0
    if rows > 1:
        qg[1, 3, :HD] *= 1e-4     # tiny head: eps matters
    return qg, k, qw, kw


def test_decode_front_is_bit_exact_with_distinct_mrope_ids():
    qg, k, qw, kw = front_inputs(0xF207, 1)
    pos = (1234, 77, 99999, 5)   # sections (11, 11, 10, 0): three of the four ids are used
    q = torch.full((N_HEADS, HD), float("nan"), device="cuda")
    gate = torch.full((N_HEADS, HD), float("nan"), device="cuda")
    kd = dev(k[0])
    attn.attn_front(dev(qg[0]), q, gate, kd, dev(qw), dev(kw), N_HEADS, N_KV, HD, N_ROT, SECTIONS,
                    torch.tensor(pos, dtype=torch.int32, device="cuda"), THETA, EPS)
    torch.cuda.synchronize()
    wq, wg, wk = orc.attn_front(qg[0], k[0], qw, kw, N_HEADS, N_KV, HD, N_ROT, SECTIONS, pos, THETA,
                                EPS, tree=True)
    assert np.array_equal(host(gate).ravel(), wg), "gate half of the joint projection"
    assert np.array_equal(host(q).ravel(), wq), "q: norm + M-RoPE bits"
    assert np.array_equal(host(kd).ravel(), wk), "k: norm + M-RoPE bits (in place)"
    cq, _, ck = orc.attn_front(qg[0], k[0], qw, kw, N_HEADS, N_KV, HD, N_ROT, SECTIONS, pos, THETA,
                               EPS, tree=False)
    ok1, _, _ = report("front q vs CPU-order definition", cq, host(q).ravel(), 1e-5, 1e-5)
    ok2, _, _ = report("front k vs CPU-order definition", ck, host(kd).ravel(), 1e-5, 1e-5)
    assert ok1 and ok2


@pytest.mark.parametrize("rows,pos0", [(37, 29), (672, 0), (5, 100_000)])
def test_chunk_front_is_bit_exact(rows, pos0):
    qg, k, qw, kw = front_inputs(0xF208 + rows, rows)
    q = torch.full((rows, N_HEADS, HD), float("nan"), device="cuda")
    gate = torch.full((rows, N_HEADS, HD), float("nan"), device="cuda")
    kd = dev(k)
    attn.chunk_front(dev(qg), kd, q, gate, dev(qw), dev(kw), N_HEADS, N_KV, HD, N_ROT, THETA, EPS, pos0,
                     rows)
    torch.cuda.synchronize()
    gq, gg, gk = host(q), host(gate), host(kd)
    for t in range(rows):
        p = pos0 + t
        wq, wg, wk = orc.attn_front(qg[t], k[t], qw, kw, N_HEADS, N_KV, HD, N_ROT, (0, 0, 0, 0),
                                    (p, p, p, p), THETA, EPS, tree=True)
        assert np.array_equal(gg[t].ravel(), wg), f"gate row {t}"
        assert np.array_equal(gq[t].ravel(), wq), f"q row {t}"
        assert np.array_equal(gk[t].ravel(), wk), f"k row {t}"


def test_front_then_existing_rope_free_path_agree():
    # with unit weights and a head already of unit RMS the norm is (nearly) the identity; the
    # rotation must be the stand-alone M-RoPE kernel's bits on the normalised values
    r = orc.Rng(0xF209)
    qg = r.normal_array((N_HEADS, 2 * HD))
    k = r.normal_array((N_KV, HD))
    ones = np.ones(HD, dtype=np.float32)
    pos = torch.tensor((40, 41, 42, 43), dtype=torch.int32, device="cuda")
    q = torch.empty((N_HEADS, HD), device="cuda")
    gate = torch.empty((N_HEADS, HD), device="cuda")
    kd = dev(k)
    attn.attn_front(dev(qg), q, gate, kd, dev(ones), dev(ones), N_HEADS, N_KV, HD, N_ROT, SECTIONS, pos,
                    THETA, EPS)
    normed = orc.head_rmsnorm(qg.reshape(N_HEADS, 2, HD)[:, 0].copy(), ones, N_HEADS, HD, EPS, tree=True)
    y = torch.empty((N_HEADS, HD), device="cuda")
    attn.mrope(dev(normed.reshape(N_HEADS, HD)), y, N_HEADS, HD, N_ROT, SECTIONS, pos, THETA)
    torch.cuda.synchronize()
    assert np.array_equal(host(q), host(y))


def test_front_rejects_other_head_dims():
    x = torch.zeros(4096, device="cuda")
    pos = torch.zeros(4, dtype=torch.int32, device="cuda")
    with pytest.raises(attn.HipmlError) as e:
        attn.attn_front(x, x, x, x, x, x, 4, 1, 128, 64, SECTIONS, pos, THETA, EPS)
    assert "head_dim" in str(e.value)
