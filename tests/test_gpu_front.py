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


@pytest.mark.parametrize("dtype", [0, 1])
def test_decode_front_with_append_has_the_bits_of_the_two_launches(dtype):
    # one token: front end, then the append of its K and V rows at step[0], against one fused launch;
    # stride > position, caches pre-filled so that a stray write shows
    qg, k, qw, kw = front_inputs(0xF30A + dtype, 1)
    r = orc.Rng(0xF30B + dtype)
    v = r.normal_array((N_KV, HD))
    stride, p = 300, 257
    row_bytes = 272 if dtype == 0 else 144
    step = torch.tensor([p, p + 1, 0, 0, p, 77, 9999, 5], dtype=torch.int32, device="cuda")

    def run(fused):
        q = torch.full((N_HEADS, HD), float("nan"), device="cuda")
        gate = torch.full((N_HEADS, HD), float("nan"), device="cuda")
        kd, vd = dev(k[0]), dev(v)
        kc = torch.full((N_KV * stride * row_bytes,), 0x5A, dtype=torch.uint8, device="cuda")
        vc = torch.full((N_KV * stride * row_bytes,), 0xA5, dtype=torch.uint8, device="cuda")
        if fused:
            attn.attn_front_encode(step, dtype, dev(qg[0]), q, gate, kd, vd, dev(qw), dev(kw), kc, vc,
                                   N_HEADS, N_KV, HD, N_ROT, SECTIONS, THETA, EPS, stride)
        else:
            attn.attn_front(dev(qg[0]), q, gate, kd, dev(qw), dev(kw), N_HEADS, N_KV, HD, N_ROT, SECTIONS,
                            step[4:], THETA, EPS)
            attn.kv_encode(step, dtype, kd, vd, kc, vc, N_KV, HD, stride)
        torch.cuda.synchronize()
        return [host(t) for t in (q, gate, kd, kc, vc)]

    two, one = run(False), run(True)
    for name, a, b in zip(("q", "gate", "k", "k cache", "v cache"), two, one):
        assert np.array_equal(a, b), name
    # the appended row is the oracle's encoding of the oracle's front end, everything else untouched
    _, _, wk = orc.attn_front(qg[0], k[0], qw, kw, N_HEADS, N_KV, HD, N_ROT, SECTIONS,
                              (p, 77, 9999, 5), THETA, EPS, tree=True)
    enc = lambda x: orc.quantize(dtype, x)  # noqa: E731
    kc = one[3].reshape(N_KV, stride, row_bytes)
    assert np.array_equal(kc[:, p].ravel(), enc(wk)), "appended K row"
    assert np.array_equal(one[4].reshape(N_KV, stride, row_bytes)[:, p].ravel(), enc(v.ravel())), "appended V row"
    mask = np.ones(stride, dtype=bool)
    mask[p] = False
    assert (kc[:, mask] == 0x5A).all() and (one[4].reshape(N_KV, stride, row_bytes)[:, mask] == 0xA5).all()


@pytest.mark.parametrize("dtype,rows,pos0", [(0, 37, 29), (0, 672, 0), (1, 5, 100_000)])
def test_chunk_front_with_append_has_the_bits_of_the_two_launches(dtype, rows, pos0):
    qg, k, qw, kw = front_inputs(0xF40C + rows, rows)
    r = orc.Rng(0xF40D + rows)
    v = r.normal_array((rows, N_KV, HD))
    stride = pos0 + rows + 3
    row_bytes = 272 if dtype == 0 else 144

    def run(fused):
        q = torch.full((rows, N_HEADS, HD), float("nan"), device="cuda")
        gate = torch.full((rows, N_HEADS, HD), float("nan"), device="cuda")
        kd, vd = dev(k), dev(v)
        kc = torch.zeros((N_KV * stride * row_bytes,), dtype=torch.uint8, device="cuda")
        vc = torch.zeros((N_KV * stride * row_bytes,), dtype=torch.uint8, device="cuda")
        if fused:
            attn.chunk_front_encode(dtype, dev(qg), kd, vd, q, gate, dev(qw), dev(kw), kc, vc, N_HEADS,
                                    N_KV, HD, N_ROT, THETA, EPS, pos0, rows, stride)
        else:
            attn.chunk_front(dev(qg), kd, q, gate, dev(qw), dev(kw), N_HEADS, N_KV, HD, N_ROT, THETA, EPS,
                             pos0, rows)
            attn.kv_encode_bulk(dtype, kd, vd, kc, vc, N_KV, HD, stride, pos0, 0, rows)
        torch.cuda.synchronize()
        return [host(t) for t in (q, gate, kd, kc, vc)]

    two, one = run(False), run(True)
    for name, a, b in zip(("q", "gate", "k", "k cache", "v cache"), two, one):
        assert np.array_equal(a, b), name
    assert one[3].any() and one[4].any()


def test_front_with_append_rejects_bad_arguments():
    t = torch.zeros(16, device="cuda")
    b = torch.zeros(16, dtype=torch.uint8, device="cuda")
    with pytest.raises(attn.HipmlError):   # rows do not fit the cache
        attn.chunk_front_encode(0, t, t, t, t, t, t, t, b, b, N_HEADS, N_KV, HD, N_ROT, THETA, EPS, 10, 5, 12)
    with pytest.raises(attn.HipmlError):   # unknown cache format
        attn.chunk_front_encode(7, t, t, t, t, t, t, t, b, b, N_HEADS, N_KV, HD, N_ROT, THETA, EPS, 0, 1, 12)
    with pytest.raises(attn.HipmlError):   # no step buffer
        attn.attn_front_encode(None, 0, t, t, t, t, t, t, t, b, b, N_HEADS, N_KV, HD, N_ROT, SECTIONS,
                               THETA, EPS, 12)


@pytest.mark.parametrize("dtype", [0, 1])
def test_batched_front_uses_each_row_s_own_position_and_cache(dtype):
    # the batched engine's step (gpu/batch/forward.rs:79-106): one row per sequence, positions that
    # differ, contiguous per-slot caches.  Against the oracle row by row, and the fused launch against
    # front_rows followed by kv_encode_rows byte for byte.
    slots, stride = 6, 96
    positions = [0, 95, 7, 7, 50, 1]
    row_bytes = 272 if dtype == 0 else 144
    slot_bytes = N_KV * stride * row_bytes
    qg, k, qw, kw = front_inputs(0xF50E + dtype, slots)
    v = orc.Rng(0xF50F + dtype).normal_array((slots, N_KV, HD))
    pos = torch.tensor([[p, p + 1] for p in positions], dtype=torch.int32, device="cuda")

    def run(fused):
        q = torch.full((slots, N_HEADS, HD), float("nan"), device="cuda")
        gate = torch.full((slots, N_HEADS, HD), float("nan"), device="cuda")
        kd, vd = dev(k), dev(v)
        kc = torch.full((slots, N_KV, stride, row_bytes), 0x3C, dtype=torch.uint8, device="cuda")
        vc = torch.full((slots, N_KV, stride, row_bytes), 0xC3, dtype=torch.uint8, device="cuda")
        if fused:
            attn.front_rows_encode(dtype, dev(qg), kd, vd, q, gate, dev(qw), dev(kw), kc, vc, N_HEADS, N_KV,
                                   HD, N_ROT, THETA, EPS, stride, pos, slot_bytes, slots)
        else:
            attn.front_rows(dev(qg), kd, q, gate, dev(qw), dev(kw), N_HEADS, N_KV, HD, N_ROT, THETA, EPS,
                            pos, slots)
            attn.kv_encode_rows(dtype, kd, vd, kc, vc, N_KV, HD, stride, pos, slot_bytes, slots)
        torch.cuda.synchronize()
        return [host(t) for t in (q, gate, kd, kc, vc)]

    two, one = run(False), run(True)
    for name, a, b in zip(("q", "gate", "k", "k cache", "v cache"), two, one):
        assert np.array_equal(a, b), name
    gq, gg, gk, kc, vc = one
    for r, p in enumerate(positions):
        wq, wg, wk = orc.attn_front(qg[r], k[r], qw, kw, N_HEADS, N_KV, HD, N_ROT, (0, 0, 0, 0),
                                    (p, p, p, p), THETA, EPS, tree=True)
        assert np.array_equal(gg[r].ravel(), wg) and np.array_equal(gq[r].ravel(), wq), f"row {r}"
        assert np.array_equal(gk[r].ravel(), wk), f"k row {r}"
        assert np.array_equal(kc[r, :, p].ravel(), orc.quantize(dtype, wk)), f"slot {r} K row"
        assert np.array_equal(vc[r, :, p].ravel(), orc.quantize(dtype, v[r].ravel())), f"slot {r} V row"
        mask = np.ones(stride, dtype=bool)
        mask[p] = False
        assert (kc[r][:, mask] == 0x3C).all() and (vc[r][:, mask] == 0xC3).all()
