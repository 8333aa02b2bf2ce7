"""Projections over Q8_0 weight matrices (the step after the attention core): HIP path through the
C ABI vs the CPU oracle on the reference's case recipes (raw random block bytes with scale 2^-10,
N(0,1) activations; crates/hipml-core/src/quant_parity.rs:80-86,125-133,
crates/hipml-core/src/prefill_parity.rs:114-119,209-219).  Tolerance: the reference's Tol::DEFAULT
(1e-4 abs OR 1e-3 rel) for its small cases; its LARGE_TOL (2e-3 / 3e-2) bounds the production
shape, where the kernel is asserted at 2e-4 abs (outputs of magnitude ~10, both sides fp32 sums of
6144 terms in different orders)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import dev, host, report  # noqa: E402

DEFAULT = (1e-4, 1e-3)


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


def run_gemv(w, x, m, k, rows):
    y = torch.full((rows, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.gemv_q8_0_rows(dev(w), dev(x), y, m, k, rows)
    torch.cuda.synchronize()
    return host(y)


def test_reference_gemv_case_64x512():
    r = orc.Rng(0x4B51_0005)
    m, k = 64, 512
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array(k)
    want = orc.gemv_q8_0(w, x, m, k)
    got = run_gemv(w, x, m, k, 1)[0]
    ok, _, _ = report("gemv_q8_0 64x512", want, got, *DEFAULT)
    assert ok


def test_reference_gemm_case_64x512_t4_and_skinny_200x512():
    for seed, m, k, t in ((0x9F11_0003, 64, 512, 4), (0x5C11_0006, 200, 512, 4)):
        r = orc.Rng(seed)
        w = orc.random_q8_0_bytes(r, m * k // 32)
        x = r.normal_array((t, k))
        want = orc.gemm_q8_0(w, x, t, m, k)
        got = run_gemv(w, x, m, k, t)
        ok, _, _ = report(f"q8_0 rows {m}x{k} t={t}", want, got, *DEFAULT)
        assert ok


def test_integer_case_is_exact():
    # d = 1 and small integer activations: every partial sum is an integer below 2^24, so any
    # summation order gives the same f32 and the result must equal the oracle's bit for bit
    r = orc.Rng(0x1234)
    m, k, rows = 80, 1024, 5
    w = orc.random_q8_0_bytes(r, m * k // 32).reshape(-1, 34)
    w[:, 0], w[:, 1] = 0x00, 0x3C
    x = np.round(r.normal_array((rows, k)) * 2).astype(np.float32)
    want = orc.gemm_q8_0(w.ravel(), x, rows, m, k)
    assert np.array_equal(run_gemv(w.ravel(), x, m, k, rows), want)


@pytest.mark.parametrize("rows", [1, 2, 3, 4, 5, 8, 9, 10, 16, 17, 24, 33, 49, 64, 70, 128])
def test_output_projection_shape(rows):
    # W_o of the model: 6144 -> 5120; activations of the size the gated attention output has
    r = orc.Rng(0x0E00 + rows)
    m, k = 5120, 6144
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array((rows, k), 0.5)
    want = orc.gemm_q8_0(w, x, rows, m, k, n_threads=8)
    got = run_gemv(w, x, m, k, rows)
    ok, ma, _ = report(f"W_o 5120x6144 rows={rows}", want, got, 2e-4, 1e-3)
    assert ok
    # a row does not depend on how many rows travel with it (the reference's batched GEMVs are bit-identical
    # per row to the single-sequence one, so that verify columns match a plain decode:
    # crates/hipml-kernels/src/attn_gpu.rs:930-932): up to 8 rows take one kernel whose per-row arithmetic
    # does not depend on the row count, more take the tile kernels
    if 2 <= rows <= 8:
        for r in {0, rows - 1}:
            assert np.array_equal(run_gemv(w, x[r], m, k, 1)[0], got[r])
    if rows == 8:
        assert np.array_equal(run_gemv(w, x[2:5], m, k, 3)[1], got[3])
    # 10 to 128 rows share one kernel (two passes of it beyond 64), 9 rows take another
    if rows in (24, 64, 70, 128):
        assert np.array_equal(run_gemv(w, x[3:13], m, k, 10)[2], got[5])
        assert np.array_equal(run_gemv(w, x[rows - 10:], m, k, 10)[9], got[rows - 1])


def test_ragged_shapes_and_scales():
    # m not a multiple of the workgroup's row tile, k with fewer block pairs than k slices, real
    # scales.  Outputs reach magnitude ~200 here, where two fp32 summation orders differ by ~1e-3: the
    # reference bounds such cases with LARGE_TOL (2e-3 / 3e-2, quant_parity.rs:20-25); on top of that
    # the kernel must be as close to the float64 value as the sequential fp32 sum is.
    r = orc.Rng(0x7A66)
    # rows 1-2 take the row kernel; more rows take full 16- or 32-row tiles (k = 5120 and 6144 in
    # straight-line code, any other k in a loop; k = 64 leaves seven of eight waves without a step)
    for m, k, rows in ((1, 64, 1), (33, 192, 2), (1000, 320, 7), (50, 4096, 16), (7, 64, 5),
                       (40, 5120, 9), (130, 704, 33), (64, 1024, 128), (20, 6144, 47)):
        w = orc.random_q8_0_bytes(r, m * k // 32).reshape(-1, 34)
        scales = (r.uniform_array(w.shape[0]) * 0.05 + 0.001).astype(np.float16)
        w[:, :2] = scales.view(np.uint8).reshape(-1, 2)
        x = r.normal_array((rows, k))
        want = orc.gemm_q8_0(w.ravel(), x, rows, m, k)
        got = run_gemv(w.ravel(), x, m, k, rows)
        ok, _, _ = report(f"q8_0 rows {m}x{k} t={rows}", want, got, 2e-3, 3e-2)
        assert ok
        blocks = w.reshape(m, k // 32, 34)
        dense = (blocks[:, :, :2].copy().view(np.float16).astype(np.float64)
                 * blocks[:, :, 2:].view(np.int8).astype(np.float64)).reshape(m, k)
        exact = x.astype(np.float64) @ dense.T
        assert np.max(np.abs(got - exact)) <= max(2 * np.max(np.abs(want - exact)), 1e-5)


@pytest.mark.parametrize("m,k", [(1, 256), (17, 512), (33, 768), (100, 2304), (5121, 1024), (6150, 512), (8200, 256),
                                 (300, 8192)])
def test_raw_row_kernel_over_ragged_shapes(m, k):
    # k a multiple of 256 and up to 8 rows take the kernel that moves the weight rows into LDS as they lie: fewer
    # rows than a workgroup takes, a last workgroup with a single row, 20 / 24 / 32 rows per workgroup (m above 4,096
    # / 5,120 / 6,144), one chunk per row (seven of eight waves idle), nine chunks (uneven shares), 32 chunks; real
    # scales.  Every row count against the oracle, and a row's bits the same whatever travels with it.
    r = orc.Rng(0x0D3A + m + k)
    w = orc.random_q8_0_bytes(r, m * k // 32).reshape(-1, 34)
    scales = (r.uniform_array(w.shape[0]) * 0.05 + 0.001).astype(np.float16)
    w[:, :2] = scales.view(np.uint8).reshape(-1, 2)
    w = w.ravel()
    x = r.normal_array((8, k))
    want = orc.gemm_q8_0(w, x, 8, m, k, n_threads=8)
    blocks = w.reshape(m, k // 32, 34)
    dense = (blocks[:, :, :2].copy().view(np.float16).astype(np.float64)
             * blocks[:, :, 2:].view(np.int8).astype(np.float64)).reshape(m, k)
    exact = x.astype(np.float64) @ dense.T
    alone = [run_gemv(w, x[i], m, k, 1)[0] for i in range(8)]
    for rows in (1, 2, 3, 4, 5, 7, 8):
        got = run_gemv(w, x[:rows], m, k, rows)
        ok, _, _ = report(f"raw-row {m}x{k} rows={rows}", want[:rows], got, 2e-3, 3e-2)
        assert ok
        # as close to the float64 value as a sequential fp32 sum is, or 21 bits of the largest output (the
        # activations enter with ~22 bits, and the offset of the weight bytes is taken out again in fp32)
        bound = max(2 * np.max(np.abs(want[:rows] - exact[:rows])), 2e-6 * np.max(np.abs(exact[:rows])) + 1e-5)
        assert np.max(np.abs(got - exact[:rows])) <= bound
        for i in range(rows):
            assert np.array_equal(got[i], alone[i]), f"rows={rows} row {i}"


@pytest.mark.parametrize("m,k", [(100, 2304), (5121, 1024), (300, 8192)])
def test_raw_row_tile_kernel_over_row_counts(m, k):
    # 10 to 128 rows over the tile kernel that moves the weight rows into LDS as they lie: one to four activation
    # tiles, a last tile with at most 8 live rows (whose other rows are not fetched), two passes beyond 64 rows with
    # a short second pass; real scales.  Every row count against the oracle, and a row's bits the same whatever
    # travels with it and whichever pass and tile it falls in.
    r = orc.Rng(0x711E + m + k)
    w = orc.random_q8_0_bytes(r, m * k // 32).reshape(-1, 34)
    scales = (r.uniform_array(w.shape[0]) * 0.05 + 0.001).astype(np.float16)
    w[:, :2] = scales.view(np.uint8).reshape(-1, 2)
    w = w.ravel()
    x = r.normal_array((128, k), 0.25)  # (outputs of magnitude ~40: two fp32 summation orders stay inside the gate)
    want = orc.gemm_q8_0(w, x, 128, m, k, n_threads=8)
    blocks = w.reshape(m, k // 32, 34)
    dense = (blocks[:, :, :2].copy().view(np.float16).astype(np.float64)
             * blocks[:, :, 2:].view(np.int8).astype(np.float64)).reshape(m, k)
    exact = x.astype(np.float64) @ dense.T
    full = run_gemv(w, x, m, k, 128)
    for rows in (10, 16, 17, 24, 32, 33, 40, 48, 49, 64, 65, 80, 96, 97, 127):
        got = run_gemv(w, x[:rows], m, k, rows)
        ok, _, _ = report(f"raw-row tiles {m}x{k} rows={rows}", want[:rows], got, 2e-3, 3e-2)
        assert ok
        bound = max(2 * np.max(np.abs(want[:rows] - exact[:rows])), 2e-6 * np.max(np.abs(exact[:rows])) + 1e-5)
        assert np.max(np.abs(got - exact[:rows])) <= bound
        assert np.array_equal(got, full[:rows]), f"rows={rows}"
    # rows taken from the middle: other tiles, other passes
    assert np.array_equal(run_gemv(w, x[60:75], m, k, 15), full[60:75])


@pytest.mark.parametrize("rows", [1, 4, 12])
def test_weights_at_a_4_byte_aligned_address(rows):
    # the raw-row kernels want W at a 16-byte boundary; a matrix that only meets the interface's 4-byte alignment
    # takes the kernels that load it in dwords, with the same answer class
    r = orc.Rng(0x0A11 + rows)
    m, k = 96, 1024
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array((rows, k), 0.5)
    want = orc.gemm_q8_0(w, x, rows, m, k)
    buf = torch.zeros(w.size + 16, dtype=torch.uint8, device="cuda")
    buf[4:4 + w.size] = torch.from_numpy(w).cuda()
    wd = buf[4:4 + w.size]
    assert wd.data_ptr() % 16 == 4
    y = torch.full((rows, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.gemv_q8_0_rows(wd, dev(x), y, m, k, rows)
    torch.cuda.synchronize()
    ok, _, _ = report(f"W at +4 bytes, rows={rows}", want, host(y), *DEFAULT)
    assert ok


def test_argument_errors():
    w = torch.zeros(34 * 4, dtype=torch.uint8, device="cuda")
    x = torch.zeros(64, device="cuda")
    y = torch.zeros(2, device="cuda")
    with pytest.raises(attn.HipmlError):
        attn.gemv_q8_0_rows(w, x, y, 2, 96, 1)     # k not a multiple of 64
    with pytest.raises(attn.HipmlError):
        attn.gemv_q8_0_rows(w, x, y, 2, 64, 129)   # too many rows
    with pytest.raises(attn.HipmlError):
        attn.gemv_q8_0_rows(w, x, y, 0, 64, 1)


# ---- the chunk GEMM (f16 operands) ---------------------------------------------------------------

# f16 operands: the reference budgets its own f16-operand kernels on these case shapes with
# 5e-2 abs / 5e-1 rel (k = 512) and 2.5e-1 / 5e-2 (k = 5120) (prefill_parity.rs:318-326); asserted here
# five and twenty-five times tighter.  Expected error: two roundings of 2^-11 per product, i.e.
# ~4e-4 of the root-sum-square of a row's terms (1.6 at k = 512 with N(0,1) activations).
F16_SMALL = (1e-2, 1e-1)
F16_LARGE = (1e-2, 5e-2)


def run_gemm(w, x, m, k, tokens):
    y = torch.full((tokens, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.gemm_q8_0_f16(dev(w), dev(x), y, m, k, tokens)
    torch.cuda.synchronize()
    return host(y)


def f16_operand_reference(w, x, m, k):
    """What the kernel is meant to compute, in float64: x rounded to f16, W as f16(d*q)."""
    blocks = w.reshape(m, k // 32, 34)
    d = blocks[:, :, :2].copy().view(np.float16).astype(np.float32)
    q = blocks[:, :, 2:].view(np.int8).astype(np.float32)
    dense = (d * q).astype(np.float16).astype(np.float64).reshape(m, k)
    return x.astype(np.float16).astype(np.float64) @ dense.T


@pytest.mark.parametrize("seed,m,k,t", [(0x9F11_0003, 64, 512, 4), (0x5C11_0006, 200, 512, 4),
                                        (0xA001, 128, 64, 128), (0xA002, 300, 1024, 37), (0xA003, 129, 192, 257)])
def test_gemm_reference_cases_and_ragged_tiles(seed, m, k, t):
    r = orc.Rng(seed)
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array((t, k))
    want = orc.gemm_q8_0(w, x, t, m, k)
    got = run_gemm(w, x, m, k, t)
    ok, _, _ = report(f"gemm_q8_0_f16 {m}x{k} t={t}", want, got, *F16_SMALL)
    assert ok
    # against its own definition the kernel is at fp32-accumulation level
    assert np.max(np.abs(got - f16_operand_reference(w, x, m, k))) < 2e-5 * np.sqrt(k)


def test_gemm_output_projection_672_tokens():
    r = orc.Rng(0x0E67)
    m, k, t = 5120, 6144, 672
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array((t, k), 0.5)
    got = run_gemm(w, x, m, k, t)
    rows = [0, 1, 127, 128, 300, 671]
    want = orc.gemm_q8_0(w, x[rows], len(rows), m, k, n_threads=8)
    ok, _, _ = report("W_o 5120x6144 t=672 (6 rows checked)", want, got[rows], *F16_LARGE)
    assert ok
    assert np.isfinite(got).all()
    # linearity over tokens holds bit for bit: a token's row does not depend on its tile neighbours
    alone = run_gemm(w, x[300:301], m, k, 1)
    assert np.array_equal(alone[0], got[300])


def test_output_chunk_equals_gate_then_gemm():
    # AttnLayer::apply_output_chunk (attn_chunk.rs:343-397) in one call: same bits as the gate kernel
    # followed by the f32-activation GEMM, with and without a gate; ragged token count
    r = orc.Rng(0x0C47)
    m, k, t = 384, 1024, 203
    w = orc.random_q8_0_bytes(r, m * k // 32)
    a = r.normal_array((t, k))
    g = r.normal_array((t, k))
    wd, ad, gd = dev(w), dev(a), dev(g)
    x16 = torch.empty((t, k), dtype=torch.float16, device="cuda")
    one = torch.full((t, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.output_chunk_q8_0(wd, ad, gd, one, m, k, t, x16)
    gated = torch.empty_like(ad)
    attn.q_gate(ad, gd, gated, t * k)
    two = torch.full((t, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.gemm_q8_0_f16(wd, gated, two, m, k, t)
    torch.cuda.synchronize()
    assert torch.equal(one, two)
    want = orc.gemm_q8_0(w, orc.q_gate(a.ravel(), g.ravel()).reshape(t, k), t, m, k)
    ok, _, _ = report("output chunk 384x1024 t=203", want, host(one), *F16_SMALL)
    assert ok
    plain = torch.full((t, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.output_chunk_q8_0(wd, ad, None, plain, m, k, t, x16)
    ref = torch.full((t, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.gemm_q8_0_f16(wd, ad, ref, m, k, t)
    torch.cuda.synchronize()
    assert torch.equal(plain, ref)
    # rows that arrive as f16 already (the chunk attention can deliver them so): only the GEMM runs
    ready = ad.to(torch.float16)
    direct = torch.full((t, m), float("nan"), dtype=torch.float32, device="cuda")
    attn.output_chunk_q8_0(wd, None, None, direct, m, k, t, ready)
    torch.cuda.synchronize()
    assert torch.equal(direct, ref)
    with pytest.raises(attn.HipmlError):   # a gate without the f32 rows it applies to
        attn.output_chunk_q8_0(wd, None, gd, direct, m, k, t, ready)


@pytest.mark.parametrize("m,k", [(1024, 5120), (12288, 5120)])
def test_qkv_projection_shapes(m, k):
    # the projections before the path use the same entry points: W_k / W_v 5120 -> 1024 and
    # W_q (q|gate) 5120 -> 12288 (attn_gpu.rs:490-498, prepare_rows :948-966)
    r = orc.Rng(0x0AB0 + m)
    w = orc.random_q8_0_bytes(r, m * k // 32)
    x = r.normal_array((3, k), 0.5)
    want = orc.gemm_q8_0(w, x, 3, m, k, n_threads=8)
    ok, _, _ = report(f"rows {m}x{k} t=3", want, run_gemv(w, x, m, k, 3), 2e-4, 1e-3)
    assert ok
    ok, _, _ = report(f"chunk {m}x{k} t=3", want, run_gemm(w, x, m, k, 3), *F16_LARGE)
    assert ok
