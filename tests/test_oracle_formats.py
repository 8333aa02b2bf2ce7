"""The oracle's KV formats against the reference's own known-answer tests
(crates/hipml-core/tests/kv_formats.rs) and against numpy's IEEE binary16."""
import numpy as np
import pytest

Q8, Q4, BLOCK = 0, 1, 32


def test_block_byte_counts(orc):
    # kv_formats.rs:16-22
    assert orc.block_bytes(Q8) == 34
    assert orc.block_bytes(Q4) == 18
    assert orc.token_bytes(Q8, 4, 256, 16) == 34_816
    assert orc.token_bytes(Q4, 4, 256, 16) == 18_432
    assert orc.row_bytes(Q8, 256) == 272


def test_f16_round_trips_and_rounds_to_nearest(orc):
    # kv_formats.rs:25-40
    for h in [0x0000, 0x3800, 0x3C00, 0xBC00, 0x7BFF, 0x0001, 0x03FF]:
        assert orc.f32_to_f16(orc.f16_to_f32(h)) == h
    assert orc.f16_to_f32(orc.f32_to_f16(0.1)) == np.float32(0.099_975_586)
    assert orc.f32_to_f16(np.inf) == 0x7C00
    assert orc.f32_to_f16(-0.0) == 0x8000


def test_f16_decode_equals_numpy_for_every_pattern(orc):
    allh = np.arange(1 << 16, dtype=np.uint16)
    want = allh.view(np.float16).astype(np.float32)
    got = np.array([orc.f16_to_f32(int(h)) for h in allh], dtype=np.float32)
    nan = np.isnan(want)  # a NaN's payload does not survive the ctypes float return
    assert np.array_equal(np.isnan(got), nan)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))


def test_f16_encode_equals_numpy_rne(orc):
    rng = np.random.default_rng(5)
    bits = rng.integers(0, 1 << 32, size=200_000, dtype=np.uint64).astype(np.uint32)
    # plus every boundary neighbourhood: halfway points between consecutive f16s
    h = np.arange(0, 0x7C00, dtype=np.uint16)
    lo = h.view(np.float16).astype(np.float64)
    hi = (h + 1).astype(np.uint16).view(np.float16).astype(np.float64)
    mid = ((lo + hi) / 2).astype(np.float32)
    near = np.concatenate([mid, np.nextafter(mid, np.float32(np.inf)),
                           np.nextafter(mid, np.float32(-np.inf)), -mid])
    bits = np.concatenate([bits, near.view(np.uint32)])
    vals = bits.view(np.float32)
    finite = np.isfinite(vals)
    with np.errstate(over="ignore"):
        want = vals.astype(np.float16).view(np.uint16)
    got = np.array([orc.f32_bits_to_f16(int(b)) for b in bits], dtype=np.uint16)
    assert np.array_equal(got[finite], want[finite])
    # NaN stays NaN, infinities keep their sign
    nan = np.isnan(vals)
    assert np.all((got[nan] & 0x7C00) == 0x7C00) and np.all((got[nan] & 0x03FF) != 0)


def test_q8_known_vector(orc):
    # kv_formats.rs:43-61
    xs = np.zeros(BLOCK, dtype=np.float32)
    xs[0], xs[1] = 63.5, -63.5
    for j in range(2, BLOCK):
        xs[j] = 0.5 * (j - 8.0)
    b = orc.quantize(Q8, xs)
    assert b.size == 34
    assert list(b[:2]) == [0x00, 0x38]
    assert b[2] == 127 and b[3] == np.uint8(np.int8(-127).view(np.uint8))
    assert np.array_equal(orc.dequantize(Q8, b), xs)


def test_q8_round_trip_error_is_half_a_step(orc):
    # kv_formats.rs:64-89
    rng = orc.Rng(0x08)
    for _ in range(64):
        xs = rng.normal_array(BLOCK, 3.0)
        step = np.abs(xs).max() / np.float32(127.0)
        back = orc.dequantize(Q8, orc.quantize(Q8, xs))
        assert np.abs(xs - back).max() <= step * 0.5625 + 1e-6
        assert np.all((back == 0) | (np.sign(xs) == np.sign(back)))
    z = orc.quantize(Q8, np.zeros(BLOCK, dtype=np.float32))
    assert list(z[:2]) == [0, 0] and not orc.dequantize(Q8, z).any()


def test_q8_matches_the_ggml_definition_in_numpy(orc):
    # docs/reference/ggml-quants.c:273-296 (quantize_row_q8_0_ref), restated in numpy.
    rng = np.random.default_rng(11)
    x = (rng.standard_normal((500, BLOCK)) * rng.uniform(1e-3, 50, (500, 1))).astype(np.float32)
    amax = np.abs(x).max(axis=1)
    d = (amax / np.float32(127.0)).astype(np.float32)
    inv = np.where(d > 0, np.float32(1.0) / d, np.float32(0)).astype(np.float32)
    t = (x * inv[:, None]).astype(np.float32)
    q = np.clip(np.sign(t) * np.floor(np.abs(t) + np.float32(0.5)), -127, 127).astype(np.int8)
    got = orc.quantize(Q8, x).reshape(500, 34)
    assert np.array_equal(got[:, :2].copy().view(np.uint16).ravel(),
                          d.astype(np.float16).view(np.uint16))
    assert np.array_equal(got[:, 2:].view(np.int8), q)


def test_q4_known_vector(orc):
    # kv_formats.rs:92-108
    xs = np.array([0.25 * ((j % 16) - 8.0) for j in range(BLOCK)], dtype=np.float32)
    b = orc.quantize(Q4, xs)
    assert b.size == 18 and list(b[:2]) == [0x00, 0x34]
    for j in range(16):
        assert b[2 + j] == ((j << 4) | j)
    assert np.array_equal(orc.dequantize(Q4, b), xs)


def test_q4_extreme_is_exact_and_error_bounded(orc):
    # kv_formats.rs:111-137
    for vmax in [2.0, -2.0, 0.125, -0.125]:
        xs = np.full(BLOCK, 0.1, dtype=np.float32)
        xs[5] = vmax
        assert orc.dequantize(Q4, orc.quantize(Q4, xs))[5] == np.float32(vmax)
    rng = orc.Rng(0x40)
    for _ in range(64):
        xs = rng.normal_array(BLOCK, 2.0)
        back = orc.dequantize(Q4, orc.quantize(Q4, xs))
        assert np.abs(xs - back).max() <= np.abs(xs).max() / 8.0 + 1e-6


@pytest.mark.parametrize("dtype", [Q8, Q4])
def test_row_layout_matches_block_order(orc, dtype):
    # kv_formats.rs:140-162
    n_kv, seq, dim = 2, 7, 64
    vals = orc.Rng(77).normal_array(n_kv * seq * dim, 0.7)
    b = orc.quantize(dtype, vals)
    nb, bb = dim // BLOCK, orc.block_bytes(dtype)
    back = orc.dequantize(dtype, b)
    for h in range(n_kv):
        for pos in range(seq):
            for d in range(dim):
                at = ((h * seq + pos) * nb + d // BLOCK) * bb
                want = orc.dequantize(dtype, b[at:at + bb])[d % BLOCK]
                assert back[(h * seq + pos) * dim + d] == want


def test_synthetic_blocks_are_well_formed(orc):
    # kv_formats.rs:230-246
    b = orc.synthetic_blocks(Q8, 1000, 7)
    assert b.size == 34_000
    back = orc.dequantize(Q8, b)
    assert np.isfinite(back).all() and np.abs(back).max() > 0
    d = b.reshape(1000, 34)[:, :2].copy().view(np.float16).astype(np.float32).ravel()
    assert np.all((d >= 0.01) & (d < 0.05))


def test_rng_integer_stream_is_xorshift64_star(orc):
    # rng.rs:19-32 restated with Python integers.
    for seed in [0, 1, 42, 0x9E00_0004, (1 << 64) - 1]:
        s = (seed | 1) & ((1 << 64) - 1)
        r = orc.Rng(seed)
        for _ in range(50):
            s ^= s >> 12
            s ^= (s << 25) & ((1 << 64) - 1)
            s ^= s >> 27
            want = (s * 0x2545F4914F6CDD1D) & ((1 << 64) - 1)
            assert r.next_u64() == want
    r1, r2 = orc.Rng(9), orc.Rng(9)
    a = r1.uniform_array(1000)
    assert np.array_equal(a, r2.uniform_array(1000)) and a.min() >= 0 and a.max() < 1
    n = orc.Rng(3).normal_array(200_000)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1) < 0.01
