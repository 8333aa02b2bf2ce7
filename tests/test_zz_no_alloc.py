"""hipml_attn_decode_kv_noalloc (split partials in the library's built-in array, nothing allocated)
against hipml_attn_decode_kv on the same inputs, through the C ABI: two calls in a row, the second
with a smaller input (fewer heads, fewer splits, shallower cache), each bit-equal to the entry point
with caller scratch and inside the kernel class of the CPU oracle."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import HD, SCALE, dev, host, quantized_cache, step_buffer, decode_scratch  # noqa: E402

KERNEL_CLASS = (1e-3, 5e-3)


def _case(seed, n_heads, n_kv, seq, stride):
    r = orc.Rng(seed)
    q = r.normal_array((n_heads, HD))
    kf = r.normal_array((n_kv, seq, HD), 0.3)
    vf = r.normal_array((n_kv, seq, HD))
    kb, vb = quantized_cache(kf, vf, stride)
    return q, kb, vb


def _both(q, kb, vb, n_heads, n_kv, seq, stride, splits):
    step = step_buffer(seq - 1, seq)
    qd, kd, vd = dev(q), dev(kb), dev(vb)
    acc, ml = decode_scratch(n_heads, splits)
    want = torch.full((n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv(step, 0, qd, kd, vd, acc, ml, want, n_heads, n_kv, HD, stride, SCALE, splits)
    got = torch.full((n_heads, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv_noalloc(step, 0, qd, kd, vd, got, n_heads, n_kv, HD, stride, SCALE, splits)
    torch.cuda.synchronize()
    return host(want), host(got)


def test_noalloc_decode_matches_decode_with_caller_scratch_twice():
    attn.init(0)
    # first call: the model's geometry at depth 5,000, 40 splits (960 partial slices of the array)
    q, kb, vb = _case(0x70A110C1, 24, 4, 5000, 5120)
    want, got = _both(q, kb, vb, 24, 4, 5000, 5120, 40)
    assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    ref = orc.attn_decode_kv(q, kb, vb, 24, 4, HD, 5000, SCALE, stride=5120)
    assert orc.compare(ref, got.ravel(), *KERNEL_CLASS)[0]
    # second call, smaller: 6 heads over 1 KV head, depth 300, 3 splits; the array still holds the first
    # call's partials in the slices this call does not use
    q, kb, vb = _case(0x70A110C2, 6, 1, 300, 300)
    want, got = _both(q, kb, vb, 6, 1, 300, 300, 3)
    assert np.array_equal(want.view(np.uint32), got.view(np.uint32))
    ref = orc.attn_decode_kv(q, kb, vb, 6, 1, HD, 300, SCALE)
    assert orc.compare(ref, got.ravel(), *KERNEL_CLASS)[0]


def test_noalloc_decode_allocates_nothing_and_replays_from_a_graph():
    # its namesake property: the device's free memory is the same before and after the calls; and the use it is
    # for: captured into a HIP graph and replayed, with eager work between the replays
    attn.init(0)
    q, kb, vb = _case(0x70A110C4, 24, 4, 2000, 2048)
    qd, kd, vd = dev(q), dev(kb), dev(vb)
    step = step_buffer(1999, 2000)
    eager = torch.full((24, HD), float("nan"), dtype=torch.float32, device="cuda")
    out = torch.full((24, HD), float("nan"), dtype=torch.float32, device="cuda")
    attn.attn_decode_kv_noalloc(step, 0, qd, kd, vd, eager, 24, 4, HD, 2048, SCALE, 16)  # (first call: code is loaded)
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
        attn.attn_decode_kv_noalloc(step, 0, qd, kd, vd, eager, 24, 4, HD, 2048, SCALE, 16)
    torch.cuda.synchronize()
    free_after, _ = torch.cuda.mem_get_info()
    assert free_after == free_before
    ref = orc.attn_decode_kv(q, kb, vb, 24, 4, HD, 2000, SCALE, stride=2048)
    assert orc.compare(ref, host(eager).ravel(), *KERNEL_CLASS)[0]
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        attn.attn_decode_kv_noalloc(step, 0, qd, kd, vd, out, 24, 4, HD, 2048, SCALE, 16)
    for i in range(3):
        out.fill_(float("nan"))
        attn.attn_decode_kv_noalloc(step, 0, qd, kd, vd, eager, 24, 4, HD, 2048, SCALE, 16)  # eager work between
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager), f"replay {i}"


def test_noalloc_decode_rejects_more_partials_than_the_array_holds():
    attn.init(0)
    q, kb, vb = _case(0x70A110C3, 24, 4, 64, 64)
    out = torch.zeros((24, HD), dtype=torch.float32, device="cuda")
    with pytest.raises(attn.HipmlError) as e:
        attn.attn_decode_kv_noalloc(step_buffer(63, 64), 0, dev(q), dev(kb), dev(vb), out, 24, 4, HD, 64,
                                    SCALE, 171)  # 24 * 171 = 4104 > 4096
    assert e.value.code == -4
    assert "4096" in e.value.message
