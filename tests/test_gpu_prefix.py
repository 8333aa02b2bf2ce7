"""Prefix snapshot / restore of quantized cache rows (crates/hipml-model/src/gpu/prefix.rs:214-239):
byte-exact copies between caches of different rows per head, and decode over a restored prefix."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

from oracle import binding as orc  # noqa: E402
from hipml_amd import attn  # noqa: E402
from gpu_util import N_HEADS, N_KV, HD, SCALE, dev, host, step_buffer  # noqa: E402


@pytest.fixture(scope="module", autouse=True)
def _init():
    attn.init(0)


@pytest.mark.parametrize("dtype", [0, 1])
@pytest.mark.parametrize("pos", [1, 37, 2049])
def test_snapshot_is_the_packed_prefix_and_restore_puts_it_back(dtype, pos):
    stride = 4096
    kv = attn.DeepKv(stride=stride, dtype=dtype)
    g = torch.Generator(device="cuda")
    g.manual_seed(pos * 7 + dtype)
    kv.k.copy_(torch.randint(0, 256, kv.k.shape, dtype=torch.uint8, device="cuda", generator=g))
    kv.v.copy_(torch.randint(0, 256, kv.v.shape, dtype=torch.uint8, device="cuda", generator=g))
    ks, vs = kv.snapshot(pos)
    torch.cuda.synchronize()
    assert torch.equal(ks, kv.k[:, :pos]) and torch.equal(vs, kv.v[:, :pos])
    other = attn.DeepKv(stride=8192, dtype=dtype)
    other.k.fill_(0xAB)
    other.v.fill_(0xCD)
    other.restore(ks, vs)
    torch.cuda.synchronize()
    assert torch.equal(other.k[:, :pos], kv.k[:, :pos]) and torch.equal(other.v[:, :pos], kv.v[:, :pos])
    assert bool((other.k[:, pos:] == 0xAB).all()) and bool((other.v[:, pos:] == 0xCD).all())


def test_decode_over_a_restored_prefix_equals_decode_over_the_original():
    seq, stride = 1500, 2048
    r = orc.Rng(0x9F1C)
    q = r.normal_array((N_HEADS, HD))
    kf = r.normal_array((N_KV, seq, HD))
    vf = r.normal_array((N_KV, seq, HD))
    a = attn.DeepKv(stride=stride)
    attn.kv_encode_bulk(0, dev(np.ascontiguousarray(kf.transpose(1, 0, 2))),
                        dev(np.ascontiguousarray(vf.transpose(1, 0, 2))), a.k, a.v, N_KV, HD, stride, 0, 0, seq)
    b = attn.DeepKv(stride=4096)
    b.restore(*a.snapshot(seq))
    outs = []
    for kvc in (a, b):
        out = torch.empty((N_HEADS, HD), device="cuda")
        splits = kvc.splits(seq)
        attn.attn_decode_kv(step_buffer(seq - 1, seq), 0, dev(q), kvc.k, kvc.v, kvc.part_acc, kvc.part_ml,
                            out, N_HEADS, N_KV, HD, kvc.seq, SCALE, splits)
        outs.append(out)
    torch.cuda.synchronize()
    want = orc.attn_decode_kv(q, host(a.k), host(a.v), N_HEADS, N_KV, HD, seq, SCALE, stride=stride)
    assert orc.compare(want, host(outs[0]).ravel(), 1e-3, 5e-3)[0]
    # the same rows at another stride: other split boundaries, same class
    assert orc.compare(want, host(outs[1]).ravel(), 1e-3, 5e-3)[0]


def test_rows_copy_argument_errors():
    kv = attn.DeepKv(stride=64)
    small = torch.empty((4, 16, 272), dtype=torch.uint8, device="cuda")
    with pytest.raises(attn.HipmlError):
        attn.kv_rows_copy(0, kv.k, kv.v, small, small, 4, 256, 64, 16, 17)   # rows beyond dst stride
    with pytest.raises(attn.HipmlError):
        attn.kv_rows_copy(7, kv.k, kv.v, small, small, 4, 256, 64, 16, 8)    # unknown format
