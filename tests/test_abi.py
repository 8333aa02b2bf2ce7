"""The C ABI without a GPU: libhipml_attn.so loads, exports every function include/hipml_attn.h
declares, the host-only entry points (split policies, RoPE table) compute, and argument errors
are reported before anything is launched."""
import ctypes as C
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from hipml_amd import attn
    return attn.lib()


def declared_functions():
    text = open(os.path.join(ROOT, "include", "hipml_attn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(hipml_\w+)\s*\(", text)))


def test_every_declared_function_is_exported(lib):
    names = declared_functions()
    assert len(names) >= 25
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_mirror_lists_every_declared_function():
    from hipml_amd import attn
    assert sorted(attn.EXPORTS) == declared_functions()


def test_split_policies(lib):
    from hipml_amd import attn
    # decode: 128 keys per split, at most two workgroups per CU over the KV heads
    assert attn.decode_splits(1, 4) == 1
    assert attn.decode_splits(8192, 4) == 64
    assert attn.decode_splits(32768, 4) == 128   # (the q8_0 launch uses 64 of them)
    assert attn.decode_splits(1 << 20, 4) == 128
    # batches: a cap on one slot's workers, never below 1
    assert 1 <= attn.batch_splits(16448, 4, 16) <= 64
    assert attn.batch_splits(16448, 4, 128) >= 1
    assert attn.batch_splits(100, 4, 16) == 1
    # prefill: no key slices once the task blocks fill the chip; slices keep n_kv*splits on the XCDs
    assert attn.chunk_splits(0, 8192, 4) == 1
    s = attn.chunk_slices(100_000, 2048, 4)
    assert s > 1 and (4 * s) % 8 == 0
    # long chunks deep in a prefix: the scratch is sized for the slices that run plus the live rows as f16
    # tiles (70,656 bytes per KV head and 64 rows) in whole slices of partial rows (2,048 x 24 x 256 f32)
    tiles = 4 * ((100_000 + 2048 + 63) // 64) * 70_656
    per_slice = 2048 * 24 * 256 * 4
    assert attn.chunk_splits(100_000, 2048, 4) == s + (tiles + per_slice - 1) // per_slice == 13
    assert attn.chunk_splits(2047, 2048, 4) == attn.chunk_slices(2047, 2048, 4)  # prefix shorter than the chunk
    assert attn.chunk_splits(2048, 2048, 4) > attn.chunk_slices(2048, 2048, 4) >= 2
    # the usual 672-token chunk: from eight times its length on
    assert attn.chunk_splits(8 * 672 - 1, 672, 4) == attn.chunk_slices(8 * 672 - 1, 672, 4)
    assert attn.chunk_splits(32768, 672, 4) > attn.chunk_slices(32768, 672, 4) >= 2
    assert attn.chunk_splits(100_000, 639, 4) == attn.chunk_slices(100_000, 639, 4)
    assert attn.chunk_slices(0, 1, 4) >= 1
    # near position 0 the keys are cut inside the workgroups (0); deep chunks and long ones are not
    assert attn.chunk_splits(0, 672, 4) == 0 and attn.chunk_splits(0, 1, 4) == 0
    assert attn.chunk_splits(512, 672, 4) == 0
    assert attn.chunk_splits(0, 2048, 4) == attn.chunk_slices(0, 2048, 4) >= 1
    assert attn.chunk_splits(1000, 64, 4) == attn.chunk_slices(1000, 64, 4) >= 2
    assert attn.chunk_slices(0, 672, 4) >= 2


def test_rope_table_on_the_host_is_the_f64_definition(lib):
    theta, n_rot, max_pos = 1e7, 64, 300
    nbytes = lib.hipml_rope_table_bytes(n_rot, max_pos)
    assert nbytes == max_pos * (n_rot // 2) * 2 * 4
    tab = np.empty(nbytes // 4, dtype=np.float32)
    assert lib.hipml_rope_table_fill_host(tab.ctypes.data_as(C.c_void_p), C.c_float(theta), n_rot, max_pos) == 0
    tab = tab.reshape(max_pos, n_rot // 2, 2)
    k = np.arange(n_rot // 2, dtype=np.float64)
    freq = np.float64(np.float32(theta)) ** (-2.0 * k / n_rot)
    ang = np.arange(max_pos, dtype=np.float64)[:, None] * freq[None, :]
    assert np.array_equal(tab[..., 0], np.cos(ang).astype(np.float32))
    assert np.array_equal(tab[..., 1], np.sin(ang).astype(np.float32))


def test_argument_errors_come_before_any_launch(lib):
    from hipml_amd import attn
    null = C.c_void_p(0)
    one = C.c_void_p(16)  # a non-null, 16-byte aligned value that is never dereferenced on these paths
    # NULL buffers
    rc = lib.hipml_attn_decode_kv(null, null, 0, null, one, one, one, one, one, 24, 4, 256, 64, C.c_float(0.0625), 1, 0, 0)
    assert rc < 0 and b"NULL" in lib.hipml_attn_last_error()
    # unknown cache format
    rc = lib.hipml_attn_decode_kv(null, one, 9, one, one, one, one, one, one, 24, 4, 256, 64, C.c_float(0.0625), 1, 0, 0)
    assert rc == -2 and b"dtype" in lib.hipml_attn_last_error()
    # head geometry the kernels are not built for
    rc = lib.hipml_attn_decode_kv(null, one, 0, one, one, one, one, one, one, 24, 4, 128, 64, C.c_float(0.0625), 1, 0, 0)
    assert rc < 0 and b"head_dim" in lib.hipml_attn_last_error()
    # head_dim 64 is a decode width only (plain fp32 kernels); the chunk entry points are 256 only
    rc = lib.hipml_attn_chunk_q8_split(null, one, one, one, one, 8, 2, 64, 0, 10, 1, 64, null, null, 1)
    assert rc < 0 and b"head_dim" in lib.hipml_attn_last_error()
    # a chunk that does not fit the cache
    rc = lib.hipml_attn_chunk_q8_split(null, one, one, one, one, 24, 4, 256, 60, 10, 1, 64, null, null, 1)
    assert rc < 0 and b"does not fit" in lib.hipml_attn_last_error()
    # key slices without scratch
    rc = lib.hipml_attn_chunk_q8_split(null, one, one, one, one, 24, 4, 256, 0, 10, 1, 64, null, null, 4)
    assert rc < 0 and b"NULL" in lib.hipml_attn_last_error()
    # the Python mirror raises where the reference's launcher returns Err(String)
    with pytest.raises(attn.HipmlError) as e:
        attn._check(rc)
    assert e.value.code == rc


def test_launching_entry_points_ask_for_init_first():
    # the MFMA kernels need the LDS limit that hipml_attn_init raises; without it a call with valid
    # arguments is refused with a message instead of failing inside the launch.  In a process of its own, so
    # that no earlier test has initialised the library (with or without a GPU: the check comes before any launch).
    import subprocess
    import sys
    from hipml_amd import attn
    code = f"""
import ctypes as C
lib = C.CDLL({attn.LIB_PATH!r})
lib.hipml_attn_last_error.restype = C.c_char_p
one = C.c_void_p(16)
rc = lib.hipml_gemv_q8_0_rows(None, one, one, one, 64, 64, 1)
assert rc == -6 and b"hipml_attn_init" in lib.hipml_attn_last_error(), (rc, lib.hipml_attn_last_error())
rc = lib.hipml_attn_decode_kv(None, one, 0, one, one, one, one, one, one, 24, 4, 256, 64, C.c_float(0.0625), 1,
                              C.c_size_t(0), C.c_size_t(0))
assert rc == -6 and b"hipml_attn_init" in lib.hipml_attn_last_error(), (rc, lib.hipml_attn_last_error())
print("refused before init")
"""
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "refused before init" in r.stdout, r.stdout + r.stderr


def test_header_is_plain_c_and_links_from_c(tmp_path):
    # the boundary is a C ABI: a C (not C++) translation unit includes the header, references every
    # declared function and links against the library; it runs the host-only entry points
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no C compiler")
    names = declared_functions()
    refs = "\n".join(f"    p[{i}] = (fn)&{n};" for i, n in enumerate(names))
    src = tmp_path / "abi_check.c"
    src.write_text(f"""
#include <stdio.h>
#include <string.h>
#include "hipml_attn.h"
typedef void (*fn)(void);
int main(void) {{
    fn p[{len(names)}];
{refs}
    for (int i = 0; i < {len(names)}; i++) if (!p[i]) return 2;
    if (strstr(hipml_attn_version(), "gfx950") == NULL) return 3;
    if (hipml_attn_decode_splits(32768, 4) != 128) return 4;
    if (hipml_rope_table_bytes(64, 10) != 10 * 32 * 2 * sizeof(float)) return 5;
    if (hipml_gemv_q8_0_rows(NULL, NULL, NULL, NULL, 1, 64, 1) != HIPML_ATTN_E_NULL) return 6;
    printf("%d functions\\n", {len(names)});
    return 0;
}}
""")
    exe = tmp_path / "abi_check"
    libdir = os.path.join(ROOT, "hipml_amd")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    str(src), "-o", str(exe), "-L", libdir, "-lhipml_attn", f"-Wl,-rpath,{libdir}",
                    "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, capture_output=True, text=True).stdout
    assert out.strip() == f"{len(names)} functions"
