"""CPU-side checks of the product's host logic and of the C-ABI library as a binary:
it loads, exports every declared symbol, and its pure-host entry points answer.
No kernel is launched here."""
import ctypes
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol(dthip):
    header = open(os.path.join(ROOT, "include", "dt_hip.h")).read()
    declared = set(re.findall(r"\b(dt_[a-z0-9_]+)\s*\(", header))
    declared -= {"dt_status", "dt_stream"}
    assert declared == set(dthip.ABI_SYMBOLS), declared ^ set(dthip.ABI_SYMBOLS)
    L = ctypes.CDLL(dthip.LIB_PATH)
    for name in declared:
        assert hasattr(L, name), name


def test_host_only_entry_points(dthip, oracle):
    L = dthip.lib()
    assert b"gfx950" in L.dt_version()
    for q, nib in [(4, 512), (5, 1024), (6, 4096), (7, 64), (8, 16384)]:
        for count in (0, 1, nib - 1, nib, 5 * nib + 3, 3072 * 3072):
            assert dthip.qx_bytes(q, nib, count) == oracle.C.qx_bytes(q, nib, count)
    assert dthip.qx_bytes(3, 32, 10) == -1 and dthip.qx_bytes(9, 32, 10) == -1 and dthip.qx_bytes(6, 0, 10) == -1
    # workspace sizing: nothing needed for the plain call, K' for the fused prep (the queries are normalised and
    # rotated inside the kernel), O for the fused projection
    assert L.dt_sdpa_workspace_bytes(1, 24, 24, 128, 4608, 4608, 0, 0) == 0
    one = 4608 * 24 * 128 * 2
    assert L.dt_sdpa_workspace_bytes(1, 24, 24, 128, 4608, 4608, 1, 0) == one
    assert L.dt_sdpa_workspace_bytes(1, 24, 24, 128, 4608, 4608, 1, 1) == 2 * one


def test_key_split_planning(dthip, monkeypatch):
    """Which attention launches get room for the key-split form (host arithmetic; without a device the plan assumes
    256 compute units): launches of whole or several rounds of workgroups never, launches well under one round with
    enough key tiles do, and the environment knob overrides the estimate either way."""
    L = dthip.lib()
    ws = lambda B, H, D, Sq, Skv: L.dt_sdpa_workspace_bytes(B, H, H, D, Sq, Skv, 0, 0)
    monkeypatch.delenv("DT_SDPA_KEY_SPLIT", raising=False)
    assert ws(1, 24, 128, 4608, 4608) == 0         # 432 workgroups = 1.69 rounds: measured slower when split
    assert ws(1, 24, 128, 16896, 16896) == 0       # 6.19 rounds
    assert ws(2, 8, 40, 4096, 4096) == 0           # exactly one round
    assert ws(2, 8, 40, 4096, 77) == 0             # two key tiles: nothing to cut
    # 64 workgroups of 64 key tiles: one run per compute unit, two partial-result slots each, plus the counters
    slot = (128 // 32 * 16 * 512 + 2 * 512) * 4
    assert ws(1, 4, 128, 4096, 4096) == 256 + 2 * 256 * slot
    # 8 workgroups: at most 8 pieces per task
    assert ws(1, 1, 128, 2048, 16384) == 256 + 2 * 64 * slot
    assert ws(1, 1, 64, 2048, 16384) == 256 + 2 * 64 * (64 // 32 * 16 * 512 + 2 * 512) * 4
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "never")
    assert ws(1, 4, 128, 4096, 4096) == 0
    monkeypatch.setenv("DT_SDPA_KEY_SPLIT", "always")
    assert ws(1, 24, 128, 4608, 4608) == 1792 + 2 * 256 * slot   # 432 counters (1728 bytes), 256-byte aligned
    assert ws(1, 1, 128, 1, 64) == 0                # a single key tile cannot be cut


def test_missing_library_fails_loudly(dthip, monkeypatch):
    monkeypatch.setattr(dthip, "_lib", None)
    monkeypatch.setattr(dthip, "LIB_PATH", os.path.join(ROOT, "no_such_dir", "libdthip.so"))
    with pytest.raises(RuntimeError, match="no CPU or PyTorch fallback"):
        dthip.lib()


@pytest.mark.parametrize("q", [4, 5, 6, 7, 8])
def test_host_packer_matches_oracle(dthip, oracle, q):
    rng = np.random.default_rng(q)
    for n in (0, 1, 7, 8, 9, 31, 32, 33, 1000):
        idx = rng.integers(0, 1 << q, size=n, dtype=np.uint8)
        assert np.array_equal(dthip.pack_indices(q, idx), oracle.C.pack_indices(q, idx))
    for nib, count in [(32, 0), (32, 31), (32, 96), (64, 64 * 3 + 5), (512, 512 * 4)]:
        nblocks = (count + nib - 1) // nib
        pal = (rng.standard_normal((nblocks, 1 << q)) * 0.02).astype(np.float16)
        idx = rng.integers(0, 1 << q, size=count, dtype=np.uint8)
        assert np.array_equal(dthip.pack_qx(q, nib, pal, idx), oracle.C.palettize_pack(q, nib, pal, idx))


def test_rotary_tables_match_oracle(dthip, oracle):
    a = dthip.Flux1RotaryPositionEmbedding(6, 5, 4, channels=128)
    assert np.array_equal(a, oracle.C.rope_flux(6, 5, 4, 128))
    a = dthip.Flux1RotaryPositionEmbedding(4, 4, 2, referenceSizes=[(2, 3), (3, 2), (5, 1)], channels=128)
    assert np.array_equal(a, oracle.C.rope_flux(4, 4, 2, 128, ref_sizes=[(2, 3), (3, 2), (5, 1)]))
    a = dthip.Flux1RotaryPositionEmbedding(3, 7, 0, channels=64)
    assert np.array_equal(a, oracle.C.rope_flux(3, 7, 0, 64))
    w = dthip.WanRotaryPositionEmbedding(4, 5, 3, channels=128)
    assert np.array_equal(w, oracle.C.rope_wan(4, 5, 3, 128))


def test_instruction_counts(dthip, oracle):
    assert dthip.DenseInstructionCount(4608, 3072, 9216) == oracle.C.dense_instruction_count(4608, 3072, 9216)
    assert dthip.ScaledDotProductAttentionInstructionCount(1, 24, 128, 4608, 4608) == \
        oracle.C.sdpa_instruction_count(1, 24, 128, 4608, 4608)


def test_operator_surface_argument_checks(dthip):
    with pytest.raises(dthip.DtError):
        dthip.ScaledDotProductAttention(scale=1.0, isCausal=True)
    d = dthip.Dense(count=8, noBias=True, name="x_q")
    with pytest.raises(RuntimeError, match="weight not loaded"):
        d(None)


def test_header_is_plain_c_and_links(dthip, tmp_path):
    """include/dt_hip.h is what a C (or Swift, through the module map) caller sees: it must compile as C99 on its
    own, and a C program linked against libdthip.so must be able to call the host-only entry points."""
    import shutil
    import subprocess

    cc = shutil.which("gcc") or shutil.which("cc")
    if cc is None:
        pytest.skip("no C compiler")
    src = tmp_path / "abi.c"
    src.write_text(r'''
#include "dt_hip.h"
#include <stdio.h>
#include <string.h>
int main(void) {
  dt_qx_weight w; dt_view4 v; dt_seq_segment s; dt_head_epilogue e; dt_dense_post p; dt_dense_group g;
  memset(&w, 0, sizeof w); memset(&v, 0, sizeof v); memset(&s, 0, sizeof s); memset(&e, 0, sizeof e);
  memset(&p, 0, sizeof p); memset(&g, 0, sizeof g);
  (void)w; (void)v; (void)s; (void)e; (void)p; (void)g;
  /* every entry point is declared with C linkage and takes only plain pointers and sizes */
  typedef void (*fn_t)(void);
  fn_t fns[] = {FNS};
  if (sizeof fns / sizeof fns[0] != NFNS) return 2;
  if (DT_OK != 0 || DT_INVALID != -1 || DT_NO_KERNEL != -2 || DT_OOM != -3) return 3;  /* ccv's exec status values */
  printf("%s %lld %zu\n", dt_version(), (long long)dt_qx_bytes(6, 4096, 3072LL * 3072),
         dt_sdpa_workspace_bytes(1, 24, 24, 128, 4608, 4608, 1, 0));
  return 0;
}
''')
    inc = os.path.join(ROOT, "include")
    text = src.read_text().replace("FNS", ", ".join(f"(fn_t){name}" for name in dthip.ABI_SYMBOLS), 1)
    src.write_text(text.replace("NFNS", str(len(dthip.ABI_SYMBOLS))))
    subprocess.check_call([cc, "-std=c99", "-Wall", "-Werror", "-pedantic", "-fsyntax-only", "-I", inc, str(src)])
    libdir = os.path.dirname(dthip.LIB_PATH)
    exe = tmp_path / "abi"
    subprocess.check_call([cc, "-std=c99", "-I", inc, str(src), "-o", str(exe), "-L", libdir, "-ldthip",
                           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib"])
    out = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert out.returncode == 0, out.stderr
    ver, qx, ws = out.stdout.split()[-3:] if len(out.stdout.split()) >= 3 else (None, None, None)
    assert "gfx950" in out.stdout
    assert int(qx) == dthip.qx_bytes(6, 4096, 3072 * 3072)
    assert int(ws) == 4608 * 24 * 128 * 2


def test_cpp_operator_mirror_compiles(dthip, tmp_path):
    """include/dt_hip.hpp (the C++ operator objects above the C ABI) compiles on its own as C++17 with warnings as
    errors, and the check program built from it exists beside the library after a build."""
    import shutil
    import subprocess

    cxx = shutil.which("g++") or shutil.which("c++")
    if cxx is None:
        pytest.skip("no C++ compiler")
    src = tmp_path / "mirror.cpp"
    src.write_text('#include "dt_hip.hpp"\nint main() { dt::Dense d(8, true); return d.count == 8 ? 0 : 1; }\n')
    subprocess.check_call([cxx, "-std=c++17", "-Wall", "-Wextra", "-Werror", "-fsyntax-only", "-I",
                           os.path.join(ROOT, "include"), str(src)])
    assert os.path.exists(os.path.join(os.path.dirname(dthip.LIB_PATH), "dt_cpp_check"))
