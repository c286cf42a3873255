"""CPU-side checks: the C-ABI library loads and exports every symbol include/vtkv.h declares (no
compute call is made), the ctypes table matches the header, host-side helpers behave, and the
product package has no path into the oracle."""
import ctypes
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "vtkv.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(vtkv_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ("vtkv_reshape_and_cache", "vtkv_decode_attention", "vtkv_swap_ranges", "vtkv_swap_blocks",
                 "vtkv_copy_blocks", "vtkv_convert_fp8", "vtkv_pool_init", "vtkv_seg_create",
                 "vtkv_extend_kv_cache_batch"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from glake_amd import _C

    assert os.path.exists(_C.LIB_PATH), "libvtkv.so has not been built (python -m glake_amd.build)"
    lib = ctypes.CDLL(_C.LIB_PATH)
    for name in declared_functions():
        assert hasattr(lib, name), f"{name} is declared in include/vtkv.h but not exported"


def test_ctypes_table_matches_header():
    from glake_amd import _C

    assert sorted(_C.SIGNATURES) == declared_functions()
    text = re.sub(r"/\*.*?\*/", "", open(os.path.join(ROOT, "include", "vtkv.h")).read(), flags=re.S)
    for name, (_, args) in _C.SIGNATURES.items():
        m = re.search(r"\b" + name + r"\s*\(([^;]*?)\)\s*;", text, flags=re.S)
        assert m, name
        params = m.group(1).strip()
        n = 0 if params in ("", "void") else params.count(",") + 1
        assert n == len(args), f"{name}: header has {n} parameters, ctypes table {len(args)}"


def test_version_and_constants_without_a_gpu():
    from glake_amd import _C

    lib = _C.lib()
    assert lib.vtkv_version() >= 100
    assert lib.vtkv_chunk_bytes() == 2 * 1024 * 1024
    ws = lib.vtkv_decode_attention_workspace_bytes
    assert ws(64, 32, 128, 4096, 0) > 64 * 32 * 130 * 4       # at least one partial per (sequence, head)
    assert ws(64, 32, 128, 4096, 256) > ws(64, 32, 128, 4096, 1024) > 0   # smaller spans, more partials
    assert ws(0, 32, 128, 4096, 0) == 0


def test_host_arena_first_fit_and_coalescing():
    from glake_amd.worker.cache_engine import _HostArena

    a = _HostArena(0)          # no pinned allocation: only the bookkeeping is exercised
    a.nbytes, a.free = 4096, [(0, 4096)]
    x = a.alloc(1000)          # rounds to 1024
    y = a.alloc(1024)
    z = a.alloc(2048)
    assert (x, y, z) == (0, 1024, 2048) and a.free == []
    from glake_amd._C import VtkvOutOfChunks
    with pytest.raises(VtkvOutOfChunks):
        a.alloc(1)
    a.release(y, 1024)
    a.release(x, 1000)
    assert a.free == [(0, 2048)]
    a.release(z, 2048)
    assert a.free == [(0, 4096)]


def test_ops_refuse_host_tensors_and_bad_arguments():
    import torch

    from glake_amd import _C, _custom_ops as ops

    k = torch.zeros(2, 8, 128, dtype=torch.bfloat16)
    with pytest.raises(_C.VtkvError):
        ops.reshape_and_cache(k, k, 0, 0, torch.zeros(2, dtype=torch.int64), torch.zeros(2, dtype=torch.int64), None,
                              None, 1, 8, 128)
    with pytest.raises(_C.VtkvError, match="block size"):
        ops.paged_attention_v1(k, k, 0, 0, 8, 1.0, torch.zeros(2, dtype=torch.int32), 16, 1, None, "auto", 1.0,
                               torch.zeros(2, dtype=torch.int64))
    with pytest.raises(_C.VtkvError, match="Invalid device combination"):
        ops.swap_blocks(k, k, torch.zeros(1, 2, dtype=torch.int64))


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from glake_amd import _C

    monkeypatch.setattr(_C, "_lib", None)
    monkeypatch.setattr(_C, "LIB_PATH", str(tmp_path / "libvtkv.so"))
    with pytest.raises(_C.VtkvLibraryMissing):
        _C.lib()


def test_product_package_never_touches_the_oracle():
    pkg = os.path.join(ROOT, "glake_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text.replace("the oracle", ""), f"{f} mentions the oracle"


def test_one_hip_runtime_whichever_import_comes_first():
    """PyTorch ships its own copy of the HIP runtime; the library has to end up on the same copy, or a
    torch stream handed to it would belong to another runtime."""
    code = ("from glake_amd import _C; _C.lib(); import torch\n"
            "libs = sorted({l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l})\n"
            "print(len(libs), libs)")
    r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, cwd=ROOT)
    assert r.returncode == 0, r.stderr
    assert r.stdout.split()[0] == "1", r.stdout


def test_bench_refuses_more_than_one_gpu():
    r = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert r.returncode != 0 and "one GPU" in r.stderr


def test_prefill_units_cover_every_query_token_once():
    """Host logic of the prompt attention: the unit table (sequence, first query row, tokens, position of
    the first token) covers each packed query row exactly once, keeps units inside one sequence, respects
    the per-unit limit, places chunk queries at the end of their sequence and lists the units in the documented order."""
    import numpy as np

    from glake_amd._custom_ops import prefill_units

    query_lens, seq_lens = [5, 0, 130, 1, 64], [5, 9, 400, 77, 64]
    for per_unit in (1, 4, 16, 32, 128):
        u = prefill_units(query_lens, seq_lens, per_unit)
        assert u.dtype == np.int32 and u.shape[1] == 4 and (u[:, 2] >= 1).all() and (u[:, 2] <= per_unit).all()
        seen = np.zeros(sum(query_lens), int)
        starts = np.concatenate([[0], np.cumsum(query_lens)])
        for b, row0, ntok, pos0 in u.tolist():
            seen[row0:row0 + ntok] += 1
            assert starts[b] <= row0 and row0 + ntok <= starts[b + 1]                 # inside its sequence
            assert pos0 == seq_lens[b] - query_lens[b] + (row0 - starts[b])           # lower-right aligned
        assert (seen == 1).all()
        # sequence by sequence, the longest context first inside each; "rows": longest first over the batch
        assert (np.diff(u[:, 0]) >= 0).all()
        for b in set(u[:, 0].tolist()):
            own = u[u[:, 0] == b]
            assert (np.diff(own[:, 2] + own[:, 3]) <= 0).all()
        by_rows = prefill_units(query_lens, seq_lens, per_unit, order="rows")
        assert (np.diff(by_rows[:, 2] + by_rows[:, 3]) <= 0).all()
        assert sorted(map(tuple, by_rows.tolist())) == sorted(map(tuple, u.tolist()))
    assert prefill_units([], [], 4).shape == (0, 4)
    import pytest

    from glake_amd import _C
    with pytest.raises(_C.VtkvError):
        prefill_units([5], [4], 4)                                                     # more queries than rows

