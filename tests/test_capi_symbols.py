"""The C-ABI library loads on a machine without a GPU and exports every function that
include/sgnn.h declares (no compute call is made here)."""
import ctypes
import os
import re

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared():
    text = open(os.path.join(ROOT, "include", "sgnn.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sgnn_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
    names = _declared()
    for must in ("sgnn_spmm_csr_f32", "sgnn_spmm_plan_create", "sgnn_quant_pack_rows_f32",
                 "sgnn_unpack_dequant_rows_f32", "sgnn_quant_v1_f32", "sgnn_dequant_v1_f32", "sgnn_last_error",
                 "sgnn_spmm_csr_dq_f32", "sgnn_quant_row_slots"):
        assert must in names


def test_library_exports_every_declared_symbol():
    so = os.path.join(ROOT, "super_gnn_amd", "libsgnn_hip.so")
    assert os.path.exists(so), "build first: make -C super_gnn_amd/csrc"
    lib = ctypes.CDLL(so)
    for name in _declared():
        assert hasattr(lib, name), f"{name} declared in include/sgnn.h but not exported"


def test_python_binding_table_matches_header():
    from super_gnn_amd import _lib
    assert sorted(_lib.SIGNATURES) == _declared()


def test_host_only_helpers():
    from super_gnn_amd import _lib
    lib = _lib.lib
    assert lib.sgnn_version() >= 1
    # reference dispatch rule (spmm.cpp:601-602): overwrite iff nnz/M/K <= 1e-4 and F > 256
    assert lib.sgnn_spmm_reference_overwrites(10, 1000, 1000, 257) == 1
    assert lib.sgnn_spmm_reference_overwrites(10, 1000, 1000, 256) == 0
    assert lib.sgnn_spmm_reference_overwrites(1000, 1000, 1000, 602) == 0
    seg = (ctypes.c_int32 * 4)(0, 5, 5, 8)
    pseg = (ctypes.c_int32 * 4)()
    assert lib.sgnn_quant_segment_offsets(seg, 3, 2, pseg) == 3 and list(pseg) == [0, 2, 2, 3]
    assert lib.sgnn_quant_segment_offsets(seg, 3, 4, pseg) == 5 and list(pseg) == [0, 3, 3, 5]
    assert lib.sgnn_quant_segment_offsets(seg, 3, 8, pseg) == 8 and list(pseg) == [0, 5, 5, 8]
    assert lib.sgnn_quant_segment_offsets(seg, 3, 3, pseg) < 0
    assert b"bits" in lib.sgnn_last_error()


def test_facade_helpers_match_reference_closed_forms():
    import torch
    from super_gnn_amd.quantizer import QuantizerForMixedBits, QuantizerForPureBits, Quantizer_for_all_procs
    # tests/test_quantizer.py:29-55 of the reference
    r = QuantizerForMixedBits.get_quantized_nodes_feat_range(6, 4, torch.tensor([8, 4, 2, 8, 4, 2]))
    assert r.tolist() == [0, 4, 6, 7, 11, 13, 14]
    r = QuantizerForMixedBits.get_quantized_nodes_feat_range(3, 3, torch.tensor([4, 4, 2]))
    assert r.tolist() == [0, 2, 4, 5]
    assert QuantizerForPureBits.get_quantized_buffer_size(5, 2, 128) == 2 * 128
    q = Quantizer_for_all_procs(4, 2)
    assert Quantizer_for_all_procs.ctx is q and q.get_quantized_splits(5) == 2 and q.get_quantized_splits(8) == 2
    assert Quantizer_for_all_procs(4, 8).get_quantized_splits(5) == 5


def test_row_split_matches_the_reference_greedy_rule():
    """distribute_work_for_row (super_gnn/ops/spmm_kernel.py:8-29) restated literally as a loop here,
    against the binary-search version the package ships."""
    import numpy as np
    import torch
    from super_gnn_amd.ops.spmm_kernel import distribute_work_for_row, disribute_work_for_col

    def literal(rowptr, value, T):
        flops = [float(value[rowptr[i]:rowptr[i + 1]].sum()) for i in range(len(rowptr) - 1)]
        target = sum(flops) // T
        splits = [len(flops)] * (T + 1)
        splits[0] = 0
        cur, tid = 0.0, 0
        for i, f in enumerate(flops):
            cur += f
            if cur > target and tid < T:
                splits[tid + 1] = i
                tid += 1
                cur = f
        splits[-1] = len(flops)
        return splits

    rng = np.random.default_rng(0)
    for M, T in [(50, 4), (200, 8), (7, 16), (1000, 3)]:
        deg = rng.integers(0, 12, M)
        deg[rng.integers(0, M, 3)] = 80  # rows heavier than the per-thread target
        rowptr = np.concatenate([[0], np.cumsum(deg)])
        value = np.ones(int(rowptr[-1]), dtype=np.float32)  # integer sums: no rounding ambiguity
        got = distribute_work_for_row(torch.from_numpy(rowptr), torch.from_numpy(value), T).tolist()
        assert got == literal(rowptr, value, T), (M, T)
    assert disribute_work_for_col(torch.zeros(3, 128), 1).tolist() == [0, 128]
    assert disribute_work_for_col(torch.zeros(3, 10), 4).tolist() == [0, 2, 4, 6, 10]


def test_package_fails_loudly_without_the_library(tmp_path):
    """No CPU fallback: a copy of the package without libsgnn_hip.so must refuse to import."""
    import shutil
    import subprocess
    import sys
    pkg = os.path.join(ROOT, "super_gnn_amd")
    shutil.copytree(pkg, tmp_path / "super_gnn_amd",
                    ignore=shutil.ignore_patterns("*.so", "csrc", "__pycache__", "obj"))
    r = subprocess.run([sys.executable, "-c", "import super_gnn_amd"], cwd=tmp_path, capture_output=True, text=True,
                       env={**os.environ, "PYTHONPATH": str(tmp_path)})
    assert r.returncode != 0
    assert "libsgnn_hip" in r.stderr


def test_product_never_imports_the_oracle():
    """The oracle is test infrastructure: nothing under super_gnn_amd/ may import or load it."""
    import re
    pkg = os.path.join(ROOT, "super_gnn_amd")
    for base, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".hpp")):
                text = open(os.path.join(base, f)).read()
                assert not re.search(r"^\s*(from|import)\s+oracle\b", text, re.M), f
                assert "liborc" not in text and "oracle/" not in text, f
