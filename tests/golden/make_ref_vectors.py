"""Writes tests/golden/ref_vectors.npz: inputs and the outputs the reference's own x86 extension
(built by oracle/build_ref.sh into oracle/_ref) produces for them.  Run in the build container only
(`python tests/golden/make_ref_vectors.py`); the committed .npz is plain data and is what travels.

Covered reference entry points: spmm (accumulate branch and overwrite branch,
super_gnn/ops/csrc/spmm.cpp:594-608), the 5-argument x86 quantize_tensor / dequantize_tensor
(super_gnn/ops/csrc/quantization_x86.cpp:17-168) and quantize_tensor_v1 / dequantize_tensor_v1
(quantization_x86.cpp:170-312)."""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
sys.path.insert(0, os.path.dirname(HERE))
from oracle import oracle as orc  # noqa: E402
from _util import random_csr  # noqa: E402


def main():
    ref = orc.ref_ops()
    assert ref is not None, "build oracle/_ref first (make -C oracle ref)"
    out = {}
    rng = np.random.default_rng(1234)
    T = torch.get_num_threads()

    def run_spmm(tag, M, K, F, deg, seed, empty, integer_init=False):
        rowptr, col, val = random_csr(M, K, deg, seed=seed, empty_frac=empty)
        x = rng.standard_normal((K, F), dtype=np.float32)
        init = rng.standard_normal((M, F), dtype=np.float32)
        if integer_init:  # compresses well; the overwrite branch discards it anyway
            init = np.round(init * 4).astype(np.float32)
            x = (np.round(x * 64) / 64).astype(np.float32)
        o = torch.from_numpy(init.copy())
        rs = torch.tensor(np.linspace(0, M, T + 1).astype(np.int32))
        ref.spmm(torch.from_numpy(rowptr), torch.from_numpy(col), torch.from_numpy(val), torch.from_numpy(x), o, M, rs,
                 torch.tensor([0, F], dtype=torch.int32))
        for k, v in dict(rowptr=rowptr, col=col, val=val, x=x, init=init, out=o.numpy()).items():
            out[f"{tag}_{k}"] = v

    run_spmm("spmm_acc", 96, 64, 70, 6, 1, 0.25)       # accumulate branch, F with a masked tail tile
    run_spmm("spmm_acc128", 40, 40, 128, 17, 2, 0.0)   # F = 128 (two full 64-wide tiles)
    # sparsity <= 1e-4 and F > 256: the overwrite branch, with a few dozen edges
    run_spmm("spmm_ovw", 640, 640, 257, 0.06, 3, 0.0, integer_init=True)
    nnz_ovw = out["spmm_ovw_col"].shape[0]
    assert nnz_ovw >= 20 and orc.takes_overwrite_branch(nnz_ovw, 640, 640, 257), nnz_ovw

    for bits in (8, 4, 2):
        n, F = 23, 37  # 23 rows: a short last group for int4 (1 of 2) and int2 (3 of 4)
        x = rng.standard_normal((n, F), dtype=np.float32)
        x[3] = 0.25  # constant row: scale 0 -> 1
        x[5, :4] = [0.0, 255.0, 0.5, 2.5]
        mn = x.min(axis=1)
        sc = ((x.max(axis=1) - mn) / np.float32((1 << bits) - 1)).astype(np.float32)
        sc[sc == 0] = 1.0
        epb = 8 // bits
        q = torch.zeros(((n + epb - 1) // epb) * F, dtype=torch.uint8)
        ref.quantize_tensor(torch.from_numpy(x), q, torch.from_numpy(mn), torch.from_numpy(sc), bits)
        deq = torch.zeros((n, F), dtype=torch.float32)
        ref.dequantize_tensor(q, deq, torch.from_numpy(mn), torch.from_numpy(sc), bits)
        for k, v in dict(x=x, min=mn, scale=sc, q=q.numpy(), deq=deq.numpy()).items():
            out[f"qrows{bits}_{k}"] = v

    n, F = 19, 29
    x = rng.standard_normal((n, F), dtype=np.float32)
    bits_per_row = rng.choice([8, 4, 2], size=n)
    rngs = orc.v1_range(bits_per_row, F)
    params = torch.zeros((n, 3), dtype=torch.float32)
    params[:, 0] = torch.from_numpy(bits_per_row.astype(np.float32))
    q = torch.zeros(int(rngs[-1]), dtype=torch.uint8)
    ref.quantize_tensor_v1(torch.from_numpy(x), q, torch.from_numpy(rngs), params)
    deq = torch.zeros((n, F), dtype=torch.float32)
    ref.dequantize_tensor_v1(q, deq, torch.from_numpy(rngs), params)
    for k, v in dict(x=x, bits=bits_per_row.astype(np.int64), range=rngs, params=params.numpy(), q=q.numpy(), deq=deq.numpy()).items():
        out[f"v1_{k}"] = v

    path = os.path.join(HERE, "ref_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")


if __name__ == "__main__":
    main()
