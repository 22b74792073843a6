"""Code written against the reference's module names runs on this build through the import shims in
super_gnn_amd/compat.  The two tests below follow the call sequences of the reference's
tests/test_spmm.py (:69-114) and tests/test_quantization_ops.py (:130-228, :362-390) with CPU tensors,
as those files do; expected values come from scipy / the CPU oracle, not from the shims."""
import math
import os
import sys

import numpy as np
import pytest
import scipy.sparse as sci_sp
import torch

from oracle import oracle as orc

pytestmark = pytest.mark.gpu
COMPAT = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "super_gnn_amd", "compat")


@pytest.fixture()
def compat_path():
    sys.path.insert(0, COMPAT)
    yield
    sys.path.remove(COMPAT)
    for name in [m for m in sys.modules if m.split(".")[0] in ("supergnn_ops", "torch_sparse", "torch_scatter", "super_gnn")]:
        del sys.modules[name]


def test_spmm_recipe_with_reference_import_names(compat_path):
    from torch_scatter import segment_csr
    from torch_sparse.matmul import matmul
    from torch_sparse.tensor import SparseTensor
    from super_gnn.ops.spmm_kernel import SPMM_forward, SPMM_backward

    A = sci_sp.rand(20020, 1020, density=0.0007, format="csr", dtype=np.float32, random_state=3)
    src = SparseTensor.from_scipy(A).requires_grad_()
    other = torch.rand(1020, 128).requires_grad_()
    rowptr, col, value = src.csr()
    assert torch.allclose(segment_csr(value, rowptr, None, "sum"), torch.from_numpy(np.asarray(A.sum(axis=1)).ravel()), atol=1e-5)

    expected = matmul(src, other, "sum")
    out = torch.zeros((20020, 128), dtype=torch.float32)
    SPMM_forward(src, other, out)
    grad_out = torch.randn_like(expected)
    expected.backward(grad_out)
    other_grad = torch.zeros((1020, 128), dtype=torch.float32)
    SPMM_backward(src, grad_out, other_grad)
    assert torch.allclose(expected, out, atol=1e-5)
    assert torch.allclose(other.grad, other_grad, atol=1e-5)
    # independent expected values
    assert torch.allclose(torch.from_numpy(A @ other.detach().numpy()), out, atol=1e-5)
    assert torch.allclose(torch.from_numpy(A.T.tocsr() @ grad_out.numpy()), other_grad, atol=1e-4)


@pytest.mark.parametrize("bits", [8, 2])
def test_quantization_script_flow_with_reference_import_names(compat_path, bits):
    import supergnn_ops

    num_nodes, feat_len = 4333, 123
    data_fp32 = torch.randn((num_nodes, feat_len), generator=torch.Generator().manual_seed(bits))
    # row-packed, one segment
    data_int8 = torch.empty((math.ceil(num_nodes / float(8 / bits)) * feat_len), dtype=torch.uint8)
    quantized_params = torch.empty((num_nodes, 2), dtype=torch.float32)
    supergnn_ops.quantize_tensor(data_fp32, data_int8, quantized_params, bits)
    deq_row = torch.empty((num_nodes, feat_len))
    supergnn_ops.dequantize_tensor(data_int8, deq_row, quantized_params, bits)
    # feature-packed with a uniform bit width
    params3 = torch.empty((num_nodes, 3)); params3[:, 0] = bits
    rng = torch.full((num_nodes + 1,), feat_len, dtype=torch.int64); rng[0] = 0
    rng[1:] = torch.ceil(rng[1:] * bits / 8.0)
    rng = torch.cumsum(rng, 0)
    q_col = torch.empty(int(rng[-1]), dtype=torch.uint8)
    supergnn_ops.quantize_tensor_v1(data_fp32, q_col, rng, params3)
    deq_col = torch.empty((num_nodes, feat_len))
    supergnn_ops.dequantize_tensor_v1(q_col, deq_col, rng, params3)
    # 256 random destination segments
    num_procs = 256
    wr = torch.randint(0, num_nodes, (num_procs + 1,), dtype=torch.int32, generator=torch.Generator().manual_seed(1)).sort()[0]
    wr[0] = 0; wr[-1] = num_nodes
    sizes = [math.ceil(int(wr[i + 1] - wr[i]) / float(8 / bits)) * feat_len for i in range(num_procs)]
    q_all = torch.empty(sum(sizes), dtype=torch.uint8)
    p_all = torch.empty((num_nodes, 2))
    supergnn_ops.quantize_tensor_for_all_procs(data_fp32, q_all, p_all, wr, num_procs, bits)
    deq_all = torch.empty((num_nodes, feat_len))
    supergnn_ops.dequantize_tensor_for_all_procs(q_all, deq_all, p_all, wr, num_procs, bits)

    # the comparisons the script prints, asserted (atol 1e-6 / rtol 1e-5 as in its diff()):
    assert torch.equal(p_all[:, 0], params3[:, 1]) and torch.equal(p_all[:, 1], params3[:, 2])
    assert torch.allclose(deq_row, deq_col, atol=1e-6, rtol=1e-5)
    assert torch.allclose(deq_col, deq_all, atol=1e-6, rtol=1e-5)
    parts = []
    for i in range(num_procs):
        xs = data_fp32[wr[i]:wr[i + 1]]
        qi = torch.empty(sizes[i], dtype=torch.uint8)
        pi = torch.empty((xs.shape[0], 2))
        supergnn_ops.quantize_tensor(xs, qi, pi, bits)
        parts.append(qi)
    assert torch.equal(q_all, torch.cat(parts))
    # and against the oracle
    q_ref, p_ref = orc.quant_rows(data_fp32.numpy(), wr.numpy(), bits)
    assert np.array_equal(q_all.numpy(), q_ref.reshape(-1)) and np.array_equal(p_all.numpy(), p_ref)
    if bits == 8:  # the script's torch.quantize_per_channel cross-check (codes only)
        scale = (data_fp32.max(dim=1)[0] - data_fp32.min(dim=1)[0]) / (2 ** bits - 1)
        codes = torch.round((data_fp32 - data_fp32.min(dim=1, keepdim=True)[0]) / scale[:, None]).to(torch.uint8)
        assert torch.equal(data_int8.view(num_nodes, feat_len), codes)


def test_aggregation_layer_with_reference_import_names(compat_path):
    # the reference's layer code: `from super_gnn.aggregator import Aggregator`, `Aggregator.apply(graph, feat, layer,
    # num_bits, is_pre_delay, training)` (layers/sageconv.py:56-60) on a partition that is the whole graph (world_size 1)
    from super_gnn.aggregator import Aggregator
    from super_gnn.data_manager import DistributedGraph
    from super_gnn.layers.sageconv import DistSAGEConvGrad
    from super_gnn_amd.data_manager import build_loopback_partitions
    from super_gnn_amd import synth
    rowptr, col = synth.uniform_degree_graph(3000, 9, seed=2)
    graph = build_loopback_partitions(rowptr, col.to(torch.int64), None, 1, 64, num_bits=32, is_pre_delay=False)[0]
    assert isinstance(graph, DistributedGraph)
    x = torch.randn(3000, 64, generator=torch.Generator().manual_seed(0))
    out = Aggregator.apply(graph, x.cuda(), 0, 32, False, True)
    want = np.zeros((3000, 64), np.float32)
    orc.spmm_accumulate(rowptr.numpy(), col.numpy().astype(np.int64), np.ones(col.numel(), np.float32), x.numpy(), want)
    assert np.array_equal(out.cpu().numpy(), want)      # 10 edges per row: the reference's fma chain, bit for bit
    conv = DistSAGEConvGrad(64, 16, 32, False).cuda()
    y = conv(graph, x.cuda(), 0)
    ref = (torch.from_numpy(want).cuda() / graph.in_degrees) @ conv.lin_neigh.weight.t() + x.cuda() @ conv.lin_self.weight.t() + conv.bias
    assert torch.allclose(y, ref, rtol=1e-4, atol=1e-4)
