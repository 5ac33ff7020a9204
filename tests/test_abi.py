"""CPU-side checks of the drop-in boundary: libmbx.so loads without a GPU, exports every symbol
declared in include/mbx.h, its scratch-size helpers work, and the host wrappers validate
arguments the way the reference's wrappers do.  No kernel is launched here."""
import ctypes
import os
import re

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, 'include', 'mbx.h')


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r'/\*.*?\*/', '', text, flags=re.S)
    return sorted(set(re.findall(r'\b(mbx_[a-z0-9_]+)\s*\(', text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for required in ['mbx_histogram', 'mbx_sort', 'mbx_sort_scratch_bytes', 'mbx_cumsum', 'mbx_topology',
                     'mbx_replicate_forward', 'mbx_replicate_backward', 'mbx_gather', 'mbx_slot_rows', 'mbx_scatter',
                     'mbx_scatter_wgrad', 'mbx_scatter_backward', 'mbx_binned_gather', 'mbx_binned_scatter', 'mbx_binned_scatter_wgrad',
                     'mbx_gmm', 'mbx_gelu_backward_inplace', 'mbx_error_string', 'mbx_version']:
        assert required in names


def test_library_loads_and_exports_every_declared_symbol():
    from megablocks_amd import _lib
    assert os.path.exists(_lib.LIB_PATH)
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(raw, name), f'{name} is declared in include/mbx.h but not exported'
    assert set(_lib._SIGNATURES) == set(declared_symbols())     # the ctypes table covers the whole header
    assert _lib.lib.mbx_version() >= 1


def test_error_strings_and_scratch_sizes():
    from megablocks_amd._lib import lib
    assert lib.mbx_error_string(0) == b'success'
    assert b'invalid' in lib.mbx_error_string(-1)
    assert b'scratch' in lib.mbx_error_string(-2)
    assert lib.mbx_sort_scratch_bytes(0, 1, 32) == 0
    one = lib.mbx_sort_scratch_bytes(16384, 1, 6)               # one radix pass: only the count table
    four = lib.mbx_sort_scratch_bytes(16384, 1, 32)             # four passes: plus two ping-pong buffers
    assert 0 < one < four and four >= one + 2 * 16384 * 4
    assert lib.mbx_sort_scratch_bytes(16384, 1, 0) == 0


def test_argument_errors_are_reported_without_touching_the_gpu():
    from megablocks_amd._lib import lib
    assert lib.mbx_histogram(None, 7, 1, 1, 4, None, None) == -1           # bad itype / null out
    assert lib.mbx_gmm(None, None, None, 0, None, 4, 16, 8, 8, 9, None) == -1   # bad layout
    assert lib.mbx_gmm(None, None, None, 0, None, 0, 0, 8, 8, 0, None) == 0     # no groups: nothing to do
    assert lib.mbx_sort(None, 1, 0, 32, None, None, None, 0, None) == 0         # empty input early-out
    assert lib.mbx_cumsum(None, 1, -1, 4, 0, None, None) == -1
    # mbx_gmm_gather(x, x_rows, indices, top_k, x_bins, b1, b2, c, c2, h, dtype, bins, groups, rows, k, n, act, stream)
    assert lib.mbx_gmm_gather(None, 8, None, 0, None, None, None, None, None, None, 0, None, 2, 16, 64, 8, 0, None) == -1  # top_k
    assert lib.mbx_gmm_gather(None, 8, None, 2, None, None, None, None, None, None, 0, None, 2, 0, 64, 8, 0, None) == 0    # no rows
    assert lib.mbx_gmm_gather(None, 8, None, 2, None, None, None, None, None, None, 0, None, 2, 16, 64, 8, 0, None) == -1  # null map
    # more tokens than 31 bits of byte offsets address: the caller gathers first
    assert lib.mbx_gmm_gather(1, 1 << 22, 1, 2, None, 1, None, 1, None, None, 0, 1, 2, 16, 4096, 8, 0, None) == -4


def test_host_wrappers_validate_like_the_reference():
    import megablocks_amd.ops as ops
    from megablocks_amd.backend import kernels
    x = torch.zeros(4, 8)
    idx = torch.zeros(4, dtype=torch.int32)
    bins = torch.tensor([4], dtype=torch.int32)
    with pytest.raises(ValueError):                              # backend/kernels.py:9-25 shape checks
        kernels.gather(x.view(-1), idx, idx, None, bins, 1)
    with pytest.raises(ValueError):
        kernels.gather(x, idx[:2], idx, None, bins, 1)
    with pytest.raises(ValueError):
        kernels.padded_scatter(x, idx, idx[:1], None, bins, bins, 1)
    with pytest.raises(RuntimeError):                            # TORCH_CHECK(x.is_cuda()) in csrc/*.h
        ops.histogram(idx, 4)
    with pytest.raises(RuntimeError):
        ops.sort(idx)
    with pytest.raises(RuntimeError):
        ops.inclusive_cumsum(idx, 0)
    with pytest.raises(AssertionError):
        ops.round_up(idx.long(), 128)                            # ops/round_up.py:9
    assert ops.round_up(torch.tensor([1, 128, 129], dtype=torch.int32), 128).tolist() == [128, 128, 256]
    assert ops.repeat(x, (1, 1)) is x and ops.repeat(x, (2, 1)).shape == (8, 8)
    assert ops.sum(x.view(1, 4, 8)).shape == (4, 8) and ops.sum(x, 0).shape == (8,)


def test_arguments_defaults_match_the_reference():
    from megablocks_amd.layers.arguments import DEFAULT_ACTIVATION_FN, Arguments
    a = Arguments(device=torch.device('cpu'))
    assert (a.hidden_size, a.ffn_hidden_size, a.moe_num_experts, a.moe_top_k) == (1024, 4096, 1, 1)
    assert a.fp16 and not a.bf16 and a.bias and a.return_bias                     # arguments.py:28-29,53-54
    assert a.mlp_type == 'mlp' and a.mlp_impl == 'grouped' and not a.memory_optimized_mlp
    assert a.activation_fn is DEFAULT_ACTIVATION_FN and a.moe_loss_weight == 0.1
    assert a.shared_expert_hidden_size == a.ffn_hidden_size
    with pytest.raises(NotImplementedError):
        Arguments(device=torch.device('cpu'), moe_expert_model_parallelism=True)


def test_synthetic_workloads_match_the_stated_sizes():
    from megablocks_amd import synthetic
    w = synthetic.WORKLOADS
    assert abs(w['c3'].gemm_flops() / 1.732e13 - 1) < 1e-3 and abs(w['c2'].gemm_flops() / 8.25e11 - 1) < 1e-2
    assert abs(w['c4'].gemm_flops() / 1.020e13 - 1) < 1e-2 and abs(w['c5'].gemm_flops() / 1.979e13 - 1) < 1e-3
    assert abs(w['c3'].permute_bytes() / 1.007e9 - 1) < 1e-3 and abs(w['c4'].permute_bytes() / 4.698e9 - 1) < 1e-3
    small = synthetic.Workload('s', 2048, 64, 128, 64, 6, 'glu', 'grouped', torch.bfloat16, 'zipf')
    inp = synthetic.make_inputs(small)
    te = inp['top_experts']
    assert te.shape == (2048, 6) and all(len(set(r)) == 6 for r in te[:50].tolist())   # distinct experts per token
    counts = torch.bincount(te.flatten(), minlength=64)
    assert int((counts == 0).sum()) == 4                                           # four empty experts
    assert torch.allclose(inp['expert_weights'].sum(-1), torch.ones(2048), atol=1e-5)


def test_bench_refuses_more_than_one_gpu():
    """The benchmark measures one GPU holding all experts; asking for more ends with a message, not a number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    run = subprocess.run([sys.executable, os.path.join(root, 'bench.py'), '--gpus', '2'], capture_output=True, text=True,
                         timeout=120)
    assert run.returncode != 0
    assert 'one GPU' in run.stderr and run.stdout.strip() == ''
