"""The dropless MoE layer: megablocks/layers/dmoe.py.

    grouped:  sort/histogram/cumsum -> gather -> grouped MLP -> weighted scatter
    sparse:   the same over 128-padded expert groups, with the block-diagonal topology
              metadata the reference builds for stk
"""
import numpy as np
import torch

import megablocks_amd.ops as ops
from megablocks_amd.ops import routing as ops_routing
from megablocks_amd import grouped_gemm_util as gg
from megablocks_amd.layers import common, dmlp_registry, moe, mpu
from megablocks_amd.layers.arguments import Arguments
from megablocks_amd.layers.mlp import Topology


def promote_scalar(x):
    return x.view(1) if not len(x.size()) else x


class ParallelDroplessMLP(moe.ParallelMLP):

    _builds_dense_mlp = False   # the reference builds a dense MLP here and replaces it at once (dmoe.py:25)

    def __init__(self, args: Arguments):
        super().__init__(args)
        self.hidden_size = args.hidden_size
        self.ffn_hidden_size = mpu.features_per_rank(args)
        self.blocking = 128
        self.mlp = dmlp_registry.get(args)
        # bits needed for a block-column index of the intermediate sparse matrix (dmoe.py:27-33)
        max_column_index = (self.ffn_hidden_size * self.num_experts) // self.blocking
        self.transpose_sort_end_bit = max(int(np.ceil(np.log2(max(max_column_index, 1)))), 1)

    def sparse_transpose(self, size, row_indices, column_indices, offsets):
        """dmoe.py:35-66: metadata of the transposed block-sparse matrix."""
        block_columns = size[1] // self.blocking
        _, gather_indices = ops.sort(column_indices.int(), self.transpose_sort_end_bit)
        column_indices_t = row_indices.gather(0, gather_indices.long())
        block_offsets_t = gather_indices.int()
        zero = torch.zeros((1,), dtype=torch.int32, device=row_indices.device)
        nnz_per_column = ops.histogram(column_indices, block_columns)
        nnz_per_column = ops.inclusive_cumsum(nnz_per_column, 0)
        if nnz_per_column.dim() == 0:
            nnz_per_column = nnz_per_column.unsqueeze(0)
        offsets_t = torch.cat([zero, nnz_per_column])
        return column_indices_t, offsets_t, block_offsets_t

    def topology(self, x, padded_bins):
        """dmoe.py:68-129."""
        padded_tokens, _ = x.size()
        assert padded_tokens % self.blocking == 0
        if self.ffn_hidden_size % self.blocking != 0:
            raise ValueError(f'The ffn_hidden_size {self.ffn_hidden_size} must be divisible by ' +
                             f'the block size {self.blocking}. Please update your configuration.')
        block_rows = padded_tokens // self.blocking
        blocks_per_row = self.ffn_hidden_size // self.blocking
        shape = (padded_tokens, self.ffn_hidden_size * mpu.experts_per_rank(self.args))
        device = x.device

        def index_arrays():
            offsets = torch.arange(0, block_rows * blocks_per_row + 1, blocks_per_row, dtype=torch.int32, device=device)
            column_indices = ops.topology(padded_bins, self.blocking, block_rows, blocks_per_row)
            # every block-row holds blocks_per_row blocks, so block b lies in block-row b // blocks_per_row
            row_indices = torch.arange(block_rows, dtype=torch.int32, device=device).repeat_interleave(
                blocks_per_row).to(torch.int16)
            column_indices_t, offsets_t, block_offsets_t = self.sparse_transpose(shape, row_indices, column_indices,
                                                                                 offsets)
            return dict(row_indices=row_indices, column_indices=column_indices, offsets=offsets,
                        column_indices_t=column_indices_t, offsets_t=offsets_t, block_offsets_t=block_offsets_t)

        padded_tokens_per_expert = torch.diff(padded_bins, prepend=padded_bins.new_zeros(1))
        gg.note_bins(padded_tokens_per_expert, padded_bins)    # the row bins of this step's grouped products
        return Topology(shape, self.blocking, padded_tokens_per_expert, index_arrays)

    def indices_and_padded_bins(self, top_experts):
        """dmoe.py:131-154."""
        top_experts = top_experts.int()
        if ops_routing.route_supported(top_experts, self.num_experts, self.sort_end_bit):
            indices, bin_ids, tokens_per_expert, bins, padded_bins = ops_routing.route(
                top_experts, self.num_experts, self.sort_end_bit, self.blocking)
            return indices, bin_ids, bins, padded_bins, tokens_per_expert
        bin_ids, indices = ops.sort(top_experts, self.sort_end_bit)
        tokens_per_expert = ops.histogram(top_experts, self.num_experts)
        padded_tokens_per_expert = ops.round_up(tokens_per_expert, self.blocking)
        padded_bins = promote_scalar(ops.inclusive_cumsum(padded_tokens_per_expert, 0))
        bins = promote_scalar(ops.inclusive_cumsum(tokens_per_expert, 0))
        return indices, bin_ids, bins, padded_bins, tokens_per_expert

    FUSE_GATHER_IN_TRAINING_FROM_TOP_K = 4

    def _fuse_gather(self, x, top_k):
        """Whether the experts get the ungathered tokens (gg.FUSED_GATHER): the built-in experts on the GPU only.  'auto':
        always without gradients; with them from top_k = 4 on, where the step is faster (the weight gradients then read
        the tokens through a row table, 1 - 4 % slower than from a copy; the gather kernel and the copy of top_k times
        the input's size, otherwise kept for the backward pass, are gone: 32768 tokens, top-6 of 64 experts: -1.2 % per
        step, 24576 tokens top-4: -0.15 %).  At top_k = 2 the step takes the same time either way ('1' then saves the
        memory of the copy), at top_k = 1 the gather is cheaper than what the indexed weight gradient loses."""
        if gg.FUSED_GATHER == '0' or not x.is_cuda or not hasattr(self.mlp, 'forward_tokens'):
            return False
        if gg.FUSED_GATHER == 'auto' and top_k < self.FUSE_GATHER_IN_TRAINING_FROM_TOP_K:
            return not (torch.is_grad_enabled() and (x.requires_grad or any(p.requires_grad for p in self.mlp.parameters())))
        return True

    def _mlp_takes_combine(self):
        """Whether the experts' forward / forward_tokens accept the layer's combine (the built-in grouped experts do; an
        expert class from the registry that overrides forward without it gets ops.scatter as before)."""
        known = getattr(self, '_takes_combine', None)
        if known is None:
            import inspect
            mlp = self.mlp
            known = bool(getattr(mlp, 'takes_combine', False)) and all(
                'combine' in inspect.signature(getattr(mlp, name)).parameters for name in ('forward', 'forward_tokens'))
            self._takes_combine = known
        return known

    def _sparse_experts(self, x, indices, bin_ids, bins, padded_bins, top_k):
        """dmoe.py:219-226: padded gather, topology, experts.  Where the experts take the ungathered tokens the gather
        is part of their first product."""
        if self._fuse_gather(x, top_k):
            padded_rows = int(padded_bins[-1].item()) if padded_bins.numel() else 0   # as ops.padded_gather reads it
            with torch.no_grad():
                topo = self.topology(x.new_empty((padded_rows, 0)), padded_bins)
            src = gg.GatheredRows(x, indices, bin_ids, bins, padded_bins, top_k, padded_rows)
            out = self.mlp.forward_tokens(src, topo.padded_tokens_per_expert)
            if out is not None:
                return out
        x = ops.padded_gather(x, indices, bin_ids, bins, padded_bins, top_k)
        with torch.no_grad():
            topo = self.topology(x, padded_bins)
        return self.mlp(x, topo)

    def sparse_forward_once(self, x, expert_weights, top_experts):
        """dmoe.py:156-193."""
        expert_weights = expert_weights.flatten()
        top_experts = top_experts.flatten()
        with torch.no_grad():
            indices, bin_ids, bins, padded_bins, tokens_per_expert = self.indices_and_padded_bins(top_experts)
        x = x.view(-1, x.shape[-1])
        x = self._sparse_experts(x, indices, bin_ids, bins, padded_bins, self.top_k)
        x = ops.padded_scatter(x, indices, bin_ids, expert_weights, bins, padded_bins, self.top_k)
        return x, tokens_per_expert

    def sparse_permute_and_compute(self, x, tokens_per_expert, indices, bin_ids, expert_weights, bins,
                                   expert_capactiy, top_k):
        """dmoe.py:196-237."""
        padded_tokens_per_expert = ops.round_up(tokens_per_expert, self.blocking)
        padded_bins = promote_scalar(ops.inclusive_cumsum(padded_tokens_per_expert, 0))
        x = x.view(-1, x.shape[-1])
        x = self._sparse_experts(x, indices, bin_ids, bins, padded_bins, top_k)
        return ops.padded_scatter(x, indices, bin_ids, expert_weights, bins, padded_bins, top_k)

    def grouped_forward_once(self, x, expert_weights, top_experts):
        """dmoe.py:239-258."""
        expert_weights = expert_weights.flatten()
        top_experts = top_experts.flatten()
        with torch.no_grad():
            indices, bin_ids, bins, tokens_per_expert = self.indices_and_bins(top_experts)
        out = self.grouped_permute_and_compute(x, tokens_per_expert, indices, bin_ids, expert_weights, bins, -1,
                                               self.args.moe_top_k)
        return out, tokens_per_expert

    def grouped_permute_and_compute(self, x, tokens_per_expert, indices, bin_ids, expert_weights, bins,
                                    expert_capactiy, top_k):
        """dmoe.py:260-280."""
        x = x.view(-1, x.shape[-1])
        # One expert per token: the combine is one output row per product row, and the built-in experts write it from
        # the store phase of their second product (gg.FUSED_COMBINE).
        combine = None
        if top_k == 1 and gg.FUSED_COMBINE != '0' and x.is_cuda and self._mlp_takes_combine() and \
                indices.dtype == torch.int32:
            combine = gg.CombinedRows(indices, bin_ids, bins, expert_weights)
        extra = () if combine is None else (combine,)
        out = None
        if self._fuse_gather(x, top_k):
            src = gg.GatheredRows(x, indices, bin_ids, bins, None, top_k, indices.shape[0])
            out = self.mlp.forward_tokens(src, tokens_per_expert, *extra)
        if out is None:
            x = ops.gather(x, indices, bin_ids, bins, top_k)
            out = self.mlp(x, tokens_per_expert, *extra)
        if combine is not None:
            return out
        return ops.scatter(out, indices, bin_ids, expert_weights, bins, top_k)

    def forward_once(self, x, expert_weights, top_experts):
        if self.args.mlp_impl == 'sparse':
            return self.sparse_forward_once(x, expert_weights, top_experts)
        return self.grouped_forward_once(x, expert_weights, top_experts)

    def permute_and_compute(self, x, tokens_per_expert, indices, bin_ids, expert_weights, bins, expert_capactiy,
                            top_k):
        fn = self.sparse_permute_and_compute if self.args.mlp_impl == 'sparse' else self.grouped_permute_and_compute
        return fn(x, tokens_per_expert, indices, bin_ids, expert_weights, bins, expert_capactiy, top_k)


class dMoE(moe.MoE):

    def _init_experts_mlp(self, args: Arguments):
        return ParallelDroplessMLP(args)
