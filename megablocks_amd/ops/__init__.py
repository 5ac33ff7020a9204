"""The operator surface of megablocks.ops (megablocks/ops/__init__.py:4-35), MI355X-native."""
from megablocks_amd.ops.permute import (binned_gather, binned_scatter, gather, padded_gather, padded_scatter,
                                        scatter)
from megablocks_amd.ops.routing import (exclusive_cumsum, histogram, inclusive_cumsum, repeat, replicate, round_up,
                                        sort, sum, topology)

__all__ = [
    'binned_gather', 'binned_scatter', 'exclusive_cumsum', 'inclusive_cumsum', 'gather', 'histogram',
    'padded_gather', 'padded_scatter', 'repeat', 'replicate', 'round_up', 'scatter', 'sort', 'sum', 'topology',
]
