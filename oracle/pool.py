"""CPU restatement of the reference's pooling over a kernel map.

TEST INFRASTRUCTURE ONLY.

Follows warpconvnet/nn/functional/sparse_pool.py:84-104: the pairs of all offsets are grouped by
output row (`IntSearchResult.to_csr`, search_results.py:136-160) and every group of gathered
feature rows is reduced (`row_reduction`, ops/reductions.py:38-56, whose torch_scatter.segment_csr
is not installed here: torch's own scatter_reduce over the output-row index is the same
reduction); output rows without pairs are zero (sparse_pool.py:92-104).  Written with torch so that
torch can differentiate it: the gradients the parity tests compare against are autograd's.

Pinned in tests/test_oracle_pins.py by torch.nn.functional.max_pool3d / avg_pool3d on a dense
cube and by a row-by-row brute force.
"""
import torch

_TORCH_NAME = {"sum": "sum", "mean": "mean", "max": "amax", "min": "amin"}


def pool_over_map(features: torch.Tensor, in_maps: torch.Tensor, out_maps: torch.Tensor,
                  num_out: int, reduction: str) -> torch.Tensor:
    gathered = features[in_maps.long()]
    index = out_maps.long()[:, None].expand(-1, features.shape[1])
    out = torch.zeros(num_out, features.shape[1], dtype=features.dtype)
    return out.scatter_reduce(0, index, gathered, _TORCH_NAME[reduction], include_self=False)
