"""GravNetOp on MI355X.  Same constructor, sub-module names and forward return
tuple as fastgraphcompute/gnn_ops.py:9-109, so state_dicts interchange; the
neighbour aggregation (gnn_ops.py:90-102) is one fused HIP kernel per
direction instead of six tensor ops over a [N, K, P] intermediate.  The module
is TorchScript-scriptable like the reference's."""
from typing import Optional, Tuple

import torch

from . import _ops  # noqa: F401  (registers the ops)
from .extensions.binned_select_knn import binned_select_knn


@torch.jit.script
def gravnet_aggregate(neighbor_idx: torch.Tensor, distsq: torch.Tensor,
                      features: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Mean and max over the K neighbour slots of features[neighbor_idx] * exp(-10 distsq): ([N, P], [N, P]).
    Slots with index -1 contribute 0; the mean always divides by K."""
    return torch.ops.fastgraphcompute_custom_ops.gravnet_aggregate(neighbor_idx, distsq, features)


@torch.jit.script
def dense(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """x W^T + b like torch.nn.functional.linear, with the weight gradient computed by the library's split
    reduction over the points instead of a tiled GEMM with a tiny output."""
    return torch.ops.fastgraphcompute_custom_ops.dense(x, weight, bias)


@torch.jit.script
def dense_split(x: torch.Tensor, a: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor]) -> torch.Tensor:
    """cat([x, a], 1) W^T + b without the concatenation (weight is [out, x.shape[1] + a.shape[1]])."""
    return torch.ops.fastgraphcompute_custom_ops.dense_split(x, a, weight, bias)


@torch.jit.script
def gravnet_layer_core(space: torch.Tensor, features: torch.Tensor, row_splits: torch.Tensor,
                       k: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """kNN in `space` and aggregation of `features` over the neighbours as one autograd node:
    (neighbor_idx [N, k], distsq [N, k], [N, 2P] = mean | max of features * exp(-10 distsq))."""
    return torch.ops.fastgraphcompute_custom_ops.gravnet_layer_core(space, features, row_splits, k)


class Dense(torch.nn.Linear):
    """torch.nn.Linear (same parameters, state_dict and results) whose weight gradient is the library's split
    reduction over the points.  For the layers around GravNetOp in a point-cloud model: their weight-gradient
    products have 10^5..10^6 rows and an output of at most a few hundred squared, the shape on which a tiled
    library GEMM leaves most of the chip idle."""

    def forward(self, input: torch.Tensor) -> torch.Tensor:
        return dense(input, self.weight, self.bias)


def use_dense_layers(module: torch.nn.Module) -> torch.nn.Module:
    """Replaces every plain torch.nn.Linear inside `module` by a Dense layer sharing its parameters (in place;
    optimizers and state_dicts built on the parameters stay valid).  Returns `module`."""
    for name, child in module.named_children():
        if type(child) is torch.nn.Linear:
            layer = Dense(child.in_features, child.out_features, bias=child.bias is not None,
                          device=child.weight.device, dtype=child.weight.dtype)
            layer.weight = child.weight
            layer.bias = child.bias
            setattr(module, name, layer)
        else:
            use_dense_layers(child)
    return module


class GravNetOp(torch.nn.Module):
    """One GravNet layer [arxiv:1902.07987]: learned coordinates -> kNN graph ->
    exp(-10 d^2)-weighted mean/max aggregation of learned features -> dense output."""

    def __init__(self, in_channels, out_channels, space_dimensions, propagate_dimensions, k,
                 output_activation=torch.nn.ReLU(), optimization_arguments: dict = {}):
        super(GravNetOp, self).__init__()
        self.k = k
        self.space_transformations = torch.nn.Linear(in_channels, space_dimensions)
        self.propagate_transformations = torch.nn.Linear(in_channels, propagate_dimensions)
        self.output_transformations = torch.nn.Sequential(
            torch.nn.Linear(in_channels + 2 * propagate_dimensions, out_channels),
            output_activation
        )
        self.optimization_arguments = optimization_arguments

    def forward(self, x: torch.Tensor, row_splits: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
        # The two projections are separate products, so that the coordinates and the features are matrices of
        # their own (rows of the features aligned to their 128 bytes: the aggregation gathers and, in the backward,
        # updates whole rows); search and aggregation are one autograd node that writes (mean | max) side by side,
        # and the output layer multiplies x and that matrix by its two weight blocks - no slice copies and no
        # concatenation, forward or backward.
        space = dense(x, self.space_transformations.weight, self.space_transformations.bias)
        propagate = dense(x, self.propagate_transformations.weight, self.propagate_transformations.bias)
        neighbor_idx, distsq, aggregated = gravnet_layer_core(space, propagate, row_splits, self.k)
        lin = self.output_transformations[0]
        out = self.output_transformations[1](dense_split(x, aggregated, lin.weight, lin.bias))
        return out, neighbor_idx, distsq, space
