"""The Linear adaptor of the reference's model/layers.py (:225-300) on MI355X.

Only the Strassen Linear path lives here; attention, RoPE and the feed-forward block of
the reference's model code are consumers of this layer, not part of it.
"""
from __future__ import annotations

import torch.nn as nn

from fixed_strassen import LinearStrassen as _LinearStrassen
from strassen import _strassen_base, strassen_matmul_two_layers


class LinearStrassen(_LinearStrassen):
    """Same module as fixed_strassen.LinearStrassen with the constructor of reference
    model/layers.py:232-244 (dtype defaults to None; depth 2 selects the two-layer product)."""

    def __init__(self, in_features: int, out_features: int, bias: bool = True, dtype=None,
                 depth: int = 1, device: str = "cuda") -> None:
        super().__init__(in_features, out_features, bias, dtype, depth, device)
        self.strassen_func = strassen_matmul_two_layers if depth == 2 else _strassen_base


def replace_linear_with_strassen(module: nn.Module, min_size: int = 128, depth: int = 1):
    """Swap every square nn.Linear of at least min_size features for LinearStrassen, in
    place, keeping weights and bias (reference model/layers.py:279-300)."""
    for name, child in module.named_children():
        if isinstance(child, nn.Linear) and not isinstance(child, _LinearStrassen):
            if child.in_features == child.out_features and child.in_features >= min_size:
                print(f"Replacing '{name}' with LinearStrassen.")
                new_layer = LinearStrassen(child.in_features, child.out_features,
                                           bias=child.bias is not None, device=child.weight.device,
                                           dtype=child.weight.dtype, depth=depth)
                new_layer.weight.data.copy_(child.weight.data)
                if child.bias is not None:
                    new_layer.bias.data.copy_(child.bias.data)
                setattr(module, name, new_layer)
            else:
                print(f"Skipping '{name}': Not square or too small.")
        elif len(list(child.children())) > 0:
            replace_linear_with_strassen(child, min_size, depth)
