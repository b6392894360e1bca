"""Vocabulary padding removal (reference: .../processors/padding_remover.py:6-12)."""

from __future__ import annotations

import torch

_VOCAB_PARAMS = {"embedding.word_embeddings.weight", "output_layer.weight"}


def strip_param_name_prefix(name: str) -> str:
    while name.startswith("module."):
        name = name[len("module."):]
    return name


def remove_padding(name: str, param: torch.Tensor, vocab_size: int) -> torch.Tensor:
    """param[:vocab_size] for the embedding / output layer, unchanged otherwise."""
    return param[:vocab_size] if strip_param_name_prefix(name) in _VOCAB_PARAMS else param
