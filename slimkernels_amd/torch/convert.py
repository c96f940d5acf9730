"""Swap the nn.Linear layers of a model for W2A8Linear.

Upstream's only model-level caller is a Hugging Face Llama loaded in fp16 and run through
``generate`` (slimkernels/torch/llama.py:15-19, 34-43); its linears are where the decode and
prefill shapes of this path come from.  ``replace_linears`` turns such a model's projections into
W2A8 layers in place: each weight is quantised where it lies (on the GPU for fp16/bf16 CUDA
weights), repacked into the streaming layout, and the fp16 original is dropped.
"""
from typing import Callable, Iterable, List, Optional

import torch

from .ops import W2A16Linear, W2A8Linear
from .w4 import W4A8Linear


def replace_linears(model: torch.nn.Module, group_size: int = 128, mode: str = "sym",
                    skip: Iterable[str] = ("lm_head",), out_dtype=None,
                    predicate: Optional[Callable[[str, torch.nn.Linear], bool]] = None, bits: int = 2,
                    weight_only: bool = False) -> List[str]:
    """Replace every eligible ``nn.Linear`` under ``model`` by a ``W2A8Linear`` (``bits=2``) or a ``W4A8Linear``
    (``bits=4``: modes "sym" and "asym", quantised on the host) and return the dotted names
    of the layers replaced.  ``weight_only=True`` (2 bits, layers whose ``in_features`` is a multiple of 128) builds
    ``W2A16Linear`` layers, which leave the activations in fp16.  Eligible: ``in_features`` a multiple of ``group_size``, the last name component
    not in ``skip`` (the output head stays in floating point by default), and ``predicate(name, layer)`` true
    when one is given.  ``out_dtype`` defaults to the dtype of each layer's weight (fp16 or bf16; other dtypes
    give fp16).  The model must already be on the GPU: the layers are built on the device of their weight."""
    if bits not in (2, 4):
        raise ValueError("bits must be 2 or 4")
    if weight_only and bits != 2:
        raise ValueError("weight_only is built for bits=2")
    layer_type = W2A16Linear if weight_only else W2A8Linear if bits == 2 else W4A8Linear
    skip = set(skip)
    done = []
    for parent_name, parent in list(model.named_modules()):
        for child_name, child in list(parent.named_children()):
            if not isinstance(child, torch.nn.Linear):
                continue
            name = f"{parent_name}.{child_name}" if parent_name else child_name
            if child_name in skip or child.in_features % group_size != 0 or (weight_only and child.in_features % 128 != 0):
                continue
            if predicate is not None and not predicate(name, child):
                continue
            w = child.weight.detach()
            if not w.is_cuda:
                raise ValueError(f"{name}: move the model to the GPU before replace_linears (weight is on {w.device})")
            dt = out_dtype or (w.dtype if w.dtype in (torch.float16, torch.bfloat16) else torch.float16)
            bias = child.bias.detach().to(dt) if child.bias is not None else None
            setattr(parent, child_name, layer_type.from_float(w, group_size, mode, bias=bias, out_dtype=dt, device=w.device))
            done.append(name)
    return done
