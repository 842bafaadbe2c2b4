"""Modifier base class and hash-weight checkpoints.

Mirror of the reference's ``Modifier`` (spotlight/modifier.py:21-88): wraps a
model, reads the JSON configuration, loads / saves the trainable parameters (the
per-layer hash functions) as a flat list of tensors.

Checkpoint format (spotlight/modifier.py:62-76): ``torch.save`` of a Python list,
one tensor per parameter in ``ft_params()`` order.  For the MLP hash that is,
per layer, ``[proj_0, bias_0, proj_1, bias_1, ...]`` with ``proj_i``
``[1, heads, in_i, out_i]`` and ``bias_i`` ``[1, heads, 1, out_i]``
(spotlight_generation.py:229-255); for the linear hash one ``[1, 32, 128, 128]``
tensor per layer (linearhashing_generation.py:224-231).  Two list lengths occur
in the reference: the generation modifier lists every layer
(spotlight_generation.py:363-369), the training modifier leaves the dense
("fix") layers out (spotlight_train.py:412-419).  ``assign_checkpoint`` takes
both; the reference asserts equality and fails on the second.

Files are read with ``torch.load(..., weights_only=True)``: a list of tensors
needs nothing else, and nothing from the file is executed.
"""
from __future__ import annotations

import json
import os
from typing import Iterable, List, Optional, Sequence

import torch


def read_checkpoint(path: str) -> List[torch.Tensor]:
    """The flat parameter list of a checkpoint file."""
    obj = torch.load(path, map_location="cpu", weights_only=True)
    if isinstance(obj, torch.Tensor):
        obj = [obj]
    if not isinstance(obj, (list, tuple)) or not all(isinstance(t, torch.Tensor) for t in obj):
        raise ValueError(f"{path}: expected a list of tensors, got {type(obj).__name__}")
    return [t.detach() for t in obj]


def write_checkpoint(params: Iterable[torch.Tensor], path: str) -> None:
    """What ``Modifier.save_checkpoint`` writes (spotlight/modifier.py:74-76)."""
    torch.save([p.detach().cpu().clone() for p in params], path)


def merge_layer_files(directory: str, num_layers: int = 32) -> List[torch.Tensor]:
    """Per-layer training results ``<layer>.pth`` (each a tensor or a list of
    tensors) merged into one flat list in layer order; layers without a file are
    skipped (train_results/convert.py:13-32 keeps a ``None`` for them, which
    ``torch.save`` then stores; a list without holes is what loads)."""
    per_layer: List[Optional[object]] = [None] * num_layers
    for name in os.listdir(directory):
        stem = name.split(".")[0]
        if not stem.isdigit():
            continue
        idx = int(stem)
        if idx >= num_layers:
            raise ValueError(f"{name}: layer index beyond num_layers={num_layers}")
        per_layer[idx] = torch.load(os.path.join(directory, name), map_location="cpu", weights_only=True)
    flat: List[torch.Tensor] = []
    for item in per_layer:
        if item is None:
            continue
        if isinstance(item, (list, tuple)):
            flat.extend(item)
        else:
            flat.append(item)
    return flat


def assign_checkpoint(layer_params: Sequence[Sequence[torch.nn.Parameter]], fix_layers: Sequence[int],
                      checkpoint: Sequence[torch.Tensor]) -> None:
    """Copies ``checkpoint`` into the parameters.  ``layer_params[i]`` are layer i's
    parameters in ``ft_params()`` order.  Accepted lengths: all layers, or all
    layers but the dense ones in ``fix_layers``.  Shapes must match exactly; dtype
    and device follow the parameter (spotlight/modifier.py:69-70)."""
    every = [p for ps in layer_params for p in ps]
    sparse_only = [p for i, ps in enumerate(layer_params) if i not in set(fix_layers) for p in ps]
    if len(checkpoint) == len(every):
        targets = every
    elif len(checkpoint) == len(sparse_only):
        targets = sparse_only
    else:
        raise ValueError(f"checkpoint holds {len(checkpoint)} tensors; the model has {len(every)} hash parameters "
                         f"({len(sparse_only)} without the dense layers {sorted(set(fix_layers))})")
    for i, (param, value) in enumerate(zip(targets, checkpoint)):
        if tuple(param.shape) != tuple(value.shape):
            raise ValueError(f"checkpoint tensor {i} has shape {tuple(value.shape)}, the parameter {tuple(param.shape)}")
    for param, value in zip(targets, checkpoint):
        param.data = value.data.to(device=param.data.device, dtype=param.data.dtype)


class Modifier(torch.nn.Module):
    """spotlight/modifier.py:21-88."""

    def __init__(self, model, save_ckp, load_ckp):
        super().__init__()
        self.model = model
        self.load_ckp = load_ckp
        self.save_ckp = save_ckp
        if self.load_ckp is not None:
            self.load_checkpoint()

    def forward(self, *args, **kwargs):
        return self.model(*args, **kwargs)

    def get_conf(self, config):
        """``config``: path of a JSON file (as in the reference) or the parsed dict."""
        if config is None:
            self.conf = None
        elif isinstance(config, dict):
            self.conf = config
        else:
            with open(config, "r") as f:
                self.conf = json.load(f)

    def freeze_model(self):
        for param in self.model.parameters():
            param.requires_grad_(False)

    def unfreeze_model(self):
        for param in self.ft_params():
            param.requires_grad_(True)

    def load_checkpoint(self, ckp: Optional[str] = None):
        ckp = ckp if ckp is not None else self.load_ckp
        assign_checkpoint(self.layer_ft_params(), self.fix_layers(), read_checkpoint(ckp))

    def save_checkpoint(self, ckp: Optional[str] = None):
        ckp = ckp if ckp is not None else self.save_ckp
        write_checkpoint(self.ft_params(), ckp)

    def generate(self, *args, **kwargs):
        return self.model.generate(*args, **kwargs)

    # -- to be provided by the concrete modifier ---------------------------------
    def ft_params(self):
        raise NotImplementedError

    def layer_ft_params(self):
        """ft_params() grouped by layer."""
        raise NotImplementedError

    def fix_layers(self):
        raise NotImplementedError

    def reset(self):
        raise NotImplementedError
