"""Models by architecture name."""
from __future__ import annotations

from pathlib import Path

import torch

from ..config.base import ModelConfig, load_config, lookup_architecture
from ..weights.loader import check_and_load, parse_dtype, tensor_shapes
from . import dapipel  # noqa: F401  (registers Dapipel)
from . import dukolorn  # noqa: F401  (registers Dukolorn)
from . import lfm2  # noqa: F401  (registers Lfm2ForCausalLM)
from . import sibodra  # noqa: F401  (registers Sibodra)
from . import zumuzen  # noqa: F401  (registers Zumuzen)
from .base import LayerCall, Model


def build_model(config: ModelConfig, dtype) -> Model:
    """The model of ``config``'s architecture, without weights."""
    dtype = parse_dtype(dtype) if isinstance(dtype, str) else dtype
    return lookup_architecture(config.architecture).build_model(config, dtype)


def load_model(model_dir, dtype, device="cuda:0") -> Model:
    """Read ``config.json``, build the model its ``architectures`` entry names, check
    ``model.safetensors`` against it and bind the tensors on ``device``."""
    dtype = parse_dtype(dtype) if isinstance(dtype, str) else dtype
    config = load_config(model_dir)
    if hasattr(config, "adopt_tensor_shapes"):
        # sizes that the architecture's config.json leaves to the tensors themselves
        config.adopt_tensor_shapes(tensor_shapes(Path(model_dir)))
    model = build_model(config, dtype)
    tensors = check_and_load(Path(model_dir), model.tensor_specs(), dtype, device,
                             may_be_unused=getattr(model, "unused_tensor_names", ()))
    model.bind(tensors)
    return model


__all__ = ["LayerCall", "Model", "build_model", "load_model"]
