"""``ModelConverter`` interface (cosmos_rl/utils/model_converter.py:26-38)."""
from __future__ import annotations

from abc import ABC, abstractmethod
from typing import List, Union

import torch
import torch.nn as nn


class ModelConverter(ABC):
    def __init__(self, config, parallel_dims):
        self.config = config
        self.parallel_dims = parallel_dims

    @abstractmethod
    def convert_model(self, model: torch.nn.Module) -> torch.nn.Module: ...

    def post_optimizer_hook(self, model: Union[nn.Module, List[nn.Module]]):
        """Runs after the optimizer step (e.g. to refresh weight statistics)."""
        ...
