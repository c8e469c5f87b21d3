"""Pre-`apply_sharding` spelling of the ZeRO-3 side-car (reference: src/tensor_parallel/legacy.py:12-20)."""
from __future__ import annotations

import logging
from typing import Collection, Optional

from torch import nn

logger = logging.getLogger(__file__)


class Sharded(nn.Module):
    def __new__(cls, module, sharded_param_names: Optional[Collection[str]] = None):
        """Applies sharding to a TensorParallel or TensorParallelPreTrainedModel and returns that same module."""
        logger.warning("`Sharded` is deprecated. Please use `.apply_sharding()` method")
        module.apply_sharding(sharded_param_names)
        return module
