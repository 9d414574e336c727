"""MI355X-native fused Adam operator: a drop-in for TorchOpt's accelerated Adam op.

    from torchopt_amd._C import adam_op                    # the 7-function native surface
    from torchopt_amd.accelerated_op import AdamOp         # the per-leaf callable
    from torchopt_amd import accelerated_op_available
"""

import sys as _sys

from torchopt_amd import accelerated_op
from torchopt_amd.accelerated_op import AdamOp, MultiAdamOp
from torchopt_amd.accelerated_op import is_available as accelerated_op_available
from torchopt_amd.alias import adam, adamw, apply_updates, chain
from torchopt_amd.func import FuncOptimizer
from torchopt_amd.meta import MetaAdam, MetaAdamW
from torchopt_amd.optim import Adam, AdamW, FusedAdam, FusedAdamW
from torchopt_amd.placement import (placed_like_tree, state_empty_like, state_zeros_like,
                                    state_zeros_like_tree, unshared)

# `import torchopt_amd._C.adam_op` should work like `from torchopt_amd._C import adam_op`
from torchopt_amd import _C  # noqa: E402

_sys.modules.setdefault('torchopt_amd._C.adam_op', _C.adam_op)

__version__ = '0.1.0'

__all__ = ['Adam', 'AdamOp', 'AdamW', 'FuncOptimizer', 'FusedAdam', 'FusedAdamW', 'MetaAdam', 'MetaAdamW', 'MultiAdamOp', 'accelerated_op',
           'accelerated_op_available', 'adam', 'adamw', 'apply_updates', 'chain', 'placed_like_tree',
           'state_empty_like', 'state_zeros_like', 'state_zeros_like_tree', 'unshared']
