"""Importing this module guarantees that ``aten.clone`` on an ``NF4Tensor`` re-quantises the dequantised
weight with the default granularity, as ``torchtune/modules/low_precision/_register_nf4_dispatch_ops.py:12-20``
arranges in the reference.  The handler itself is registered next to the tensor class."""
from ...nf4_tensor import NF4_OPS_TABLE, _nf4_clone

import torch

assert NF4_OPS_TABLE[torch.ops.aten.clone.default] is _nf4_clone
