"""MI355X-native AlphaFold3 Pairformer / diffusion-transformer hot path.

Host side: thin PyTorch modules that keep the module `forward` signatures and
parameter names of hasaki321/Distributed-xfold (src/distributed_xfold/nn/*) and
call hand-written gfx950 kernels through the C ABI of `libaf3hip.so`
(include/af3_hip.h).  There is no eager or CPU fallback: without the built
library, or with tensors that are not on the GPU, every operator raises.
"""

from . import lib, ops  # noqa: F401
from . import check, nn  # noqa: F401
from . import torch_ops  # noqa: F401  (nothing is registered until torch_ops.register() is called)

__all__ = ["lib", "ops", "nn", "check", "torch_ops"]
