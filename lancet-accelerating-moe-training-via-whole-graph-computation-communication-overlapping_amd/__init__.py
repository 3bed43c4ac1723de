"""MI355X-native MoE token dispatch and fused LANS behind RAF's operator surface.

  capi  - ctypes bindings of the C ABI (include/lancet_hip.h)
  ops   - the six RAF operators (moe_encode, moe_encode_batch_prioritized, moe_decode,
          moe_merge_masks, moe_redispatch, lans) over torch tensors that live on the GPU
  grad  - the gradient rules of the MoE operators (src/op/grad/moe.cc) as torch.autograd functions
  moe_layer - Gate / Experts / MOELayerImpl, the layer that calls the operators (models/benchmark/pytorch/utils.py)
  pipeline - the partitioned encode / exchange / decode call pattern of Lancet's partition pass on two streams
  raf_executor - a minimal executor over the C++ op layer (raf_hip/: OpEnv, dialect registry,
          dispatch), the path a RAF build would take
  build - compiles the in-tree libraries with hipcc

torch is used for device memory and streams only; every operator runs hand-written HIP
kernels through the C ABI and raises when the library is missing.
"""
from . import capi  # noqa: F401
from . import ops  # noqa: F401
from . import grad  # noqa: F401
from . import moe_layer  # noqa: F401
from . import pipeline  # noqa: F401
from . import raf_executor  # noqa: F401

__all__ = ["capi", "ops", "grad", "moe_layer", "pipeline", "raf_executor"]
