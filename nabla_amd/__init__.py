"""nabla_amd -- MI355X (gfx950) fused optimizer-step engine for fumishiki/nabla.

Only the optimizer-step path is here: ``nabla_amd.optim`` mirrors
nabla-train's ``Sgd`` / ``Adam`` / ``AdamW`` / ``GradScaler`` /
``clip_grad_norm`` / ``zero_grad`` over the C ABI of ``include/nabla_optim.h``
(``libnabla_optim.so``: hand-written HIP kernels, embedded gfx950 code object);
``nabla_amd.groups`` (GroupOptimizer), ``nabla_amd.schedule`` (LrSchedule),
``nabla_amd.trainer`` (the Trainer's loop body after backward) and
``nabla_amd.checkpoint`` (NBLA / meta.txt) are the callers and file formats
either side of it; ``nabla_amd.backend`` is nabla-core's Backend primitives as
multi-tensor launches.
"""
from . import _lib  # noqa: F401
from .optim import (Adam, AdamW, GradScaler, GradScalerState, NablaPanic, OptimMeta,  # noqa: F401
                    OptimStateError, Sgd, TensorList, accumulate, clip_grad_norm, has_non_finite,
                    scale_grad, sync, unscale_accumulate, zero_grad)

__version__ = "0.1.0"
