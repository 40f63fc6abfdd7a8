"""MI355X (gfx950) implementation of the MoE context-encoding path of aws-neuron/nki-library.

Import paths mirror the reference package (``nkilib.core.moe.moe_cte``,
``nkilib.core.rmsnorm.rmsnorm_quant``, ``nkilib.core.utils.common_types``) so that
model code written against it keeps working.  Tensors are torch tensors on a
ROCm device; the compute runs in hand-written HIP kernels loaded from
``nkilib/_lib/libmoe_gfx950.so`` through a C ABI (``include/moe_gfx950.h``).
There is no CPU fallback: calling a kernel without the library raises.
"""

__all__ = ["core"]
