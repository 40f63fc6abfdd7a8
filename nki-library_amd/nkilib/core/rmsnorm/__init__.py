from .rmsnorm_quant import RmsNormQuantKernelArgs, rmsnorm_quant_kernel

__all__ = ["RmsNormQuantKernelArgs", "rmsnorm_quant_kernel"]
