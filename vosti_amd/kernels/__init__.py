from .ops import KernelError, Kernels, dtype_name, kernels_for

__all__ = ["KernelError", "Kernels", "dtype_name", "kernels_for"]
