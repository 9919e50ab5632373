from .library import ACTIVATIONS, HipKernels, KernelError, get_kernels, set_kernels

__all__ = ["ACTIVATIONS", "HipKernels", "KernelError", "get_kernels", "set_kernels"]
