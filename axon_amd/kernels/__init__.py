from .lib import KernelError, Kernels, kernels, MODE_STORE, MODE_ADD_F32, MODE_STORE_F32, MODE_SWIGLU

__all__ = ["KernelError", "Kernels", "kernels", "MODE_STORE", "MODE_ADD_F32", "MODE_STORE_F32", "MODE_SWIGLU"]
