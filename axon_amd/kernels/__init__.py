from .lib import KernelError, Kernels, PackedMatrix, kernels, MODE_STORE, MODE_ADD_F32, MODE_STORE_F32, MODE_SWIGLU

__all__ = ["KernelError", "Kernels", "PackedMatrix", "kernels", "MODE_STORE", "MODE_ADD_F32", "MODE_STORE_F32", "MODE_SWIGLU"]
