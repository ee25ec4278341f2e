from .lib import (KernelError, Kernels, PackedMatrix, kernels, MODE_STORE, MODE_ADD_F32, MODE_STORE_F32, MODE_SWIGLU,
                  current_stream, ptr, register_kernel_source)

__all__ = ["KernelError", "Kernels", "PackedMatrix", "kernels", "MODE_STORE", "MODE_ADD_F32", "MODE_STORE_F32", "MODE_SWIGLU",
           "current_stream", "ptr", "register_kernel_source"]
