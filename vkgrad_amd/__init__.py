"""vkgrad's training-GEMM path for MI355X (gfx950).

The package mirrors the reference's call surface for this one path:

    vkgrad_amd.vk        Device, Buffer, Graph, VkError      (reference vk.py)
    vkgrad_amd.kernels   Matmul, autotune_matmul, CONFIGS,
                         warmup, make_kernels, Elementwise   (reference kernels.py)
    vkgrad_amd.autograd  Ctx, Param, Linear, MLP, AdamW,
                         TrainStep, pick_config              (reference autograd.py)

Everything executes in libmigemm.so (hand-written HIP for gfx950) through
ctypes; there is no CPU fallback, and importing a module that needs the library
raises if it has not been built.
"""

__all__ = ["vk", "kernels", "autograd"]
