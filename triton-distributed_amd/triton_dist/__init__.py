"""MI355X-native implementation of the per-GPU compute half of Triton-distributed's overlapped ops.

The op-level entry points keep the call signatures and tensor layouts of the reference's
``triton_dist.kernels`` (AG-GEMM, GEMM-RS, low-latency MoE all-to-all, SP flash decode) and route through
the C ABI of ``libtdist_hip.so`` (hand-written gfx950 HIP kernels). There is no CPU or PyTorch fallback:
calling an op without the built library, or without a GPU, raises.
"""

__version__ = "0.1.0"
