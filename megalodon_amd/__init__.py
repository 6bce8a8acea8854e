"""megalodon_amd: gfx950-native fused ops for the Megalodon hot path.

Host side in PyTorch-ROCm, kernels in ``lib/libmegalodon_hip.so`` (plain C ABI,
``include/megalodon_hip.h``).
"""
__version__ = "0.1.0"
