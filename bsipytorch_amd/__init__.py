"""MI355X-native implementation of the ``bsi_ops`` fixed-bit BSI tensor-dot path.

``bsipytorch_amd.bsi_ops`` mirrors the reference extension's Python API; ``bsipytorch_amd.linear``
holds the ``BSIQuantizedLinear`` drop-in.  All compute runs in ``libbsi_hip.so`` (hand-written HIP
for gfx950, C ABI in ``include/bsi_hip.h``); PyTorch only provides device memory and streams.
"""
__all__ = ["bsi_ops", "linear"]
