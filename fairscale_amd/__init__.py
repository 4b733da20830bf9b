"""MI355X-native fused multi-tensor Adam behind the ``fairscale.optim.Adam`` interface.

``fairscale_amd.optim.Adam`` / ``Precision`` mirror ``fairscale/optim/adam.py``;
``fairscale_amd.fused_adam_hip.adam`` mirrors the native entry point ``fairscale.fused_adam_cuda.adam``
(``fairscale/clib/fused_adam_cuda/fused_adam_cuda.cpp:4-8``) over the C ABI in ``include/fsadam.h``.
"""

__version__ = "0.1.0"
