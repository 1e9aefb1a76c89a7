"""MI355X-native implementation of the NervanaGPU compute core.

    from nervanagpu_amd import NervanaGPU, GPUTensor

mirrors `from nervanagpu import NervanaGPU, GPUTensor` of the reference
(nervanagpu/__init__.py:15).  The device is initialised lazily on the first
allocation; there is no CPU fallback.
"""
from .nervanagpu import NervanaGPU, GPUTensor, OpTreeNode  # noqa: F401
from ._lib import NervanaGPUError  # noqa: F401
