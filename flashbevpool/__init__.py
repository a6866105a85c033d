"""Import-name shim: ``from flashbevpool import flash_bevpool, FlashBEVPool`` resolves to the
MI355X implementation, so code written against the reference package
(flashbev/flashbevpool/__init__.py:3-6) runs unchanged."""
from flashbev_amd import FlashBEVPool, SamplingVT, flash_bevpool, sampling_vt_pillarpool_fused

__all__ = ["FlashBEVPool", "flash_bevpool", "SamplingVT", "sampling_vt_pillarpool_fused"]
