"""MI355X-native FlashOverlap hot path: signal/reorder GEMM, wait + consumer,
reorder+RMSNorm.  Kernels live in lib/libfo_kernels.so (C ABI, include/flashoverlap.h);
lib/libst_pybinding.so registers the reference's torch.classes / torch.ops names."""
from . import _capi, layout, config  # noqa: F401
from ._capi import F16, BF16, FlashOverlapError  # noqa: F401

__all__ = ["_capi", "layout", "config", "ops", "layers", "tune", "F16", "BF16", "FlashOverlapError"]


def __getattr__(name):
    # ops / layers / tune import torch lazily so that `import flashoverlap_amd` stays cheap
    if name in ("ops", "layers", "tune"):
        import importlib
        return importlib.import_module(f".{name}", __name__)
    raise AttributeError(name)
