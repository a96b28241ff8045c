"""cgnet_amd: the Clebsch-Gordan layer hot path of CGNet on MI355X (gfx950).

``CG_layers`` / ``CGNet`` mirror the reference's module API, ``CG_cuda_ops`` its native
operator module, ``CGutils`` its host-side metadata helpers.  The arithmetic lives in
``csrc/`` (HIP kernels behind the C ABI of ``include/cgnet_hip.h``).
"""
from . import CGutils  # noqa: F401

__all__ = ["CGutils", "CG_cuda_ops", "CG_layers", "CGNet"]
