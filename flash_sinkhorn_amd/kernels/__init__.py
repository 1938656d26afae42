"""Kernel launchers (HIP, gfx950) with the reference's ``flash_sinkhorn.kernels`` names.

Eager exports follow the reference's ``kernels/__init__.py:41-55``; the internal
helpers it only bridges lazily with a DeprecationWarning (:62-97) are bridged the
same way.
"""
from flash_sinkhorn_amd.kernels._common import epsilon_schedule, max_diameter
from flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid import (
    sinkhorn_flashstyle_alternating,
    sinkhorn_flashstyle_symmetric,
)
from flash_sinkhorn_amd.kernels.apply_flash import (
    apply_plan_mat_flashstyle,
    apply_plan_vec_flashstyle,
)
from flash_sinkhorn_amd.kernels.sinkhorn_triton_grad_sqeuclid import (
    sinkhorn_geomloss_online_grad_sqeuclid,
)
from flash_sinkhorn_amd.kernels.c_transform_sqeuclid import c_transform_kernel

__all__ = [
    "epsilon_schedule", "max_diameter",
    "sinkhorn_flashstyle_alternating", "sinkhorn_flashstyle_symmetric",
    "apply_plan_vec_flashstyle", "apply_plan_mat_flashstyle",
    "sinkhorn_geomloss_online_grad_sqeuclid", "c_transform_kernel",
]

_BRIDGED = {
    "log_weights": "flash_sinkhorn_amd.kernels._common",
    "mat5_sqeuclid": "flash_sinkhorn_amd.kernels.apply_ott",
    "precompute_flashsinkhorn_inputs": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "compute_bias_f": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "compute_bias_g": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "flashsinkhorn_lse": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "flashsinkhorn_lse_fused": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "flashsinkhorn_symmetric_step": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "shifted_to_standard_potentials": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
    "standard_to_shifted_potentials": "flash_sinkhorn_amd.kernels.sinkhorn_flashstyle_sqeuclid",
}


def __getattr__(name):
    if name in _BRIDGED:
        import importlib
        import warnings

        target = _BRIDGED[name]
        warnings.warn(
            f"Importing {name} from flash_sinkhorn_amd.kernels is deprecated. "
            f"Import from {target} directly.", DeprecationWarning, stacklevel=2)
        return getattr(importlib.import_module(target), name)
    raise AttributeError(f"module 'flash_sinkhorn_amd.kernels' has no attribute {name!r}")
