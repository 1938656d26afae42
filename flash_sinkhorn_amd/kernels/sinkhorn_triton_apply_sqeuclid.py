"""Import-path shim: plan products under the reference's older module name
(``kernels/sinkhorn_triton_apply_sqeuclid.py:9-17``)."""
from flash_sinkhorn_amd.kernels.apply_flash import (  # noqa: F401
    apply_plan_mat_flashstyle,
    apply_plan_vec_flashstyle,
)
from flash_sinkhorn_amd.kernels.apply_ott import mat5_sqeuclid  # noqa: F401
