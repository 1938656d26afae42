"""MI355X-native FlashSinkhorn: streaming entropic optimal transport on hand-written
gfx950 kernels, behind the public names of the reference package (``flash_sinkhorn``)."""
from flash_sinkhorn_amd.samples_loss import SamplesLoss
from flash_sinkhorn_amd.c_transform import c_transform_cost, c_transform_fwd
from flash_sinkhorn_amd.cg import CGInfo, conjugate_gradient
from flash_sinkhorn_amd.hvp import (
    HvpInfo,
    geomloss_to_ott_potentials,
    hvp_x_sqeuclid,
    hvp_x_sqeuclid_from_potentials,
    inverse_hvp_x_sqeuclid_from_potentials,
)
from flash_sinkhorn_amd.implicit_grad import (
    ImplicitGradInfo,
    implicit_grad_x,
    implicit_grad_x_from_potentials,
)

__all__ = ["SamplesLoss", "CGInfo", "conjugate_gradient", "HvpInfo",
           "geomloss_to_ott_potentials", "hvp_x_sqeuclid", "hvp_x_sqeuclid_from_potentials",
           "inverse_hvp_x_sqeuclid_from_potentials", "ImplicitGradInfo", "implicit_grad_x",
           "implicit_grad_x_from_potentials", "c_transform_fwd", "c_transform_cost",
           "__version__"]
__version__ = "0.1.0"
