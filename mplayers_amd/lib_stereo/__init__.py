"""Same import name as the reference's compiled package (`from lib_stereo import TRWP, ISGMR`,
pytorch/MP_module.py:5-8).  The reference builds it twice with different MAX_DISPARITY limits
(MPLayers/setup.py:58-61); here one HIP library serves both names, up to 256 labels."""
from ..ops import ISGMR, TRWP, TRWP_hard_soft  # noqa: F401
from .. import compute_terms  # noqa: F401  (`from lib_stereo import compute_terms`, MPLayers/test_compute_terms.py:10)
