"""MI355X-native min-sum message-passing layers (TRWP, ISGMR) behind the reference's surface."""
from . import lib_seg, lib_stereo  # noqa: F401
from .MP_module import ISGMRFunction, MPModule, TRWPFunction  # noqa: F401
