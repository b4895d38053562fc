"""MI355X-native device data path behind the ROC_SHMEM interface.

Python mirror of the host interface: one process stands for all PEs, every
PE's symmetric-heap slice lives in the one GPU's HBM.  Calls go through the C
ABI of ``librocshmem_mi355x.so`` (``include/rocshmem_mi355x.h``); data moves
only in hand-written gfx950 kernels.
"""
from .api import *  # noqa: F401,F403
from .api import __all__  # noqa: F401
