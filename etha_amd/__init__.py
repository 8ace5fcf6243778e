"""etha_amd — MI355X-native redistribute hot path (pack / unpack / self-copy / Partial reduce).

The host planner lives in :mod:`etha_amd.comm`; the device work is done by hand-written HIP
kernels in ``libetha_reshard.so`` (C ABI in ``include/etha_reshard.h``), bound through
:mod:`etha_amd._native`.
"""

__version__ = "0.1.0"
