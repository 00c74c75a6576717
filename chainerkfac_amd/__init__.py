"""MI355X-native K-FAC per-layer hot path behind the chainerkfac API.

``chainerkfac_amd.optimizers.KFAC`` / ``fisher_blocks`` / ``inverse`` mirror
``chainerkfac.optimizers``; ``chainerkfac_amd.communicators.ArrayPacker`` holds
the pack/unpack half of the reference communicator.  Everything numerical runs
in hand-written HIP kernels (libkfac_hip.so, C ABI in include/kfac_hip.h).
"""
from chainerkfac_amd import communicators  # NOQA
from chainerkfac_amd import optimizers  # NOQA
from chainerkfac_amd import links  # NOQA
