from chainerkfac_amd.communicators import _utility  # NOQA
from chainerkfac_amd.communicators.packing import ArrayPacker  # NOQA
from chainerkfac_amd.communicators.packing import _ArraysInfo  # NOQA
