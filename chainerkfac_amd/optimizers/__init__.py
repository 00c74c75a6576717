from chainerkfac_amd.optimizers import fisher_blocks  # NOQA
from chainerkfac_amd.optimizers.cholesky_inverse import inverse  # NOQA
from chainerkfac_amd.optimizers.kfac import KFAC  # NOQA
from chainerkfac_amd.optimizers.kfac import fblock_constructor  # NOQA
