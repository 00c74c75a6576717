from chainerkfac_amd.optimizers.fisher_blocks.connection import FisherBlockConnection  # NOQA
from chainerkfac_amd.optimizers.fisher_blocks.connections import FisherBlockLinear  # NOQA
from chainerkfac_amd.optimizers.fisher_blocks.connections import FisherBlockConvolution2D  # NOQA
from chainerkfac_amd.optimizers.fisher_blocks.normalizations import FisherBlockBatchNormalization  # NOQA
