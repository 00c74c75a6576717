from chainerkfac_amd.optimizers.fisher_blocks.connections.linear import FisherBlockLinear  # NOQA
from chainerkfac_amd.optimizers.fisher_blocks.connections.convolution_2d import FisherBlockConvolution2D  # NOQA
