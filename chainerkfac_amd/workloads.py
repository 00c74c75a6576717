"""Layer-shape tables of the benchmark configurations (synthetic workloads).

Each layer is a dict:
  conv   : kind, name, c_in, c_out, k, s, p, h, w (input size), bias
  linear : kind, name, d_in, d_out, bias
  bn     : kind, name, c, h, w   (h = w = 1 for a 2-D input)
The tables are derived from the model definitions the reference trains:
examples/mnist/train.py:18-33 (MLP), examples/cifar10/models/resnet50.py:6-73
(bottleneck v1 topology; ImageNet stem and per-conv bias added as the
configuration states) and examples/imagenet/models/resnet50_d.py:55-253.
"""


def conv_out(size, k, s, p):
    return (size + 2 * p - k) // s + 1


def _conv(name, c_in, c_out, k, s, p, h, w, bias):
    return dict(kind='conv', name=name, c_in=c_in, c_out=c_out, k=k, s=s, p=p, h=h, w=w, bias=bias)


def _bn(name, c, h, w):
    return dict(kind='bn', name=name, c=c, h=h, w=w)


def _linear(name, d_in, d_out, bias=True):
    return dict(kind='linear', name=name, d_in=d_in, d_out=d_out, bias=bias)


def mlp_mnist():
    """784-1000-1000-10 with bias."""
    return [_linear('l1', 784, 1000), _linear('l2', 1000, 1000), _linear('l3', 1000, 10)]


def cifar_cnn():
    """conv3x3 3->64, 64->128, 128->256 (2x2/2 max-pool after each), FC 4096->10."""
    return [_conv('conv1', 3, 64, 3, 1, 1, 32, 32, True),
            _conv('conv2', 64, 128, 3, 1, 1, 16, 16, True),
            _conv('conv3', 128, 256, 3, 1, 1, 8, 8, True),
            _linear('fc', 4096, 10)]


def resnet50_v1(insize=224, n_class=1000, bias=True):
    """ResNet-50 bottleneck v1: 53 conv + 53 BN + 1 FC (161 factors)."""
    layers = []
    h = insize
    layers.append(_conv('conv1', 3, 64, 7, 2, 3, h, h, bias))
    h = conv_out(h, 7, 2, 3)
    layers.append(_bn('bn1', 64, h, h))
    h = conv_out(h, 3, 2, 1)                      # 3x3/2 max-pool, pad 1
    n_in = 64
    for si, (n_mid, n_out, blocks, stride) in enumerate(
            [(64, 256, 3, 1), (128, 512, 4, 2), (256, 1024, 6, 2), (512, 2048, 3, 2)]):
        for b in range(blocks):
            s = stride if b == 0 else 1
            pre = 'res{}/{}'.format(si + 2, b)
            ho = conv_out(h, 1, s, 0)
            layers.append(_conv(pre + '/conv1', n_in, n_mid, 1, s, 0, h, h, bias))
            layers.append(_bn(pre + '/bn1', n_mid, ho, ho))
            layers.append(_conv(pre + '/conv2', n_mid, n_mid, 3, 1, 1, ho, ho, bias))
            layers.append(_bn(pre + '/bn2', n_mid, ho, ho))
            layers.append(_conv(pre + '/conv3', n_mid, n_out, 1, 1, 0, ho, ho, bias))
            layers.append(_bn(pre + '/bn3', n_out, ho, ho))
            if b == 0:
                layers.append(_conv(pre + '/conv4', n_in, n_out, 1, s, 0, h, h, bias))
                layers.append(_bn(pre + '/bn4', n_out, ho, ho))
            n_in = n_out
            h = ho
    layers.append(_linear('fc', 2048, n_class))
    return layers


def resnet50_d(insize=224):
    """ResNet-50-D: 55 conv + 55 BN + 1 FC (167 factors); only the first stem
    conv and the FC carry a bias."""
    layers = []
    h = insize
    layers.append(_conv('conv1_1', 3, 32, 3, 2, 1, h, h, True))
    h = conv_out(h, 3, 2, 1)
    layers.append(_bn('bn1_1', 32, h, h))
    layers.append(_conv('conv1_2', 32, 32, 3, 1, 1, h, h, False))
    layers.append(_bn('bn1_2', 32, h, h))
    layers.append(_conv('conv1_3', 32, 64, 3, 1, 1, h, h, False))
    layers.append(_bn('bn1_3', 64, h, h))
    h = -(-(h - 3) // 2) + 1                      # 3x3/2 max-pool, cover_all
    n_in = 64
    for si, (ch, n_out, blocks, stride) in enumerate(
            [(64, 256, 3, 1), (128, 512, 4, 2), (256, 1024, 6, 2), (512, 2048, 3, 2)]):
        for b in range(blocks):
            pre = 'res{}/{}'.format(si + 2, b)
            if b == 0:
                ho = conv_out(h, 3, stride, 1)
                layers.append(_conv(pre + '/conv1', n_in, ch, 1, 1, 0, h, h, False))
                layers.append(_bn(pre + '/bn1', ch, h, h))
                layers.append(_conv(pre + '/conv2', ch, ch, 3, stride, 1, h, h, False))
                layers.append(_bn(pre + '/bn2', ch, ho, ho))
                layers.append(_conv(pre + '/conv3', ch, n_out, 1, 1, 0, ho, ho, False))
                layers.append(_bn(pre + '/bn3', n_out, ho, ho))
                # projection on the (average-pooled when strided) block input
                layers.append(_conv(pre + '/conv4', n_in, n_out, 1, 1, 0, ho, ho, False))
                layers.append(_bn(pre + '/bn4', n_out, ho, ho))
                h = ho
            else:
                layers.append(_conv(pre + '/conv1', n_out, ch, 1, 1, 0, h, h, False))
                layers.append(_bn(pre + '/bn1', ch, h, h))
                layers.append(_conv(pre + '/conv2', ch, ch, 3, 1, 1, h, h, False))
                layers.append(_bn(pre + '/bn2', ch, h, h))
                layers.append(_conv(pre + '/conv3', ch, n_out, 1, 1, 0, h, h, False))
                layers.append(_bn(pre + '/bn3', n_out, h, h))
            n_in = n_out
    layers.append(_linear('fc', 2048, 1000))
    return layers


def factor_dims(layer):
    """Dimensions of the Kronecker factors of one layer: (dA, dG) or (dF,)."""
    if layer['kind'] == 'conv':
        return (layer['c_in'] * layer['k'] ** 2 + (1 if layer['bias'] else 0), layer['c_out'])
    if layer['kind'] == 'linear':
        return (layer['d_in'] + (1 if layer['bias'] else 0), layer['d_out'])
    return (2 * layer['c'],)


def all_factor_dims(layers):
    return [d for layer in layers for d in factor_dims(layer)]


def cov_rows(layer, batch):
    """Rows of the matrix whose Gram matrix is the layer's factor(s)."""
    if layer['kind'] == 'conv':
        ho = conv_out(layer['h'], layer['k'], layer['s'], layer['p'])
        wo = conv_out(layer['w'], layer['k'], layer['s'], layer['p'])
        return batch * ho * wo
    return batch


def flops(layers, batch):
    """Algorithmic work of one K-FAC step: cov = M d (d+1) per factor,
    inverse = d^3 per factor, precondition = 2 dG^2 dA + 2 dG dA^2 per
    connection layer and 2 (2C)^2 per batch-norm layer."""
    cov = inv = pre = 0
    for layer in layers:
        m = cov_rows(layer, batch)
        dims = factor_dims(layer)
        for d in dims:
            cov += m * d * (d + 1)
            inv += d ** 3
        if len(dims) == 2:
            dA, dG = dims
            pre += 2 * dG * dG * dA + 2 * dG * dA * dA
        else:
            pre += 2 * dims[0] ** 2
    return dict(cov=cov, inverse=inv, precondition=pre)


def takes_shift_route(layer):
    """Whether the library computes the layer's A factor from shifted correlations of
    the input (3x3, stride 1, padding 1, at least 64 channels or 28..32, images of at
    least 4 x 4: the conditions of try_conv_shift in csrc/cov.hip) rather than as a
    product of patch matrices."""
    return (layer['kind'] == 'conv' and layer['k'] == 3 and layer['s'] == 1 and layer['p'] == 1 and
            (layer['c_in'] >= 64 or 28 <= layer['c_in'] <= 32) and layer['h'] >= 4 and layer['w'] >= 4)


def cov_flops_executed(layers, batch):
    """Multiply-add work (2 flop each) that the covariance kernels issue for one step,
    where it differs from the algorithmic M d (d+1) of flops(): a factor on the
    shifted-correlation route takes 13 whole-image products of C x C, 6 over one image
    row, 6 over one image column and 4 over one pixel, each computed in full."""
    total = 0
    for layer in layers:
        m = cov_rows(layer, batch)
        dims = factor_dims(layer)
        for i, d in enumerate(dims):
            if i == 0 and takes_shift_route(layer):
                c, h, w = layer['c_in'], layer['h'], layer['w']
                if c <= 32:
                    # stacked tiles: 18 blocks of 32 x 32 over the whole image (13 of them needed),
                    # strips and corners as three-shift groups on a 64 x 64 tile
                    total += 2 * batch * (18 * 32 * 32 * h * w + 3 * 64 * 64 * (2 * w + 2 * h + 4))
                else:
                    total += 2 * c * c * batch * (13 * h * w + 6 * w + 6 * h + 4)
            else:
                total += m * d * (d + 1)
    return total


def build_resnet50_v1(device='cuda', generator=None, n_class=1000, bias=True):
    """The network behind the ``resnet50_v1`` layer table as a callable chain of
    ``chainerkfac_amd.links``: bottleneck topology of the reference's
    examples/cifar10/models/resnet50.py:6-73 (1x1 -> 3x3 -> 1x1 with a batch
    normalisation after every convolution, stride on the first 1x1, a projection
    shortcut in the first bottleneck of every stage, no activation after the
    sum) behind the ImageNet stem (7x7/2 convolution, 3x3/2 max-pooling), global
    average pooling and an ``n_class``-way linear layer.  ``bias`` gives every
    convolution a bias, as the benchmark configuration states."""
    import torch.nn.functional as TF
    from chainerkfac_amd import links as L

    def conv(c_in, c_out, k, s, p):
        return L.Convolution2D(c_in, c_out, k, s, p, nobias=not bias, device=device, generator=generator)

    class Bottleneck(L.Chain):
        def __init__(self, n_in, n_mid, n_out, stride, project):
            super(Bottleneck, self).__init__()
            self.conv1, self.bn1 = conv(n_in, n_mid, 1, stride, 0), L.BatchNormalization(n_mid, device=device)
            self.conv2, self.bn2 = conv(n_mid, n_mid, 3, 1, 1), L.BatchNormalization(n_mid, device=device)
            self.conv3, self.bn3 = conv(n_mid, n_out, 1, 1, 0), L.BatchNormalization(n_out, device=device)
            if project:
                self.conv4, self.bn4 = conv(n_in, n_out, 1, stride, 0), L.BatchNormalization(n_out, device=device)
            self.project = project

        def __call__(self, x):
            h = TF.relu(self.bn1(self.conv1(x)))
            h = TF.relu(self.bn2(self.conv2(h)))
            h = self.bn3(self.conv3(h))
            return h + (self.bn4(self.conv4(x)) if self.project else x)

    class Net(L.Chain):
        def __init__(self):
            super(Net, self).__init__()
            self.conv1, self.bn1 = conv(3, 64, 7, 2, 3), L.BatchNormalization(64, device=device)
            n_in = 64
            for si, (n_mid, n_out, blocks, stride) in enumerate(
                    [(64, 256, 3, 1), (128, 512, 4, 2), (256, 1024, 6, 2), (512, 2048, 3, 2)]):
                stage = L.ChainList(*[Bottleneck(n_in if b == 0 else n_out, n_mid, n_out,
                                                 stride if b == 0 else 1, b == 0) for b in range(blocks)])
                setattr(self, 'res{}'.format(si + 2), stage)
                n_in = n_out
            self.fc = L.Linear(2048, n_class, device=device, generator=generator)

        def __call__(self, x):
            h = TF.max_pool2d(TF.relu(self.bn1(self.conv1(x))), 3, 2, 1)
            for name in ('res2', 'res3', 'res4', 'res5'):
                for block in getattr(self, name):
                    h = block(h)
            return self.fc(h.mean(dim=(2, 3)))

    return Net()
