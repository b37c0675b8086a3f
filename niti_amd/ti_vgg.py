"""VGG-style CIFAR networks with the reference's ``ti_vgg.TiVGG_cifar`` interface (ti_vgg.py:10-42)."""
from torch.nn.modules import Sequential

from .ti_net import TiNet
from .ti_torch import TiConv2d, TiDropout, TiFlat, TiLinear, TiMaxpool2d, TiReLU

cifar_cfg = {
    7: [128, 128, 'M', 256, 256, 'M', 512, 512, 'M'],
    8: [128, 128, 128, 'M', 256, 256, 'M', 512, 512, 'M'],
    9: [128, 128, 128, 'M', 256, 256, 256, 'M', 512, 512, 'M'],
    # ten-conv VGG-13 widths (no counterpart in the reference's code, only in its result figure)
    13: [64, 64, 'M', 128, 128, 'M', 256, 256, 'M', 512, 512, 'M', 512, 512, 'M'],
}


class TiVGG_cifar(TiNet):
    def __init__(self, depth=None, fuse=True, dropout=True):
        super().__init__()
        self.forward_layers = self._make_layers(cifar_cfg[depth], dropout)
        self.regime = [{'epoch': 0, 'gb': 5},
                       {'epoch': 100, 'gb': 4},
                       {'epoch': 150, 'gb': 3}]
        if fuse:
            self.fuse()

    def _make_layers(self, cfg, dropout=True):
        layers = []
        in_channels = 3
        image_size = 32
        for idx, x in enumerate(cfg):
            if x == 'M':
                layers += [TiMaxpool2d(2, 2)]
                image_size = image_size // 2
            else:
                layers += [TiConv2d(in_channels, x, first_layer=(idx == 0)), TiReLU()]
                in_channels = x
        layers += [TiFlat()]
        if dropout:
            layers += [TiDropout()]
        layers += [TiLinear(512 * image_size * image_size, 10, last_layer=True)]
        return Sequential(*layers)
