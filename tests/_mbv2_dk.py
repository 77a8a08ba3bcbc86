"""MobileNetV2 (width 1.0, 224 x 224) with every 3 x 3 depthwise convolution replaced by DeformKernel2d
at scope 4 x 4 -- the whole-network stress configuration of the benchmark.  The reference ships no
network (its README lists models as under construction), so this is the textbook architecture
(inverted residuals: 1 x 1 expand, 3 x 3 depthwise, 1 x 1 project; t, c, n, s table of the paper) with
the library's layer dropped into the depthwise slot, as the reference's README describes its use.
Shared by the GPU test of the network and by `bench.py --workload mbv2_net`.
"""
import torch
from torch import nn

from deformable_kernels.modules import DeformKernel2d

# expansion t, output channels c, repeats n, stride s
SETTINGS = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2), (6, 320, 1, 1)]


def _bn_relu(ch):
    return [nn.BatchNorm2d(ch), nn.ReLU6(inplace=True)]


class InvertedResidualDK(nn.Module):
    def __init__(self, cin, cout, stride, expand, scope=(4, 4)):
        super().__init__()
        hidden = cin * expand
        self.residual = stride == 1 and cin == cout
        layers = []
        if expand != 1:
            layers += [nn.Conv2d(cin, hidden, 1, bias=False)] + _bn_relu(hidden)
        self.depthwise = DeformKernel2d(scope, hidden, hidden, kernel_size=3, stride=stride, padding=1,
                                        groups=hidden)
        layers += [self.depthwise] + _bn_relu(hidden)
        layers += [nn.Conv2d(hidden, cout, 1, bias=False), nn.BatchNorm2d(cout)]
        self.block = nn.Sequential(*layers)

    def forward(self, x):
        return x + self.block(x) if self.residual else self.block(x)


class MobileNetV2DK(nn.Module):
    def __init__(self, classes=1000, scope=(4, 4)):
        super().__init__()
        features = [nn.Conv2d(3, 32, 3, 2, 1, bias=False)] + _bn_relu(32)
        cin = 32
        for t, c, n, s in SETTINGS:
            for i in range(n):
                features.append(InvertedResidualDK(cin, c, s if i == 0 else 1, t, scope))
                cin = c
        features += [nn.Conv2d(cin, 1280, 1, bias=False)] + _bn_relu(1280)
        self.features = nn.Sequential(*features)
        self.classifier = nn.Linear(1280, classes)
        self.reset_parameters()

    def reset_parameters(self):
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                if getattr(m, "zero_init", False):
                    # offset branch: small random offsets instead of the customary zeros, so that a
                    # synthetic run exercises the deformed sampling and not the zero-offset special case
                    nn.init.normal_(m.weight, 0.0, 0.02)
                    nn.init.normal_(m.bias, 0.0, 0.3)
                else:
                    nn.init.kaiming_normal_(m.weight, mode="fan_out")
            elif isinstance(m, nn.Linear):
                nn.init.normal_(m.weight, 0.0, 0.01)
                nn.init.zeros_(m.bias)

    def dk_layers(self):
        return [m for m in self.modules() if isinstance(m, DeformKernel2d)]

    def forward(self, x):
        x = self.features(x)
        return self.classifier(x.mean((2, 3)))
