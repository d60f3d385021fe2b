"""ResNet-18 written against the layer API exactly as the reference's timing script does
(tests/resnet/resnet18_dg.py:12-75): BasicBlock = conv3x3(s)/BN/ReLU/conv3x3/BN + shortcut
[1x1(s) conv/BN when the shape changes], add, ReLU; stages [2, 2, 2, 2]; 7x7/2 stem, 3x3/2 max-pool.
``pool`` and ``classes`` choose the tail: the reference script uses AvgPooling2D(2) and 100 classes on 56x56
inputs; the 224x224 benchmark configuration uses a global 7x7 average pool and 1000 classes.
"""
import numpy as np

from xshinnosuke_amd.layers import Conv2D, BatchNormalization, ReLU, MaxPooling2D, AvgPooling2D, Flatten, Dense
from xshinnosuke_amd.nn.models import Module, Sequential


class BasicBlock(Module):
    def __init__(self, in_channels, out_channels, stride, init='he_normal'):
        super().__init__()
        self.conv1 = Sequential(
            Conv2D(out_channels, 3, stride=stride, padding=1, kernel_initializer=init),
            BatchNormalization(),
            ReLU(True),
            Conv2D(out_channels, 3, stride=1, padding=1, kernel_initializer=init),
            BatchNormalization(),
        )
        if stride != 1 or in_channels != out_channels:
            self.shortcut = Sequential(Conv2D(out_channels, 1, stride=stride, kernel_initializer=init),
                                       BatchNormalization())
        else:
            self.shortcut = Sequential()
        self.relu = ReLU(inplace=True)

    def forward(self, x, *args):
        out = self.conv1(x)
        out += self.shortcut(x)
        return self.relu(out)


class ResNet18(Module):
    def __init__(self, classes=1000, pool=7, init='he_normal', dense_init='he_normal'):
        super().__init__()
        self.conv1 = Sequential(Conv2D(out_channels=64, kernel_size=7, stride=2, padding=3, kernel_initializer=init),
                                BatchNormalization(), ReLU(inplace=True))
        self.pool1 = MaxPooling2D(kernel_size=3, stride=2, padding=1)
        self.in_channels = 64
        self.layer1 = self._stage(64, 2, 1, init)
        self.layer2 = self._stage(128, 2, 2, init)
        self.layer3 = self._stage(256, 2, 2, init)
        self.layer4 = self._stage(512, 2, 2, init)
        self.pool2 = AvgPooling2D(pool)
        self.flat = Flatten()
        self.fc = Dense(classes, kernel_initializer=dense_init)

    def _stage(self, channels, blocks, stride, init):
        layers = []
        for s in [stride] + [1] * (blocks - 1):
            layers.append(BasicBlock(self.in_channels, channels, s, init))
            self.in_channels = channels
        return Sequential(*layers)

    def forward(self, x, *args):
        x = self.conv1(x)
        x = self.pool1(x)
        x = self.layer1(x)
        x = self.layer2(x)
        x = self.layer3(x)
        x = self.layer4(x)
        x = self.pool2(x)
        x = self.flat(x)
        return self.fc(x)


def named_params(net):
    """Parameters in a reproducible order: walk the modules the way forward() uses them."""
    out = []

    def seq(s):
        for layer in s._graph:
            if hasattr(layer, '_graph'):
                seq(layer)
            elif hasattr(layer, 'conv1'):
                seq(layer.conv1); seq(layer.shortcut)
            else:
                out.extend(p for p in layer.parameters() if p is not None)
    seq(net.conv1)
    for stage in (net.layer1, net.layer2, net.layer3, net.layer4):
        seq(stage)
    out.extend(net.fc.parameters())
    return out


def oracle_forward(net, x):
    """ResNet-18 inference (moving-statistics batch norm) in NumPy: convolutions and the max-pool through the
    oracle (float64 GEMM, one rounding), the rest in float64 rounded to float32 per op."""
    import oracle            # the CPU checker: test / benchmark-baseline use only

    def bn(layer, a):
        g, b = (p.numpy().astype(np.float64).reshape(1, -1, 1, 1) for p in layer.parameters())
        mm = layer.moving_mean.numpy().astype(np.float64).reshape(1, -1, 1, 1)
        mv = layer.moving_variance.numpy().astype(np.float64).reshape(1, -1, 1, 1)
        return (g * (a - mm) / np.sqrt(mv + layer.epsilon) + b).astype(np.float32)

    def run(layer, a):
        name = type(layer).__name__
        if name == 'Sequential':
            for sub in layer._graph:
                a = run(sub, a)
            return a
        if name == 'BasicBlock':
            out = run(layer.conv1, a) + run(layer.shortcut, a)
            return np.maximum(out, 0)
        if name == 'Conv2D':
            w, b = (p.numpy() for p in layer.parameters())
            return oracle.conv2d_fwd(a, w.astype(np.float32), b.reshape(-1).astype(np.float32), layer.stride, layer.pad_size)[0]
        if name == 'BatchNormalization':
            return bn(layer, a)
        if name == 'ReLU':
            return np.maximum(a, 0)
        raise AssertionError(name)

    a = run(net.conv1, x)
    a = oracle.max_pool2d_fwd(a, 3, (2, 2), 1)[0]
    for stage in (net.layer1, net.layer2, net.layer3, net.layer4):
        a = run(stage, a)
    k = net.pool2.kernel_size
    n, c, h, w = a.shape
    a = a.astype(np.float64).reshape(n, c, h // k, k, w // k, k).mean(axis=(3, 5)).astype(np.float32)
    wfc, bfc = (p.numpy().astype(np.float64) for p in net.fc.parameters())
    return (a.reshape(n, -1).astype(np.float64) @ wfc + bfc).astype(np.float32)
