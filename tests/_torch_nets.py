"""Small torch networks in the styles of the served model families, used by the ONNX import tests: each is exported
with torch's own ONNX exporter and the imported graph must reproduce the module's forward pass."""
import torch
import torch.nn as nn
import torch.nn.functional as F


def randomize(module, seed):
    """Non-trivial parameters everywhere, including batch-norm statistics."""
    g = torch.Generator().manual_seed(seed)
    with torch.no_grad():
        for m in module.modules():
            if isinstance(m, nn.BatchNorm2d):
                m.weight.copy_(torch.rand(m.weight.shape, generator=g) + 0.5)
                m.bias.copy_(torch.randn(m.bias.shape, generator=g) * 0.1)
                m.running_mean.copy_(torch.randn(m.running_mean.shape, generator=g) * 0.2)
                m.running_var.copy_(torch.rand(m.running_var.shape, generator=g) + 0.5)
            elif isinstance(m, (nn.Conv2d, nn.Linear)):
                fan_in = m.weight[0].numel()
                m.weight.copy_(torch.randn(m.weight.shape, generator=g) * (2.0 / fan_in) ** 0.5)
                if m.bias is not None:
                    m.bias.copy_(torch.randn(m.bias.shape, generator=g) * 0.05)
            elif isinstance(m, nn.PReLU):
                m.weight.copy_(torch.rand(m.weight.shape, generator=g) * 0.4)
    return module.eval()


class BasicBlock(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.conv1 = nn.Conv2d(cin, cout, 3, stride, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(cout)
        self.conv2 = nn.Conv2d(cout, cout, 3, 1, 1, bias=False)
        self.bn2 = nn.BatchNorm2d(cout)
        self.downsample = None
        if stride != 1 or cin != cout:
            self.downsample = nn.Sequential(nn.Conv2d(cin, cout, 1, stride, bias=False), nn.BatchNorm2d(cout))

    def forward(self, x):
        out = F.relu(self.bn1(self.conv1(x)))
        out = self.bn2(self.conv2(out))
        identity = x if self.downsample is None else self.downsample(x)
        return F.relu(out + identity)


class ResNet(nn.Module):
    """torchvision's ResNet layout (BasicBlock): layers=[2,2,2,2], width 64, 224x224 is ResNet-18."""

    def __init__(self, layers=(2, 2, 2, 2), width=64, classes=1000):
        super().__init__()
        self.conv1 = nn.Conv2d(3, width, 7, 2, 3, bias=False)
        self.bn1 = nn.BatchNorm2d(width)
        blocks, cin = [], width
        for stage, count in enumerate(layers):
            for b in range(count):
                cout = width * 2 ** stage
                blocks.append(BasicBlock(cin, cout, 2 if (stage > 0 and b == 0) else 1))
                cin = cout
        self.blocks = nn.Sequential(*blocks)
        self.fc = nn.Linear(cin, classes)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.bn1(self.conv1(x))), 3, 2, 1)
        x = self.blocks(x)
        return self.fc(torch.flatten(F.adaptive_avg_pool2d(x, 1), 1))


class Fire(nn.Module):
    def __init__(self, cin, squeeze, e1, e3):
        super().__init__()
        self.squeeze, self.e1, self.e3 = nn.Conv2d(cin, squeeze, 1), nn.Conv2d(squeeze, e1, 1), nn.Conv2d(squeeze, e3, 3, padding=1)

    def forward(self, x):
        s = F.relu(self.squeeze(x))
        return torch.cat([F.relu(self.e1(s)), F.relu(self.e3(s))], 1)


class SqueezeStyle(nn.Module):
    def __init__(self):
        super().__init__()
        self.stem = nn.Conv2d(3, 16, 3, 2)
        self.f1, self.f2 = Fire(16, 4, 8, 8), Fire(16, 4, 12, 12)
        self.head = nn.Conv2d(24, 10, 1)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.stem(x)), 3, 2, ceil_mode=True)
        x = F.max_pool2d(self.f2(self.f1(x)), 3, 2, ceil_mode=True)
        return torch.flatten(F.adaptive_avg_pool2d(F.relu(self.head(x)), 1), 1)


class InvertedResidual(nn.Module):
    def __init__(self, cin, cout, stride, expand):
        super().__init__()
        hidden = cin * expand
        self.use_res = stride == 1 and cin == cout
        self.body = nn.Sequential(
            nn.Conv2d(cin, hidden, 1, bias=False), nn.BatchNorm2d(hidden), nn.ReLU6(),
            nn.Conv2d(hidden, hidden, 3, stride, 1, groups=hidden, bias=False), nn.BatchNorm2d(hidden), nn.ReLU6(),
            nn.Conv2d(hidden, cout, 1, bias=False), nn.BatchNorm2d(cout))

    def forward(self, x):
        return x + self.body(x) if self.use_res else self.body(x)


class MobileStyle(nn.Module):
    def __init__(self):
        super().__init__()
        self.stem = nn.Sequential(nn.Conv2d(3, 8, 3, 2, 1, bias=False), nn.BatchNorm2d(8), nn.ReLU6())
        self.blocks = nn.Sequential(InvertedResidual(8, 8, 1, 4), InvertedResidual(8, 16, 2, 4), InvertedResidual(16, 16, 1, 4))
        self.fc = nn.Linear(16, 7)

    def forward(self, x):
        x = self.blocks(self.stem(x))
        return self.fc(torch.flatten(F.adaptive_avg_pool2d(x, 1), 1))


class DenseStyle(nn.Module):
    """Pre-activation dense layers (norm -> relu -> conv), concatenation of every layer's output, a transition."""

    def __init__(self, growth=6, layers=3):
        super().__init__()
        self.stem = nn.Conv2d(3, 12, 3, 1, 1, bias=False)
        self.layers = nn.ModuleList()
        c = 12
        for _ in range(layers):
            self.layers.append(nn.Sequential(nn.BatchNorm2d(c), nn.ReLU(), nn.Conv2d(c, 2 * growth, 1, bias=False),
                                             nn.BatchNorm2d(2 * growth), nn.ReLU(), nn.Conv2d(2 * growth, growth, 3, 1, 1, bias=False)))
            c += growth
        self.transition = nn.Sequential(nn.BatchNorm2d(c), nn.ReLU(), nn.Conv2d(c, c // 2, 1, bias=False), nn.AvgPool2d(2, 2))
        self.norm = nn.BatchNorm2d(c // 2)
        self.fc = nn.Linear(c // 2, 5)

    def forward(self, x):
        x = F.max_pool2d(self.stem(x), 3, 2, 1)
        for layer in self.layers:
            x = torch.cat([x, layer(x)], 1)
        x = F.relu(self.norm(self.transition(x)))
        return self.fc(torch.flatten(F.adaptive_avg_pool2d(x, 1), 1))


class InceptionStyle(nn.Module):
    """Asymmetric kernels, an average-pool branch that counts its padding, a strided reduction block, softmax."""

    def __init__(self):
        super().__init__()
        bn = lambda c: nn.BatchNorm2d(c, eps=0.001)
        self.stem = nn.Sequential(nn.Conv2d(3, 16, 3, 2, bias=False), bn(16), nn.ReLU())
        self.b1 = nn.Sequential(nn.Conv2d(16, 8, 1, bias=False), bn(8), nn.ReLU())
        self.b7 = nn.Sequential(nn.Conv2d(16, 6, 1, bias=False), bn(6), nn.ReLU(), nn.Conv2d(6, 6, (1, 7), padding=(0, 3), bias=False), bn(6), nn.ReLU(),
                                nn.Conv2d(6, 8, (7, 1), padding=(3, 0), bias=False), bn(8), nn.ReLU())
        self.bp = nn.Sequential(nn.Conv2d(16, 4, 1, bias=False), bn(4), nn.ReLU())
        self.r3 = nn.Sequential(nn.Conv2d(20, 12, 3, 2, bias=False), bn(12), nn.ReLU())
        self.fc = nn.Linear(32, 9)

    def forward(self, x):
        x = self.stem(x)
        x = torch.cat([self.b1(x), self.b7(x), self.bp(F.avg_pool2d(x, 3, 1, 1))], 1)
        x = torch.cat([self.r3(x), F.max_pool2d(x, 3, 2)], 1)
        return F.softmax(self.fc(torch.flatten(F.adaptive_avg_pool2d(x, 1), 1)), 1)


class FaceStyle(nn.Module):
    """Per-channel PReLU after a conv, a norm in front of a zero-padded conv (not foldable), residual without activation,
    a flatten of a spatial map into the embedding layer, leaky relu."""

    def __init__(self):
        super().__init__()
        self.conv0, self.bn0, self.act0 = nn.Conv2d(3, 8, 3, 1, 1, bias=False), nn.BatchNorm2d(8), nn.PReLU(8)
        self.bn1, self.conv1, self.bn2, self.act1 = nn.BatchNorm2d(8), nn.Conv2d(8, 8, 3, 1, 1, bias=False), nn.BatchNorm2d(8), nn.PReLU(8)
        self.conv2, self.bn3 = nn.Conv2d(8, 8, 3, 2, 1, bias=False), nn.BatchNorm2d(8)
        self.short = nn.Sequential(nn.Conv2d(8, 8, 1, 2, bias=False), nn.BatchNorm2d(8))
        self.bn4 = nn.BatchNorm2d(8)
        self.fc = nn.Linear(8 * 6 * 6, 16)

    def forward(self, x):
        x = self.act0(self.bn0(self.conv0(x)))
        y = self.bn3(self.conv2(self.act1(self.bn2(self.conv1(self.bn1(x))))))
        x = y + self.short(x)
        x = F.leaky_relu(self.bn4(x), 0.1)
        return self.fc(torch.flatten(x, 1))


class PreActBlock(nn.Module):
    """ResNet v2 unit (the layout of the resnet*-v2-7 zoo files): norm and relu come BEFORE each conv, the shortcut
    branches off after the first norm+relu when it projects, and nothing follows the addition."""

    def __init__(self, cin, cout, stride):
        super().__init__()
        self.bn1, self.conv1 = nn.BatchNorm2d(cin), nn.Conv2d(cin, cout, 3, stride, 1, bias=False)
        self.bn2, self.conv2 = nn.BatchNorm2d(cout), nn.Conv2d(cout, cout, 3, 1, 1, bias=False)
        self.project = nn.Conv2d(cin, cout, 1, stride, bias=False) if (stride != 1 or cin != cout) else None

    def forward(self, x):
        a = F.relu(self.bn1(x))
        shortcut = x if self.project is None else self.project(a)
        y = self.conv1(a)
        y = self.conv2(F.relu(self.bn2(y)))
        return y + shortcut


class ResNetV2Style(nn.Module):
    def __init__(self):
        super().__init__()
        self.bn_data = nn.BatchNorm2d(3)
        self.conv0, self.bn0 = nn.Conv2d(3, 8, 7, 2, 3, bias=False), nn.BatchNorm2d(8)
        self.blocks = nn.Sequential(PreActBlock(8, 8, 1), PreActBlock(8, 16, 2), PreActBlock(16, 16, 1))
        self.bn_last, self.fc = nn.BatchNorm2d(16), nn.Linear(16, 11)

    def forward(self, x):
        x = F.max_pool2d(F.relu(self.bn0(self.conv0(self.bn_data(x)))), 3, 2, 1)
        x = F.relu(self.bn_last(self.blocks(x)))
        return self.fc(torch.flatten(F.adaptive_avg_pool2d(x, 1), 1))


NETS = {
    "resnet_v2_style": (ResNetV2Style, (1, 3, 40, 40)),
    "resnet_style": (lambda: ResNet((1, 2), 8, 10), (1, 3, 32, 32)),
    "squeeze_style": (SqueezeStyle, (1, 3, 47, 47)),
    "mobile_style": (MobileStyle, (1, 3, 32, 32)),
    "dense_style": (DenseStyle, (1, 3, 24, 24)),
    "inception_style": (InceptionStyle, (1, 3, 35, 35)),
    "face_style": (FaceStyle, (1, 3, 12, 12)),
}
