"""ResNet-50 (v1.5: stride on the 3x3 convolution) in the standard public layout, built from
plain torch.nn layers (and AddReLU for the closing relu(out + identity) of a block) so that QModule
can convert it; relu(bn(x)) pairs and the closing relu(bn(x) + identity) are handed to layers.bn_relu /
bn_add_relu, which are the separate calls for plain layers.  torchvision is not available in this
environment; the reference benchmarks torchvision's resnet50
(mem_speed_benchmark/train.py:170,203-206)."""
import torch
import torch.nn as nn

from .layers import AddReLU, bn_add_relu, bn_relu, skip_connection


class Bottleneck(nn.Module):
    expansion = 4

    def __init__(self, inplanes, planes, stride=1, downsample=None):
        super().__init__()
        self.conv1 = nn.Conv2d(inplanes, planes, 1, bias=False)
        self.bn1 = nn.BatchNorm2d(planes)
        self.conv2 = nn.Conv2d(planes, planes, 3, stride=stride, padding=1, bias=False)
        self.bn2 = nn.BatchNorm2d(planes)
        self.conv3 = nn.Conv2d(planes, planes * self.expansion, 1, bias=False)
        self.bn3 = nn.BatchNorm2d(planes * self.expansion)
        # three separate modules: a converted ReLU keeps one mask per call site
        self.relu1 = nn.ReLU(inplace=True)
        self.relu2 = nn.ReLU(inplace=True)
        self.relu3 = AddReLU()          # relu(out + identity), fused into one pass when converted
        self.downsample = downsample

    def forward(self, x):
        # a block without a downsample branch adds its own input back: tie the two uses of it together
        x, identity = skip_connection(self.relu3, x) if self.downsample is None else (x, None)
        out = bn_relu(self.bn1, self.relu1, self.conv1(x))
        out = bn_relu(self.bn2, self.relu2, self.conv2(out))
        if self.downsample is not None:
            identity = self.downsample(x)
        return bn_add_relu(self.bn3, self.relu3, self.conv3(out), identity)


class ResNet(nn.Module):
    def __init__(self, layers=(3, 4, 6, 3), num_classes=1000, width=64):
        super().__init__()
        self.inplanes = width
        self.conv1 = nn.Conv2d(3, width, 7, stride=2, padding=3, bias=False)
        self.bn1 = nn.BatchNorm2d(width)
        self.relu = nn.ReLU(inplace=True)
        self.maxpool = nn.MaxPool2d(3, stride=2, padding=1)
        self.layer1 = self._make_layer(width, layers[0])
        self.layer2 = self._make_layer(width * 2, layers[1], stride=2)
        self.layer3 = self._make_layer(width * 4, layers[2], stride=2)
        self.layer4 = self._make_layer(width * 8, layers[3], stride=2)
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(width * 8 * Bottleneck.expansion, num_classes)
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out", nonlinearity="relu")

    def _make_layer(self, planes, blocks, stride=1):
        downsample = None
        if stride != 1 or self.inplanes != planes * Bottleneck.expansion:
            downsample = nn.Sequential(
                nn.Conv2d(self.inplanes, planes * Bottleneck.expansion, 1, stride=stride, bias=False),
                nn.BatchNorm2d(planes * Bottleneck.expansion))
        layers = [Bottleneck(self.inplanes, planes, stride, downsample)]
        self.inplanes = planes * Bottleneck.expansion
        layers += [Bottleneck(self.inplanes, planes) for _ in range(1, blocks)]
        return nn.Sequential(*layers)

    def forward(self, x):
        x = self.maxpool(bn_relu(self.bn1, self.relu, self.conv1(x)))
        x = self.layer4(self.layer3(self.layer2(self.layer1(x))))
        return self.fc(torch.flatten(self.avgpool(x), 1))


def resnet50(num_classes=1000):
    return ResNet((3, 4, 6, 3), num_classes)
