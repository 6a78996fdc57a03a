"""The two networks the benchmark configurations name, built from the SC layers.

TinyConvSC   conv3x3 3->32->32, maxpool2, ->64->64, maxpool2, fc 4096->10 (float fc).
ResNet18SC   topology of the reference's resnet_sc.py (:48-99 BasicBlock, :158-260 ResNet):
             float 7x7 stem + BatchNorm(eps 1e-3) + Hardtanh(0,1) + AvgPool(3,2,1), BasicBlocks whose
             3x3 and 1x1 convs are SC layers, Hardtanh(0,1) activations, float fc; Kaiming init.
"""
import torch
import torch.nn as nn

import sc_functional as utils_f
from sc_layers import Conv2d_Add_Partial


def _sc3x3(cin, cout, stride, **sc):
    return Conv2d_Add_Partial(cin, cout, kernel_size=3, stride=stride, padding=1, bias=False, **sc)


def _sc1x1(cin, cout, stride, **sc):
    return Conv2d_Add_Partial(cin, cout, kernel_size=1, stride=stride, bias=False, **sc)


class TinyConvSC(nn.Module):
    def __init__(self, num_classes=10, **sc):
        super().__init__()
        act = lambda: nn.Hardtanh(0, 1)
        self.features = nn.Sequential(
            _sc3x3(3, 32, 1, **sc), nn.BatchNorm2d(32), act(),
            _sc3x3(32, 32, 1, **sc), nn.BatchNorm2d(32), act(), nn.MaxPool2d(2),
            _sc3x3(32, 64, 1, **sc), nn.BatchNorm2d(64), act(),
            _sc3x3(64, 64, 1, **sc), nn.BatchNorm2d(64), act(), nn.MaxPool2d(2))
        self.fc = nn.Linear(64 * 8 * 8, num_classes)
        self.sync = 1
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out", nonlinearity="relu")

    def forward(self, x):
        utils_f.update_sync(self, self.sync)
        x = self.features(x)
        return self.fc(torch.flatten(x, 1))


class BasicBlock(nn.Module):
    def __init__(self, inplanes, planes, stride=1, downsample=None, **sc):
        super().__init__()
        self.conv1 = _sc3x3(inplanes, planes, stride, **sc)
        self.bn1 = nn.BatchNorm2d(planes)
        self.relu = nn.Hardtanh(0, 1)
        self.conv2 = _sc3x3(planes, planes, 1, **sc)
        self.bn2 = nn.BatchNorm2d(planes)
        self.downsample = downsample

    def forward(self, x):
        identity = x
        out = self.relu(self.bn1(self.conv1(x)))
        out = self.bn2(self.conv2(out))
        if self.downsample is not None:
            identity = self.downsample(x)
        out = out + identity
        return self.relu(out)


class ResNet18SC(nn.Module):
    def __init__(self, num_classes=1000, **sc):
        super().__init__()
        self.inplanes = 64
        strides = [1, 1, 2, 2] if num_classes < 1000 else [2, 2, 2, 2]
        self.conv1 = nn.Conv2d(3, 64, kernel_size=7, stride=strides[0], padding=3, bias=False)
        self.bn1 = nn.BatchNorm2d(64, eps=1e-3)
        self.relu = nn.Hardtanh(0, 1)
        self.maxpool = nn.AvgPool2d(kernel_size=3, stride=2, padding=1)
        self.layer1 = self._make_layer(64, 2, 1, sc)
        self.layer2 = self._make_layer(128, 2, strides[1], sc)
        self.layer3 = self._make_layer(256, 2, strides[2], sc)
        self.layer4 = self._make_layer(512, 2, strides[3], sc)
        self.avgpool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(512, num_classes)
        self.sync = 1
        for m in self.modules():
            if isinstance(m, nn.Conv2d):
                nn.init.kaiming_normal_(m.weight, mode="fan_out", nonlinearity="relu")
            elif isinstance(m, nn.BatchNorm2d):
                nn.init.constant_(m.weight, 1)
                nn.init.constant_(m.bias, 0)

    def _make_layer(self, planes, blocks, stride, sc):
        downsample = None
        if stride != 1 or self.inplanes != planes:
            downsample = nn.Sequential(_sc1x1(self.inplanes, planes, stride, **sc), nn.BatchNorm2d(planes))
        layers = [BasicBlock(self.inplanes, planes, stride, downsample, **sc)]
        self.inplanes = planes
        for _ in range(1, blocks):
            layers.append(BasicBlock(planes, planes, **sc))
        return nn.Sequential(*layers)

    def forward(self, x):
        utils_f.update_sync(self, self.sync)
        x = self.maxpool(self.relu(self.bn1(self.conv1(x))))
        x = self.layer4(self.layer3(self.layer2(self.layer1(x))))
        x = torch.flatten(self.avgpool(x), 1)
        return self.fc(x)
