"""Shape-equivalent CIFAR networks for the benchmarks (32x32 inputs): ResNet-18 with a 3x3 stem and no
max-pool (same layer shapes as the reference's ``micronet+/models.py:86-120,151-211``) and the VGG-16
convolution stack (``models.py:35-65``).  Plain ``nn.Module``s; ``app_layers.prepare`` rewrites them."""
import torch.nn as nn


def _conv_bn_relu(cin, cout, stride=1):
    return [nn.Conv2d(cin, cout, 3, stride=stride, padding=1, bias=False), nn.BatchNorm2d(cout), nn.ReLU(inplace=True)]


class BasicBlock(nn.Module):
    def __init__(self, cin, cout, stride):
        super().__init__()
        self.residual_function = nn.Sequential(*_conv_bn_relu(cin, cout, stride),
                                               nn.Conv2d(cout, cout, 3, padding=1, bias=False), nn.BatchNorm2d(cout))
        self.shortcut = nn.Sequential()
        if stride != 1 or cin != cout:
            self.shortcut = nn.Sequential(nn.Conv2d(cin, cout, 1, stride=stride, bias=False), nn.BatchNorm2d(cout))
        self.relu = nn.ReLU(inplace=True)

    def forward(self, x):
        return self.relu(self.residual_function(x) + self.shortcut(x))


class ResNet18(nn.Module):
    def __init__(self, num_classes=10):
        super().__init__()
        self.conv1 = nn.Sequential(*_conv_bn_relu(3, 64))
        stages, cin = [], 64
        for cout, stride in ((64, 1), (128, 2), (256, 2), (512, 2)):
            stages.append(nn.Sequential(BasicBlock(cin, cout, stride), BasicBlock(cout, cout, 1)))
            cin = cout
        self.conv2_x, self.conv3_x, self.conv4_x, self.conv5_x = stages
        self.avg_pool = nn.AdaptiveAvgPool2d((1, 1))
        self.fc = nn.Linear(512, num_classes)

    def forward(self, x):
        x = self.conv5_x(self.conv4_x(self.conv3_x(self.conv2_x(self.conv1(x)))))
        return self.fc(self.avg_pool(x).flatten(1))


class VGG16(nn.Module):
    CFG = (64, 64, 'M', 128, 128, 'M', 256, 256, 256, 'M', 512, 512, 512, 'M', 512, 512, 512, 'M')

    def __init__(self, num_classes=10):
        super().__init__()
        layers, cin = [], 3
        for v in self.CFG:
            if v == 'M':
                layers.append(nn.MaxPool2d(2, 2))
            else:
                layers += [nn.Conv2d(cin, v, 3, padding=1), nn.BatchNorm2d(v), nn.ReLU(inplace=True)]
                cin = v
        self.features = nn.Sequential(*layers)
        self.classifier = nn.Linear(512, num_classes)

    def forward(self, x):
        return self.classifier(self.features(x).flatten(1))


def resnet18(num_classes=10):
    return ResNet18(num_classes)


def vgg16(num_classes=10):
    return VGG16(num_classes)
