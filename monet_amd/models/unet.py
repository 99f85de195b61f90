"""The U-Net the reference benchmarks (models/unet/unet_model.py:8-39,
unet_parts.py:8-77): four max-pool / double-convolution stages down, four
stages up in which "upsampling" is an adaptive average pool to the skip
connection's size followed by a channel concatenation, and a 1x1 head."""
import torch
import torch.nn as nn


def _double_conv(cin, cout, mid=None):
    mid = mid or cout
    return nn.Sequential(
        nn.Conv2d(cin, mid, 3, padding=1), nn.BatchNorm2d(mid), nn.ReLU(inplace=True),
        nn.Conv2d(mid, cout, 3, padding=1), nn.BatchNorm2d(cout), nn.ReLU(inplace=True))


class DoubleConv(nn.Module):
    def __init__(self, cin, cout, mid=None):
        super().__init__()
        self.double_conv = _double_conv(cin, cout, mid)

    def forward(self, x):
        return self.double_conv(x)


class Down(nn.Module):
    def __init__(self, cin, cout):
        super().__init__()
        self.maxpool_conv = nn.Sequential(nn.MaxPool2d(2), DoubleConv(cin, cout))

    def forward(self, x):
        return self.maxpool_conv(x)


class Up(nn.Module):
    def __init__(self, cin, cout, height, width):
        super().__init__()
        self.up = nn.AdaptiveAvgPool2d((height, width))
        self.conv = DoubleConv(cin, cout, cin // 2)

    def forward(self, low, skip):
        return self.conv(torch.cat([skip, self.up(low)], dim=1))


class OutConv(nn.Module):
    def __init__(self, cin, cout):
        super().__init__()
        self.conv = nn.Conv2d(cin, cout, 1)

    def forward(self, x):
        return self.conv(x)


class UNet(nn.Module):
    def __init__(self, n_channels, n_classes, height, width):
        super().__init__()
        self.n_channels, self.n_classes = n_channels, n_classes
        self.inc = DoubleConv(n_channels, 64)
        self.down1, self.down2 = Down(64, 128), Down(128, 256)
        self.down3, self.down4 = Down(256, 512), Down(512, 512)
        self.up1 = Up(1024, 256, height // 8, width // 8)
        self.up2 = Up(512, 128, height // 4, width // 4)
        self.up3 = Up(256, 64, height // 2, width // 2)
        self.up4 = Up(128, 64, height, width)
        self.outc = OutConv(64, n_classes)

    def forward(self, x):
        x1 = self.inc(x)
        x2 = self.down1(x1)
        x3 = self.down2(x2)
        x4 = self.down3(x3)
        x5 = self.down4(x4)
        x = self.up1(x5, x4)
        x = self.up2(x, x3)
        x = self.up3(x, x2)
        x = self.up4(x, x1)
        return self.outc(x)
