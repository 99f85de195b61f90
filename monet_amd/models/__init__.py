"""Model definitions the headline configurations are quoted on."""
from .resnet import resnet18, resnet50  # noqa: F401
from .unet import UNet  # noqa: F401
