"""Model definitions the headline configurations are quoted on."""
from .resnet import resnet18, resnet50  # noqa: F401
from .unet import UNet  # noqa: F401

UNET_SIZE = (416, 608)
UNET_CLASSES = 2


def build_model(spec):
    """(model, input_shape, short name) for a model given the way the reference's command
    lines name it: "unet", or an expression such as "torchvision.models.resnet50()"
    (monet/cvxpy_solver.py:358-365).  torchvision is used when it is installed; otherwise
    the architectures restated in this package stand in for the ones they cover."""
    if spec == "unet":
        # two output classes (softmax cross entropy over the class dimension); the reference's
        # own command lines build it with one (monet/schedule.py:391)
        h, w = UNET_SIZE
        return UNet(n_channels=3, n_classes=UNET_CLASSES, height=h, width=w), (3, h, w), "unet"
    name = spec.split(".")[-1]
    name = name[:-2] if name.endswith("()") else name
    try:
        import torchvision
        return getattr(torchvision.models, name)(), (3, 224, 224), name
    except ImportError:
        own = {"resnet18": resnet18, "resnet50": resnet50}
        if name not in own:
            raise ValueError("torchvision is not installed and %r is not restated here" % name)
        return own[name](), (3, 224, 224), name
