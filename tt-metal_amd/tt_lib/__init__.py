"""tt_lib mirror for the block-float hot path on MI355X (tensor, operations.primary, device)."""
from . import tensor  # noqa: F401
from . import operations  # noqa: F401


class device:  # namespace mirror of tt_lib.device
    @staticmethod
    def CreateDevice(device_id: int = 0):
        return tensor.Device(device_id)

    @staticmethod
    def CloseDevice(dev) -> None:
        import torch

        torch.cuda.synchronize(dev.torch_device)

    @staticmethod
    def Synchronize(dev=None) -> None:
        import torch

        torch.cuda.synchronize()
