import torch


class LinearBase(torch.nn.Module):
    """Common base of the quantized Linear modules (nn_models/modules/linear/linear_base.py:2-12)."""

    def __init__(self):
        super().__init__()

    def forward(self, x):
        raise NotImplementedError
