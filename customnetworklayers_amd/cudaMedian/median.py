"""Autograd surface of the median layer: the names, arguments and tensor layouts of the reference's
cudaMedian/median.py (MedianFunction, Median)."""
from torch import nn
from torch.autograd import Function

from . import median_cuda_ext


class MedianFunction(Function):
    @staticmethod
    def forward(ctx, in_vol):  # median.py:18-44
        outputs = median_cuda_ext.forward(in_vol.contiguous())
        ctx.save_for_backward(in_vol)
        return outputs[0]

    @staticmethod
    def backward(ctx, grad_sol):  # median.py:47-56
        (in_vol,) = ctx.saved_tensors
        outputs = median_cuda_ext.backward(grad_sol.contiguous(), in_vol.contiguous())
        return outputs[0]


class Median(nn.Module):
    def __init__(self, device):
        super(Median, self).__init__()
        self.device = device

    def forward(self, t_vol):
        """t_vol: H x W x D histogram per pixel.  Returns the H x W map of median positions (median.py:69-80
        drops the second output channel, the mass of the median's bin)."""
        sol = MedianFunction.apply(t_vol.unsqueeze(0))
        return sol.squeeze(0).permute(1, 2, 0)[:, :, 0]

    def init(self):
        pass
