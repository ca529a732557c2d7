"""Autograd surface of the quadratic-fit layer: the names, arguments and tensor layouts of the
reference's cudaQuadFit/QuadFitting.py (QuadFittingFromFlowFunction, QuadFittingFromFlow)."""
import torch
from torch import nn
from torch.autograd import Function

from . import QuadFit_cuda_ext


class QuadFittingFromFlowFunction(Function):
    """sol = fit(feat0, feat1, flow); gradients flow to the two feature maps only: the fit is piecewise
    constant in the flow (cudaQuadFit/cudaCode/quadFit.h:11-12)."""

    @staticmethod
    def forward(ctx, feat0, feat1, flow):  # QuadFitting.py:20-30
        outputs = QuadFit_cuda_ext.forward(feat0.contiguous(), feat1.contiguous(), flow.contiguous())
        ctx.save_for_backward(feat0, feat1, flow)
        return outputs[0]

    @staticmethod
    def backward(ctx, grad_sol):  # QuadFitting.py:33-40 (which returns two values for three inputs)
        feat0, feat1, flow = ctx.saved_tensors
        d_oGfeat0, d_oGfeat1 = QuadFit_cuda_ext.backward(grad_sol.contiguous(), feat0.contiguous(),
                                                         feat1.contiguous(), flow.contiguous())
        return d_oGfeat0, d_oGfeat1, None


class QuadFittingFromFlow(nn.Module):
    def __init__(self, device):
        super(QuadFittingFromFlow, self).__init__()
        self.device = device

    def forward(self, t_feat0, t_feat1, t_flow):
        """t_feat0, t_feat1: H x W x C; t_flow: H x W x 3 (QuadFitting.py:50-53 asserts three channels although
        only the first two, the x and y displacement, are read).  Returns H x W x 3."""
        Yi, Xi, Li = t_flow.shape
        assert Li == 3, "flow should have 3 channels: the displacement in X and Y direction and one more\n"
        t_feat0_in = t_feat0.permute(2, 0, 1).unsqueeze(0)
        t_feat1_in = t_feat1.permute(2, 0, 1).unsqueeze(0)
        t_flow_in = t_flow.permute(2, 0, 1).unsqueeze(0)
        sol = QuadFittingFromFlowFunction.apply(t_feat0_in, t_feat1_in, t_flow_in)
        return sol.squeeze(0).permute(1, 2, 0).contiguous()

    def init(self):
        pass
