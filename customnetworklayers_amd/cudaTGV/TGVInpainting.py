"""Python surface of the TGV inpainting layer: the names, signatures and tensor conventions of the
reference's cudaTGV/TGVInpainting.py (TGVInpaintingFunction at lines 18-43, TGVInpaint at 46-74).

The first channel of the diffusion tensors is assumed to lie in [0, 1]; the second (the weight of
the auxiliary variables' regulariser) may be any value >= 0 (TGVInpainting.py:16-17)."""
import numpy as np
import torch
from torch import nn
from torch.autograd import Function

from . import tgvInpaint_cuda_ext


class TGVInpaintingFunction(Function):

    @staticmethod
    def forward(ctx, dx, dy, dc, db, di, its, pid):
        # a forward nobody differentiates keeps no intermediate iterates
        outputs = tgvInpaint_cuda_ext.forward(dx.contiguous(), dy.contiguous(), dc.contiguous(),
                                              db.contiguous(), di.contiguous(), its, pid,
                                              keep=None if any(ctx.needs_input_grad[:5]) else 0)
        sol = outputs[0]
        variables = [dx, dy, dc, db, torch.from_numpy(np.array([its, pid]))]
        ctx.save_for_backward(*variables)
        return sol

    @staticmethod
    def backward(ctx, grad_sol):
        dx, dy, dc, db, ii = ctx.saved_tensors
        its, pid = (int(v) for v in ii.tolist())
        outputs = tgvInpaint_cuda_ext.backward(grad_sol.contiguous(), dx.contiguous(), dy.contiguous(),
                                               dc.contiguous(), db.contiguous(), its, pid)
        d_oGx, d_oGy, d_oGc, d_oGb, d_oGi = outputs
        return d_oGx, d_oGy, d_oGc, d_oGb, d_oGi, None, None


class TGVInpaint(nn.Module):
    """Unbatched H x W x C interface of the reference module (cudaTGV/TGVInpainting.py:46-74).
    pid is a unique number between 0 and 9."""

    def __init__(self, device, its, pid=3, corrected_gradient=False):
        super(TGVInpaint, self).__init__()
        self.its = its
        self.id = pid
        self.device = device
        # not in the reference: back-propagate the corrected gradient instead of the reference's (gradient_mode)
        self.corrected_gradient = bool(corrected_gradient)

    def forward(self, t_dx, t_dy, t_dc, t_db, t_di):
        tgvInpaint_cuda_ext.gradient_mode(self.id, 1 if self.corrected_gradient else 0)
        Yx, Xx, Lx = t_dx.shape  # no batches here
        assert Lx == 2, "tensors should have 2 channels\n"
        Yi, Xi, Li = t_di.shape
        Lb = t_db.shape[2]
        assert Li == 3 * Lb, "input should have 3! channels (primary and two auxilliary variables) per channel of b\n"

        t_dx_in = t_dx.permute(2, 0, 1).unsqueeze(0)  # order is 1,Channel,Height,Width
        t_dy_in = t_dy.permute(2, 0, 1).unsqueeze(0)
        t_dc_in = t_dc.permute(2, 0, 1).unsqueeze(0)
        t_db_in = t_db.permute(2, 0, 1).unsqueeze(0)
        t_di_in = t_di.permute(2, 0, 1).unsqueeze(0)

        # the output has 3 channels per channel of b (primary and two auxiliary variables)
        sol = TGVInpaintingFunction.apply(t_dx_in, t_dy_in, t_dc_in, t_db_in, t_di_in, self.its, self.id)
        return sol.squeeze(0).permute(1, 2, 0).contiguous()

    def init(self):
        pass
