"""MSD network for regression (reference msd_regression_model.py:8-82)."""
import torch.nn as nn

from .msd_model import MSDModel

loss_functions = {"L1": nn.L1Loss(), "L2": nn.MSELoss()}


class MSDRegressionModel(MSDModel):
    def __init__(self, c_in, c_out, depth, width, *, dilations=[1, 2, 3, 4, 5, 6, 7, 8, 9, 10], loss="L2",
                 parallel=False, ndim=2):
        """c_in/c_out channels, ``depth`` layers of ``width`` channels;
        ``loss`` is "L1" or "L2"; ``parallel`` wraps the net in nn.DataParallel
        (batch size must then be a multiple of the GPU count)."""
        super().__init__(c_in, c_out, depth, width, dilations, ndim=ndim)
        self.criterion = loss_functions.get(loss)
        if self.criterion is None:
            raise ValueError(f"The loss must be one of {list(loss_functions.keys())}. Supplied {loss}. ")

        self.net = nn.Sequential(self.scale_in, self.msd, self.scale_out)
        self.net.cuda()
        if parallel:
            self.net = nn.DataParallel(self.net)
        # only the MSD module is trained; the scaling layers are frozen
        self.init_optimizer(self.msd)

    def _fused_forward_loss(self):
        kind = self._loss_kind()
        if kind is None or not isinstance(self.net, nn.Sequential) or len(self.net) != 3 \
                or self.net[1] is not self.msd or self.net[2] is not self.scale_out:
            return None
        return self.msd.forward_loss(self.net[0](self.input), self.target, kind, scale=self.scale_out)
