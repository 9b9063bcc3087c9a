"""MSD network for segmentation (reference msd_segmentation_model.py:10-119)."""
import torch
import torch.nn as nn

from .msd_model import MSDModel, _moments, scaling_module_set_bias, scaling_module_set_scale


class MSDSegmentationModel(MSDModel):
    def __init__(self, c_in, num_labels, depth, width, *, dilations=[1, 2, 3, 4, 5, 6, 7, 8, 9, 10],
                 parallel=False, ndim=2):
        """``num_labels`` output classes; log-softmax over channels + NLL loss."""
        self.num_labels = num_labels
        super().__init__(c_in, num_labels, depth, width, dilations, ndim=ndim)
        self.criterion = nn.NLLLoss()

        net_trained = nn.Sequential(self.msd, nn.LogSoftmax(dim=1))
        self.net = nn.Sequential(self.scale_in, net_trained)
        self.net.cuda()
        if parallel:
            self.net = nn.DataParallel(self.net)
        self.init_optimizer(net_trained)

    def set_normalization(self, dataloader):
        """Only the input is normalised; the targets are labels."""
        mean, std, _, _ = _moments(dataloader)
        if std == 0:
            raise ValueError("set_normalization: the input data has zero variance")
        scaling_module_set_scale(self.scale_in, 1 / std)
        scaling_module_set_bias(self.scale_in, -mean / std)

    def set_target(self, target):
        """Labels in [0, num_labels), checked here as msd_segmentation_model.py:105-119 does (for
        a tensor on the GPU that read-back waits for the device; ``train`` defers it)."""
        target = target.long()
        lo, hi = target.min(), target.max()
        if lo < 0 or self.num_labels <= hi:
            raise ValueError(
                f"Target invalid: expected values in range {[0, self.num_labels - 1]}, but got {[lo, hi]}")
        # NLLLoss takes (B, *spatial) class indices: drop the channel axis
        self.target = target.squeeze(1).cuda()

    def _set_target_deferred(self, target):
        if not target.is_cuda:
            return self.set_target(target)      # a host tensor is checked on the host: no device wait
        target = target.long()
        # lowest and highest label seen since the last verdict, kept on the device; the step
        # itself runs on labels clamped into range, so no loss kernel ever sees an invalid one
        lo, hi = target.min(), target.max()
        seen = getattr(self, "_label_range", None)
        self._label_range = (lo, hi) if seen is None else (torch.minimum(seen[0], lo), torch.maximum(seen[1], hi))
        self.target = target.squeeze(1).clamp(0, self.num_labels - 1)

    def _raise_deferred_target_error(self):
        seen, self._label_range = getattr(self, "_label_range", None), None
        if seen is None:
            return
        lo, hi = int(seen[0]), int(seen[1])
        if lo < 0 or self.num_labels <= hi:
            raise ValueError(
                f"Target invalid: expected values in range {[0, self.num_labels - 1]}, but got {[lo, hi]}")

    def _fused_forward_loss(self):
        if self._loss_kind() != "nll" or not isinstance(self.net, nn.Sequential) or len(self.net) != 2:
            return None
        trained = self.net[1]
        if not isinstance(trained, nn.Sequential) or len(trained) != 2 or trained[0] is not self.msd \
                or type(trained[1]) is not nn.LogSoftmax or trained[1].dim != 1:
            return None
        return self.msd.forward_loss(self.net[0](self.input), self.target, "nll")
