"""Training wrapper shared by the regression and segmentation models
(reference msd_model.py:8-342): frozen 1x1 input/output scaling layers, Adam
on the trainable part, normalisation from a data loader, save/load."""
import numpy as np
import torch
import torch.nn as nn
import torch.optim as optim

from .msd_module import MSDModule


def scaling_module(num_channels, *, conv3d=False):
    """A frozen 1x1 convolution initialised to the identity.  It is saved with
    the network and never touched by the optimiser."""
    conv = nn.Conv3d if conv3d else nn.Conv2d
    c = conv(num_channels, num_channels, 1)
    c.bias.requires_grad = False
    c.weight.requires_grad = False
    scaling_module_set_scale(c, 1.0)
    scaling_module_set_bias(c, 0.0)
    return c


def scaling_module_set_scale(sm, s):
    c_out, c_in = sm.weight.shape[:2]
    assert c_out == c_in
    sm.weight.data.zero_()
    for i in range(c_out):
        sm.weight.data[i, i] = s


def scaling_module_set_bias(sm, bias):
    sm.bias.data.fill_(bias)


def _moments(batches):
    """Mean and standard deviation from per-batch means of x and x**2."""
    mean = square = 0
    n = 0
    for x in batches:
        mean = mean + x.mean()
        square = square + x.pow(2).mean()
        n += 1
    mean, square = mean / n, square / n
    return float(mean), float(np.sqrt(float(square) - float(mean) ** 2))


class MSDModel:
    """Base class; use MSDRegressionModel or MSDSegmentationModel.

    Subclasses build ``self.net`` and ``self.criterion`` and call
    ``init_optimizer`` with the trainable sub-network."""

    def __init__(self, c_in, c_out, depth, width, dilations=[1, 2, 3, 4, 5, 6, 7, 8, 9, 10], ndim=2):
        if ndim not in (2, 3):
            raise ValueError(f"Expected 2D or 3D convolutions (ndim=2 or 3). Got: {ndim}")
        self.c_in, self.c_out = c_in, c_out
        self.depth, self.width = depth, width
        self.dilations = dilations
        self.ndim = ndim

        # construction order fixes the RNG draw order (msd_model.py:109-111)
        self.scale_in = scaling_module(c_in, conv3d=ndim == 3)
        self.scale_out = scaling_module(c_out, conv3d=ndim == 3)
        self.msd = MSDModule(c_in, c_out, depth, width, dilations, ndim=ndim)

    def init_optimizer(self, trainable_net):
        self.optimizer = optim.Adam(trainable_net.parameters())

    def set_normalization(self, dataloader):
        """Make scale_in map the training inputs to zero mean / unit variance
        and scale_out map the network output back to the targets' mean / std."""
        mean_in, std_in = _moments(d[0] for d in dataloader)
        mean_out, std_out = _moments(d[1] for d in dataloader)
        scaling_module_set_scale(self.scale_in, 1 / std_in)
        scaling_module_set_bias(self.scale_in, -mean_in / std_in)
        scaling_module_set_scale(self.scale_out, std_out)
        scaling_module_set_bias(self.scale_out, mean_out)

    def set_input(self, data):
        assert self.c_in == data.shape[1], "Wrong number of input channels"
        self.input = data.cuda()

    def set_target(self, data):
        assert self.c_out == data.shape[1], "Wrong number of output channels"
        self.target = data.cuda()

    def forward(self, input=None, target=None):
        """Loss of one (input, target) pair; arguments left out keep their last value."""
        if input is not None:
            self.set_input(input)
        if target is not None:
            self.set_target(target)
        self.output = None
        self.loss = None
        self.output = self.net(self.input)
        self.loss = self.criterion(self.output, self.target)
        return self.loss.item()

    def learn(self, input=None, target=None):
        """One optimisation step on one (input, target) pair; returns the loss."""
        loss = self.forward(input, target)
        self.optimizer.zero_grad()
        self.loss.backward()
        self.optimizer.step()
        return loss

    def train(self, dataloader, num_epochs):
        for _ in range(num_epochs):
            for input, target in dataloader:
                self.learn(input, target)

    def validate(self, dataloader):
        """Mean loss per (input, target) pair of the loader."""
        total = 0
        for input, target in dataloader:
            total += self.forward(input, target)
        return total / len(dataloader)

    def print(self):
        print(self.net)

    def get_loss(self):
        return self.loss.data.mean().item()

    def get_output(self):
        """Output of the last forward/learn/train/validate call, else None."""
        return getattr(self, "output", None)

    def save(self, path, epoch):
        state = {
            "epoch": int(epoch),
            "state_dict": self.net.state_dict(),
            "optimizer": self.optimizer.state_dict(),
        }
        torch.save(state, path)

    def load(self, path):
        """Restore network and optimiser; returns the stored epoch."""
        state = torch.load(path, weights_only=True)
        self.net.load_state_dict(state["state_dict"])
        self.optimizer.load_state_dict(state["optimizer"])
        self.net.cuda()
        return state["epoch"]
