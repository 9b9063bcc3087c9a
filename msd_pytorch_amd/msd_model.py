"""Training wrapper shared by the regression and segmentation models
(reference msd_model.py:8-342): frozen 1x1 input/output scaling layers, Adam
on the trainable part, normalisation from a data loader, save/load."""
import numpy as np
import torch
import torch.nn as nn
import torch.optim as optim

from . import msd_custom_convolutions as cc
from .msd_module import MSDFinalFunction, MSDModule


class _NativePointwise:
    """forward of a 1x1 convolution as one native pass over the voxels (the kernel of the
    network's final layer) for GPU tensors with contiguous channel planes; torch's
    convolution otherwise.  Parameters, state-dict keys and initialisation are those of
    the torch class it is mixed into."""

    def forward(self, input):
        w = self.weight
        if self.bias is not None and input.dim() == w.dim() and input.dtype == w.dtype \
                and w.is_cuda and cc.final_layer_supported(input):
            return MSDFinalFunction.apply(input, w.view(w.shape[0], w.shape[1]), self.bias)
        return super().forward(input)


class ScalingConv2d(_NativePointwise, nn.Conv2d):
    pass


class ScalingConv3d(_NativePointwise, nn.Conv3d):
    pass


def scaling_module(num_channels, *, conv3d=False):
    """A frozen 1x1 convolution initialised to the identity.  It is saved with
    the network and never touched by the optimiser."""
    conv = ScalingConv3d if conv3d else ScalingConv2d
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


def _moments(pairs):
    """Mean and standard deviation of the inputs and of the targets of an iterable of
    (input, target) batches, from per-batch means of x and x**2 as msd_model.py:140-153
    computes them, in one pass and in double precision on the host."""
    sums = [0.0, 0.0, 0.0, 0.0]
    n = 0
    for pair in pairs:
        x, y = pair[0], pair[1]
        for i, t in enumerate((x, y)):
            t = t.detach().double()
            sums[2 * i] += float(t.mean())
            sums[2 * i + 1] += float(t.pow(2).mean())
        n += 1
    if n == 0:
        raise ValueError("set_normalization: the data loader yields no batches")
    out = []
    for i in range(2):
        mean, square = sums[2 * i] / n, sums[2 * i + 1] / n
        out += [mean, float(np.sqrt(max(square - mean ** 2, 0.0)))]
    return tuple(out)


def match_module_prefix(state_dict, wanted_keys):
    """Rename the keys of a checkpoint so that it loads into a network with or without the
    ``module.`` prefix that nn.DataParallel adds (``parallel=True`` models,
    msd_regression_model.py:78-79): the prefix is added or dropped to agree with
    ``wanted_keys``; a dictionary that already agrees is returned as it is."""
    wanted = list(wanted_keys)
    have_prefix = bool(state_dict) and all(k.startswith("module.") for k in state_dict)
    want_prefix = bool(wanted) and all(k.startswith("module.") for k in wanted)
    if have_prefix == want_prefix:
        return state_dict
    if have_prefix:
        return type(state_dict)((k[len("module."):], v) for k, v in state_dict.items())
    return type(state_dict)(("module." + k, v) for k, v in state_dict.items())


class GraphedStep:
    """One train step of an MSDModel recorded as a HIP graph and replayed.

    ``GraphedStep(model)`` runs ``model.step_async(update=update)`` a few times on the
    model's current input and target (set them first with ``set_input`` / ``set_target``),
    then captures one more run.  Calling the object copies a new input and target (when
    given; same shapes) into the captured buffers and replays the whole step, scaling
    layers, loss and backward pass included, as a single launch: what a network this small
    needs, since its step is otherwise bound by launch overhead, not by the kernels.
    ``loss()`` reads the loss of the last replay; the parameters' ``.grad`` hold its
    gradients.  With ``update=True`` the optimiser step is part of the graph, which torch
    only allows for an optimiser built with ``capturable=True``
    (``model.optimizer = torch.optim.Adam(params, capturable=True)``); the ``warmup`` runs
    (at least one) are then real optimisation steps on the current batch, and they are what
    creates the optimiser's state outside the graph.

    The captured work is the eager work, launch for launch, so replays give the same bits."""

    def __init__(self, model, update=False, warmup=3):
        if update and not model.optimizer.defaults.get("capturable", False):
            raise ValueError("GraphedStep(update=True) needs an optimiser built with capturable=True")
        if update and warmup < 1:
            raise ValueError("GraphedStep(update=True) needs warmup >= 1: the optimiser creates its state in its "
                             "first step, which must not be part of the graph")
        if getattr(model, "input", None) is None or getattr(model, "target", None) is None:
            raise ValueError("GraphedStep: call set_input and set_target first")
        self.model = model
        model.loss = model.output = None          # no autograd graph of an earlier step kept alive
        # the graph's static buffers are its own: set_input / set_target keep a tensor that is
        # already on the GPU as it is, and every replay overwrites these
        model.input, model.target = model.input.clone(), model.target.clone()
        # warm-up and capture run on ONE side stream: the gradient accumulators of the
        # parameters are made in the first backward pass and stay with the stream they were made on
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            for _ in range(warmup):
                model.step_async(update=update)
            model.loss = model.output = None
            model.optimizer.zero_grad(set_to_none=True)
        torch.cuda.current_stream().wait_stream(side)
        self.graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(self.graph, stream=side):
            model.step_async(update=update)
        self._input, self._target = model.input, model.target
        self.shapes = (model.input.shape, model.target.shape)
        # the values only: the recorded autograd graph would keep the parameters' gradient
        # accumulators (and their stream) alive for every eager step that follows
        self._loss, self._output = model.loss.detach(), model.output.detach()
        model.loss, model.output = self._loss, self._output
        # the gradient tensors the graph writes (an eager step in between replaces .grad)
        self._grads = [(p, p.grad) for group in model.optimizer.param_groups for p in group["params"]
                       if p.grad is not None]

    def __call__(self, input=None, target=None):
        if input is not None:
            self._input.copy_(input, non_blocking=True)
        if target is not None:
            self._target.copy_(target.reshape(self._target.shape), non_blocking=True)
        self.graph.replay()
        self.model.loss, self.model.output = self._loss, self._output
        for p, g in self._grads:
            p.grad = g

    def loss(self):
        return self._loss.item()


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
        mean_in, std_in, mean_out, std_out = _moments(dataloader)
        if std_in == 0 or std_out == 0:
            raise ValueError("set_normalization: the data has zero variance "
                             f"(std of inputs {std_in}, of targets {std_out})")
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

    def _launch_forward(self, input=None, target=None):
        """Network and criterion on one (input, target) pair, without waiting for the GPU."""
        if input is not None:
            self.set_input(input)
        if target is not None:
            self.set_target(target)
        self.output = None
        self.loss = None
        fused = self._fused_forward_loss() if self.fuse_loss and not self._net_hooked() else None
        if fused is not None:
            self.loss, self.output = fused
            return
        self.output = self.net(self.input)
        self.loss = self.criterion(self.output, self.target)

    # Loss computed in the pass of the final layer (MSDModule.forward_loss) where the model has
    # the standard structure; set to False to run network and criterion as separate modules.
    # With the fused node ``model.output`` is detached from the autograd graph: a further loss
    # built on it gets no gradient.  Hooks on any module of ``net`` switch the fusion off for
    # that call, since the hooks' modules are then not called one by one.
    fuse_loss = True

    def _net_hooked(self):
        """True when any module of ``net`` (the Sequential containers, the scaling layers, the
        MSD module and its parts, LogSoftmax) carries a forward, pre-forward or backward hook."""
        for m in self.net.modules():
            if m._forward_hooks or m._forward_pre_hooks or m._backward_hooks or m._backward_pre_hooks:
                return True
        return False

    def _loss_kind(self):
        """"mse", "l1" or "nll" when the criterion is torch's with default settings, else None."""
        c = self.criterion
        if getattr(c, "reduction", None) != "mean":
            return None
        if type(c) is nn.MSELoss:
            return "mse"
        if type(c) is nn.L1Loss:
            return "l1"
        if type(c) is nn.NLLLoss and c.weight is None and c.ignore_index == -100:
            return "nll"
        return None

    def _fused_forward_loss(self):
        """(loss, output) through the fused node, or None when the model is not the plain
        scale_in -> msd [-> scale_out | -> LogSoftmax] -> criterion chain on the GPU."""
        return None

    def forward(self, input=None, target=None):
        """Loss of one (input, target) pair; arguments left out keep their last value."""
        self._launch_forward(input, target)
        return self.loss.item()

    def step_async(self, input=None, target=None, update=True):
        """Launch forward, zero_grad, backward and (``update``) the optimiser step of
        msd_model.py:225-244 without waiting for the GPU.  Nothing is returned: ``get_loss()``
        reads the loss when it is wanted, and waits then."""
        self._launch_forward(input, target)
        self.optimizer.zero_grad()
        self.loss.backward()
        if update:
            self.optimizer.step()

    def gradients(self, input=None, target=None):
        """forward + zero_grad + backward: what ``learn`` does short of the optimiser step.
        Returns the loss."""
        self.step_async(input, target, update=False)
        return self.loss.item()

    def learn(self, input=None, target=None):
        """One optimisation step on one (input, target) pair; returns the loss (read back
        after the whole step has been launched)."""
        self.step_async(input, target)
        return self.loss.item()

    def train(self, dataloader, num_epochs, graph=False):
        """``num_epochs`` passes over the loader, one optimisation step per batch
        (msd_model.py:246-261).  ``graph=True`` records the step as a HIP graph on the first
        batch and replays it for every later batch of the same shape (GraphedStep): for
        networks so small that a step is bound by launch overhead rather than by the kernels
        (depth 10 at 256 x 256: 0.25 against 0.7 ms per step).  The optimiser is then switched
        to its capturable form, keeping its state."""
        # the loss of each batch is not looked at here (the reference drops it too):
        # the host keeps launching ahead of the GPU; targets that are on the GPU already are
        # validated there and the verdict is read once per epoch (_set_target_deferred)
        steps = {}        # one recorded step per batch shape (a loader's last batch may be smaller)
        for _ in range(num_epochs):
            for input, target in dataloader:
                self.set_input(input)
                self._set_target_deferred(target)
                if not graph:
                    self.step_async()
                    continue
                shapes = (self.input.shape, self.target.shape)
                step = steps.get(shapes)
                if step is None:
                    self._make_optimizer_capturable()
                    steps[shapes] = GraphedStep(self, update=True, warmup=1)   # the warm-up run is this batch's step
                else:
                    step(self.input, self.target)
            self._raise_deferred_target_error()

    def _set_target_deferred(self, target):
        """set_target for a training loop that must not wait for the GPU per batch.  Models whose
        set_target inspects values (segmentation labels) override this for GPU tensors."""
        self.set_target(target)

    def _raise_deferred_target_error(self):
        pass

    def _make_optimizer_capturable(self):
        if self.optimizer.defaults.get("capturable", False):
            return
        state = self.optimizer.state_dict()
        for group in state["param_groups"]:
            group["capturable"] = True
        params = [p for group in self.optimizer.param_groups for p in group["params"]]
        self.optimizer = type(self.optimizer)(params, capturable=True)
        self.optimizer.load_state_dict(state)

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
        """Restore network and optimiser; returns the stored epoch.

        Reads the files that ``save`` and the reference's ``save`` (msd_model.py:310-324)
        write: ``{"epoch", "state_dict", "optimizer"}`` with the parameter names of the
        reference (``weight{i}``, one flat ``bias``, ``final_layer.linear.*`` under the
        position of the module in ``net``).  A checkpoint of a ``parallel=True`` model loads
        into a plain one and the other way round.  Only tensors and plain containers are
        accepted from the file (nothing in it is executed)."""
        device = "cuda" if torch.cuda.is_available() else "cpu"
        state = torch.load(path, map_location=device, weights_only=True)
        missing = [k for k in ("epoch", "state_dict", "optimizer") if k not in state]
        if missing:
            raise RuntimeError(f"{path} is not an MSD checkpoint: no {missing} entry")
        own = self.net.state_dict()
        weights = match_module_prefix(state["state_dict"], own.keys())
        for key, value in weights.items():
            if key in own and tuple(own[key].shape) != tuple(value.shape):
                raise RuntimeError(f"{path}: {key} has shape {tuple(value.shape)}, this model expects "
                                   f"{tuple(own[key].shape)} (other depth, width or channel counts?)")
        self.net.load_state_dict(weights)
        self.optimizer.load_state_dict(state["optimizer"])
        self.net.cuda()
        return state["epoch"]
