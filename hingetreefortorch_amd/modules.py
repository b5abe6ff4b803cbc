"""nn.Modules with the reference's public names and constructor semantics.

RandomHingeForest / RandomHingeFern follow RandomHingeForest/_RandomHingeForest.py:42-142,153-231 and the
HingeTreeConv{1,2,3}d / HingeFernConv{1,2,3}d modules follow RandomHingeForest/_HingeTreeConv.py:34-302:
  * parameters `weights`, `thresholds` (trainable) and `ordinals` (int64, requires_grad=False);
  * the random draws happen in the order thresholds -> ordinals -> weights with the same torch calls, so a model built
    under the same torch.manual_seed gets the same initial parameters as the reference;
  * init_type "random" | "sequential"; extra_outputs None | int | iterable (forest/fern), int (conv);
  * thresholds are made consistent on the CPU at construction;
  * load_state_dict re-casts `ordinals` to int64 (old snapshots stored them as floats).
Unlike the reference, the fern convolution modules do not run the *tree* threshold fix on fern-shaped tensors (which
fails there for depth >= 2); ferns need no fix.
"""
import operator
from functools import reduce

import torch
import torch.nn as nn

from . import functions as _fn


def _draw_parameters(nodes_shape, leaves_shape, modulus, extra, init_type, conv):
    thresholds = 6.0 * torch.rand(nodes_shape) - 3.0
    if init_type == "random":
        ordinals = torch.randint_like(thresholds, low=0, high=modulus, dtype=torch.long)
    elif init_type == "sequential":
        ordinals = torch.arange(thresholds.numel(), dtype=torch.long)
        ordinals -= modulus * (ordinals // modulus)
        ordinals = torch.reshape(ordinals, thresholds.shape)
    else:
        raise RuntimeError(f"Unknown init_type {init_type}. Must be one of 'random' or 'sequential'.")
    if conv:
        tail = [extra] if extra > 1 else []
    elif extra is None:
        tail = []
    elif hasattr(extra, "__iter__"):
        tail = list(extra)
    else:
        tail = [extra]
    weights = torch.randn(list(leaves_shape) + tail)
    return thresholds, ordinals, weights


class _ForestBase(nn.Module):
    __constants__ = ["in_channels", "out_channels", "depth", "extra_outputs", "init_type"]
    _function = None
    _fern = False

    def __init__(self, in_channels: int, out_channels: int, depth: int, extra_outputs=None, init_type: str = "random"):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.depth = depth
        self.extra_outputs = extra_outputs
        self.init_type = init_type
        nodes = depth if self._fern else 2 ** depth - 1
        thresholds, ordinals, weights = _draw_parameters([out_channels, nodes], [out_channels, 2 ** depth], in_channels,
                                                         extra_outputs, init_type, conv=False)
        self._function.fix_thresholds(thresholds, ordinals, weights)
        self.weights = nn.Parameter(weights, requires_grad=True)
        self.thresholds = nn.Parameter(thresholds, requires_grad=True)
        self.ordinals = nn.Parameter(ordinals, requires_grad=False)

    def forward(self, x):
        return self._function.apply(x, self.thresholds, self.ordinals, self.weights)

    def reachability(self, x):
        return self._function.reachability(x, self.thresholds, self.ordinals, self.weights)

    def leafmap(self, x):
        return self._function.leafmap(x, self.thresholds, self.ordinals, self.weights)

    def marginmap(self, x):
        return self._function.marginmap(x, self.thresholds, self.ordinals, self.weights)

    def check_thresholds(self):
        return self._function.check_thresholds(self.thresholds.data, self.ordinals.data, self.weights.data)

    def fix_thresholds(self):
        return self._function.fix_thresholds(self.thresholds.data, self.ordinals.data, self.weights.data)

    def init_medians(self, x):
        return self._function.init_medians(x, self.thresholds.data, self.ordinals.data, self.weights.data)

    def load_state_dict(self, *args, **kwargs):
        # float ordinals of old snapshots are cast by the copy into the int64 parameter; keep the reference's guard
        result = super().load_state_dict(*args, **kwargs)
        if self.ordinals.dtype != torch.long:
            self.ordinals = nn.Parameter(self.ordinals.data.type(torch.long), requires_grad=False)
        return result


class RandomHingeForest(_ForestBase):
    _function = _fn.HingeTree

    def pathmap(self, x):
        """Ordinals of the ancestors of each (sample, tree)'s leaf, root first: shape leafmap.shape + [depth].
        Same arithmetic as the reference (_RandomHingeForest.py:88-121): the leaf key is read as the index of a heap
        leaf (vertex = key + 2^depth - 1) and its parents are followed up to the root."""
        leaf = self.leafmap(x).to(torch.long)
        trees = torch.arange(leaf.shape[1], device=leaf.device).view([1, -1] + [1] * (leaf.dim() - 2)).expand_as(leaf)
        vertex = leaf + (2 ** self.depth - 1)
        steps = []
        for _ in range(self.depth):
            vertex = torch.div(vertex - 1, 2, rounding_mode="floor")
            steps.append(self.ordinals[trees, vertex])
        return torch.stack(steps[::-1], dim=-1)

    def init_greedy(self, x, y):
        return _fn.HingeTree.init_greedy(x, y, self.thresholds.data, self.ordinals.data, self.weights.data)


class RandomHingeFern(_ForestBase):
    _function = _fn.HingeFern
    _fern = True

    def pathmap(self, x):
        """A fern tests the same ordinals for every sample: ordinals broadcast to leafmap.shape + [depth]
        (_RandomHingeForest.py:190-206)."""
        if x.dim() < 2:
            raise RuntimeError("Input batch should be at least 2 dimensions.")
        shape = [x.shape[0], self.out_channels] + list(x.shape[2:]) + [self.depth]
        view = [1, self.out_channels] + [1] * (x.dim() - 2) + [self.depth]
        return self.ordinals.view(view).expand(shape).clone()


def _as_tuple(x, n: int):
    if isinstance(x, int):
        return tuple([x] * n)
    if len(x) != n:
        raise RuntimeError(f"Expected size {n} list/tuple.")
    return tuple(x)


class _ConvBase(nn.Module):
    __constants__ = ["in_channels", "out_channels", "depth", "extra_outputs", "kernel_size", "stride", "padding",
                     "dilation", "init_type"]
    _function = None
    _fern = False
    _nd = 0

    def __init__(self, in_channels: int, out_channels: int, depth: int, kernel_size, stride=1, padding=0, dilation=1,
                 extra_outputs: int = 1, init_type: str = "random"):
        super().__init__()
        self.in_channels = in_channels
        self.out_channels = out_channels
        self.depth = depth
        self.extra_outputs = extra_outputs
        self.init_type = init_type
        self.kernel_size = _as_tuple(kernel_size, self._nd)
        self.stride = _as_tuple(stride, self._nd)
        self.padding = _as_tuple(padding, self._nd)
        self.dilation = _as_tuple(dilation, self._nd)
        taps = reduce(operator.mul, self.kernel_size)
        nodes = depth if self._fern else 2 ** depth - 1
        thresholds, ordinals, weights = _draw_parameters([out_channels, in_channels, nodes],
                                                         [out_channels, in_channels, 2 ** depth], taps, extra_outputs,
                                                         init_type, conv=True)
        if not self._fern:
            _fn.HingeTree.fix_thresholds(thresholds.view([out_channels * in_channels, -1]),
                                         ordinals.view([out_channels * in_channels, -1]),
                                         weights.view([out_channels * in_channels, 2 ** depth, -1]))
        self.weights = nn.Parameter(weights, requires_grad=True)
        self.thresholds = nn.Parameter(thresholds, requires_grad=True)
        self.ordinals = nn.Parameter(ordinals, requires_grad=False)

    def forward(self, x):
        return self._function.apply(x, self.thresholds, self.ordinals, self.weights, self.kernel_size, self.stride,
                                    self.padding, self.dilation)


class HingeTreeConv1d(_ConvBase):
    _function, _nd = _fn.HingeTreeConv1d, 1


class HingeTreeConv2d(_ConvBase):
    _function, _nd = _fn.HingeTreeConv2d, 2


class HingeTreeConv3d(_ConvBase):
    _function, _nd = _fn.HingeTreeConv3d, 3


class HingeFernConv1d(_ConvBase):
    _function, _nd, _fern = _fn.HingeFernConv1d, 1, True


class HingeFernConv2d(_ConvBase):
    _function, _nd, _fern = _fn.HingeFernConv2d, 2, True


class HingeFernConv3d(_ConvBase):
    _function, _nd, _fern = _fn.HingeFernConv3d, 3, True


class _FusedLinearMixin:
    """Adds the linear layer over the tree axis (RandomHingeForest/_RandomHingeForest.py:296-330): `linear_weights`
    [out_channels, number_of_trees] initialised like nn.Linear, `linear_bias` [out_channels] (zeros and frozen when
    bias=False)."""

    def _init_linear(self, number_of_trees, out_channels, bias):
        import math
        from torch.nn import init
        self.linear_weights = nn.Parameter(torch.empty([out_channels, number_of_trees]))
        self.linear_bias = nn.Parameter(torch.zeros([out_channels]), requires_grad=bias)
        init.kaiming_uniform_(self.linear_weights, a=math.sqrt(5))
        if bias:
            fan_in, _ = init._calculate_fan_in_and_fan_out(self.linear_weights)
            bound = 1 / math.sqrt(fan_in) if fan_in > 0 else 0
            init.uniform_(self.linear_bias, -bound, bound)


class RandomHingeForestFusedLinear(RandomHingeForest, _FusedLinearMixin):
    def __init__(self, in_channels: int, number_of_trees: int, out_channels: int, depth: int, extra_outputs=None,
                 init_type: str = "random", bias: bool = True):
        super().__init__(in_channels, number_of_trees, depth, extra_outputs, init_type)
        self._init_linear(number_of_trees, out_channels, bias)

    def forward(self, x):
        return _fn.HingeTreeFusedLinear.apply(x, self.thresholds, self.ordinals, self.weights, self.linear_weights,
                                              self.linear_bias)


class RandomHingeFernFusedLinear(RandomHingeFern, _FusedLinearMixin):
    def __init__(self, in_channels: int, number_of_trees: int, out_channels: int, depth: int, extra_outputs=None,
                 init_type: str = "random", bias: bool = True):
        super().__init__(in_channels, number_of_trees, depth, extra_outputs, init_type)
        self._init_linear(number_of_trees, out_channels, bias)

    def forward(self, x):
        return _fn.HingeFernFusedLinear.apply(x, self.thresholds, self.ordinals, self.weights, self.linear_weights,
                                              self.linear_bias)


class RandomHingeForestExpanded(RandomHingeForest):
    """RandomHingeForest with tile-shaped extra_outputs followed by Expand(padding) (the head of the reference's
    segmentation model, rcc/Net.py:99-109) as one module: same parameters and state dict as RandomHingeForest, same
    values as the two modules in sequence, one pass over memory less."""

    def __init__(self, in_channels: int, out_channels: int, depth: int, extra_outputs, init_type: str = "random",
                 padding=0):
        super().__init__(in_channels, out_channels, depth, extra_outputs, init_type)
        self.padding = padding

    def forward(self, x):
        return _fn.HingeTreeExpanded.apply(x, self.thresholds, self.ordinals, self.weights, self.padding)


class RandomHingeFernExpanded(RandomHingeFern):
    """RandomHingeFern followed by Expand(padding) as one module; see RandomHingeForestExpanded."""

    def __init__(self, in_channels: int, out_channels: int, depth: int, extra_outputs, init_type: str = "random",
                 padding=0):
        super().__init__(in_channels, out_channels, depth, extra_outputs, init_type)
        self.padding = padding

    def forward(self, x):
        return _fn.HingeFernExpanded.apply(x, self.thresholds, self.ordinals, self.weights, self.padding)


class LinearHingeForest(nn.Module):
    """Linear(bias=False) -> BatchNorm1d(affine=False) -> RandomHingeForest(init_type="sequential") as one module: the
    model of the reference's README (README.md:117-129; experiments/run_letter_seq.py:45-52), where the linear layer
    produces one private feature per decision vertex (out_channels * (2^depth - 1) of them). The projection and the
    batch statistics run in one matrix-core kernel of the HIP library; in eval mode the running statistics are used.

    Sub-module names and parameter shapes equal those of the three separate torch / reference modules (`fc.weight`,
    `bn.running_mean`, `bn.running_var`, `bn.num_batches_tracked`, `forest.weights`, `forest.thresholds`,
    `forest.ordinals`), so a state dict moves between the two forms unchanged."""

    def __init__(self, in_features: int, out_channels: int, depth: int, extra_outputs=None, eps: float = 1e-5,
                 momentum: float = 0.1):
        super().__init__()
        hidden = out_channels * (2 ** depth - 1)
        self.fc = nn.Linear(in_features, hidden, bias=False)
        self.bn = nn.BatchNorm1d(hidden, eps=eps, momentum=momentum, affine=False)
        self.forest = RandomHingeForest(hidden, out_channels, depth, extra_outputs=extra_outputs,
                                        init_type="sequential")

    def forward(self, x):
        if not self.training or not x.is_cuda or x.dtype != torch.float32:
            return self.forest(self.bn(self.fc(x)))
        out, mean, var = _fn.LinearBatchNormForest.apply(x.contiguous(), self.fc.weight, self.bn.eps,
                                                         self.forest.thresholds, self.forest.ordinals,
                                                         self.forest.weights, False)
        if self.bn.track_running_stats:
            with torch.no_grad():
                n = x.shape[0]
                self.bn.num_batches_tracked += 1
                m = self.bn.momentum if self.bn.momentum is not None else 1.0 / float(self.bn.num_batches_tracked)
                self.bn.running_mean.mul_(1 - m).add_(mean, alpha=m)
                self.bn.running_var.mul_(1 - m).add_(var * (n / max(n - 1, 1)), alpha=m)
        return out
