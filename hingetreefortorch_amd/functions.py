"""Autograd functions with the reference's public names (HingeTree/_HingeTree.py:92-186, 370-506).

`HingeTree`, `HingeFern` and the six convolution functions keep the reference's `apply` signatures, static helper
methods and the rule that `torch.use_deterministic_algorithms(True)` selects the deterministic backward
(_HingeTree.py:24-30,103-106). The convolutions have no deterministic backward in the reference either and raise the
same RuntimeError under that switch (_HingeTree.py:384-385).
"""
import torch

from . import hingetree_cpp as _ops


def _is_deterministic():
    if hasattr(torch, "are_deterministic_algorithms_enabled"):
        return torch.are_deterministic_algorithms_enabled()
    if hasattr(torch, "is_deterministic"):
        return torch.is_deterministic()
    raise RuntimeError("Unable to query torch deterministic mode.")


class _ForestFunction(torch.autograd.Function):
    """forward(ctx, inData, inThresholds, inOrdinals, inWeights); gradients for data, thresholds and weights."""
    _prefix = None  # "tree" | "fern"

    @classmethod
    def _op(cls, name):
        return getattr(_ops, f"{cls._prefix}_{name}")

    @staticmethod
    def _forward(cls, ctx, inData, inThresholds, inOrdinals, inWeights):
        # When a backward pass will follow, the forward pass also keeps what its tree walks found, so that the backward
        # does not walk again (the reference's backward re-walks, hingetree_gpu.cu:619-730; same gradients).
        records = None
        if any(ctx.needs_input_grad) and inData.is_cuda:
            out, records = cls._op("forward_records")(inData, inThresholds, inOrdinals, inWeights)
        else:
            out = cls._op("forward")(inData, inThresholds, inOrdinals, inWeights)
        ctx.has_records = records is not None
        if records is not None:
            ctx.save_for_backward(inData, inThresholds, inOrdinals, inWeights, records)
        else:
            ctx.save_for_backward(inData, inThresholds, inOrdinals, inWeights)
        return out

    @staticmethod
    def _backward(cls, ctx, outDataGrad):
        inData, inThresholds, inOrdinals, inWeights = ctx.saved_tensors[:4]
        need = ctx.needs_input_grad
        args = (inData, need[0], inThresholds, need[1], inOrdinals, need[2], inWeights, need[3],
                outDataGrad.contiguous())
        if ctx.has_records:
            grads = cls._op("backward_records")(ctx.saved_tensors[4], _is_deterministic(), *args)
        else:
            grads = cls._op("backward_deterministic" if _is_deterministic() else "backward")(*args)
        return tuple(grads)

    # static helpers of the reference classes
    @classmethod
    def check_thresholds(cls, inThresholds, inOrdinals, inWeights):
        return cls._op("check_thresholds")(inThresholds, inOrdinals, inWeights)

    @classmethod
    def fix_thresholds(cls, inThresholds, inOrdinals, inWeights):
        return cls._op("fix_thresholds")(inThresholds, inOrdinals, inWeights)

    @classmethod
    def reachability(cls, inData, inThresholds, inOrdinals, inWeights):
        return cls._op("reachability")(inData, inThresholds, inOrdinals, inWeights)

    @classmethod
    def leafmap(cls, inData, inThresholds, inOrdinals, inWeights):
        return cls._op("leafmap")(inData, inThresholds, inOrdinals, inWeights)

    @classmethod
    def marginmap(cls, inData, inThresholds, inOrdinals, inWeights):
        return cls._op("marginmap")(inData, inThresholds, inOrdinals, inWeights)

    @classmethod
    def speedtest(cls, inData):
        return cls._op("speedtest")(inData, _is_deterministic())

    @classmethod
    def init_medians(cls, inData, inThresholds, inOrdinals, inWeights):
        return cls._op("init_medians")(inData, inThresholds, inOrdinals, inWeights)


class HingeTree(_ForestFunction):
    _prefix = "tree"

    @staticmethod
    def forward(ctx, inData, inThresholds, inOrdinals, inWeights):
        return _ForestFunction._forward(HingeTree, ctx, inData, inThresholds, inOrdinals, inWeights)

    @staticmethod
    def backward(ctx, outDataGrad):
        return _ForestFunction._backward(HingeTree, ctx, outDataGrad)

    @staticmethod
    def init_greedy(inData, inLabels, inThresholds, inOrdinals, inWeights):
        return _ops.tree_init_greedy(inData, inLabels, inThresholds, inOrdinals, inWeights)


class HingeFern(_ForestFunction):
    _prefix = "fern"

    @staticmethod
    def forward(ctx, inData, inThresholds, inOrdinals, inWeights):
        return _ForestFunction._forward(HingeFern, ctx, inData, inThresholds, inOrdinals, inWeights)

    @staticmethod
    def backward(ctx, outDataGrad):
        return _ForestFunction._backward(HingeFern, ctx, outDataGrad)


def _conv_function(name, prefix, nd, label):
    fwd = getattr(_ops, f"{prefix}_conv{nd}d_forward")
    bwd = getattr(_ops, f"{prefix}_conv{nd}d_backward")

    def forward(ctx, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation):
        ctx.save_for_backward(inData, inThresholds, inOrdinals, inWeights)
        ctx.kernelSize, ctx.stride, ctx.padding, ctx.dilation = kernelSize, stride, padding, dilation
        return fwd(inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation)

    def backward(ctx, outDataGrad):
        if _is_deterministic() and outDataGrad.device.type != "cpu":
            raise RuntimeError(f"No deterministic implementation of backpropagation for hinge {label} convolution on "
                               "GPUs.")
        inData, inThresholds, inOrdinals, inWeights = ctx.saved_tensors
        need = ctx.needs_input_grad
        grads = bwd(inData, need[0], inThresholds, need[1], inOrdinals, need[2], inWeights, need[3],
                    outDataGrad.contiguous(), ctx.kernelSize, ctx.stride, ctx.padding, ctx.dilation)
        return tuple(grads) + (None, None, None, None)

    return type(name, (torch.autograd.Function,), {"forward": staticmethod(forward), "backward": staticmethod(backward),
                                                   "__doc__": f"{nd}-d hinge {label} convolution."})


HingeTreeConv1d = _conv_function("HingeTreeConv1d", "tree", 1, "tree")
HingeTreeConv2d = _conv_function("HingeTreeConv2d", "tree", 2, "tree")
HingeTreeConv3d = _conv_function("HingeTreeConv3d", "tree", 3, "tree")
HingeFernConv1d = _conv_function("HingeFernConv1d", "fern", 1, "fern")
HingeFernConv2d = _conv_function("HingeFernConv2d", "fern", 2, "fern")
HingeFernConv3d = _conv_function("HingeFernConv3d", "fern", 3, "fern")


class _FusedLinearFunction(torch.autograd.Function):
    """forward(ctx, inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias) =
    inLinearBias + inLinearWeights @ forest(inData) over the tree axis (_HingeTree.py:218-258). Unlike the reference,
    whose GPU forward accumulates with atomics and therefore refuses to run under
    torch.use_deterministic_algorithms(True), this one is deterministic and selects the deterministic forest backward
    under that switch."""
    _prefix = None

    @staticmethod
    def _forward(cls, ctx, inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias):
        args = (inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias)
        # when a backward pass will follow, the forest's output and walk records are kept for it (the reference's
        # backward computes the forest again, hingetree_fused_linear.cpp:200-412; same gradients)
        ctx.kept = 0
        if any(ctx.needs_input_grad) and inData.is_cuda:
            out, f, records = getattr(_ops, f"{cls._prefix}_fused_linear_forward_records")(*args)
            ctx.kept = 1 if records is None else 2
            ctx.save_for_backward(*args, f, *([] if records is None else [records]))
            return out
        ctx.save_for_backward(*args)
        return getattr(_ops, f"{cls._prefix}_fused_linear_forward")(*args)

    @staticmethod
    def _backward(cls, ctx, outDataGrad):
        inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias = ctx.saved_tensors[:6]
        need = ctx.needs_input_grad
        args = (inData, need[0], inThresholds, need[1], inOrdinals, need[2], inWeights, need[3], inLinearWeights,
                need[4], inLinearBias, need[5], outDataGrad.contiguous())
        if ctx.kept:
            state = (ctx.saved_tensors[6], ctx.saved_tensors[7] if ctx.kept == 2 else None)
            return tuple(getattr(_ops, f"{cls._prefix}_fused_linear_backward_records")(state, _is_deterministic(), *args))
        name = f"{cls._prefix}_fused_linear_backward" + ("_deterministic" if _is_deterministic() else "")
        return tuple(getattr(_ops, name)(*args))


class HingeTreeFusedLinear(_FusedLinearFunction):
    _prefix = "tree"

    @staticmethod
    def forward(ctx, *args):
        return _FusedLinearFunction._forward(HingeTreeFusedLinear, ctx, *args)

    @staticmethod
    def backward(ctx, outDataGrad):
        return _FusedLinearFunction._backward(HingeTreeFusedLinear, ctx, outDataGrad)


class HingeFernFusedLinear(_FusedLinearFunction):
    _prefix = "fern"

    @staticmethod
    def forward(ctx, *args):
        return _FusedLinearFunction._forward(HingeFernFusedLinear, ctx, *args)

    @staticmethod
    def backward(ctx, outDataGrad):
        return _FusedLinearFunction._backward(HingeFernFusedLinear, ctx, outDataGrad)


class LinearBatchNorm(torch.autograd.Function):
    """zhat = BatchNorm1d(affine=False, training)(Linear(bias=False)(x)) as one operator on the HIP library: the dense
    front of the reference's README model (README.md:117-129). forward(ctx, inData, inLinearWeights, eps) returns
    (zhat, mean, var); mean and the biased batch variance are for the caller's running statistics and carry no
    gradient."""

    @staticmethod
    def forward(ctx, inData, inLinearWeights, eps):
        zhat, mean, rstd, var = _ops.linear_bn_forward(inData, inLinearWeights, eps)
        ctx.save_for_backward(inData, inLinearWeights, zhat, rstd)
        ctx.mark_non_differentiable(mean, var)
        return zhat, mean, var

    @staticmethod
    def backward(ctx, outDataGrad, _mean_grad, _var_grad):
        inData, inLinearWeights, zhat, rstd = ctx.saved_tensors
        g = outDataGrad.contiguous().clone()  # the operator works in place on the upstream gradient
        dx, dlin = _ops.linear_bn_backward(inData, ctx.needs_input_grad[0], inLinearWeights, ctx.needs_input_grad[1],
                                           zhat, rstd, g)
        return dx, dlin, None


class LinearBatchNormForest(torch.autograd.Function):
    """Linear(bias=False) -> BatchNorm1d(affine=False, training) -> HingeTree / HingeFern as one operator: the whole
    README model (README.md:117-129). forward(ctx, inData, inLinearWeights, eps, inThresholds, inOrdinals, inWeights,
    fern) returns (out, mean, var). Forward values are those of LinearBatchNorm followed by the forest function; what
    the fusion buys is the backward pass: when inData wants no gradient (a first layer), the gradient of the linear
    weights comes straight from the forest's walk records -- the forest's input gradient has one non-zero per sample
    and tree, so its dense [batch, features] form, the batch-norm backward over it and the dense product with the inputs
    are all skipped (tree_linear_bn_backward_records). Deterministic mode, inputs that want gradients and shapes the
    library does not serve that way take the two separate backward passes."""

    @staticmethod
    def forward(ctx, inData, inLinearWeights, eps, inThresholds, inOrdinals, inWeights, fern):
        pre = "fern" if fern else "tree"
        # one call: the forest reads the un-normalised product z and normalises it on the way (no pass over [batch,
        # features] to write zhat); the walk records are kept when a backward pass will follow
        out, records, z, mean, rstd, var = getattr(_ops, pre + "_linear_bn_forward_records")(
            inData, inLinearWeights, eps, inThresholds, inOrdinals, inWeights, want_records=any(ctx.needs_input_grad))
        ctx.pre = pre
        ctx.has_records = records is not None
        saved = [inData, inLinearWeights, z, mean, rstd, inThresholds, inOrdinals, inWeights]
        ctx.save_for_backward(*(saved + ([records] if records is not None else [])))
        ctx.mark_non_differentiable(mean, var)
        return out, mean, var

    @staticmethod
    def backward(ctx, outDataGrad, _mean_grad, _var_grad):
        inData, inLinearWeights, z, mean, rstd, inThresholds, inOrdinals, inWeights = ctx.saved_tensors[:8]
        need_x, need_lin, _, need_thr, need_ord, need_w, _ = ctx.needs_input_grad
        up = outDataGrad.contiguous()
        deterministic = _is_deterministic()
        if ctx.has_records and not need_x and not deterministic:
            got = getattr(_ops, ctx.pre + "_linear_bn_backward_records")(
                ctx.saved_tensors[8], inData, inLinearWeights, need_lin, z, rstd, inThresholds, need_thr, inOrdinals,
                inWeights, need_w, up, mean=mean)
            if got is not None:
                return None, got[0], None, got[1], None, got[2], None
        # the two separate backward passes, on the normalised product
        zhat = (z - mean) * rstd
        args = (zhat, need_x or need_lin, inThresholds, need_thr, inOrdinals, need_ord, inWeights, need_w, up)
        if ctx.has_records:
            dz, dthr, _, dw = getattr(_ops, ctx.pre + "_backward_records")(ctx.saved_tensors[8], deterministic, *args)
        else:
            dz, dthr, _, dw = getattr(_ops, ctx.pre + ("_backward_deterministic" if deterministic else "_backward"))(*args)
        dx = dlin = None
        if dz is not None:
            dx, dlin = _ops.linear_bn_backward(inData, need_x, inLinearWeights, need_lin, zhat, rstd, dz)
        return dx, dlin, None, dthr, None, dw, None


def contract(inData, window, padding=0):
    """HingeTree/_HingeTree.py:32-39."""
    if isinstance(window, int):
        window = [window] * (inData.dim() - 2)
    if isinstance(padding, int):
        padding = [padding] * (inData.dim() - 2)
    return _ops.contract(inData, window, padding)


def expand(inData, padding=0):
    """HingeTree/_HingeTree.py:40-44."""
    if isinstance(padding, int):
        padding = [padding] * ((inData.dim() - 2) // 2)
    return _ops.expand(inData, padding)


class _Expand(torch.autograd.Function):
    """Tiles -> image; the gradient is the contraction of the upstream gradient (_HingeTree.py:46-59)."""

    @staticmethod
    def forward(ctx, inData, padding):
        dim = (inData.dim() - 2) // 2
        ctx.window = list(inData.shape[-dim:])
        ctx.padding = padding
        return expand(inData, padding)

    @staticmethod
    def backward(ctx, outDataGrad):
        if ctx.needs_input_grad[0]:
            return contract(outDataGrad.contiguous(), ctx.window, ctx.padding), None
        return None, None


class _Contract(torch.autograd.Function):
    """Image -> tiles; the gradient is the expansion of the upstream gradient (_HingeTree.py:61-73)."""

    @staticmethod
    def forward(ctx, inData, window, padding=0):
        ctx.padding = padding
        return contract(inData, window, padding)

    @staticmethod
    def backward(ctx, outDataGrad):
        if ctx.needs_input_grad[0]:
            return expand(outDataGrad.contiguous(), ctx.padding), None, None
        return None, None, None


class _ForestExpandedFunction(torch.autograd.Function):
    """Forest with tile-shaped outputs per leaf followed by Expand, as one operator: the forward pass stores the image
    directly (the tile-major intermediate [B, T, *tiles, *window] is never written); the backward pass reads the upstream
    gradient as the image where the library serves the shape, and otherwise contracts it and runs the forest's backward. Same values as Expand(padding)(HingeTree.apply(...)), which is
    how the reference's segmentation model composes the two (rcc/Net.py:99-109)."""
    _prefix = None

    @staticmethod
    def _forward(cls, ctx, inData, inThresholds, inOrdinals, inWeights, padding):
        nd = inWeights.dim() - 2
        ctx.padding = [padding] * nd if isinstance(padding, int) else list(padding)
        ctx.save_for_backward(inData, inThresholds, inOrdinals, inWeights)
        return getattr(_ops, f"{cls._prefix}_forward_expanded")(inData, inThresholds, inOrdinals, inWeights, ctx.padding)

    @staticmethod
    def _backward(cls, ctx, outDataGrad):
        inData, inThresholds, inOrdinals, inWeights = ctx.saved_tensors
        need = ctx.needs_input_grad
        grads = getattr(_ops, f"{cls._prefix}_backward_expanded")(
            _is_deterministic(), ctx.padding, inData, need[0], inThresholds, need[1], inOrdinals, need[2], inWeights,
            need[3], outDataGrad.contiguous())
        return tuple(grads) + (None,)


class HingeTreeExpanded(_ForestExpandedFunction):
    _prefix = "tree"

    @staticmethod
    def forward(ctx, inData, inThresholds, inOrdinals, inWeights, padding=0):
        return _ForestExpandedFunction._forward(HingeTreeExpanded, ctx, inData, inThresholds, inOrdinals, inWeights,
                                                padding)

    @staticmethod
    def backward(ctx, outDataGrad):
        return _ForestExpandedFunction._backward(HingeTreeExpanded, ctx, outDataGrad)


class HingeFernExpanded(_ForestExpandedFunction):
    _prefix = "fern"

    @staticmethod
    def forward(ctx, inData, inThresholds, inOrdinals, inWeights, padding=0):
        return _ForestExpandedFunction._forward(HingeFernExpanded, ctx, inData, inThresholds, inOrdinals, inWeights,
                                                padding)

    @staticmethod
    def backward(ctx, outDataGrad):
        return _ForestExpandedFunction._backward(HingeFernExpanded, ctx, outDataGrad)


class Expand(torch.nn.Module):
    """_HingeTree.py:75-81."""

    def __init__(self, padding=0):
        super().__init__()
        self.padding = padding

    def forward(self, inData):
        return _Expand.apply(inData, self.padding)


class Contract(torch.nn.Module):
    """_HingeTree.py:83-90."""

    def __init__(self, window, padding=0):
        super().__init__()
        self.window = window
        self.padding = padding

    def forward(self, inData):
        return _Contract.apply(inData, self.window, self.padding)
