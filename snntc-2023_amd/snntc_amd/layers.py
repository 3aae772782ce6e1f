"""PyTorch-ROCm counterparts of the reference's Keras layers (SNN_TC_Modules.py).

Constructor argument names, order and defaults, the weight layout ``[in_size + bias, out_size]``,
the two ``Params`` vectors and the padding rules are the reference's; only the framework differs
(``torch.nn.Module`` + ``torch.autograd.Function`` instead of ``tf.keras.layers.Layer`` +
``RegisterGradient``).  ``SNN_dense``, ``SNN_conv``, the earliest-spike pooling layers, the SAME padding
and the loss run gfx950 kernels and, like the four ops, take float32 tensors on a ROCm device only: there
is no host fallback.  ``SNN_avgpool2d`` and ``SNN_LRN`` are compositions of stock PyTorch ops, as they are
stock TF ops in the reference.
"""
import math

import numpy as np
import torch
import torch.nn.functional as F

from ._lib import SnntcLibraryError
from .ops import SnnCvSame, SnnCvTimes, SnnFcTimes, SnnMinPool, SnnPadTime, SoftmaxTimeLoss

# Mirrors the reference's module-level switch (SNN_TC_Modules.py:11): when True the layers keep
# the largest batch and element count they have seen in ``maxD`` (every tensor must stay below
# 2**31 elements).
Check_Dim = False


def init_weight(in_size=1, out_size=1, bias_volt=1.0, init_param=15.0):
    """randn * sqrt(init_param / in_size), plus a zero bias row when bias_volt > 1e-8
    (SNN_TC_Modules.py:19-25).  Returns float32 numpy [in_size (+1), out_size]."""
    weight = np.random.randn(in_size, out_size) * np.sqrt(init_param / in_size)
    if bias_volt > 1e-8:
        weight = np.concatenate((weight, np.zeros([1, out_size])), axis=0)
    return weight.astype(np.float32)


def _pair(v):
    return [v[0], v[1]] if isinstance(v, (list, tuple)) else [v, v]


def _same_pad(size, kernel, stride):
    """SAME padding along one axis as the reference computes it (SNN_TC_Modules.py:147-158):
    total = (ceil(size/stride) - 1) * stride + kernel - size, before = int(total/2)."""
    total = int((math.ceil(size / stride) - 1.0) * stride + kernel) - size
    before = int(total / 2)
    return before, total - before


def _require_device(t, what):
    """The kernels behind these layers exist for float32 NHWC tensors on a ROCm device only."""
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{what} must be a torch.Tensor")
    if not t.is_cuda:
        raise SnntcLibraryError(f"{what} lives on {t.device}: this layer runs on a ROCm GPU only (no CPU fallback)")
    if t.dtype != torch.float32:
        raise TypeError(f"{what} must be float32, got {t.dtype}")


def _pad_hw(x, kh, kw, sh, sw, value):
    """Pads NHWC ``x`` for SAME mode with ``value`` in one kernel pass (a negative total is refused: tf.pad
    would fail there and the reference never reaches that case)."""
    _require_device(x, "input")
    if x.dim() != 4:
        raise ValueError(f"input must be [B,H,W,C], got shape {tuple(x.shape)}")
    H, W = x.shape[1], x.shape[2]
    top, bottom = _same_pad(H, kh, sh)
    left, right = _same_pad(W, kw, sw)
    if min(top, bottom, left, right) < 0:
        raise ValueError("negative SAME padding: kernel smaller than stride is not supported")
    if top or bottom or left or right:
        return SnnPadTime.apply(x.contiguous(), top, bottom, left, right, float(value))
    return x


class _CostsMixin:
    def w_sum_cost(self):
        """mean(max(0, theta - sum_i w_ij))  (SNN_TC_Modules.py:77-80, 172-175)."""
        part1 = self._theta - torch.sum(self.weight, 0)
        return torch.mean(torch.where(part1 > 0, part1, torch.zeros_like(part1)))

    def l2_cost(self):
        """mean(w^2)  (SNN_TC_Modules.py:82-84, 177-179)."""
        return torch.mean(torch.square(self.weight))


class SNN_dense(torch.nn.Module, _CostsMixin):
    """SNN-TC fully connected layer (SNN_TC_Modules.py:36-84).  call(X[B,in_size]) -> [B,out_size]."""

    def __init__(self, in_size=1, out_size=1, biasvolt=1.0, MAX_SPIKE_TIME=1e5, Epsilon=1e-10,
                 Spike_Threshold=1.0, Thread_per_Block=0, Blocks=0, weight=None, name=None):
        super().__init__()
        self.in_size = in_size
        self.out_size = out_size
        self.biasvolt = float(biasvolt)
        self.Params = np.array([MAX_SPIKE_TIME, Epsilon, Spike_Threshold, Thread_per_Block, Blocks, self.biasvolt],
                               dtype=np.float32)
        self._theta = float(self.Params[2])
        self.maxD = [1, 1]
        if weight is None:
            weight = init_weight(in_size=self.in_size, out_size=self.out_size, bias_volt=self.biasvolt)
        else:
            weight = np.array(weight).astype(np.float32)
        self.name = 'fckernel' if name is None else name
        if self.biasvolt > 1e-8:
            self.in_size += 1
        if tuple(weight.shape) != (self.in_size, self.out_size):
            raise ValueError(f"weight shape {tuple(weight.shape)} != {(self.in_size, self.out_size)}")
        self.weight = torch.nn.Parameter(torch.from_numpy(weight))

    def forward(self, X):
        B = X.shape[0]
        if Check_Dim:
            self.maxD[0] = max(self.maxD[0], int(B))
            self.maxD[1] = max(self.maxD[1], int(B) * int(X.shape[1]))
        return SnnFcTimes.apply(X, self.weight, self.Params)      # Y[:B] of the [2B,J] op output


class SNN_conv(torch.nn.Module, _CostsMixin):
    """SNN-TC 2-D convolution on NHWC input (SNN_TC_Modules.py:96-179).
    SAME pads with MAX_SPIKE_TIME (split int(pad/2) / rest); VALID crops to (N-1)*S+K."""

    def __init__(self, in_channel=1, out_channel=1, kernel_sizes=1, strides=1, padding='SAME', rates=1,
                 biasvolt=1.0, MAX_SPIKE_TIME=1e5, Spike_Threshold=1.0, Epsilon=1e-10,
                 Thread_per_Block=0, Blocks=0, weight=None, name=None):
        super().__init__()
        self.Kh, self.Kw = _pair(kernel_sizes)
        self.C = in_channel
        self.Kc = out_channel
        self.Sh, self.Sw = _pair(strides)
        self.padding = padding.upper()
        self.cudaflag = 0
        self.rates = _pair(rates)          # accepted, not implemented (as in the reference)
        self.biasvolt = float(biasvolt)
        self.Params = np.array([MAX_SPIKE_TIME, Thread_per_Block, Blocks, Epsilon, Spike_Threshold, self.cudaflag,
                                self.Kh, self.Kw, self.Sh, self.Sw, (self.padding == 'SAME'), self.biasvolt],
                               dtype=np.float32)
        self._theta = float(self.Params[4])
        self.maxD = [0, 0]
        self.in_size = self.Kh * self.Kw * self.C
        if weight is None:
            weight = init_weight(in_size=self.in_size, out_size=self.Kc, bias_volt=self.biasvolt)
        else:
            weight = np.array(weight).astype(np.float32)
        self.name = 'convkernel' if name is None else name
        if self.biasvolt > 1e-8:
            self.in_size += 1
        if tuple(weight.shape) != (self.in_size, self.Kc):
            raise ValueError(f"weight shape {tuple(weight.shape)} != {(self.in_size, self.Kc)}")
        self.weight = torch.nn.Parameter(torch.from_numpy(weight))
        self._padded = {}                  # padded input buffers by (B, H, W, device), see padded_input_buffer

    def prepare_input(self, input):
        """The padded (SAME) or cropped (VALID) tensor handed to the op."""
        H, W = input.shape[1], input.shape[2]
        if self.padding == 'SAME':
            return _pad_hw(input, self.Kh, self.Kw, self.Sh, self.Sw, self.Params[0])
        nh = int((H - self.Kh) / self.Sh + 1.0)
        nw = int((W - self.Kw) / self.Sw + 1.0)
        return input[:, 0:(nh - 1) * self.Sh + self.Kh, 0:(nw - 1) * self.Sw + self.Kw, :]

    def same_pads(self, H, W):
        """(top, bottom, left, right) of the SAME padding of an H x W image."""
        top, bottom = _same_pad(H, self.Kh, self.Sh)
        left, right = _same_pad(W, self.Kw, self.Sw)
        if min(top, bottom, left, right) < 0:
            raise ValueError("negative SAME padding: kernel smaller than stride is not supported")
        return top, bottom, left, right

    def padded_input_buffer(self, B, H, W, device):
        """The layer's own padded input for B images of H x W (SAME mode): a tensor [B,Hp,Wp,C] that lives as
        long as the layer, its border filled with MAX_SPIKE_TIME once, and (top, left), where the image
        goes.  The layer before writes its output straight into the interior (`feed`), so no padding pass
        runs between the two; the content belongs to the latest forward pass (a backward pass of an
        earlier one is refused by autograd: the writes advance the buffer's version counter).  The
        layer keeps the buffers of the MAX_PADDED_BUFFERS input shapes used last; release_buffers() drops
        them all."""
        top, bottom, left, right = self.same_pads(H, W)
        key = (B, H, W, str(device))
        buf = self._padded.pop(key, None)
        if buf is None:
            buf = torch.full((B, top + H + bottom, left + W + right, self.C), float(self.Params[0]),
                             dtype=torch.float32, device=device)
            while len(self._padded) >= self.MAX_PADDED_BUFFERS:
                self._padded.pop(next(iter(self._padded)))          # the shape used longest ago
        self._padded[key] = buf                                     # most recently used last
        return buf, (top, left)

    MAX_PADDED_BUFFERS = 4

    def release_buffers(self):
        """Drops the padded input buffers (they are re-created on demand)."""
        self._padded.clear()

    def output_hw(self, H, W):
        if self.padding == 'SAME':
            return -(-H // self.Sh), -(-W // self.Sw)
        return int((H - self.Kh) / self.Sh + 1.0), int((W - self.Kw) / self.Sw + 1.0)

    def forward(self, input, prefilled=False, feed=None):
        """prefilled: the layer before has written `input` into this layer's padded_input_buffer.
        feed: the SNN_conv that follows; its padded input buffer receives this layer's output as well."""
        _require_device(input, "input")
        if input.dim() != 4:
            raise ValueError(f"input must be [B,H,W,C], got shape {tuple(input.shape)}")
        B = input.shape[0]
        if self.padding == 'SAME':
            H, W = input.shape[1], input.shape[2]
            xpad = self.padded_input_buffer(B, H, W, input.device)[0] if prefilled else None
            next_xpad, next_offset = None, (0, 0)
            if feed is not None:
                nh, nw = self.output_hw(H, W)
                next_xpad, next_offset = feed.padded_input_buffer(B, nh, nw, input.device)
            if Check_Dim:
                self.maxD[0] = max(self.maxD[0], int(B))
            return SnnCvSame.apply(input.contiguous(), self.weight, self.Params, self.same_pads(H, W), xpad, next_xpad,
                                   next_offset)
        if prefilled or feed is not None:
            raise ValueError("chaining needs SAME padding")
        X = self.prepare_input(input)
        if Check_Dim:
            self.maxD[0] = max(self.maxD[0], int(B))
            self.maxD[1] = max(self.maxD[1], int(X.numel()))
        return SnnCvTimes.apply(X.contiguous(), self.weight, self.Params)   # Y[:B] of the op output


class SNN_LRN(torch.nn.Module):
    """Local response normalisation over channels with 1e5-padded squares (SNN_TC_Modules.py:182-212)."""

    def __init__(self, depth_radius=5, bias=2, alpha=0.0001, beta=0.75):
        super().__init__()
        self.depth_radius, self.bias, self.alpha, self.beta = depth_radius, bias, alpha, beta

    def forward(self, x):
        c = x.shape[3]
        half_n = self.depth_radius // 2
        sq = F.pad(torch.square(x), (half_n, half_n), mode="constant", value=1e5)
        scale = self.bias
        for i in range(self.depth_radius):
            scale = scale + self.alpha * sq[:, :, :, i:i + c]
        return x / scale ** self.beta

    def get_config(self):
        return {"alpha": self.alpha, "depth_radius": self.depth_radius, "beta": self.beta, "bias": self.bias}


class _Pool2d(torch.nn.Module):
    def __init__(self, kernel_sizes=1, strides=1, padding='SAME', padvalue=1e5, name=None):
        super().__init__()
        self.Kh, self.Kw = _pair(kernel_sizes)
        self.Sh, self.Sw = _pair(strides)
        self.padding = padding.upper()
        self.padvalue = padvalue
        self.name = name

    def _padded_nchw(self, input):
        """Stock-op padding (any device), for the layers that are stock ops in the reference too."""
        if self.padding == 'SAME':
            top, bottom = _same_pad(input.shape[1], self.Kh, self.Sh)
            left, right = _same_pad(input.shape[2], self.Kw, self.Sw)
            if min(top, bottom, left, right) < 0:
                raise ValueError("negative SAME padding: kernel smaller than stride is not supported")
            input = F.pad(input, (0, 0, left, right, top, bottom), mode="constant", value=float(self.padvalue))
        return input.permute(0, 3, 1, 2)


class SNN_maxpool2d(_Pool2d):
    """Earliest-spike pooling: pad with 1e5, then -maxpool(-x), VALID (SNN_TC_Modules.py:215-246)."""

    def forward(self, input, feed=None):
        """feed: the SNN_conv that follows; its padded input buffer receives the pooled times as well."""
        _require_device(input, "input")
        if input.dim() != 4:
            raise ValueError(f"input must be [B,H,W,C], got shape {tuple(input.shape)}")
        # one kernel each way: the padding is implicit and the minimum is taken directly
        H, W = input.shape[1], input.shape[2]
        top = bottom = left = right = 0
        if self.padding == 'SAME':
            top, bottom = _same_pad(H, self.Kh, self.Sh)
            left, right = _same_pad(W, self.Kw, self.Sw)
            if min(top, bottom, left, right) < 0:
                raise ValueError("negative SAME padding: kernel smaller than stride is not supported")
        nh = (H + top + bottom - self.Kh) // self.Sh + 1
        nw = (W + left + right - self.Kw) // self.Sw + 1
        next_xpad, next_offset = None, (0, 0)
        if feed is not None:
            next_xpad, next_offset = feed.padded_input_buffer(input.shape[0], nh, nw, input.device)
        return SnnMinPool.apply(input.contiguous(), (self.Kh, self.Kw), (self.Sh, self.Sw), (top, left), (nh, nw),
                                float(self.padvalue), next_xpad, next_offset)


class SNN_globalminpool2d(torch.nn.Module):
    """Global earliest-spike pooling, [B,H,W,C] -> [B,C]: every channel keeps its first spike over the
    whole image.  It is SNN_maxpool2d with one VALID window the size of the image; the reference's
    ImageNet example reduces with a stock global pooling layer at this place
    (snntc-imagenet-example/snntc-imagenet.py:125)."""

    def __init__(self, padvalue=1e5, name=None):
        super().__init__()
        self.padvalue = padvalue
        self.name = name

    def forward(self, input):
        _require_device(input, "input")
        B, H, W, C = input.shape
        y = SnnMinPool.apply(input.contiguous(), (H, W), (H, W), (0, 0), (1, 1), float(self.padvalue))
        return y.reshape(B, C)


class SNN_flatten(torch.nn.Module):
    """[B,H,W,C] -> [B,H*W*C] in NHWC order, what Keras' Flatten does between the reference's conv and
    dense layers (tf.reshape in snntc-cifar10.py:105)."""

    def forward(self, input):
        return input.reshape(input.shape[0], -1)


class SNN_avgpool2d(_Pool2d):
    """Average pooling after padding with 1e5 (SNN_TC_Modules.py:251-281)."""

    def forward(self, input):
        x = self._padded_nchw(input)
        y = F.avg_pool2d(x, (self.Kh, self.Kw), (self.Sh, self.Sw))
        return y.permute(0, 2, 3, 1)


def loss_func(logit=None, label=None):
    """Mean categorical cross-entropy of one-hot ``label`` against softmax(-logit): the earliest
    output spike is the predicted class (SNN_TC_Modules.py:286-288)."""
    _require_device(logit, "logit")
    _require_device(label, "label")
    if logit.dim() != 2 or label.shape != logit.shape:
        raise ValueError(f"logit and label must both be [B, classes], got {tuple(logit.shape)} and {tuple(label.shape)}")
    if label.requires_grad:
        raise ValueError("label must not require a gradient: the loss kernel differentiates the spike times only")
    return SoftmaxTimeLoss.apply(logit, label)               # one fused kernel for loss and gradient
