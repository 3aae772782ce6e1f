"""MI355X (gfx950) implementation of the SNN-TC custom ops behind the reference's Python API.

Public names follow the reference module ``SNN_TC_Modules``: the op handles ``snnfc``,
``snnfc_grad``, ``snncv``, ``snncv_grad`` and the layers ``SNN_dense``, ``SNN_conv``,
``SNN_maxpool2d``, ``SNN_avgpool2d``, ``SNN_LRN``, plus ``init_weight`` and ``loss_func``.
"""
from . import _lib
from ._lib import SnntcError, SnntcLibraryError
from .ops import SnnCv, SnnCvSame, SnnCvTimes, SnnFc, SnnFcTimes, SnnMinPool, SnnPadTime, SoftmaxTimeLoss, min_pool, min_pool_grad, pad_time, pad_time_grad, sgd_update, softmax_time_loss, snncv, snncv_grad, snncv_output_dims, snnfc, snnfc_grad, snnfc_static, init, check_scan_health
from . import train
from . import networks
from .layers import (SNN_LRN, SNN_avgpool2d, SNN_conv, SNN_dense, SNN_flatten, SNN_globalminpool2d, SNN_maxpool2d,
                     init_weight, loss_func)

__all__ = [
    "snnfc", "snnfc_grad", "snnfc_static", "init", "check_scan_health", "snncv", "snncv_grad", "snncv_output_dims", "SnnFc", "SnnCv", "SnnFcTimes", "SnnCvTimes", "SoftmaxTimeLoss", "softmax_time_loss", "sgd_update", "SnnMinPool", "min_pool", "min_pool_grad", "SnnPadTime", "pad_time", "pad_time_grad",
    "SNN_dense", "SNN_conv", "SNN_maxpool2d", "SNN_avgpool2d", "SNN_globalminpool2d", "SNN_flatten", "SNN_LRN", "init_weight", "loss_func",
    "SnntcError", "SnntcLibraryError", "train", "networks",
]
