"""Drop-in for the fused "V3" losses of pytorch-loss, running on hand-written HIP kernels (MI355X).

    from pytorch_loss import LabelSmoothSoftmaxCEV3, FocalLossV3, LargeMarginSoftmaxV3, LovaszSoftmaxV3

Plus the relabelling step in front of that path in segmentation training, ``OhemCELoss`` /
``OhemLargeMarginLoss``, and the target encoder ``OnehotEncoder``. Only this path is provided; the kernels live in libpytorch_loss_hip.so (built by
``python pytorch-loss_amd/build.py``) and there is no CPU fallback.
"""
from .label_smooth import LabelSmoothSoftmaxCEV3, LSRCrossEntropyFunctionV3
from .focal_loss import FocalLossV3, FocalSigmoidLossFuncV3, FocalSigmoidLossFuncV3FB
from .large_margin_softmax import LargeMarginSoftmaxV3, LargeMarginSoftmaxFuncV3, LargeMarginSoftmaxFuncV3FB
from .lovasz_softmax import LovaszSoftmaxV3, LovaszSoftmaxFunctionV3
from .ohem_loss import OhemCELoss, OhemLargeMarginLoss, score_ohem_label
from .one_hot import convert_to_one_hot, convert_to_one_hot_cu, OnehotEncoder
from .soft_dice_loss import SoftDiceLossV3, SoftDiceLossV3Func
from .layer_norm import LayerNormV3, LayerNormV3Func
from .taylor_softmax import (TaylorSoftmaxV3, LogTaylorSoftmaxV3, TaylorCrossEntropyLossV3, TaylorSoftmaxFunc,
                             TaylorCrossEntropyFunctionV3, taylor_softmax_v3)

__all__ = [
    "LabelSmoothSoftmaxCEV3", "LSRCrossEntropyFunctionV3",
    "FocalLossV3", "FocalSigmoidLossFuncV3", "FocalSigmoidLossFuncV3FB",
    "LargeMarginSoftmaxV3", "LargeMarginSoftmaxFuncV3", "LargeMarginSoftmaxFuncV3FB",
    "LovaszSoftmaxV3", "LovaszSoftmaxFunctionV3",
    "OhemCELoss", "OhemLargeMarginLoss", "score_ohem_label",
    "convert_to_one_hot", "convert_to_one_hot_cu", "OnehotEncoder",
    "SoftDiceLossV3", "SoftDiceLossV3Func",
    "LayerNormV3", "LayerNormV3Func",
    "TaylorSoftmaxV3", "LogTaylorSoftmaxV3", "TaylorCrossEntropyLossV3", "TaylorSoftmaxFunc",
    "TaylorCrossEntropyFunctionV3", "taylor_softmax_v3",
]
