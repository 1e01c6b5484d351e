"""aether: the reference's layer / model API on hand-written HIP kernels for
MI355X (gfx950).  ``from aether import *`` gives the names the reference's
``CNN.models.CNN_model_cupy`` star-import gives."""
from .layers import (Activation_Softmax_Loss_CategoricalCrossEntropy, Batch_Norm, Conv_Layer, Flatten,
                     Layer_Dense, Layer_Dropout, Layer_Dropout_Spatial, Leaky_ReLU, Loss,
                     Loss_CategoricalCrossEntropy, Optimizer_Adam, Pooling, ReLU, SoftMax)
from .model import (Accuracy, Accuracy_Categorical, Accuracy_Regression, Layer_Input, Model)
from .tensor import DeviceTensor, as_device
from . import _lib

__all__ = [
    "Activation_Softmax_Loss_CategoricalCrossEntropy", "Batch_Norm", "Conv_Layer", "Flatten", "Layer_Dense",
    "Layer_Dropout", "Layer_Dropout_Spatial", "Leaky_ReLU", "Loss", "Loss_CategoricalCrossEntropy",
    "Optimizer_Adam", "Pooling", "ReLU", "SoftMax", "Accuracy", "Accuracy_Categorical", "Accuracy_Regression",
    "Layer_Input", "Model", "DeviceTensor", "as_device",
]
