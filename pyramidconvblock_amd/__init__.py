"""MI355X-native implementation of the PyramidConvBlock hot path: channels-last large-kernel
depthwise conv2d with the adaptive average pooling, gate and bilinear upsampling that
``ConvBlock`` composes around it, forward and backward, on hand-written gfx950 kernels."""
from .avgpool import AdaptiveAvgPool2dFunction, OptimizedAdaptiveAvgPool2d
from .conv_block import ConvBlock, GateFunction, SimpleGate
from .dwconv import DepthwiseConv2DFunction, OptimizedDepthwiseConv2d
from .up import BilinearInterp2dFunction, OptimizedBilinearInterp2d

__all__ = [
    "ConvBlock", "SimpleGate", "GateFunction",
    "OptimizedDepthwiseConv2d", "DepthwiseConv2DFunction",
    "OptimizedAdaptiveAvgPool2d", "AdaptiveAvgPool2dFunction",
    "OptimizedBilinearInterp2d", "BilinearInterp2dFunction",
]
