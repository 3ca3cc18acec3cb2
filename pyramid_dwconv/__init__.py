"""Drop-in import name of the reference package (pyramid_dwconv/__init__.py:1-2):
``from pyramid_dwconv import ConvBlock`` resolves to the MI355X implementation."""
from pyramidconvblock_amd import ConvBlock, DepthwiseConv2DFunction, OptimizedDepthwiseConv2d  # noqa: F401
