"""MI355X-native deformable convolution (2-D bilinear, 3-D trilinear) with the module / function
API of lshiwjx/deform_conv3d_pytorch_op.  Host code is Python on PyTorch-ROCm; the arithmetic
runs in hand-written HIP kernels for gfx950 behind the C ABI of include/dcn_amd.h."""
from .functions import ConvOffset2dFunction, ConvOffset3dFunction, output_size
from .modules import ConvOffset2d, ConvOffset2dPack, ConvOffset3d, ConvOffset3dPack
from .conv2d import Conv2d, Conv2dFunction

__all__ = ["ConvOffset2d", "ConvOffset3d", "ConvOffset2dPack", "ConvOffset3dPack", "ConvOffset2dFunction",
           "ConvOffset3dFunction", "output_size", "Conv2d", "Conv2dFunction"]
