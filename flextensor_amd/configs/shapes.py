"""Shape tables of the registered tasks.

Tuple formats are those of the reference's tables so that drivers index them
the same way:
  gemm       (N, K, M)                                    configs/gemm_config.py:11-15
  conv2d     (batch, C, H, W, K, _, kh, kw, _, stride, pad, dilation, groups)
                                                          configs/conv2d_config.py:19
  depthwise  (batch, C, H, W, factor, kh, kw, stride, pad, dilation)
                                                          configs/depthwise_config.py:1-9
  grouped / dilation
             (batch, C, H, W, K, kh, kw, stride, pad, dilation, groups)
                                                          configs/grouped_config.py:1-6,
                                                          configs/dilation_config.py:8-24
"""


def _conv(batch, c, hw, k, ksize, stride, pad, dilation=1, groups=1):
    return (batch, c, hw, hw, k, c, ksize, ksize, 1, stride, pad, dilation, groups)


# every power-of-two triple 2^5..2^12, enumerated as the reference does
gemm_shapes = [(2 ** i, 2 ** k, 2 ** j)
               for i in range(5, 13) for j in range(5, 13) for k in range(5, 13)]

# YOLO-v1 convolution layers (C, H=W, K, kernel, stride, pad), batch 1
_yolo_layers = [
    (3, 448, 64, 7, 2, 3), (64, 112, 192, 3, 1, 1), (192, 56, 128, 1, 1, 0),
    (128, 56, 256, 3, 1, 1), (256, 56, 256, 1, 1, 0), (256, 56, 512, 3, 1, 1),
    (512, 28, 256, 1, 1, 0), (256, 28, 512, 3, 1, 1), (512, 28, 512, 1, 1, 0),
    (512, 28, 1024, 3, 1, 1), (1024, 14, 512, 1, 1, 0), (512, 14, 1024, 3, 1, 1),
    (1024, 14, 1024, 3, 1, 1), (1024, 14, 1024, 3, 2, 1), (1024, 7, 1024, 3, 1, 1),
]
yolo_shapes = [_conv(1, c, hw, k, ks, st, pd) for (c, hw, k, ks, st, pd) in _yolo_layers]
yolo_shapes_b8 = [_conv(8, c, hw, k, ks, st, pd) for (c, hw, k, ks, st, pd) in _yolo_layers]

# MobileNet-style depthwise layers
depthwise_shapes = [
    (1, 32, 112, 112, 1, 3, 3, 1, 1, 1),
    (1, 16, 112, 112, 6, 3, 3, 2, 1, 1),
    (1, 24, 56, 56, 6, 3, 3, 2, 1, 1),
    (1, 32, 28, 28, 6, 3, 3, 2, 1, 1),
    (1, 64, 14, 14, 6, 3, 3, 1, 1, 1),
    (1, 96, 14, 14, 6, 3, 3, 2, 1, 1),
    (1, 160, 7, 7, 6, 3, 3, 1, 1, 1),
]

# 1x1 convolution 1024 -> 512 on 14x14 with 4..32 groups
grouped_shapes = [(1, 1024, 14, 14, 512, 1, 1, 1, 0, 1, g) for g in (4, 8, 16, 32)]

# YOLO layers 5..15 with dilation 2 (same padding as the undilated layers)
dilation_shapes = [(1, c, hw, hw, k, ks, ks, st, pd, 2, 1)
                   for (c, hw, k, ks, st, pd) in _yolo_layers[4:]]

# The five benchmark configurations of this backend (index = config number):
#   gemm fp32 1024^3 | conv 1x64x56x56->64 3x3 | conv 8x256x14x14->512 3x3 and
#   conv 8x512x7x7->2048 1x1 | depthwise 8x512x28x28 3x3 | gemm int8 4096^3
baseline_gemm_shapes = [(1024, 1024, 1024)]
baseline_conv_shapes = [
    _conv(1, 64, 56, 64, 3, 1, 1),
    _conv(8, 256, 14, 512, 3, 1, 1),
    _conv(8, 512, 7, 2048, 1, 1, 0),
]
baseline_depthwise_shapes = [(8, 512, 28, 28, 1, 3, 3, 1, 1, 1)]
baseline_gemm_int8_shapes = [(4096, 4096, 4096)]
