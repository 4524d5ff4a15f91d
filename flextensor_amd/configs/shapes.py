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

# The other networks of the reference's conv2d tables (configs/conv2d_config.py:9-16, 58-67,
# 83-268), as (C, H=W, K, kernel, stride, pad[, groups]); batch as the reference registers them.
_overfeat_layers = [
    (3, 192, 96, 11, 4, 5), (96, 24, 256, 5, 1, 2), (256, 12, 512, 3, 1, 1),
    (512, 12, 1024, 3, 1, 1), (1024, 12, 1024, 3, 1, 1),
]
_google_layers = [
    (3, 224, 64, 7, 2, 3), (64, 56, 64, 1, 1, 0), (64, 56, 192, 3, 1, 1), (192, 28, 64, 1, 1, 0),
    (192, 28, 96, 1, 1, 0), (96, 28, 128, 3, 1, 1), (192, 28, 16, 1, 1, 0), (16, 28, 32, 5, 1, 2),
    (192, 28, 32, 1, 1, 0), (256, 28, 128, 1, 1, 0), (128, 28, 192, 3, 1, 1),
    (256, 28, 32, 1, 1, 0), (32, 28, 96, 5, 1, 2), (256, 28, 64, 1, 1, 0), (480, 14, 192, 1, 1, 0),
    (480, 14, 96, 1, 1, 0), (96, 14, 208, 3, 1, 1), (480, 14, 16, 1, 1, 0), (16, 14, 48, 5, 1, 2),
    (480, 14, 64, 1, 1, 0), (512, 14, 160, 1, 1, 0), (512, 14, 112, 1, 1, 0),
    (112, 14, 224, 3, 1, 1), (512, 14, 24, 1, 1, 0), (24, 14, 64, 5, 1, 2), (512, 14, 64, 1, 1, 0),
    (512, 14, 128, 1, 1, 0), (128, 14, 256, 3, 1, 1), (512, 14, 144, 1, 1, 0),
    (144, 14, 288, 3, 1, 1), (512, 14, 32, 1, 1, 0), (32, 14, 64, 5, 1, 2),
    (528, 14, 256, 1, 1, 0), (528, 14, 160, 1, 1, 0), (160, 14, 320, 3, 1, 1),
    (528, 14, 32, 1, 1, 0), (32, 14, 128, 5, 1, 2), (528, 14, 128, 1, 1, 0),
    (832, 7, 256, 1, 1, 0), (832, 7, 160, 1, 1, 0), (160, 7, 320, 3, 1, 1), (832, 7, 32, 1, 1, 0),
    (32, 7, 128, 5, 1, 2), (832, 7, 128, 1, 1, 0), (832, 7, 384, 1, 1, 0), (832, 7, 192, 1, 1, 0),
    (192, 7, 384, 3, 1, 1), (832, 7, 48, 1, 1, 0), (48, 7, 128, 5, 1, 2),
]
_squeeze_layers = [
    (3, 227, 96, 7, 2, 0), (96, 55, 16, 1, 1, 0), (16, 55, 64, 1, 1, 0), (16, 55, 64, 3, 1, 1),
    (128, 55, 16, 1, 1, 0), (128, 55, 32, 1, 1, 0), (32, 55, 128, 1, 1, 0), (32, 55, 128, 3, 1, 1),
    (256, 27, 32, 1, 1, 0), (32, 27, 128, 1, 1, 0), (32, 27, 128, 3, 1, 1), (256, 27, 48, 1, 1, 0),
    (48, 27, 192, 1, 1, 0), (48, 27, 192, 3, 1, 1), (384, 27, 48, 1, 1, 0), (384, 27, 64, 1, 1, 0),
    (64, 27, 256, 1, 1, 0), (64, 27, 256, 3, 1, 1), (512, 13, 64, 1, 1, 0), (64, 13, 256, 1, 1, 0),
    (64, 13, 256, 3, 1, 1), (512, 13, 1000, 1, 1, 0),
]
_res_layers = [
    (3, 224, 64, 7, 2, 3), (64, 56, 256, 1, 1, 0), (64, 56, 64, 1, 1, 0), (64, 56, 64, 3, 1, 1),
    (256, 56, 64, 1, 1, 0), (256, 56, 512, 1, 2, 0), (256, 56, 128, 1, 2, 0),
    (128, 28, 128, 3, 1, 1), (128, 28, 512, 1, 1, 0), (512, 28, 128, 1, 1, 0),
    (512, 28, 1024, 1, 2, 0), (512, 28, 256, 1, 2, 0), (256, 14, 256, 3, 1, 1),
    (256, 14, 1024, 1, 1, 0), (1024, 14, 256, 1, 1, 0), (1024, 14, 2048, 1, 2, 0),
    (1024, 14, 512, 1, 2, 0), (512, 7, 512, 3, 1, 1), (512, 7, 2048, 1, 1, 0),
    (2048, 7, 512, 1, 1, 0),
]
_vgg_16_layers = [
    (3, 224, 64, 3, 1, 1), (64, 224, 64, 3, 1, 1), (64, 112, 128, 3, 1, 1),
    (128, 112, 128, 3, 1, 1), (128, 56, 256, 3, 1, 1), (256, 56, 256, 3, 1, 1),
    (256, 28, 512, 3, 1, 1), (512, 28, 512, 3, 1, 1), (512, 14, 512, 3, 1, 1),
]
# MobileNet-v2 depthwise stages written as grouped convolutions (groups = C)
_mobilev2_layers = [
    (32, 112, 32, 3, 1, 1, 32), (16, 112, 96, 3, 2, 1, 16), (24, 56, 144, 3, 2, 1, 24),
    (32, 28, 192, 3, 2, 1, 32), (64, 14, 384, 3, 1, 1, 64), (96, 14, 576, 3, 2, 1, 96),
    (160, 7, 960, 3, 1, 1, 160),
]


def _table(batch, layers):
    return [_conv(batch, l[0], l[1], l[2], l[3], l[4], l[5], 1, l[6] if len(l) > 6 else 1) for l in layers]


overfeat_shapes = _table(1, _overfeat_layers)
google_shapes = _table(1, _google_layers)
squeeze_shapes = _table(1, _squeeze_layers)
res_shapes = _table(64, _res_layers)                 # the reference tunes ResNet at batch 64
vgg_16_shapes = _table(1, _vgg_16_layers)
vgg_19_shapes = []                                   # empty upstream as well (every entry commented out)
mobilev2_shapes = _table(1, _mobilev2_layers)
# one 1x1 layer at batch 256; its bias slot is 0 where the others carry 1 (never read by the drivers)
test_conv_shapes = [(256, 256, 14, 14, 512, 256, 1, 1, 0, 1, 0, 1, 1)]

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
# the same layers at batch 8 and 16 (flextensor/configs/depthwise_config.py:12-31)
depthwise_shapes_b8 = [(8,) + s[1:] for s in depthwise_shapes]
depthwise_shapes_b16 = [(16,) + s[1:] for s in depthwise_shapes]

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
# further int8 GEMMs (M, K, N): smaller cubes and two products with few tiles and a long K,
# where the reduce split decides (across workgroups or across wavefront groups)
gemm_int8_shapes = [(512, 512, 512), (1024, 1024, 1024), (2048, 2048, 2048),
                    (1024, 4096, 1024), (512, 8192, 512)]
