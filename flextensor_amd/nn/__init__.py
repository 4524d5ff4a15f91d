from .ops import (zero_pad2d, conv2d_nchw, depthwise_conv2d_nchw, gemm, gemm_int8, bias_add_nchw, batch_gemm,
                  im2col_nchw_naive, col2img_nchw, gemm_conv2d_nchw)
