// What the graph rewrite needs to know about the image-convolution kernel (conv_stem7_mfma.hip), in plain integers so
// that host-only translation units can include it.
#pragma once

namespace cinn_hip_kernels {

// True when the kernel takes this convolution (NCHW input [n][c][h][w], filter [oc][c][kh][kw], element type given as
// cinn_type_code_t value and bit width) together with a 3x3 / stride 2 / padding 1 max pooling after its relu.
bool StemPoolFusableShape(int n, int c, int h, int w, int oc, int kh, int kw, int stride_h, int stride_w, int pad_h,
                          int pad_w, int dil_h, int dil_w, int type_code, int type_bits);

}  // namespace cinn_hip_kernels
