// Program passes that prepare convolutional networks for the gfx950 convolution kernels.
//
// ConvertConvLayoutToNHWC: the MFMA convolution kernels want the reduction index (input channel) contiguous in
// memory, i.e. channels-last activations and [O][KH][KW][I] filters.  Programs are written in NCHW (the layout of
// the paddle models the reference compiles), so this pass moves every chain
//     conv2d -> batch_norm / pool2d / element-wise ops -> conv2d ...
// to NHWC: tensors inside the chain only exist channels-last, transposes appear where a chain starts from or
// returns to an op that needs NCHW (reshape, matmul, fetched outputs), and filters are transposed once (a
// pre-run instruction when the filter is marked const).  The reference has the same kind of pass for its x86
// NCHWc kernels (cinn/hlir/pass/alterlayout.cc).
//
// FuseConvBatchNorm: folds `conv2d -> batch_norm [-> + residual] [-> relu]` on channels-last tensors into one
// hip_conv2d_bn_relu call whose epilogue applies y = conv * s + t with s = scale / sqrt(variance + eps),
// t = bias - mean * s (computed by ordinary fp32 instructions, pre-run for const statistics).
#pragma once
#include <set>
#include <string>

#include "frontend/syntax.h"

namespace cinn {
namespace frontend {

Program ConvertConvLayoutToNHWC(const Program& program, const std::set<std::string>& fetch_ids);
// With fuse_stem_pool, a 3x3 / stride 2 / padding 1 max pooling that follows the relu of a folded image convolution
// (7x7 / stride 2 / padding 3 over 3 NCHW channels, 16-bit) is folded in as well (attribute max_pool): the
// full-resolution activation then never reaches memory.
Program FuseConvBatchNorm(const Program& program, const std::set<std::string>& fetch_ids, bool fuse_stem_pool = true);
// matmul(x, W) with a const 2-D W stored [K][N]: multiply by a pre-run transposed copy instead (trans_b), so that
// both operands of the GEMM kernel have K contiguous whatever the sizes of x
Program PretransposeConstMatmulWeights(const Program& program);
// matmul(x [M][K], W stored [N][K]) + bias [N] in a 16-bit type, the bias known before the first run: one
// hip_conv2d_bn_relu call on the operands seen as 1x1 images (x as [M,1,1,K], W as [N,1,1,K]) with scale 1 and the
// bias in fp32 as shift - a classifier's bias then costs no kernel of its own.  The sum is rounded once, from the
// fp32 accumulator plus bias, where the two operators round the product first.
Program FuseMatmulBias(const Program& program, const std::set<std::string>& fetch_ids);
// Two folded 1x1, stride 1, unpadded channels-last convolutions of which the second reads the first one's result
// (the expansion that ends a ResNet bottleneck, with its shortcut and relu, and the reduction that starts the next):
// one hip_conv2d_bn_relu_chain call with two outputs, when the kernel behind it takes the channel counts
// (kernels/conv_chain.h).  The call is placed in front of the first result's earliest reader (a projection shortcut
// may come before the reduction); the instructions that compute the second convolution's scale and shift move there
// with it.  The first result stays an output - the next shortcut reads it - but is written once and not read back;
// the results are those of the two calls.
Program FuseConvChain(const Program& program, const std::set<std::string>& fetch_ids);

// A folded 1x1 convolution whose residual input is the result of a folded 1x1 projection (any stride, no relu, read by
// nothing else) - the last layer of a bottleneck block and its projection shortcut - becomes one
// hip_conv2d_pointwise_pair call over both inputs, when the kernel behind it takes the shape (kernels/conv_chain.h,
// ConvPairShape): y = act(s1 (w1 x) + t1 + s2 (w2 x2) + t2) is computed as act([s1 w1 | s2 w2] [x; x2] + (t1 + t2)).
// The scaled, concatenated filter and the summed shift are computed by ordinary instructions in front of the call
// (from parameters alone, so they run once); the scales are multiplied in fp32 and the products rounded once to the
// 16-bit storage type, which moves a result by at most one rounding of a filter value per term.
Program FuseShortcutProjection(const Program& program, const std::set<std::string>& fetch_ids);

}  // namespace frontend
}  // namespace cinn
