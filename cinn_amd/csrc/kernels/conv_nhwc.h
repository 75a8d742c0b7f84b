// Internal interface between the convolution intrinsics (conv_mfma.hip) and the channels-last MFMA kernels
// (conv_nhwc_mfma.hip).
#pragma once
#include <hip/hip_runtime.h>

#include "cinn_hip_runtime.h"
#include "kernels/conv_chain.h"
#include "runtime/scratch.h"

namespace cinn_hip_kernels {

struct ConvNhwcArgs {
  const void* x;         // NHWC activations, or NCHW when nchw_input is set
  const void* w;         // [OC][KH][KW][IC], or [OC][IC][KH][KW] when nchw_input is set
  void* y;               // NHWC [N][OH][OW][OC]
  const float* scale;    // per output channel, may be null (then alpha is used)
  const float* shift;    // per output channel, may be null
  const void* residual;  // NHWC tensor of y's shape added before the activation, may be null
  float alpha;           // used when scale is null
  float residual_scale;  // factor of the residual (beta of the alpha / beta form)
  bool relu;
  bool nchw_input;
  // a 3x3, stride 2, padding 1 max pooling follows the epilogue inside the kernel: y is the pooled tensor, oh / ow stay
  // the convolution's own output extents.  Only conv_stem7_mfma.hip implements it (StemPoolFusableShape says when).
  bool pool_after = false;
  int n, h, w_in, c;  // input extents
  int oc, kh, kw;
  int oh, ow;
  int pad_h, pad_w, stride_h, stride_w, dil_h, dil_w;
  cinn_type_t type;  // element type of x, w, y and residual
  // A second channels-last input [N][h2][w2][c2] read through a 1x1 window on the output's pixel grid, or null:
  //   y[n, oy, ox, :] = act(conv(x, w[:, :kh kw c]) + w[:, kh kw c:] x2[n, oy stride2_h, ox stride2_w, :] + ...)
  // The filter rows are then [kh][kw][c] followed by c2 more values.  Only the implicit-GEMM kernels take it
  // (TryPointwiseConvAsGemm; ConvPairShape says for which shapes).
  const void* x2 = nullptr;
  int h2 = 0, w2 = 0, c2 = 0, stride2_h = 1, stride2_w = 1;
};

// true when the channels-last kernels can run this convolution (groups are not supported; the general path needs
// the input channel count to be a multiple of one 16-byte chunk)
bool ConvNhwcSupported(const ConvNhwcArgs& a);
void RunConvNhwc(const ConvNhwcArgs& a, hipStream_t stream);

// 16-bit convolutions whose shape the direct-to-LDS GEMM kernels take (gemm_mfma.hip): a 1x1, stride 1, unpadded
// convolution is the GEMM pixels x channels; any other one with a multiple of 64 input channels runs as an implicit GEMM
// (K = kh * kw * c); both with this epilogue.  false when the shape does not qualify.
bool TryPointwiseConvAsGemm(const ConvNhwcArgs& a, hipStream_t stream);
// 3x3, stride 1, padding 1 convolutions with 16-bit operands and multiples of 64 channels on both sides whose input
// rows fit LDS (conv_patch_mfma.hip): the input patch of a band of output rows stays resident in LDS, only the filter
// streams; same epilogue.  false when the shape does not qualify.
bool TryConvPatch(const ConvNhwcArgs& a, hipStream_t stream);
// Two 1x1, stride 1, unpadded convolutions in a row on channels-last 16-bit tensors, seen as matrix products over the
// m = N * H * W pixels: e = act1(x w1^T * scale1 + shift1 + residual) [m][n1], y = act2(e w2^T * scale2 + shift2)
// [m][n2], with x [m][k1], w1 [n1][k1], w2 [n2][n1]; both e and y are written (conv_chain_mfma.hip).
struct ConvChainArgs {
  const void* x;
  const void* w1;
  const float* scale1;
  const float* shift1;
  const void* residual;  // may be null
  bool relu1;
  void* e;
  const void* w2;
  const float* scale2;
  const float* shift2;
  bool relu2;
  void* y;
  int64_t m;
  int k1, n1, n2;
  cinn_type_t type;
  // a second input of the first product, [m][k1b], or null: e = act1([x | x2] w1^T * scale1 + shift1) with w1
  // [n1][k1 + k1b]; no residual then
  const void* x2 = nullptr;
  int k1b = 0;
};
// false when the shape or the types do not qualify (the caller then runs the two convolutions one after the other)
bool TryConvChain(const ConvChainArgs& a, hipStream_t stream);
// 256 bytes of zeros in device memory (what masked-out chunks are read from)
inline const void* ConvZeroPage() { return ZeroPage(); }

// depthwise convolutions (groups == channels in == channels out) on channels-last tensors, filter [C][KH][KW]
// (conv_depthwise.hip): same epilogue; false when the shape does not qualify
bool DepthwiseNhwcSupported(const ConvNhwcArgs& a, int groups);
void RunDepthwiseNhwc(const ConvNhwcArgs& a, hipStream_t stream);

// NCHW-input convolutions whose filter and input patch fit LDS (conv_stem_mfma.hip): staged instead of gathered
bool ConvStemSupported(const ConvNhwcArgs& a);
void RunConvStem(const ConvNhwcArgs& a, hipStream_t stream);

// the 7x7, stride 2, padding 3 convolution of a 3-channel NCHW image in 16-bit types (conv_stem7_mfma.hip): persistent
// blocks with the next tile's input rows fetched while the current tile is multiplied; false when the shape does not
// qualify
bool TryConvStem7(const ConvNhwcArgs& a, hipStream_t stream);

}  // namespace cinn_hip_kernels

// Test hook, exported from the shared library but deliberately absent from the public header: the `s_waitcnt vmcnt`
// count a feeding wavefront of conv3x3_patch_chunks_kernel uses before the barrier of K step (chunk, tap) - how many of
// its loads may still be in flight while the next filter stage (and, at tap 7, the next chunk's patch) is known to have
// landed.  Host-side evaluation of the kernel's own constexpr, pure (no state).
extern "C" int cinn_hip_conv_patch_loads_in_flight(int tap, int first_chunk, int last_chunk, int patch_loads_per_step);

// Measurement hook of the direct-to-LDS GEMM kernel (gemm_mfma.hip), exported like the one above: while a device buffer
// is set, thread 0 of every block of that kernel writes four (100 MHz clock, core clock counter) pairs - block start,
// first operands landed, K loop done, last store issued - at buffer + 64 bytes * linear block index.  Null switches it
// off.  bench_gemm.py --clock reads the stamps.
extern "C" void cinn_hip_gemm_set_probe(void* device_buffer);

// The same for conv3x3_c64_stream_kernel (conv_patch_mfma.hip): six pairs per block at buffer + 128 bytes * linear
// block index - block start, filter and first patch rows landed, first tile multiplied, whole patch landed, fourth
// tile stored, last store issued.  bench_conv.py --clock reads the stamps.
extern "C" void cinn_hip_conv_patch_set_probe(void* device_buffer);
