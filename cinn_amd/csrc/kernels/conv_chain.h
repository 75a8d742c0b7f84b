// What the graph rewrite needs to know about the kernel that runs two 1x1 convolutions in a row (conv_chain_mfma.hip),
// in plain integers so that host-only translation units can include it.
#pragma once
#include <cstdint>

namespace cinn_hip_kernels {

// True when one kernel computes e = act(x w1^T ...) [m][n1] and y = act(e w2^T ...) [m][n2] from x [m][k1] in a 16-bit
// type: the channel counts it is instantiated for, m a multiple of 16.
bool ConvChainShape(int64_t m, int k1, int n1, int n2);
// The same with a second input of the first product: e = act([x | x2] w1^T ...) with x2 [m][k1b], w1 [n1][k1 + k1b].
bool ConvChainShape2(int64_t m, int k1, int k1b, int n1, int n2);

// True when the implicit-GEMM kernels (gemm_mfma.hip) compute a 1x1 convolution over two channels-last 16-bit inputs
// that share the output's pixel grid - y = act([x | x2] w^T + shift) with x [m][c1], x2 read at a stride, w [oc][c1 + c2]
// - in one launch: both channel counts multiples of the 64-deep K step and enough output tiles to fill the chip.
bool ConvPairShape(int64_t m, int c1, int c2, int oc);

}  // namespace cinn_hip_kernels
