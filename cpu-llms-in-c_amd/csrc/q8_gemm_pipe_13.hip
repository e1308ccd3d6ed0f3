// The pipelined GEMM kernel on 8-bit codes, 13 tiles per workgroup (three per wave and one
// shared): the shape whose blocks fill the compute units best on matrices like the 1600-tile
// conditioner gate.  A file of its own, like the other instantiations.
#include "q4_gemm_device.h"

namespace mi355q {

template __global__ void q4_gemm_pipe_kernel<128, 3, true, false, true>(const GemmParams);

}  // namespace mi355q
