// The pipelined GEMM kernel on 8-bit codes, 16 tiles per workgroup (a file of its own, like the
// affine-Q4 instantiations, so that they compile side by side).
#include "q4_gemm_device.h"

namespace mi355q {

template __global__ void q4_gemm_pipe_kernel<128, 4, false, false, true>(const GemmParams);

}  // namespace mi355q
