// The pipelined affine-Q4 GEMM kernel, 17 tiles per workgroup (the 17th shared by the four waves): one instantiation per file so that they
// compile side by side.
#include "q4_gemm_device.h"

namespace mi355q {

template __global__ void q4_gemm_pipe_kernel<128, 4, true, false>(const GemmParams);

}  // namespace mi355q
