// The kernels of the streaming affine-Q4 linear and the list of launch shapes they are built
// for.  Every row count's instantiations are compiled in a file of their own
// (q4_stream_rows_*.hip), so that they build side by side; q4_stream.hip, which launches them,
// only declares them.
#pragma once

#include "q4_stream_device.h"

namespace mi355q {

template <int MP, int TB, int D, int W, bool BF, bool WRAP = false>
__global__ void __launch_bounds__(64 * W) q4_stream_kernel(const StreamParams p)
{
    extern __shared__ uint4 lds[];
    stream_workgroup<MP, TB, D, W, BF, WRAP, kStreamPlain>(p, ChainParams{}, blockIdx.x, blockIdx.y, lds);
}

// The half-tile form (see stream_workgroup): MP operand rows = two per activation row.
template <int MP, int W, bool BF>
__global__ void __launch_bounds__(64 * W) q4_stream_half_kernel(const StreamParams p)
{
    extern __shared__ uint4 lds[];
    stream_workgroup<MP, 1, 2, W, BF, false, kStreamPlain, true>(p, ChainParams{}, blockIdx.x, 0u, lds);
}

// (tiles per workgroup, steps in flight, waves) built for every row count MP; sixteen waves
// exist for single tiles at one and two rows only
#define MI355Q_STREAM_SHAPES(X, MP)                                                                            \
    X(MP, 1, 2, 2) X(MP, 1, 2, 4) X(MP, 1, 2, 8) X(MP, 1, 4, 4) X(MP, 1, 4, 8) X(MP, 2, 2, 2) X(MP, 2, 2, 4) \
    X(MP, 2, 2, 8) X(MP, 3, 2, 4) X(MP, 4, 2, 2) X(MP, 4, 2, 4) X(MP, 4, 2, 8)
#define MI355Q_STREAM_SHAPES_SIXTEEN_WAVES(X, MP) X(MP, 1, 2, 16)
// (operand rows, waves) of the half-tile kernels
#define MI355Q_STREAM_HALF_SHAPES(X) X(2, 4) X(2, 8) X(2, 16) X(4, 4) X(4, 8) X(8, 4) X(8, 8)

// one shape = four kernels: metadata in bf16 planes or fp16 pairs, activation row repeated or not
#define MI355Q_STREAM_KERNELS(PREFIX, MP, TB, D, W)                                             \
    PREFIX template __global__ void q4_stream_kernel<MP, TB, D, W, true, true>(const StreamParams);   \
    PREFIX template __global__ void q4_stream_kernel<MP, TB, D, W, false, true>(const StreamParams);  \
    PREFIX template __global__ void q4_stream_kernel<MP, TB, D, W, true, false>(const StreamParams);  \
    PREFIX template __global__ void q4_stream_kernel<MP, TB, D, W, false, false>(const StreamParams);
#define MI355Q_STREAM_HALF_KERNELS(PREFIX, MP, W)                                               \
    PREFIX template __global__ void q4_stream_half_kernel<MP, W, true>(const StreamParams);     \
    PREFIX template __global__ void q4_stream_half_kernel<MP, W, false>(const StreamParams);

#define MI355Q_STREAM_DECLARE(MP, TB, D, W) MI355Q_STREAM_KERNELS(extern, MP, TB, D, W)
#define MI355Q_STREAM_DEFINE(MP, TB, D, W) MI355Q_STREAM_KERNELS(, MP, TB, D, W)
#define MI355Q_STREAM_HALF_DECLARE(MP, W) MI355Q_STREAM_HALF_KERNELS(extern, MP, W)
#define MI355Q_STREAM_HALF_DEFINE(MP, W) MI355Q_STREAM_HALF_KERNELS(, MP, W)

}  // namespace mi355q
