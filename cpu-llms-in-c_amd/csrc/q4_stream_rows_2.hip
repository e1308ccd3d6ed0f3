// The streaming kernels for two activation rows (and the half-tile kernels) (a file per row count: they compile side by side).
#include "q4_stream_kernels.h"

namespace mi355q {

MI355Q_STREAM_SHAPES(MI355Q_STREAM_DEFINE, 2)
MI355Q_STREAM_SHAPES_SIXTEEN_WAVES(MI355Q_STREAM_DEFINE, 2)
MI355Q_STREAM_HALF_SHAPES(MI355Q_STREAM_HALF_DEFINE)

}  // namespace mi355q
