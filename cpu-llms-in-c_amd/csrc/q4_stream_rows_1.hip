// The streaming kernels for one activation row (a file per row count: they compile side by side).
#include "q4_stream_kernels.h"

namespace mi355q {

MI355Q_STREAM_SHAPES(MI355Q_STREAM_DEFINE, 1)
MI355Q_STREAM_SHAPES_SIXTEEN_WAVES(MI355Q_STREAM_DEFINE, 1)

}  // namespace mi355q
