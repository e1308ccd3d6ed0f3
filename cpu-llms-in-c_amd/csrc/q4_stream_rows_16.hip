// The streaming kernels for nine to sixteen activation rows (a file per row count: they compile side by side).
#include "q4_stream_kernels.h"

namespace mi355q {

MI355Q_STREAM_SHAPES(MI355Q_STREAM_DEFINE, 16)

}  // namespace mi355q
