// The streaming kernels for five to eight activation rows (a file per row count: they compile side by side).
#include "q4_stream_kernels.h"

namespace mi355q {

MI355Q_STREAM_SHAPES(MI355Q_STREAM_DEFINE, 8)

}  // namespace mi355q
