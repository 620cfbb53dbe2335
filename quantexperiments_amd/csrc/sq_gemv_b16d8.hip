// Decode-time kernels for 16-bit tags, chunk width 8.
#include "sq_rows_mfma.h"
namespace sq {
SQ_GEMV_FORMAT(16, 8)
SQ_MMA_FORMAT(16, 8)
}
