// Decode-time kernels for 12-bit tags, chunk width 4.
#include "sq_rows_mfma.h"
namespace sq {
SQ_GEMV_FORMAT(12, 4)
SQ_MMA_FORMAT(12, 4)
}
