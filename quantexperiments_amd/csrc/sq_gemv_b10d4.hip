// Decode-time kernels for 10-bit tags, chunk width 4.
#include "sq_rows_mfma.h"
namespace sq {
SQ_GEMV_FORMAT(10, 4)
SQ_MMA_FORMAT(10, 4)
}
