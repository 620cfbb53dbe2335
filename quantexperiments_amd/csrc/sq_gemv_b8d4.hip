// Decode-time kernels for 8-bit tags, chunk width 4.
#include "sq_rows_mfma.h"
namespace sq {
SQ_GEMV_FORMAT(8, 4)
SQ_MMA_FORMAT(8, 4)
}
