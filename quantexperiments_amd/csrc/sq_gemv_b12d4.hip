// Decode-time kernels for 12-bit tags, chunk width 4.
#include "sq_gemv_kernel.h"
namespace sq {
SQ_GEMV_FORMAT(12, 4)
}
