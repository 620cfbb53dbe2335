// Decode-time kernels for 16-bit tags, chunk width 8.
#include "sq_gemv_kernel.h"
namespace sq {
SQ_GEMV_FORMAT(16, 8)
}
