// Instantiates the streaming GEMV / skinny GEMM kernels for one block format.
#include "gemv_kernel.hpp"

namespace cuthip {
template int launch_fmt<CUTHIP_Q8_0>(GemvParams, hipStream_t);
}
