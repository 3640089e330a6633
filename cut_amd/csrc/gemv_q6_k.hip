// Instantiates the streaming GEMV / skinny GEMM kernels for one block format.
#include "gemv_kernel.hpp"

namespace cuthip {
template int launch_fmt<CUTHIP_Q6_K>(GemvParams, hipStream_t);
}
