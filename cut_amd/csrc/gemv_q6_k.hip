// Instantiates the streaming GEMV / skinny GEMM kernels for one block format.
#include "gemv_kernel.hpp"
#include "gemv_rows8.hpp"

namespace cuthip {
template int launch_fmt<CUTHIP_Q6_K>(GemvParams, hipStream_t);
template int launch_rows8_fmt<CUTHIP_Q6_K>(const GemvParams &, hipStream_t);
template bool rows8_fits<CUTHIP_Q6_K>(const GemvParams &);
template int launch_rows8_ksplit<CUTHIP_Q6_K>(const GemvParams &, float *, uint32_t *, hipStream_t);
}
