// Pair launches of the 8-row GEMV (two weight tensors, one activation vector) for the K-quant formats.
#include "gemv_rows8.hpp"

namespace cuthip {
template bool launch_rows8_pair_fmt<CUTHIP_Q4_K, CUTHIP_Q4_K>(const GemvParams &, const GemvParams &, hipStream_t, int *);
template bool launch_rows8_pair_fmt<CUTHIP_Q4_K, CUTHIP_Q6_K>(const GemvParams &, const GemvParams &, hipStream_t, int *);
template bool launch_rows8_pair_fmt<CUTHIP_Q6_K, CUTHIP_Q4_K>(const GemvParams &, const GemvParams &, hipStream_t, int *);
template bool launch_rows8_pair_fmt<CUTHIP_Q6_K, CUTHIP_Q6_K>(const GemvParams &, const GemvParams &, hipStream_t, int *);
}  // namespace cuthip
