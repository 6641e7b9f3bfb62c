// Every dense GEMM kernel in the GEMM_BLOCK_FP8 scaling mode (see gemm_dispatch.h).
#include "gemm_dispatch.h"

namespace sglamd {
template int dispatch_out<GEMM_BLOCK_FP8>(const GemmArgs&, int, hipStream_t, void*, int64_t);
}  // namespace sglamd
