// Grouped expert GEMM tiles for f16 operands, EPI_PLAIN epilogue.
#include "moe_gemm_tiles.h"

namespace fr {
template int dispatch_block<f16_t, EPI_PLAIN>(GemmArgs, int, int, int64_t, hipStream_t);
template int prepare_tiles<f16_t, EPI_PLAIN>();
}  // namespace fr
