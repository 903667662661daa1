// Grouped expert GEMM tiles for fp8 operands, EPI_SILU epilogue.
#include "moe_gemm_tiles.h"

namespace fr {
template int dispatch_block<fp8_t, EPI_SILU>(GemmArgs, int, int, int64_t, hipStream_t);
template int prepare_tiles<fp8_t, EPI_SILU>();
}  // namespace fr
