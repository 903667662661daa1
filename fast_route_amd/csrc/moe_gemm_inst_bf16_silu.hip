// Grouped expert GEMM tiles for bf16 operands, EPI_SILU epilogue.
#include "moe_gemm_tiles.h"

namespace fr {
template int dispatch_block<bf16_t, EPI_SILU>(GemmArgs, int, int, int64_t, hipStream_t);
template int prepare_tiles<bf16_t, EPI_SILU>();
}  // namespace fr
