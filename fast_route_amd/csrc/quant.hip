// Per-row dynamic quantisation to OCP fp8 e4m3 on gfx950.
//
// One wavefront per row: max|x| across the row (16-byte loads, cross-lane
// butterfly), scale = amax/448 (1 for an all-zero row), then x/scale converted
// with v_cvt_pk_fp8_f32 (round to nearest even).  Rows of up to 16384 elements
// are read once, by a workgroup each, and wait in registers for their scale;
// longer rows are read twice by one wavefront each.
#include "quant_core.h"

namespace fr {
namespace {

constexpr int kQuantThreads = 256;
constexpr int kQuantRowsPerBlock = kQuantThreads / kWave;

// Rows of up to 2048 * NC elements: one workgroup per row, the row in registers (NC 16-byte chunks per thread).
template <typename T, int NC>
__global__ __launch_bounds__(kQuantThreads) void quant_rows_block_kernel(const T* __restrict__ x, int64_t rows,
                                                                         const int32_t* __restrict__ rows_dev, int K,
                                                                         int64_t ldx, unsigned char* __restrict__ q,
                                                                         float* __restrict__ scale) {
  __shared__ float red[kQuantRowsPerBlock];
  const int64_t row = blockIdx.x;
  if (rows_dev && row >= rows_dev[0]) return;
  quant_row_block<T, NC, kQuantRowsPerBlock>(x + row * ldx, K, q + row * static_cast<int64_t>(K), scale + row, threadIdx.x, red);
}

// Longer rows: one wavefront per row, two passes over it.
template <typename T>
__global__ __launch_bounds__(kQuantThreads) void quant_rows_kernel(const T* __restrict__ x, int64_t rows,
                                                                   const int32_t* __restrict__ rows_dev, int K,
                                                                   int64_t ldx, unsigned char* __restrict__ q,
                                                                   float* __restrict__ scale) {
  const int lane = threadIdx.x % kWave;
  const int64_t row = static_cast<int64_t>(blockIdx.x) * kQuantRowsPerBlock + threadIdx.x / kWave;
  if (row >= rows || (rows_dev && row >= rows_dev[0])) return;
  quant_row(x + row * ldx, K, q + row * static_cast<int64_t>(K), scale + row, lane);
}

template <typename T>
void launch_quant_rows(const void* x, int64_t rows, const int32_t* rows_dev, int64_t K, int64_t ldx, void* q_out,
                       float* scale_out, hipStream_t st) {
  const dim3 per_row(static_cast<unsigned>(rows)), block(kQuantThreads);
  const T* xp = static_cast<const T*>(x);
  unsigned char* qp = static_cast<unsigned char*>(q_out);
  constexpr int64_t kPerChunk = 8 * kQuantThreads;  // elements one chunk per thread covers
  if (K <= 2 * kPerChunk) hipLaunchKernelGGL((quant_rows_block_kernel<T, 2>), per_row, block, 0, st, xp, rows, rows_dev, (int)K, ldx, qp, scale_out);
  else if (K <= 4 * kPerChunk) hipLaunchKernelGGL((quant_rows_block_kernel<T, 4>), per_row, block, 0, st, xp, rows, rows_dev, (int)K, ldx, qp, scale_out);
  else if (K <= 8 * kPerChunk) hipLaunchKernelGGL((quant_rows_block_kernel<T, 8>), per_row, block, 0, st, xp, rows, rows_dev, (int)K, ldx, qp, scale_out);
  else
    hipLaunchKernelGGL((quant_rows_kernel<T>), dim3(static_cast<unsigned>(ceil_div(rows, kQuantRowsPerBlock))), block, 0, st, xp,
                       rows, rows_dev, (int)K, ldx, qp, scale_out);
}

}  // namespace
}  // namespace fr

namespace fr {
// rows_dev (optional, device): only rows below *rows_dev are touched
int quant_rows(const void* x, int dtype, int64_t rows, const int32_t* rows_dev, int64_t K, int64_t ldx, void* q_out,
               float* scale_out, hipStream_t st) {
  if (rows == 0) return FR_OK;
  if (dtype == FR_BF16) launch_quant_rows<bf16_t>(x, rows, rows_dev, K, ldx, q_out, scale_out, st);
  else if (dtype == FR_F16) launch_quant_rows<f16_t>(x, rows, rows_dev, K, ldx, q_out, scale_out, st);
  else
    return fail(FR_E_DTYPE, "quantisation source dtype %d not in {f16, bf16}", dtype);
  return check_launch("quant_rows_kernel");
}
}  // namespace fr

extern "C" int fr_quant_e4m3_rows(const void* x, int dtype, int64_t rows, int64_t K, int64_t ldx, void* q_out,
                                  float* scale_out, void* stream) {
  using namespace fr;
  FR_REQUIRE(rows >= 0, FR_E_SHAPE, "fr_quant_e4m3_rows: rows=%lld < 0", (long long)rows);
  if (rows == 0) return FR_OK;
  FR_REQUIRE(x && q_out && scale_out, FR_E_NULL, "fr_quant_e4m3_rows: null pointer");
  FR_REQUIRE(K > 0 && K % 16 == 0 && K < (int64_t(1) << 30), FR_E_SHAPE, "fr_quant_e4m3_rows: K=%lld must be a positive multiple of 16", (long long)K);
  FR_REQUIRE(ldx >= K && ldx % 8 == 0 && aligned16(x) && aligned16(q_out), FR_E_ALIGN, "fr_quant_e4m3_rows: 16-byte alignment, ldx %% 8 == 0, ldx >= K");
  FR_REQUIRE(dtype == FR_BF16 || dtype == FR_F16, FR_E_DTYPE, "fr_quant_e4m3_rows: dtype %d not in {f16, bf16}", dtype);
  return quant_rows(x, dtype, rows, nullptr, K, ldx, q_out, scale_out, static_cast<hipStream_t>(stream));
}
