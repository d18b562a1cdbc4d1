// Packed-int4 matmul for shapes the tiled kernels do not cover (group sizes that are not
// 32, 64 or a multiple of 128).  Same definition as packed_int4_gemm_scalar
// (crates/yscv-kernels/src/ops/int4_matmul.rs:387-435): one wavefront per output row, the
// lanes stride over the row's bytes, fp32 arithmetic, one cross-lane reduction per result.
// It is a correctness path, not a fast one: the row is re-read once per activation row.
#include "int4_common.hpp"
#include "kernels.hpp"

namespace yscv {

template <typename ST>
__global__ void __launch_bounds__(256) int4_generic_kernel(const uint8_t *__restrict__ raw,
                                                           const ST *__restrict__ scales,
                                                           const uint8_t *__restrict__ zps,
                                                           const void *__restrict__ x, int x_dtype,
                                                           void *__restrict__ y, int y_dtype, size_t m,
                                                           size_t n, size_t k, size_t g) {
  const size_t groups = k / g;
  const int lane = threadIdx.x & 63;
  const size_t wave = (blockIdx.x * (size_t)blockDim.x + threadIdx.x) >> 6;
  const size_t nwaves = ((size_t)gridDim.x * blockDim.x) >> 6;
  for (size_t item = wave; item < m * n; item += nwaves) {
    const size_t mi = item / n, row = item % n;
    const uint8_t *rb = raw + row * (k / 2);
    float acc = 0.0f;
    for (size_t b = lane; b < k / 2; b += 64) {
      const size_t grp = (2 * b) / g;
      const float sc = (float)scales[row * groups + grp];
      const float zp = zps ? (float)zps[row * groups + grp] : 8.0f;
      const int byte = rb[b];
      const float q0 = (float)(byte & 15) - zp, q1 = (float)(byte >> 4) - zp;
      const float x0 = load_in(x, mi * k + 2 * b, x_dtype), x1 = load_in(x, mi * k + 2 * b + 1, x_dtype);
      acc = fmaf(sc, fmaf(q0, x0, q1 * x1), acc);
    }
    for (int off = 32; off > 0; off >>= 1) acc += __shfl_xor(acc, off, 64);
    if (lane == 0) store_out(y, mi * n + row, acc, y_dtype);
  }
}

int32_t launch_int4_generic(const yscv_hip_int4_weight *w, const void *x, int x_dtype, void *y,
                            int y_dtype, size_t m, hipStream_t s) {
  if (!w->raw) return set_error(YSCV_HIP_ERR_UNSUPPORTED, "weight has no generic layout");
  size_t items = m * w->n;
  size_t blocks = ceil_div(items, (size_t)4);
  if (blocks > 65535 * 4) blocks = 65535 * 4;
  if (blocks < 1) blocks = 1;
  if (w->scale_dtype == YSCV_HIP_F32)
    hipLaunchKernelGGL(int4_generic_kernel<float>, dim3((unsigned)blocks), dim3(256), 0, s, w->raw,
                       static_cast<const float *>(w->rscales), w->rzps, x, x_dtype, y, y_dtype, m, w->n,
                       w->k, w->g);
  else
    hipLaunchKernelGGL(int4_generic_kernel<_Float16>, dim3((unsigned)blocks), dim3(256), 0, s, w->raw,
                       static_cast<const _Float16 *>(w->rscales), w->rzps, x, x_dtype, y, y_dtype, m,
                       w->n, w->k, w->g);
  YSCV_HIP_TRY(hipGetLastError());
  return YSCV_HIP_OK;
}

}  // namespace yscv
