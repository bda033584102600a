// C[m, n] = X[m, k] W[n, k]^T for a weight of few rows (n up to 256: a router's, say), any number of rows of X,
// bfloat16 operands, 32-bit sums and a 32-bit result.  The library's products round their result to bfloat16, which
// a router's scores must not be; the plain 32-bit product takes as long for 64 columns as for thousands.
//
// A workgroup owns 16 rows of X and all columns; its four wavefronts take a quarter of k each (whole steps of 32) and
// add their sums through LDS in wavefront order.  Per step one A fragment (a lane's 16 bytes of its row) and one B
// fragment per 16 columns (a lane's 16 bytes of a row of W), both straight from memory, W staying in the caches;
// accumulators of ceil(n / 16) tiles.  The order of every sum follows k alone, whatever m is.
#include "common.h"
#include "api.h"

namespace pa {

template <int NT>
__global__ __launch_bounds__(256) void gemm_narrow_kernel(const bf16* __restrict__ x, const bf16* __restrict__ w,
                                                         float* __restrict__ c, int m, int n, int k, long ldx, long ldc) {
  __shared__ float sums[3][NT][4][kWave];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int m0 = blockIdx.x * 16;
  const int nt = (n + 15) / 16;
  const int row = m0 + r < m ? m0 + r : m - 1;
  const bf16* xr = x + (size_t)row * ldx + 8 * g;
  f32x4 acc[NT];
#pragma unroll
  for (int j = 0; j < NT; ++j) acc[j] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16x8 zero;
#pragma unroll
  for (int i = 0; i < 8; ++i) zero[i] = (bf16)0.f;
  const int steps = (k + 31) / 32, per = (steps + 3) / 4;
  const int s_end = (wave + 1) * per < steps ? (wave + 1) * per : steps;
  for (int s = wave * per; s < s_end; ++s) {
    const int k0 = 32 * s;
    const bool in = k0 + 8 * g < k;   // k is a multiple of 8: a lane's piece lies inside or outside whole
    const bf16x8 a = in ? *reinterpret_cast<const bf16x8*>(xr + k0) : zero;
#pragma unroll
    for (int j = 0; j < NT; ++j) {
      if (j < nt) {
        const int col = 16 * j + r < n ? 16 * j + r : n - 1;
        const bf16x8 b = in ? *reinterpret_cast<const bf16x8*>(w + (size_t)col * k + k0 + 8 * g) : zero;
        acc[j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc[j], 0, 0, 0);
      }
    }
  }
  if (wave > 0) {
#pragma unroll
    for (int j = 0; j < NT; ++j)
#pragma unroll
      for (int i = 0; i < 4; ++i) sums[wave - 1][j][i][lane] = acc[j][i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int j = 0; j < NT; ++j) {
    const int col = 16 * j + r;
    if (j < nt && col < n) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int orow = m0 + 4 * g + i;
        const float v = ((acc[j][i] + sums[0][j][i][lane]) + sums[1][j][i][lane]) + sums[2][j][i][lane];
        if (orow < m) c[(size_t)orow * ldc + col] = v;
      }
    }
  }
}

}  // namespace pa

using namespace pa;

extern "C" int pa_gemm_narrow(void* stream, const void* x, const void* w, float* c, int m, int n, int k, long ldx, long ldc) {
  if (m == 0) return 0;
  PA_REQUIRE(m > 0 && n > 0 && k > 0 && ldx >= k && ldc >= n, "gemm_narrow: bad sizes m=%d n=%d k=%d", m, n, k);
  PA_REQUIRE(n <= 256, "gemm_narrow: %d columns are more than the 256 the kernel takes", n);
  PA_REQUIRE(k % 8 == 0 && ldx % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)w & 15) == 0,
             "gemm_narrow: rows of %d elements (stride %ld) are no whole 16-byte pieces", k, ldx);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((m + 15) / 16);
#define PA_NARROW(NT)                                                                                             \
  hipLaunchKernelGGL(gemm_narrow_kernel<NT>, grid, dim3(256), 0, st, (const bf16*)x, (const bf16*)w, c, m, n, k, ldx, ldc)
  if (n <= 64) PA_NARROW(4);
  else if (n <= 128) PA_NARROW(8);
  else if (n <= 256) PA_NARROW(16);
  else return pa::fail("gemm_narrow: %d columns are more than the 256 the kernel takes", n);
#undef PA_NARROW
  return check_launch("gemm_narrow");
}
