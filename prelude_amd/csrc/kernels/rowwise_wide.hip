// Row-wise kernels for models that carry their residual stream in 32-bit beside activations in the engine's
// element type, and activations of feed-forwards that the gated epilogues of the products do not have:
//   - RMSNorm of (x + residual) with the residual kept in 32-bit, whatever the element type of x and the output;
//   - a gated pair with both halves clamped: g = min(g, limit), u = clamp(u, -limit, limit),
//     y = g * sigmoid(alpha * g) * (u + 1);
//   - the square of relu.
#include "common.h"
#include "api.h"

namespace pa {

// s = x (+ residual), all in 32-bit; residual <- s unrounded (unless `rows`); out = round(s * rsqrt(mean(s^2) + eps) * w).
// x may come as `slices` 32-bit partial sums, [slices, rows, hidden], added in order in place of the load of x.
// One workgroup a row; NV elements a thread held in registers between the two passes when the row fits.
template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_wide_kernel(const T* __restrict__ x, const float* __restrict__ parts,
                                                          int slices, size_t slice_stride, float* residual,
                                                          const float* __restrict__ w, T* __restrict__ out,
                                                          const int* __restrict__ rows, int hidden, float eps) {
  __shared__ float scratch[16];
  const int r = blockIdx.x;
  const size_t src = rows ? (size_t)rows[r] : (size_t)r;
  const T* xr = x ? x + src * hidden : nullptr;
  const float* pr = parts ? parts + src * hidden : nullptr;
  float* rr = residual ? residual + src * hidden : nullptr;
  T* orow = out + (size_t)r * hidden;
  auto value = [&](int i) {
    float v;
    if (pr) {
      v = pr[i];
      for (int p = 1; p < slices; ++p) v += pr[(size_t)p * slice_stride + i];
    } else {
      v = to_f32(xr[i]);
    }
    if (rr) v += rr[i];
    return v;
  };
  float ss = 0.f;
  if (NV > 0) {
    float v[NV > 0 ? NV : 1];
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = threadIdx.x + j * 256;
      v[j] = i < hidden ? value(i) : 0.f;
      ss += v[j] * v[j];
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)hidden + eps);
#pragma unroll
    for (int j = 0; j < NV; ++j) {
      const int i = threadIdx.x + j * 256;
      if (i < hidden) {
        if (rr && !rows) rr[i] = v[j];
        orow[i] = from_f32<T>(v[j] * inv * w[i]);
      }
    }
  } else {
    for (int i = threadIdx.x; i < hidden; i += 256) {
      const float s = value(i);
      ss += s * s;
    }
    ss = block_sum(ss, scratch);
    const float inv = rsqrtf(ss / (float)hidden + eps);
    for (int i = threadIdx.x; i < hidden; i += 256) {
      const float s = value(i);
      if (rr && !rows) rr[i] = s;
      orow[i] = from_f32<T>(s * inv * w[i]);
    }
  }
}

// gate_up [T, 2I] with columns alternating gate_j, up_j -> [T, I]
template <typename T>
__global__ void clamped_gate_kernel(const T* __restrict__ gate_up, T* __restrict__ out, size_t total, float limit,
                                    float alpha) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  out[i] = from_f32<T>(clamped_gate(to_f32(gate_up[2 * i]), to_f32(gate_up[2 * i + 1]), limit, alpha));
}

template <typename T>
__global__ void relu_squared_kernel(const T* __restrict__ x, T* __restrict__ out, size_t total) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= total) return;
  const float v = fmaxf(to_f32(x[i]), 0.f);
  out[i] = from_f32<T>(v * v);
}

// The same in 16-byte pieces for bfloat16: a thread takes eight pairs (two loads) and writes eight outputs.
__global__ void clamped_gate_vec_kernel(const bf16* __restrict__ gate_up, bf16* __restrict__ out, size_t groups, float limit,
                                        float alpha) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const bf16x8 a = *reinterpret_cast<const bf16x8*>(gate_up + 16 * i);
  const bf16x8 b = *reinterpret_cast<const bf16x8*>(gate_up + 16 * i + 8);
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    o[j] = (bf16)clamped_gate((float)a[2 * j], (float)a[2 * j + 1], limit, alpha);
    o[4 + j] = (bf16)clamped_gate((float)b[2 * j], (float)b[2 * j + 1], limit, alpha);
  }
  *reinterpret_cast<bf16x8*>(out + 8 * i) = o;
}

__global__ void relu_squared_vec_kernel(const bf16* __restrict__ x, bf16* __restrict__ out, size_t groups) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i >= groups) return;
  const bf16x8 a = *reinterpret_cast<const bf16x8*>(x + 8 * i);
  bf16x8 o;
#pragma unroll
  for (int j = 0; j < 8; ++j) {
    const float v = fmaxf((float)a[j], 0.f);
    o[j] = (bf16)(v * v);
  }
  *reinterpret_cast<bf16x8*>(out + 8 * i) = o;
}

template <typename T>
static void launch_wide(hipStream_t st, const T* x, const float* parts, int slices, size_t slice_stride, float* residual,
                        const float* w, T* out, const int* rows, int nrows, int hidden, float eps) {
#define PA_WIDE(NV)                                                                                                  \
  hipLaunchKernelGGL((rmsnorm_wide_kernel<T, NV>), dim3(nrows), dim3(256), 0, st, x, parts, slices, slice_stride,    \
                     residual, w, out, rows, hidden, eps)
  if (hidden <= 256) PA_WIDE(1);
  else if (hidden <= 1024) PA_WIDE(4);
  else if (hidden <= 2048) PA_WIDE(8);
  else if (hidden <= 4096) PA_WIDE(16);
  else if (hidden <= 8192) PA_WIDE(32);
  else PA_WIDE(0);
#undef PA_WIDE
}

}  // namespace pa

using namespace pa;

extern "C" int pa_rmsnorm_wide(void* stream, int dtype, const void* x, const float* parts, int slices, long slice_stride,
                               float* residual, const float* w, void* out, const int* rows, int nrows, int hidden,
                               float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && hidden > 0, "rmsnorm_wide: bad sizes rows=%d hidden=%d", nrows, hidden);
  PA_REQUIRE((x != nullptr) != (parts != nullptr), "rmsnorm_wide: give x or partial sums (one of them)");
  PA_REQUIRE(!parts || slices >= 1, "rmsnorm_wide: %d slices", slices);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    launch_wide<float>(st, (const float*)x, parts, slices, (size_t)slice_stride, residual, w, (float*)out, rows, nrows, hidden, eps);
  else if (dtype == kBF16)
    launch_wide<bf16>(st, (const bf16*)x, parts, slices, (size_t)slice_stride, residual, w, (bf16*)out, rows, nrows, hidden, eps);
  else
    return pa::fail("rmsnorm_wide: unknown element type code %d", dtype);
  return check_launch("rmsnorm_wide");
}

extern "C" int pa_clamped_gate(void* stream, int dtype, const void* gate_up, void* out, int tokens, int inter, float limit,
                               float alpha) {
  if (tokens == 0) return 0;
  PA_REQUIRE(tokens > 0 && inter > 0 && limit > 0.f, "clamped_gate: bad sizes tokens=%d inter=%d limit=%g", tokens, inter,
             (double)limit);
  const size_t total = (size_t)tokens * inter;
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kBF16 && total % 8 == 0 && ((uintptr_t)gate_up & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    hipLaunchKernelGGL(clamped_gate_vec_kernel, dim3((unsigned)((total / 8 + 255) / 256)), dim3(256), 0, st, (const bf16*)gate_up,
                       (bf16*)out, total / 8, limit, alpha);
    return check_launch("clamped_gate");
  }
  if (dtype == kF32)
    hipLaunchKernelGGL(clamped_gate_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)gate_up, (float*)out, total, limit, alpha);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(clamped_gate_kernel<bf16>, dim3(blocks), dim3(256), 0, st, (const bf16*)gate_up, (bf16*)out, total, limit, alpha);
  else
    return pa::fail("clamped_gate: unknown element type code %d", dtype);
  return check_launch("clamped_gate");
}

extern "C" int pa_relu_squared(void* stream, int dtype, const void* x, void* out, long total) {
  if (total == 0) return 0;
  PA_REQUIRE(total > 0, "relu_squared: bad size %ld", total);
  const unsigned blocks = (unsigned)((total + 255) / 256);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kBF16 && total % 8 == 0 && ((uintptr_t)x & 15) == 0 && ((uintptr_t)out & 15) == 0) {
    hipLaunchKernelGGL(relu_squared_vec_kernel, dim3((unsigned)((total / 8 + 255) / 256)), dim3(256), 0, st, (const bf16*)x, (bf16*)out,
                       (size_t)(total / 8));
    return check_launch("relu_squared");
  }
  if (dtype == kF32)
    hipLaunchKernelGGL(relu_squared_kernel<float>, dim3(blocks), dim3(256), 0, st, (const float*)x, (float*)out, (size_t)total);
  else if (dtype == kBF16)
    hipLaunchKernelGGL(relu_squared_kernel<bf16>, dim3(blocks), dim3(256), 0, st, (const bf16*)x, (bf16*)out, (size_t)total);
  else
    return pa::fail("relu_squared: unknown element type code %d", dtype);
  return check_launch("relu_squared");
}
