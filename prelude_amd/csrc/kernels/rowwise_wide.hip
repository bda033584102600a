// Row-wise kernels for models that carry their residual stream in 32-bit beside activations in the engine's
// element type, and activations of feed-forwards that the gated epilogues of the products do not have:
//   - RMSNorm of (x + residual) with the residual kept in 32-bit, whatever the element type of x and the output;
//   - a gated pair with both halves clamped: g = min(g, limit), u = clamp(u, -limit, limit),
//     y = g * sigmoid(alpha * g) * (u + 1);
//   - the square of relu;
//   - a branch's output brought to unit RMS, scaled and added to the 32-bit stream (a layer whose norm sits on the
//     sublayer's output: x <- x + norm(f(x))), with a copy of the new stream in the engine's type for the next reader;
//   - a row of 32-bit values brought to unit RMS, scaled, and multiplied by the sigmoid of a gate.
#include "common.h"
#include "api.h"

namespace pa {

// s = x (+ residual) (or the residual's rows alone, x and parts null), all in 32-bit; residual <- s unrounded (unless `rows`); out = round(s * rsqrt(mean(s^2) + eps) * w).
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
      v = xr ? to_f32(xr[i]) : 0.f;   // neither: the norm of the residual's rows alone
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

// residual <- residual + y * rsqrt(mean(y^2) + eps) * w, all in 32-bit; copy (or null) = the new residual rounded to
// T.  y is x, or `slices` partial sums added in order.  One workgroup a row; up to NV * 256 elements are held in
// registers between the two passes, longer rows are read twice.
template <typename T, int NV>
__global__ __launch_bounds__(256) void rmsnorm_branch_kernel(const T* __restrict__ x, const float* __restrict__ parts,
                                                            int slices, size_t slice_stride, float* __restrict__ residual,
                                                            const float* __restrict__ w, T* __restrict__ copy, int hidden,
                                                            float eps) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const T* xr = x ? x + r * hidden : nullptr;
  const float* pr = parts ? parts + r * hidden : nullptr;
  float* rr = residual + r * hidden;
  T* cr = copy ? copy + r * hidden : nullptr;
  auto value = [&](int i) {
    if (!pr) return to_f32(xr[i]);
    float v = pr[i];
    for (int p = 1; p < slices; ++p) v += pr[(size_t)p * slice_stride + i];
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
        const float s = rr[i] + v[j] * inv * w[i];
        rr[i] = s;
        if (cr) cr[i] = from_f32<T>(s);
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
      const float s = rr[i] + value(i) * inv * w[i];
      rr[i] = s;
      if (cr) cr[i] = from_f32<T>(s);
    }
  }
}

// out[t, i] = o[t, i] * rsqrt(mean_i(o[t, :]^2) + eps) * w[i] * sigmoid(gate[t, i]); o 32-bit, gate of type T in rows
// gate_stride elements apart (it may lie inside a wider projection).  One workgroup a row.
template <typename T, int NV>
__global__ __launch_bounds__(256) void gated_rmsnorm_kernel(const float* __restrict__ o, const T* __restrict__ gate,
                                                           size_t gate_stride, const float* __restrict__ w,
                                                           T* __restrict__ out, int width, float eps) {
  __shared__ float scratch[16];
  const size_t r = blockIdx.x;
  const float* orow = o + r * width;
  const T* grow = gate + r * gate_stride;
  T* dst = out + r * width;
  float ss = 0.f;
  float v[NV];
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * 256;
    v[j] = i < width ? orow[i] : 0.f;
    ss += v[j] * v[j];
  }
  ss = block_sum(ss, scratch);
  const float inv = rsqrtf(ss / (float)width + eps);
#pragma unroll
  for (int j = 0; j < NV; ++j) {
    const int i = threadIdx.x + j * 256;
    if (i < width) dst[i] = from_f32<T>(v[j] * inv * w[i] / (1.0f + expf(-to_f32(grow[i]))));
  }
}

template <typename T>
static void launch_branch(hipStream_t st, const T* x, const float* parts, int slices, size_t slice_stride, float* residual,
                          const float* w, T* copy, int nrows, int hidden, float eps) {
#define PA_BRANCH(NV)                                                                                                 \
  hipLaunchKernelGGL((rmsnorm_branch_kernel<T, NV>), dim3(nrows), dim3(256), 0, st, x, parts, slices, slice_stride,  \
                     residual, w, copy, hidden, eps)
  if (hidden <= 256) PA_BRANCH(1);
  else if (hidden <= 1024) PA_BRANCH(4);
  else if (hidden <= 2048) PA_BRANCH(8);
  else if (hidden <= 4096) PA_BRANCH(16);
  else if (hidden <= 8192) PA_BRANCH(32);
  else PA_BRANCH(0);
#undef PA_BRANCH
}

template <typename T>
static int launch_gated(hipStream_t st, const float* o, const T* gate, size_t gate_stride, const float* w, T* out, int nrows,
                        int width, float eps) {
#define PA_GATED(NV)                                                                                                  \
  hipLaunchKernelGGL((gated_rmsnorm_kernel<T, NV>), dim3(nrows), dim3(256), 0, st, o, gate, gate_stride, w, out, width, eps)
  if (width <= 256) PA_GATED(1);
  else if (width <= 1024) PA_GATED(4);
  else if (width <= 2048) PA_GATED(8);
  else if (width <= 4096) PA_GATED(16);
  else if (width <= 8192) PA_GATED(32);
  else return pa::fail("gated_rmsnorm: rows of %d elements are more than the 8192 the kernel takes", width);
#undef PA_GATED
  return 0;
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
  PA_REQUIRE(!(x && parts) && (x || parts || (residual && rows)),
             "rmsnorm_wide: give x or partial sums (one of them), or the residual and the rows to norm alone");
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

extern "C" int pa_rmsnorm_branch(void* stream, int dtype, const void* x, const float* parts, int slices, long slice_stride,
                                 float* residual, const float* w, void* copy, int nrows, int hidden, float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && hidden > 0 && residual && w, "rmsnorm_branch: bad sizes rows=%d hidden=%d", nrows, hidden);
  PA_REQUIRE((x != nullptr) != (parts != nullptr), "rmsnorm_branch: give x or partial sums (one of them)");
  PA_REQUIRE(!parts || slices >= 1, "rmsnorm_branch: %d slices", slices);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    launch_branch<float>(st, (const float*)x, parts, slices, (size_t)slice_stride, residual, w, (float*)copy, nrows, hidden, eps);
  else if (dtype == kBF16)
    launch_branch<bf16>(st, (const bf16*)x, parts, slices, (size_t)slice_stride, residual, w, (bf16*)copy, nrows, hidden, eps);
  else
    return pa::fail("rmsnorm_branch: unknown element type code %d", dtype);
  return check_launch("rmsnorm_branch");
}

extern "C" int pa_gated_rmsnorm(void* stream, int dtype, const float* o, const void* gate, long gate_stride, const float* w,
                                void* out, int nrows, int width, float eps) {
  if (nrows == 0) return 0;
  PA_REQUIRE(nrows > 0 && width > 0 && gate_stride >= width, "gated_rmsnorm: bad sizes rows=%d width=%d gate stride=%ld", nrows,
             width, gate_stride);
  hipStream_t st = (hipStream_t)stream;
  int rc;
  if (dtype == kF32)
    rc = launch_gated<float>(st, o, (const float*)gate, (size_t)gate_stride, w, (float*)out, nrows, width, eps);
  else if (dtype == kBF16)
    rc = launch_gated<bf16>(st, o, (const bf16*)gate, (size_t)gate_stride, w, (bf16*)out, nrows, width, eps);
  else
    return pa::fail("gated_rmsnorm: unknown element type code %d", dtype);
  return rc ? rc : check_launch("gated_rmsnorm");
}
