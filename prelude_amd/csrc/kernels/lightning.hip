// Linear attention with a decaying state of fixed size per request and head ("lightning attention"):
//
//   S_t = a_h S_(t-1) + k_t v_t^T          S [dim, vdim], 32-bit, one per (request, head), kept in a state slot
//   o_t = S_t^T q_t                         o [vdim], 32-bit
//
// q, k [tokens, heads, dim] and v [tokens, heads, vdim] lie inside one merged projection (row stride ld, column
// offsets q_off, k_off, v_off) and may pass through an activation on their way in (act 0 none, 1 SiLU), taken in
// 32-bit.  a_h is the head's decay.  A sequence s of the step owns the packed rows cu_q[s] .. cu_q[s+1] and the
// state slot state_slots[s]; a request's portions may be cut anywhere, the state carries over.
//
// pa_lightning_attn: the recurrence as it stands, on the vector ALU, for any sizes and both element types.  A
// workgroup owns (64 value columns, head, sequence): four wavefronts split the rows of S between them (row d to
// wavefront d % 4), each thread keeps its rows of one column in registers and walks the tokens in order, sixteen at
// a time through LDS; the four partial dot products of a token are added in wavefront order.  The order of every sum
// follows the token's place in its sequence alone, so a token's output is the same bits however its prompt was cut.
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kLaTokens = 16;    // tokens staged at a time
constexpr int kLaCols = 64;      // value columns a workgroup
constexpr int kLaParts = 4;      // wavefronts, each with a share of the state's rows

__device__ __forceinline__ float la_act(float x, int act) { return act == 1 ? x / (1.0f + expf(-x)) : x; }

// R: rows of the state a thread keeps (dim <= 4 R)
template <typename T, int R>
__global__ __launch_bounds__(kLaParts* kLaCols) void lightning_attn_kernel(
    const T* __restrict__ qkv, long ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ cu_q, float* __restrict__ out,
    int heads, int dim, int vdim, int act) {
  __shared__ float qs[kLaTokens][4 * R];
  __shared__ float ks[kLaTokens][4 * R];
  __shared__ float vs[kLaTokens][kLaCols];
  __shared__ float part[kLaParts][kLaTokens][kLaCols];
  const int col = threadIdx.x % kLaCols, w = threadIdx.x / kLaCols;
  const int c0 = blockIdx.x * kLaCols, h = blockIdx.y, seq = blockIdx.z;
  const int row0 = cu_q[seq], row1 = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (slot < 0 || row1 <= row0) return;   // the same for the whole workgroup
  const bool live = c0 + col < vdim;
  const float a = decay[h];
  float* sp = state + (((size_t)slot * heads + h) * dim) * vdim + c0 + col;
  float S[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = r * kLaParts + w;
    S[r] = (live && d < dim) ? sp[(size_t)d * vdim] : 0.f;
  }
  for (int t0 = row0; t0 < row1; t0 += kLaTokens) {
    const int n = row1 - t0 < kLaTokens ? row1 - t0 : kLaTokens;
    __syncthreads();   // the block before has been read
    for (int i = threadIdx.x; i < n * dim; i += kLaParts * kLaCols) {
      const int t = i / dim, d = i % dim;
      const T* src = qkv + (size_t)(t0 + t) * ld + (size_t)h * dim + d;
      qs[t][d] = la_act(to_f32(src[q_off]), act);
      ks[t][d] = la_act(to_f32(src[k_off]), act);
    }
    for (int i = threadIdx.x; i < n * kLaCols; i += kLaParts * kLaCols) {
      const int t = i / kLaCols, c = i % kLaCols;
      vs[t][c] = c0 + c < vdim ? la_act(to_f32(qkv[(size_t)(t0 + t) * ld + v_off + (size_t)h * vdim + c0 + c]), act) : 0.f;
    }
    __syncthreads();
    for (int t = 0; t < n; ++t) {
      const float v = vs[t][col];
      float acc = 0.f;
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = r * kLaParts + w;
        if (d < dim) {
          S[r] = fmaf(a, S[r], ks[t][d] * v);
          acc = fmaf(S[r], qs[t][d], acc);
        }
      }
      part[w][t][col] = acc;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n * kLaCols; i += kLaParts * kLaCols) {
      const int t = i / kLaCols, c = i % kLaCols;
      if (c0 + c < vdim)
        out[((size_t)(t0 + t) * heads + h) * vdim + c0 + c] = ((part[0][t][c] + part[1][t][c]) + part[2][t][c]) + part[3][t][c];
    }
  }
  if (live) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = r * kLaParts + w;
      if (d < dim) sp[(size_t)d * vdim] = S[r];
    }
  }
}

template <typename T>
static int launch_lightning(hipStream_t st, const T* qkv, long ld, int q_off, int k_off, int v_off, const float* decay,
                            float* state, const int* state_slots, const int* cu_q, float* out, int nseq, int heads, int dim,
                            int vdim, int act) {
  dim3 grid((vdim + kLaCols - 1) / kLaCols, heads, nseq);
#define PA_LA(R)                                                                                                        \
  hipLaunchKernelGGL((lightning_attn_kernel<T, R>), grid, dim3(kLaParts* kLaCols), 0, st, qkv, ld, q_off, k_off, v_off, \
                     decay, state, state_slots, cu_q, out, heads, dim, vdim, act)
  if (dim <= 32) PA_LA(8);
  else if (dim <= 64) PA_LA(16);
  else if (dim <= 128) PA_LA(32);
  else PA_LA(64);
#undef PA_LA
  return 0;
}

}  // namespace pa

using namespace pa;

extern "C" int pa_lightning_attn(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off,
                                 const float* decay, float* state, const int* state_slots, const int* cu_q, float* out,
                                 int nseq, int tokens, int heads, int dim, int vdim, int act) {
  if (nseq == 0 || tokens == 0) return 0;
  PA_REQUIRE(nseq > 0 && tokens > 0 && heads > 0 && vdim > 0, "lightning_attn: bad sizes seqs=%d tokens=%d heads=%d vdim=%d", nseq,
             tokens, heads, vdim);
  PA_REQUIRE(dim > 0 && dim <= 256, "lightning_attn: a key width of %d is outside 1..256", dim);
  PA_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && ld >= (long)heads * dim, "lightning_attn: bad offsets or row stride %ld", ld);
  PA_REQUIRE(act == 0 || act == 1, "lightning_attn: unknown activation code %d", act);
  PA_REQUIRE(nseq <= 65535 && heads <= 65535, "lightning_attn: %d sequences x %d heads exceed the grid", nseq, heads);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    launch_lightning<float>(st, (const float*)qkv, ld, q_off, k_off, v_off, decay, state, state_slots, cu_q, out, nseq, heads, dim,
                            vdim, act);
  else if (dtype == kBF16)
    launch_lightning<bf16>(st, (const bf16*)qkv, ld, q_off, k_off, v_off, decay, state, state_slots, cu_q, out, nseq, heads, dim,
                           vdim, act);
  else
    return pa::fail("lightning_attn: unknown element type code %d", dtype);
  return check_launch("lightning_attn");
}
