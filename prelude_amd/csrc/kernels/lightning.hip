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
// workgroup owns (64 or 128 value columns, head, sequence).  A lane keeps a quarter of the rows of S for one column
// (or two, 64 apart) in registers: the 16-lane rows of a wavefront are the four quarters, its wavefront picks the 16
// columns.  It walks the tokens in order, sixteen at a time through LDS; a token's four partial dot products are
// added across the wavefront's rows, (0 + 1) + (2 + 3).  The order of every sum follows the token's place in its
// sequence alone, so a token's output is the same bits however its prompt was cut.
//
// pa_lightning_attn_chunked: the same sums for long portions with the whole chip at work.  A portion is cut into
// chunks of C tokens; with S_b the state before a chunk and i a token's place in it,
//
//   o_i   = sum_{j <= i} a^(i-j) (q_i . k_j) v_j  +  a^(i+1) S_b^T q_i        (inside the chunk  +  from before it)
//   S_b'  = a^n S_b + U,   U = sum_j a^(n-1-j) k_j v_j^T                      (n tokens in the chunk)
//
// so (1) every chunk runs the recurrence from a zero state on its own, which gives the first sum and U, (2) one pass
// over the chunks of a sequence in order turns the U into the S_b and leaves the final state in the slot, (3) every
// chunk adds the second term.  All three keep to 32-bit and to non-negative powers of a.  Sequences of at most one
// chunk are left to pa_lightning_attn.
#include "common.h"
#include "api.h"

namespace pa {

constexpr int kLaTokens = 16;    // tokens staged at a time
constexpr int kLaLanes = 64;     // value columns a workgroup, times NC
constexpr int kLaThreads = 256;
constexpr int kLaMaxChunk = 256;

__device__ __forceinline__ float la_act(float x, int act) { return act == 1 ? x / (1.0f + expf(-x)) : x; }

// The sum over the four 16-lane rows of a wavefront, (row 0 + row 1) + (row 2 + row 3), in every lane.
__device__ __forceinline__ float la_sum_rows(float v) {
  const unsigned u = __float_as_uint(v);
  const auto a = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  v = __uint_as_float(a[0]) + __uint_as_float(a[1]);
  const unsigned w = __float_as_uint(v);
  const auto b = __builtin_amdgcn_permlane32_swap(w, w, false, false);
  return __uint_as_float(b[0]) + __uint_as_float(b[1]);
}

enum LaMode : int { kLaWhole = 0, kLaLocal = 1, kLaApply = 2 };

// Where chunk j of the sequence that starts at packed row `row0` and is the z-th of the launch keeps its state: every
// sequence adds at most one partial chunk, so floor(row0 / C) + z + j is different for every chunk of the launch and
// below tokens / C + sequences.
__device__ __forceinline__ size_t la_chunk_index(int row0, int chunk, int z, int j) { return (size_t)(row0 / chunk + z + j); }

// R: rows of the state a lane keeps (dim <= 4 R, R a multiple of 4); NC: columns a lane keeps (64 apart).
// kLaWhole: grid (column tiles, heads, sequences); sequences longer than `max_len` tokens (> 0) or shorter than
// `min_len` are left alone.
// kLaLocal / kLaApply: grid (column tiles, heads, listed sequences x max_chunks); sequences of at most one chunk and
// chunks past a sequence's end leave at once.
template <typename T, int R, int NC, int MODE>
__global__ __launch_bounds__(kLaThreads, 2) void lightning_attn_kernel(
    const T* __restrict__ qkv, long ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ cu_q,
    const int* __restrict__ seq_ids, float* __restrict__ out, float* __restrict__ work, int heads, int dim, int vdim, int act,
    int max_len, int chunk, int max_chunks, int min_len) {
  constexpr int kCols = kLaLanes * NC;
  // a quarter's rows lie R + 4 floats apart: the four 16-byte reads of a wavefront (one a quarter) then fall into
  // different banks (R is a multiple of 8, so R floats apart they would all fall into the same four)
  constexpr int kQuarter = R + 4;
  __shared__ __align__(16) float qs[kLaTokens][4 * kQuarter];
  __shared__ __align__(16) float ks[MODE == kLaApply ? 1 : kLaTokens][4 * kQuarter];
  __shared__ float vs[MODE == kLaApply ? 1 : kLaTokens][kCols];
  __shared__ float pw[MODE == kLaApply ? kLaMaxChunk : 1];
  const int w = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int dp = lane / 16;                      // which quarter of the rows
  const int cl = 16 * w + lane % 16;             // column within a run of 64
  const int c0 = blockIdx.x * kCols, h = blockIdx.y;
  int seq, z = 0, j = 0;
  if (MODE == kLaWhole) {
    seq = blockIdx.z;
  } else {
    z = blockIdx.z / max_chunks, j = blockIdx.z % max_chunks;
    seq = seq_ids[z];
  }
  int row0 = cu_q[seq], row1 = cu_q[seq + 1];
  const int slot = state_slots[seq];
  if (slot < 0 || row1 <= row0) return;   // the same for the whole workgroup
  if (MODE == kLaWhole && ((max_len > 0 && row1 - row0 > max_len) || row1 - row0 < min_len)) return;
  float* sp;
  if (MODE == kLaWhole) {
    sp = state + (((size_t)slot * heads + h) * dim) * vdim;
  } else {
    if (row1 - row0 <= chunk || row0 + j * chunk >= row1) return;
    sp = work + ((la_chunk_index(row0, chunk, z, j) * heads + h) * dim) * vdim;
    row0 += j * chunk;
    row1 = row1 < row0 + chunk ? row1 : row0 + chunk;
  }
  const float a = decay[h];
  if (MODE == kLaApply) {
    for (int i = threadIdx.x; i < chunk; i += kLaThreads) pw[i] = powf(a, (float)(i + 1));
  }
  int col[NC];
  bool live[NC];
  float S[NC][R];
#pragma unroll
  for (int c = 0; c < NC; ++c) {
    col[c] = c0 + kLaLanes * c + cl;
    live[c] = col[c] < vdim;
    // every load is unconditional (rows and columns that do not exist are clamped to ones that do, and zeroed by a
    // select): loads under branches are waited for one by one
    const int cc = live[c] ? col[c] : vdim - 1;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int d = dp * R + r;
      if (MODE == kLaLocal) {
        S[c][r] = 0.f;
      } else {
        const float v = sp[(size_t)(d < dim ? d : dim - 1) * vdim + cc];
        S[c][r] = (live[c] && d < dim) ? v : 0.f;
      }
    }
  }
  // A block of sixteen tokens on its way from memory: element e of the block is token e / kPerToken's query row d,
  // key row d or value column, by its place inside the token.  All of a thread's loads are asked for together, a
  // block ahead of their use, so the walk over a block's tokens hides them.
  constexpr int kPerToken = (MODE == kLaApply ? 4 * R : 8 * R + kCols);
  constexpr int kRaw = (kLaTokens * kPerToken + kLaThreads - 1) / kLaThreads;
  T raw[kRaw];
  auto fetch = [&](int t0) {
#pragma unroll
    for (int i = 0; i < kRaw; ++i) {
      const int e = threadIdx.x + kLaThreads * i;
      const int t = e / kPerToken, x = e % kPerToken;
      // rows past dim, columns past vdim and tokens past the end are zeros (they leave the sums alone); their loads
      // are clamped to places that exist, so that none stands under a branch
      const int tt = t0 + t < row1 ? t0 + t : row1 - 1;
      const int part = x < 4 * R ? 0 : (x < 8 * R ? 1 : 2);
      const int idx = x - (part == 0 ? 0 : (part == 1 ? 4 * R : 8 * R));
      const int width = part == 2 ? vdim : dim;
      const int at = part == 2 ? c0 + idx : idx;
      const size_t base = part == 0 ? (size_t)q_off + (size_t)h * dim : (part == 1 ? (size_t)k_off + (size_t)h * dim : (size_t)v_off + (size_t)h * vdim);
      const T v = qkv[(size_t)tt * ld + base + (at < width ? at : width - 1)];
      raw[i] = (t0 + t < row1 && t < kLaTokens && at < width) ? v : from_f32<T>(0.f);
    }
  };
  auto stage = [&]() {
#pragma unroll
    for (int i = 0; i < kRaw; ++i) {
      const int e = threadIdx.x + kLaThreads * i;
      const int t = e / kPerToken, x = e % kPerToken;
      if (t >= kLaTokens) continue;
      const float v = la_act(to_f32(raw[i]), act);
      if (x < 4 * R) {
        qs[t][(x / R) * kQuarter + x % R] = v;
      } else if (MODE != kLaApply) {
        if (x < 8 * R) ks[t][((x - 4 * R) / R) * kQuarter + (x - 4 * R) % R] = v;
        else vs[t][x - 8 * R] = v;
      }
    }
  };
  fetch(row0);
  for (int t0 = row0; t0 < row1; t0 += kLaTokens) {
    const int n = row1 - t0 < kLaTokens ? row1 - t0 : kLaTokens;
    __syncthreads();   // the block before has been read
    stage();
    __syncthreads();
    if (t0 + kLaTokens < row1) fetch(t0 + kLaTokens);
    // The block's tokens in groups whose results leave together.  The third pass adds to what the stream holds: it
    // asks for a whole block's places before the walk (its state is fixed, so it has the registers); the passes
    // that carry the state along take four tokens at a time, which keeps two wavefronts on a SIMD.
    constexpr int kGroup = MODE == kLaApply ? kLaTokens : 4;
#pragma unroll 1
    for (int tb = 0; tb < n; tb += kGroup) {
      float res[kGroup][NC];
      if (MODE == kLaApply) {
#pragma unroll
        for (int u = 0; u < kGroup; ++u)
#pragma unroll
          for (int c = 0; c < NC; ++c)
            res[u][c] = (dp == 0 && live[c] && tb + u < n) ? out[((size_t)(t0 + tb + u) * heads + h) * vdim + col[c]] : 0.f;
      }
#pragma unroll
      for (int u = 0; u < kGroup; ++u) {
        const int t = tb + u;
        if (t < n) {
          float acc[NC];
          float v[NC];
#pragma unroll
          for (int c = 0; c < NC; ++c) {
            acc[c] = 0.f;
            v[c] = MODE == kLaApply ? 0.f : vs[t][kLaLanes * c + cl];
          }
#pragma unroll
          for (int r = 0; r < R; r += 4) {
            const f32x4 q4 = *reinterpret_cast<const f32x4*>(&qs[t][dp * kQuarter + r]);
            f32x4 k4 = f32x4{0.f, 0.f, 0.f, 0.f};
            if (MODE != kLaApply) k4 = *reinterpret_cast<const f32x4*>(&ks[t][dp * kQuarter + r]);
#pragma unroll
            for (int e = 0; e < 4; ++e) {
#pragma unroll
              for (int c = 0; c < NC; ++c) {
                if (MODE != kLaApply) S[c][r + e] = fmaf(a, S[c][r + e], k4[e] * v[c]);
                acc[c] = fmaf(S[c][r + e], q4[e], acc[c]);
              }
            }
          }
#pragma unroll
          for (int c = 0; c < NC; ++c) {
            const float sum = la_sum_rows(acc[c]);
            res[u][c] = MODE == kLaApply ? res[u][c] + pw[t0 + t - row0] * sum : sum;
          }
        }
      }
      if (dp == 0) {
#pragma unroll
        for (int u = 0; u < kGroup; ++u)
#pragma unroll
          for (int c = 0; c < NC; ++c)
            if (tb + u < n && live[c]) out[((size_t)(t0 + tb + u) * heads + h) * vdim + col[c]] = res[u][c];
      }
    }
  }
  if (MODE != kLaApply) {
#pragma unroll
    for (int c = 0; c < NC; ++c) {
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const int d = dp * R + r;
        if (live[c] && d < dim) sp[(size_t)d * vdim + col[c]] = S[c][r];
      }
    }
  }
}

// Sequences of exactly one token (a decode step): the same sums as the kernel above gives for them, bit for bit, in a
// kernel small enough that a step's many launches do not wait for its code.  Grid (tiles of 64 columns, heads,
// sequences); a wavefront owns a quarter of the rows (the quarters of the kernel above), a lane a column: a row's 64
// columns are one run of memory.  All of a lane's rows of S are asked for at once, updated and stored; the quarters'
// dot products meet in LDS and are added (0 + 1) + (2 + 3).
template <typename T, int R>
__global__ __launch_bounds__(kLaThreads) void lightning_step_kernel(
    const T* __restrict__ qkv, long ld, int q_off, int k_off, int v_off, const float* __restrict__ decay,
    float* __restrict__ state, const int* __restrict__ state_slots, const int* __restrict__ cu_q, float* __restrict__ out,
    int heads, int dim, int vdim, int act) {
  __shared__ float qs[4 * R], ks[4 * R];
  __shared__ float part[4][kLaLanes];
  const int w = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int h = blockIdx.y, seq = blockIdx.z;
  const int row = cu_q[seq];
  const int slot = state_slots[seq];
  if (slot < 0 || cu_q[seq + 1] - row != 1) return;   // the same for the whole workgroup
  const int col = blockIdx.x * kLaLanes + lane;
  const bool live = col < vdim;
  float* sp = state + (((size_t)slot * heads + h) * dim) * vdim + (live ? col : vdim - 1);
  float s[R];
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = w * R + r;
    s[r] = sp[(size_t)(d < dim ? d : dim - 1) * vdim];
  }
  const T* src = qkv + (size_t)row * ld;
  if ((int)threadIdx.x < 4 * R) {
    const int d = (int)threadIdx.x < dim ? threadIdx.x : dim - 1;
    qs[threadIdx.x] = la_act(to_f32(src[q_off + (size_t)h * dim + d]), act);
    ks[threadIdx.x] = la_act(to_f32(src[k_off + (size_t)h * dim + d]), act);
  }
  const float v = la_act(to_f32(src[v_off + (size_t)h * vdim + (live ? col : vdim - 1)]), act);
  const float a = decay[h];
  __syncthreads();
  float acc = 0.f;
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = w * R + r;
    s[r] = fmaf(a, s[r], ks[d] * v);
    if (d < dim) acc = fmaf(s[r], qs[d], acc);
  }
#pragma unroll
  for (int r = 0; r < R; ++r) {
    const int d = w * R + r;
    if (live && d < dim) sp[(size_t)d * vdim] = s[r];
  }
  part[w][lane] = acc;
  __syncthreads();
  if (w == 0 && live) out[((size_t)row * heads + h) * vdim + col] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
}

// The chunks of one listed sequence in order: work[chunk] holds U coming in and the state before the chunk going
// out; the state slot gives the start and receives the end.  A thread an element of a head's state.
__global__ __launch_bounds__(256) void lightning_scan_kernel(const float* __restrict__ decay, float* __restrict__ state,
                                                            const int* __restrict__ state_slots, const int* __restrict__ cu_q,
                                                            const int* __restrict__ seq_ids, float* __restrict__ work,
                                                            int heads, int per_head, int chunk) {
  const int z = blockIdx.z, h = blockIdx.y;
  const int seq = seq_ids[z];
  const int row0 = cu_q[seq], len = cu_q[seq + 1] - row0;
  const int slot = state_slots[seq];
  if (slot < 0 || len <= chunk) return;
  const int e = blockIdx.x * 256 + threadIdx.x;
  if (e >= per_head) return;
  const float a = decay[h];
  const float a_chunk = powf(a, (float)chunk);
  float* sp = state + ((size_t)slot * heads + h) * per_head + e;
  float S = *sp;
  const int chunks = (len + chunk - 1) / chunk;
  for (int j = 0; j < chunks; ++j) {
    float* wp = work + (la_chunk_index(row0, chunk, z, j) * heads + h) * per_head + e;
    const float U = *wp;
    *wp = S;
    const int n = len - j * chunk;
    S = fmaf(n >= chunk ? a_chunk : powf(a, (float)n), S, U);
  }
  *sp = S;
}

template <typename T, int MODE>
static void launch_lightning(hipStream_t st, int zdim, const T* qkv, long ld, int q_off, int k_off, int v_off,
                             const float* decay, float* state, const int* state_slots, const int* cu_q, const int* seq_ids,
                             float* out, float* work, int heads, int dim, int vdim, int act, int max_len, int chunk,
                             int max_chunks, int min_len = 0) {
  // two columns a lane where the state is wide enough and its rows leave the registers for them
  // ... and there are workgroups enough without halving the columns of each (a step of few single tokens wants the
  // workgroups)
  const bool two = vdim > kLaLanes && dim <= 128 && (long)zdim * heads * ((vdim + 2 * kLaLanes - 1) / (2 * kLaLanes)) >= 256;
  const int cols = two ? 2 * kLaLanes : kLaLanes;
  dim3 grid((vdim + cols - 1) / cols, heads, zdim);
#define PA_LA(R, NC)                                                                                                       \
  hipLaunchKernelGGL((lightning_attn_kernel<T, R, NC, MODE>), grid, dim3(kLaThreads), 0, st, qkv, ld, q_off, k_off, v_off, \
                     decay, state, state_slots, cu_q, seq_ids, out, work, heads, dim, vdim, act, max_len, chunk, max_chunks, min_len)
  if (dim <= 32) { if (two) PA_LA(8, 2); else PA_LA(8, 1); }
  else if (dim <= 64) { if (two) PA_LA(16, 2); else PA_LA(16, 1); }
  else if (dim <= 128) { if (two) PA_LA(32, 2); else PA_LA(32, 1); }
  else PA_LA(64, 1);
#undef PA_LA
}

static int lightning_check(const char* what, int nseq, int tokens, int heads, int dim, int vdim, long ld, int q_off, int k_off,
                           int v_off, int act) {
  PA_REQUIRE(nseq > 0 && tokens > 0 && heads > 0 && vdim > 0, "%s: bad sizes seqs=%d tokens=%d heads=%d vdim=%d", what, nseq,
             tokens, heads, vdim);
  PA_REQUIRE(dim > 0 && dim <= 256, "%s: a key width of %d is outside 1..256", what, dim);
  PA_REQUIRE(q_off >= 0 && k_off >= 0 && v_off >= 0 && ld >= (long)heads * dim, "%s: bad offsets or row stride %ld", what, ld);
  PA_REQUIRE(act == 0 || act == 1, "%s: unknown activation code %d", what, act);
  PA_REQUIRE(heads <= 65535, "%s: %d heads exceed the grid", what, heads);
  return 0;
}

}  // namespace pa

using namespace pa;

// max_len > 0: sequences of more tokens are left alone (they go to pa_lightning_attn_chunked); sequences of fewer
// than min_len tokens are left alone too (single tokens go to pa_lightning_step).
extern "C" int pa_lightning_attn(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off,
                                 const float* decay, float* state, const int* state_slots, const int* cu_q, float* out,
                                 int nseq, int tokens, int heads, int dim, int vdim, int act, int max_len, int min_len) {
  if (nseq == 0 || tokens == 0) return 0;
  if (int rc = lightning_check("lightning_attn", nseq, tokens, heads, dim, vdim, ld, q_off, k_off, v_off, act)) return rc;
  PA_REQUIRE(nseq <= 65535, "lightning_attn: %d sequences exceed the grid", nseq);
  hipStream_t st = (hipStream_t)stream;
  if (dtype == kF32)
    launch_lightning<float, kLaWhole>(st, nseq, (const float*)qkv, ld, q_off, k_off, v_off, decay, state, state_slots, cu_q,
                                      nullptr, out, nullptr, heads, dim, vdim, act, max_len, 0, 1, min_len);
  else if (dtype == kBF16)
    launch_lightning<bf16, kLaWhole>(st, nseq, (const bf16*)qkv, ld, q_off, k_off, v_off, decay, state, state_slots, cu_q,
                                     nullptr, out, nullptr, heads, dim, vdim, act, max_len, 0, 1, min_len);
  else
    return pa::fail("lightning_attn: unknown element type code %d", dtype);
  return check_launch("lightning_attn");
}

// The sequences of exactly one token among the step's nseq (the others are left alone).
extern "C" int pa_lightning_step(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off,
                                 const float* decay, float* state, const int* state_slots, const int* cu_q, float* out,
                                 int nseq, int heads, int dim, int vdim, int act) {
  if (nseq == 0) return 0;
  if (int rc = lightning_check("lightning_step", nseq, nseq, heads, dim, vdim, ld, q_off, k_off, v_off, act)) return rc;
  PA_REQUIRE(nseq <= 65535, "lightning_step: %d sequences exceed the grid", nseq);
  hipStream_t st = (hipStream_t)stream;
  dim3 grid((vdim + kLaLanes - 1) / kLaLanes, heads, nseq);
#define PA_LS(T, R)                                                                                                       \
  hipLaunchKernelGGL((lightning_step_kernel<T, R>), grid, dim3(kLaThreads), 0, st, (const T*)qkv, ld, q_off, k_off, v_off, \
                     decay, state, state_slots, cu_q, out, heads, dim, vdim, act)
#define PA_LS_R(T)                    \
  do {                                \
    if (dim <= 32) PA_LS(T, 8);       \
    else if (dim <= 64) PA_LS(T, 16); \
    else if (dim <= 128) PA_LS(T, 32); \
    else PA_LS(T, 64);                \
  } while (0)
  if (dtype == kF32)
    PA_LS_R(float);
  else if (dtype == kBF16)
    PA_LS_R(bf16);
  else
    return pa::fail("lightning_step: unknown element type code %d", dtype);
#undef PA_LS_R
#undef PA_LS
  return check_launch("lightning_step");
}

// 32-bit words of workspace for the listed sequences' chunk states
extern "C" long pa_lightning_attn_workspace(int nlisted, int tokens, int heads, int dim, int vdim, int chunk) {
  if (chunk <= 0) return 0;
  return ((long)tokens / chunk + nlisted) * heads * dim * vdim;
}

// The sequences seq_ids[0 .. nlisted) that have more than `chunk` tokens (at most max_len each), in chunks.
extern "C" int pa_lightning_attn_chunked(void* stream, int dtype, const void* qkv, long ld, int q_off, int k_off, int v_off,
                                         const float* decay, float* state, const int* state_slots, const int* cu_q,
                                         const int* seq_ids, float* out, float* work, int nlisted, int tokens, int max_len,
                                         int heads, int dim, int vdim, int act, int chunk) {
  if (nlisted == 0 || tokens == 0 || max_len <= chunk) return 0;
  if (int rc = lightning_check("lightning_attn_chunked", nlisted, tokens, heads, dim, vdim, ld, q_off, k_off, v_off, act)) return rc;
  PA_REQUIRE(chunk >= kLaTokens && chunk % kLaTokens == 0 && chunk <= kLaMaxChunk,
             "lightning_attn_chunked: chunks of %d tokens are not a multiple of %d up to %d", chunk, kLaTokens, kLaMaxChunk);
  PA_REQUIRE(seq_ids && work, "lightning_attn_chunked: no list of sequences or no workspace");
  const int max_chunks = (max_len + chunk - 1) / chunk;
  PA_REQUIRE((long)nlisted * max_chunks <= 65535, "lightning_attn_chunked: %d sequences x %d chunks exceed the grid", nlisted, max_chunks);
  hipStream_t st = (hipStream_t)stream;
  const int per_head = dim * vdim;
  dim3 scan_grid((per_head + 255) / 256, heads, nlisted);
#define PA_LA_PASS(T, MODE)                                                                                               \
  launch_lightning<T, MODE>(st, nlisted * max_chunks, (const T*)qkv, ld, q_off, k_off, v_off, decay, state, state_slots, cu_q, seq_ids, out, \
                            work, heads, dim, vdim, act, 0, chunk, max_chunks)
#define PA_LA_SCAN()                                                                                                      \
  hipLaunchKernelGGL(lightning_scan_kernel, scan_grid, dim3(256), 0, st, decay, state, state_slots, cu_q, seq_ids, work,   \
                     heads, per_head, chunk)
  if (dtype == kF32) {
    PA_LA_PASS(float, kLaLocal);
    PA_LA_SCAN();
    PA_LA_PASS(float, kLaApply);
  } else if (dtype == kBF16) {
    PA_LA_PASS(bf16, kLaLocal);
    PA_LA_SCAN();
    PA_LA_PASS(bf16, kLaApply);
  } else {
    return pa::fail("lightning_attn_chunked: unknown element type code %d", dtype);
  }
#undef PA_LA_PASS
#undef PA_LA_SCAN
  return check_launch("lightning_attn_chunked");
}
