// Attention over a cache of latents on the matrix cores (bfloat16 in, 32-bit scores, softmax and sums).
//
// All heads read the same cached vectors, so the rows of the score matrix are (token, head) pairs: a workgroup
// of four wavefronts owns 64 consecutive rows of one sequence's portion (row = token * heads + head), 16 a
// wavefront, and walks the keys in blocks of 32.  A block is brought into LDS once per workgroup: the vectors as
// they lie in the cache (rows of rank + rot elements, the score's operand), and the first `rank` elements of each
// again transposed ([element][key]: the operand of the weighted sum, whose contraction runs over keys).  The cache
// keeps that transposed copy itself ([pages, rank, page]), written once per token, so both are copied in 16-byte
// pieces, from memory straight into LDS.
//
//   S^T = K Q^T     A = 16 keys x 32 elements from LDS, B = the wavefront's queries, kept in registers
//   O^T = V^T P^T   A = 16 elements x 32 keys from the transposed copy, B = the probabilities just computed
//
// v_mfma_f32_16x16x32_bf16 (lane l, g = l / 16, r = l % 16): A row r, columns 8g..8g+7; B column r, rows 8g..8g+7;
// C column r, rows 4g..4g+3.  A block's 32 keys are two score tiles; row 4a + i of tile t stands for key
// 8a + 4t + i, so lane group g ends up with the scores of keys 8g..8g+7 of its query: packed, they are the B
// operand of the second product as they stand.
//
// Few rows a sequence (single decoded tokens) would leave the chip empty: then the keys are cut into splits of
// `split_keys` (grid.z), each leaving an unnormalised partial (maximum, sum, weighted sum) that a merge kernel adds
// up in split order.  The sink joins last, as one more term exp(sink_h) of the denominator.
#include "common.h"
#include "api.h"

namespace pa {

constexpr float kLog2eL = 1.4426950408889634f;
constexpr int kLmRows = 64;      // query rows a workgroup
constexpr int kLmKeys = 32;      // keys a block
constexpr int kLmPad = 8;        // elements of padding behind an LDS row

// 64 pieces of 16 bytes from memory straight into LDS: lane l's piece lands at `lds_base` + 16 l.  Written as the
// instruction itself: through the compiler's own builtin every later read of LDS first waited for all such loads
// (it cannot tell the two buffers apart), which put the staging in line with the products instead of behind them.
// The kernel waits for them itself (vmcnt 0) before the barrier that publishes a buffer.
__device__ __forceinline__ void load_to_lds_16(const void* src, void* lds_base) {
  const unsigned base = __builtin_amdgcn_readfirstlane((unsigned)(uintptr_t)(__attribute__((address_space(3))) char*)lds_base);
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(base), "v"(src) : "memory");
}

__device__ __forceinline__ f32x4 mfma16l(bf16x8 a, bf16x8 b, f32x4 c) {
  return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
}

// RT: value tiles of 16 elements held in registers (rank <= 16 RT); QS: steps of 32 elements of a query held in
// registers (rank + rot <= 32 QS).
template <int RT, int QS>
__global__ __launch_bounds__(256) void latent_attn_mfma_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ cache, const bf16* __restrict__ cache_t,
    const float* __restrict__ sink, const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, bf16* __restrict__ out,
    float* __restrict__ ws, int nh, int rank, int rot, int page_size, int window, float scale, int split_keys,
    int n_splits) {
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int dk = rank + rot;
  const int dk_steps = (dk + 31) / 32;
  const int k_stride = dk_steps * 32 + kLmPad;                 // elements
  const int v_tiles = (rank + 15) / 16;
  constexpr int v_stride = kLmKeys + kLmPad;

  const int seq = seq_ids ? seq_ids[blockIdx.y] : blockIdx.y;
  const int q0 = cu_q[seq], qn = cu_q[seq + 1] - q0;
  const int rows = qn * nh;
  const int rb = blockIdx.x * kLmRows;
  if (rb >= rows) return;
  const int ctx = context_lens[seq];
  const int p0 = ctx - qn;                                     // position of the portion's first token
  const int* table = block_table + (size_t)seq * table_stride;
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;

  // this lane's query row (clamped: rows past the end repeat the last one and are not stored)
  const int row = rb + wave * 16 + r;
  const bool row_ok = row < rows;
  const int rowc = row_ok ? row : rows - 1;
  const int tq = rowc / nh, head = rowc % nh;
  const int pos = p0 + tq;
  const int lo_row = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;

  // keys the workgroup walks: up to its last row's position, from its first row's window edge, inside its split
  const int last_row = (rb + kLmRows - 1 < rows ? rb + kLmRows - 1 : rows - 1);
  const int hi_wg = p0 + last_row / nh;
  const int first_pos = p0 + rb / nh;
  int lo_wg = (window > 0 && first_pos - window + 1 > 0) ? first_pos - window + 1 : 0;
  int end_wg = hi_wg + 1;
  if (n_splits > 1) {
    const int s0 = blockIdx.z * split_keys;
    lo_wg = lo_wg > s0 ? lo_wg : s0;
    end_wg = end_wg < s0 + split_keys ? end_wg : s0 + split_keys;
  }
  lo_wg = (lo_wg / kLmKeys) * kLmKeys;                         // blocks stand at multiples of 32 keys

  // queries: B operand, column r = this lane's row, rows 8g..8g+7 of every step of 32 elements
  bf16x8 qf[QS];
  {
    const bf16* qr = q + ((size_t)(q0 + tq) * nh + head) * dk;
#pragma unroll
    for (int s = 0; s < QS; ++s) {
      const int d = 32 * s + 8 * g;
      bf16x8 v = {};
      if (d + 8 <= dk) v = *reinterpret_cast<const bf16x8*>(qr + d);
      qf[s] = v;
    }
  }
  f32x4 o[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float c = scale * kLog2eL;
  const bool wave_active = rb + wave * 16 < rows;              // a wavefront without rows of its own only helps staging

  // Staging goes from memory straight into LDS (no registers in between: with the queries and the output tiles a
  // wavefront holds, staged pieces parked in registers were waited for one by one).  One such load fills 64
  // consecutive 16-byte pieces of LDS, a piece a lane, from 64 addresses of the lanes' own; the two regions are
  // laid out piece by piece: rows of k_pieces (a row's pieces and one of padding), then the transposed copy's rows
  // of five (four runs of 8 keys and one of padding).  Pieces of padding, keys past the range and pages given back
  // are loaded from clamped addresses: what they bring is finite and is masked or multiplied by zero.  Two buffers:
  // the next block's loads are in flight while this block is worked on.
  const int k_pieces = dk_steps * 4 + 1;
  const int k_loads = (kLmKeys * k_pieces + 63) / 64, v_loads = (v_tiles * 16 * 5 + 63) / 64;
  const int buf_elems = (k_loads + v_loads) * 512;             // 64 pieces of 8 elements a load
  const int ch_last = dk / 8 - 1;
  // Where this lane's piece of each load lies does not change from block to block: piece i = 64 * load + lane of
  // the rows is key i / k_pieces, piece i % k_pieces; of the transposed copy element i / 5, run i % 5 of 8 keys (the
  // fifth is padding).  So each load's share of the address is worked out once, before the first block: the offset
  // inside the block's run of 8 keys (24 bits) and which of the block's four runs it is (the bits above).  A block
  // then costs a load a choice among four bases and an addition.  (Pages hold multiples of 8 keys, so a run lies in
  // one page.  Pieces of padding, elements and keys that do not exist take the place of ones that do.)
  constexpr int KS = ((kLmKeys * (QS * 4 + 1) + 63) / 64 + 3) / 4;      // loads of rows a wavefront, at most
  constexpr int VS = ((RT * 16 * 5 + 63) / 64 + 3) / 4;                 // loads of the copy a wavefront, at most
  unsigned kinfo[KS], vinfo[VS];
#pragma unroll
  for (int sl = 0; sl < KS; ++sl) {
    const int i = (wave + 4 * sl) * 64 + lane;
    int key = i / k_pieces, ch = i % k_pieces;
    key = key < kLmKeys ? key : kLmKeys - 1;
    ch = ch < ch_last ? ch : ch_last;
    kinfo[sl] = (unsigned)((key & 7) * dk + 8 * ch) | ((unsigned)(key >> 3) << 24);
  }
#pragma unroll
  for (int sl = 0; sl < VS; ++sl) {
    const int i = (wave + 4 * sl) * 64 + lane;
    int vrow = i / 5, j = i % 5;
    vrow = vrow < rank ? vrow : rank - 1;
    j = j < 4 ? j : 0;
    vinfo[sl] = (unsigned)(vrow * page_size) | ((unsigned)j << 24);
  }
  auto issue_block = [&](int b0, bf16* buf) {
    const int last = end_wg - 1;
    const int rel_last = last - b0;                              // >= 0: the block holds a key of the range
    // where the block's four runs of 8 keys start, in the cache and in the copy (the same for every lane); a run past
    // the range takes the place of the last one inside it
    const bf16* krun[4];
    const bf16* vrun[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int kc = 8 * j <= rel_last ? b0 + 8 * j : (last & ~7);
      const int at = kc / page_size;
      const int page = table[at];
      const size_t pg = page >= 0 ? page : 0, place = kc - at * page_size;
      krun[j] = cache + (pg * page_size + place) * dk;
      vrun[j] = cache_t + pg * rank * page_size + place;
    }
#pragma unroll
    for (int sl = 0; sl < KS; ++sl) {
      const int sI = wave + 4 * sl;
      if (sI < k_loads) {
        const unsigned j = kinfo[sl] >> 24;
        const bf16* base = j == 0 ? krun[0] : (j == 1 ? krun[1] : (j == 2 ? krun[2] : krun[3]));
        load_to_lds_16(base + (kinfo[sl] & 0xffffffu), buf + (size_t)sI * 512);
      }
    }
#pragma unroll
    for (int sl = 0; sl < VS; ++sl) {
      const int sI = wave + 4 * sl;
      if (sI < v_loads) {
        const unsigned j = vinfo[sl] >> 24;
        const bf16* base = j == 0 ? vrun[0] : (j == 1 ? vrun[1] : (j == 2 ? vrun[2] : vrun[3]));
        load_to_lds_16(base + (vinfo[sl] & 0xffffffu), buf + (size_t)(k_loads + sI) * 512);
      }
    }
  };

  const int wave_pos_min = __shfl(pos, 0, kWave);              // the wavefront's rows ascend: its first row sees least,
  const int wave_lo_max = __shfl(lo_row, 15, kWave);           // its last row's window starts last
  bf16* const buf0 = reinterpret_cast<bf16*>(lds_raw);
  if (lo_wg < end_wg) issue_block(lo_wg, buf0);
  int it = 0;
  for (int b0 = lo_wg; b0 < end_wg; b0 += kLmKeys, ++it) {
    bf16* const cur = buf0 + (it & 1) * buf_elems;
    __builtin_amdgcn_s_waitcnt(0);                             // this wavefront's share of the block has landed
    __syncthreads();                                           // ... and everyone's; all are done with the other buffer
    if (b0 + kLmKeys < end_wg) issue_block(b0 + kLmKeys, buf0 + ((it + 1) & 1) * buf_elems);
    if (!wave_active) continue;
    const bf16* k_lds = cur;
    const bf16* v_lds = cur + k_loads * 512;
    // ---- scores of 32 keys for this wavefront's 16 rows ----
    // Operands are read from LDS in batches ahead of the products that use them (a wavefront is alone on its SIMD:
    // a read waited for right before its product costs the LDS's latency every time), and the two tiles' chains of
    // dependent products run interleaved.
    f32x4 s[2];
    s[0] = f32x4{0.f, 0.f, 0.f, 0.f};
    s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    {
      const bf16* kr0 = k_lds + (8 * (r / 4) + (r % 4)) * k_stride + 8 * g;
      const bf16* kr1 = kr0 + 4 * k_stride;
      constexpr int kBatch = 6;
#pragma unroll
      for (int k0 = 0; k0 < QS; k0 += kBatch) {
        bf16x8 ka[kBatch], kb[kBatch];
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          // (offsets known when compiled: a step past the latent's own width reads on into the buffer -- the rows
          // are followed by the transposed copy, so it stays inside -- and is not multiplied)
          const int ks = k0 + j < QS ? k0 + j : QS - 1;
          ka[j] = *reinterpret_cast<const bf16x8*>(kr0 + 32 * ks);
          kb[j] = *reinterpret_cast<const bf16x8*>(kr1 + 32 * ks);
        }
#pragma unroll
        for (int j = 0; j < kBatch; ++j) {
          if (k0 + j < QS && k0 + j < dk_steps) {
            s[0] = mfma16l(ka[j], qf[k0 + j], s[0]);
            s[1] = mfma16l(kb[j], qf[k0 + j], s[1]);
          }
        }
      }
    }
    // ---- mask, running maximum, probabilities ----
    // (a block that every row of the wavefront sees whole, which is most of them, skips the mask)
    float bm = -INFINITY;
    if (b0 + kLmKeys - 1 <= wave_pos_min && b0 >= wave_lo_max && b0 + kLmKeys <= end_wg) {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) bm = fmaxf(bm, s[t][i]);
    } else {
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int kidx = b0 + 8 * g + 4 * t + i;
          const bool ok = kidx <= pos && kidx >= lo_row && kidx < end_wg;
          s[t][i] = ok ? s[t][i] : -INFINITY;
          bm = fmaxf(bm, s[t][i]);
        }
    }
    bm = fmaxf(bm, __shfl_xor(bm, 16, kWave));
    bm = fmaxf(bm, __shfl_xor(bm, 32, kWave));
    // The exponentials are taken against a reference that follows the running maximum lazily: it moves, and the
    // sums are rescaled, only when a score exceeds it by 2^8 (then probabilities stay below 256, which 32-bit sums
    // and bfloat16 operands hold as well as values below 1); after the first blocks that is rare.
    const bool move = m == -INFINITY || (bm - m) * c > 8.f;
    const float m_new = move ? bm : m;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float shift = -m_use * c;
    const float alpha = move ? __builtin_amdgcn_exp2f(fmaf(m, c, shift)) : 1.0f;
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[t][i], c, shift));       // 2^-inf = 0 for masked keys
        psum += p;
        pf[4 * t + i] = (bf16)p;
      }
    l = l * alpha + psum;
    m = m_new;
    // ---- weighted sum: O^T += V^T P^T ----
    // (the sums are rescaled only in blocks where some row's maximum moved: early ones, and rarely later)
    const bool rescale = __any(alpha != 1.0f);
    {
      const bf16* vr = v_lds + r * v_stride + 8 * g;
      constexpr int vBatch = 8;
#pragma unroll
      for (int t0 = 0; t0 < RT; t0 += vBatch) {
        if (t0 < v_tiles) {
          bf16x8 vf[vBatch];
#pragma unroll
          for (int j = 0; j < vBatch; ++j) {
            const int t = t0 + j < RT ? t0 + j : RT - 1;
            vf[j] = *reinterpret_cast<const bf16x8*>(vr + 16 * (t < v_tiles ? t : 0) * v_stride);
          }
#pragma unroll
          for (int j = 0; j < vBatch; ++j) {
            if (t0 + j < RT && t0 + j < v_tiles) {
              if (rescale) o[t0 + j] *= alpha;
              o[t0 + j] = mfma16l(vf[j], pf, o[t0 + j]);
            }
          }
        }
      }
    }
  }

  // ---- the row's sum over its four lanes; then the sink and the division, or the partial for the merge ----
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (!row_ok) return;
  const float mn = m * scale;                                  // the maximum in the exponent's own unit
  if (n_splits > 1) {
    // (splits are for sequences of one token: the partial's row is the sequence's place in the launch and the head)
    float* w = ws + (((size_t)blockIdx.y * nh + head) * n_splits + blockIdx.z) * (rank + 2);
    if (g == 0) {
      w[0] = mn;
      w[1] = l;
    }
#pragma unroll
    for (int t = 0; t < RT; ++t)
      if (t < v_tiles)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int d = 16 * t + 4 * g + i;
          if (d < rank) w[2 + d] = o[t][i];
        }
    return;
  }
  float a = 1.f;
  if (sink) {
    const float sk = sink[head];
    const float top = fmaxf(mn, sk);
    a = expf(mn - top);
    l = l * a + expf(sk - top);
  }
  const float inv = a / l;
  bf16* orow = out + ((size_t)(q0 + tq) * nh + head) * rank;
#pragma unroll
  for (int t = 0; t < RT; ++t)
    if (t < v_tiles) {
      const int d = 16 * t + 4 * g;
      if (d + 4 <= rank) {
        bf16x4 v = {(bf16)(o[t][0] * inv), (bf16)(o[t][1] * inv), (bf16)(o[t][2] * inv), (bf16)(o[t][3] * inv)};
        *reinterpret_cast<bf16x4*>(orow + d) = v;
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if (d + i < rank) orow[d + i] = (bf16)(o[t][i] * inv);
      }
    }
}

// Steps of single tokens: a sequence brings only `heads` rows, one tile of 16 for 16 heads, so staging a block in LDS
// for four wavefronts serves one of them, and a workgroup walking its blocks one after the other is bound by the
// latency of each.  Here a wavefront is a split of its own: it takes 16 heads of one sequence and its own range of
// keys, reads both operands straight from the cache in 16-byte pieces (a row of a key for the scores; eight keys of an
// element from the transposed copy for the weighted sum: what the cache's two layouts are for), batches of loads in
// flight, no LDS and no barrier; four such wavefronts a workgroup keep four blocks of a compute unit's memory
// traffic in flight.  Every wavefront leaves a partial for the merge kernel.
// Grid (sequences, ceil(splits / 4), tiles of 16 heads); split z = 4 blockIdx.y + wavefront.
template <int RT, int QS>
__global__ __launch_bounds__(256) void latent_attn_decode_kernel(
    const bf16* __restrict__ q, const bf16* __restrict__ cache, const bf16* __restrict__ cache_t,
    const int* __restrict__ block_table, int table_stride, const int* __restrict__ seq_ids,
    const int* __restrict__ cu_q, const int* __restrict__ context_lens, float* __restrict__ ws, int nh, int rank, int rot,
    int page_size, int window, float scale, int split_keys, int n_splits) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int g = lane / 16, r = lane % 16;
  const int z = blockIdx.y * 4 + wave;
  if (z >= n_splits) return;
  const int seq = seq_ids ? seq_ids[blockIdx.x] : blockIdx.x;
  const int tok = cu_q[seq];
  const int pos = context_lens[seq] - 1;
  const int dk = rank + rot;
  const int dk_steps = (dk + 31) / 32;
  const int v_tiles = (rank + 15) / 16;
  const int* table = block_table + (size_t)seq * table_stride;
  const int head0 = blockIdx.z * 16;
  const int head = head0 + r < nh ? head0 + r : nh - 1;
  const bool row_ok = head0 + r < nh;
  const int lo_row = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  int lo = z * split_keys, end = lo + split_keys;
  lo = lo > lo_row ? lo : lo_row;
  end = end < pos + 1 ? end : pos + 1;
  const int b_first = (lo / kLmKeys) * kLmKeys;

  bf16x8 qf[QS];
  {
    const bf16* qr = q + ((size_t)tok * nh + head) * dk;
#pragma unroll
    for (int s = 0; s < QS; ++s) {
      const int d = 32 * s + 8 * g;
      bf16x8 v = {};
      if (d + 8 <= dk) v = *reinterpret_cast<const bf16x8*>(qr + d);
      qf[s] = v;
    }
  }
  f32x4 o[RT];
#pragma unroll
  for (int t = 0; t < RT; ++t) o[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  const float c = scale * kLog2eL;
  const int last = end - 1;

  for (int b0 = b_first; b0 < end; b0 += kLmKeys) {
    // this lane's two key rows (tile t: key 8 (r / 4) + 4 t + r % 4) and its run of 8 keys in the copy, clamped into
    // the range (what a clamped key brings is masked)
    const bf16* kr[2];
#pragma unroll
    for (int t = 0; t < 2; ++t) {
      int kidx = b0 + 8 * (r / 4) + 4 * t + (r % 4);
      kidx = kidx < last ? kidx : last;
      const int at = kidx / page_size;
      const int page = table[at];
      kr[t] = cache + ((size_t)(page >= 0 ? page : 0) * page_size + (kidx - at * page_size)) * dk + 8 * g;
    }
    const bf16* vr;
    {
      int kidx = b0 + 8 * g;
      kidx = kidx < (last & ~7) ? kidx : (last & ~7);
      const int at = kidx / page_size;
      const int page = table[at];
      vr = cache_t + ((size_t)(page >= 0 ? page : 0) * rank + r) * page_size + (kidx - at * page_size);
    }
    f32x4 s[2];
    s[0] = f32x4{0.f, 0.f, 0.f, 0.f};
    s[1] = f32x4{0.f, 0.f, 0.f, 0.f};
    constexpr int kBatch = 6;
#pragma unroll
    for (int k0 = 0; k0 < QS; k0 += kBatch) {
      bf16x8 ka[kBatch], kb[kBatch];
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        int ks = k0 + j < QS ? k0 + j : QS - 1;
        ks = ks < dk_steps ? ks : dk_steps - 1;
        const int d = 32 * ks + 8 * g + 8 <= dk ? 32 * ks : dk - 8 - 8 * g;      // (a piece past the row's end: the last one; q is zero there)
        ka[j] = *reinterpret_cast<const bf16x8*>(kr[0] + d);
        kb[j] = *reinterpret_cast<const bf16x8*>(kr[1] + d);
      }
#pragma unroll
      for (int j = 0; j < kBatch; ++j) {
        if (k0 + j < QS && k0 + j < dk_steps) {
          s[0] = mfma16l(ka[j], qf[k0 + j], s[0]);
          s[1] = mfma16l(kb[j], qf[k0 + j], s[1]);
        }
      }
    }
    float bm = -INFINITY;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int kidx = b0 + 8 * g + 4 * t + i;
        const bool ok = kidx >= lo && kidx < end;
        s[t][i] = ok ? s[t][i] : -INFINITY;
        bm = fmaxf(bm, s[t][i]);
      }
    bm = fmaxf(bm, __shfl_xor(bm, 16, kWave));
    bm = fmaxf(bm, __shfl_xor(bm, 32, kWave));
    const bool move = m == -INFINITY || (bm - m) * c > 8.f;
    const float m_new = move ? bm : m;
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float shift = -m_use * c;
    const float alpha = move ? __builtin_amdgcn_exp2f(fmaf(m, c, shift)) : 1.0f;
    float psum = 0.f;
    bf16x8 pf;
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(fmaf(s[t][i], c, shift));
        psum += p;
        pf[4 * t + i] = (bf16)p;
      }
    l = l * alpha + psum;
    m = m_new;
    const bool rescale = __any(alpha != 1.0f);
    constexpr int vBatch = 8;
#pragma unroll
    for (int t0 = 0; t0 < RT; t0 += vBatch) {
      if (t0 < v_tiles) {
        bf16x8 vf[vBatch];
#pragma unroll
        for (int j = 0; j < vBatch; ++j) {
          int e = 16 * (t0 + j) + r;                           // this lane's element of tile t0 + j, clamped into the latent
          e = e < rank ? e : rank - 1;
          vf[j] = *reinterpret_cast<const bf16x8*>(vr + (size_t)(e - r) * page_size);
        }
#pragma unroll
        for (int j = 0; j < vBatch; ++j) {
          if (t0 + j < RT && t0 + j < v_tiles) {
            if (rescale) o[t0 + j] *= alpha;
            o[t0 + j] = mfma16l(vf[j], pf, o[t0 + j]);
          }
        }
      }
    }
  }
  l += __shfl_xor(l, 16, kWave);
  l += __shfl_xor(l, 32, kWave);
  if (!row_ok) return;
  float* w = ws + (((size_t)blockIdx.x * nh + head) * n_splits + z) * (rank + 2);
  if (g == 0) {
    w[0] = m * scale;
    w[1] = l;
  }
#pragma unroll
  for (int t = 0; t < RT; ++t)
    if (t < v_tiles)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = 16 * t + 4 * g + i;
        if (d < rank) w[2 + d] = o[t][i];
      }
}

// out[row] = sum over the splits' partials, each scaled by exp(its maximum - the largest), then the sink.
// One workgroup a row; the splits' factors are worked out once (in LDS), then every thread adds its elements over
// the splits in order, eight loads in flight.
constexpr int kMergeMaxSplits = 4096;
__global__ __launch_bounds__(256) void latent_attn_merge_kernel(const float* __restrict__ ws, const float* __restrict__ sink,
                                                               const int* __restrict__ seq_ids, const int* __restrict__ cu_q,
                                                               bf16* __restrict__ out, int nh, int rank, int n_splits) {
  __shared__ float factor[kMergeMaxSplits];
  __shared__ float scratch[16];
  const int row = blockIdx.x;                                  // (place in the launch) * heads + head
  const int seq = seq_ids ? seq_ids[row / nh] : row / nh;
  const size_t out_row = (size_t)cu_q[seq] * nh + row % nh;
  const size_t stride = (size_t)rank + 2;
  const float* w = ws + (size_t)row * n_splits * stride;
  float top = -INFINITY;
  for (int z = threadIdx.x; z < n_splits; z += blockDim.x) top = fmaxf(top, w[z * stride]);
  top = wave_max(top);
  {
    const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
    if (lane == 0) scratch[wave] = top;
    __syncthreads();
    for (int i = 0; i < (int)(blockDim.x / kWave); ++i) top = fmaxf(top, scratch[i]);
    __syncthreads();
  }
  const float sk = sink ? sink[row % nh] : -INFINITY;
  top = fmaxf(top, sk);
  float lpart = 0.f;
  for (int z = threadIdx.x; z < n_splits; z += blockDim.x) {
    const float mz = w[z * stride];
    const float f = mz == -INFINITY ? 0.f : expf(mz - top);
    factor[z] = f;
    lpart += f * w[z * stride + 1];
  }
  float l = block_sum(lpart, scratch);                         // (its barriers also publish the factors)
  if (sink) l += expf(sk - top);
  const float inv = 1.f / l;
  for (int d = threadIdx.x; d < rank; d += blockDim.x) {
    float acc = 0.f;
    int z = 0;
    for (; z + 8 <= n_splits; z += 8) {
      float v[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) v[j] = w[(z + j) * stride + 2 + d];
#pragma unroll
      for (int j = 0; j < 8; ++j) acc += v[j] * factor[z + j];
    }
    for (; z < n_splits; ++z) acc += w[z * stride + 2 + d] * factor[z];
    out[out_row * rank + d] = (bf16)(acc * inv);
  }
}

template <int RT, int QS>
static int launch_latent_mfma(hipStream_t st, dim3 grid, size_t lds, const bf16* q, const bf16* cache, const bf16* cache_t, const float* sink,
                              const int* block_table, int table_stride, const int* seq_ids, const int* cu_q,
                              const int* context_lens, bf16* out, float* ws, int nh, int rank, int rot, int page_size,
                              int window, float scale, int split_keys, int n_splits) {
  static bool raised = false;
  if (!raised) {
    hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&latent_attn_mfma_kernel<RT, QS>),
                                       hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024);
    if (e != hipSuccess) return pa::fail("latent_attn_mfma: cannot raise the LDS limit: %s", hipGetErrorString(e));
    raised = true;
  }
  hipLaunchKernelGGL((latent_attn_mfma_kernel<RT, QS>), grid, dim3(256), lds, st, q, cache, cache_t, sink, block_table, table_stride,
                     seq_ids, cu_q, context_lens, out, ws, nh, rank, rot, page_size, window, scale, split_keys, n_splits);
  return 0;
}

static size_t latent_mfma_lds(int rank, int rot) {
  const int dk_steps = (rank + rot + 31) / 32, v_tiles = (rank + 15) / 16;
  const int k_loads = (kLmKeys * (dk_steps * 4 + 1) + 63) / 64, v_loads = (v_tiles * 16 * 5 + 63) / 64;
  return (size_t)2 * (k_loads + v_loads) * 1024;               // two buffers of whole 64-piece loads
}

}  // namespace pa

using namespace pa;

// Sizes the matrix-core kernel takes: 16-byte rows, at most 512 + 64 elements, pages of a multiple of 8 keys.
extern "C" int pa_latent_attn_mfma_supports(int rank, int rot, int page_size) {
  return rank > 0 && rot >= 0 && rank % 8 == 0 && rot % 8 == 0 && rank <= 512 && rot <= 64 && page_size > 0 && page_size % 8 == 0 &&
         page_size <= 16384 &&   // (an element's offset in the transposed copy, rank * page_size, is kept in 24 bits)
         latent_mfma_lds(rank, rot) <= 160 * 1024;
}

// 32-bit words of workspace for `n_seqs` sequences of one token in `n_splits` splits
extern "C" long pa_latent_attn_mfma_workspace(int n_seqs, int nh, int rank, int n_splits) {
  return n_splits > 1 ? (long)n_seqs * nh * n_splits * (rank + 2) : 0;
}

// q [tokens, heads, rank + rot], cache [pages, page, rank + rot] and its latents transposed, cache_t [pages, rank, page]
// -> out [tokens, heads, rank] for the sequences seq_ids[0..n_seqs) (null: sequences
// 0..n_seqs), each with cu_q[s+1] - cu_q[s] tokens ending at context_lens[s]; max_q_len bounds their tokens.
// n_splits > 1 (sequences of one token only): the keys in splits of split_keys, partials in ws, merged here; a split is
// a workgroup of the staged kernel, or with `wave_splits` a wavefront of the kernel that reads the cache directly.
extern "C" int pa_latent_attn_mfma(void* stream, const void* q, const void* cache, const void* cache_t, const float* sink, const int* block_table,
                                   int table_stride, const int* seq_ids, const int* cu_q, const int* context_lens, void* out,
                                   void* ws, int n_seqs, int max_q_len, int nh, int rank, int rot, int page_size,
                                   int window, float scale, int split_keys, int n_splits, int wave_splits) {
  if (n_seqs == 0) return 0;
  PA_REQUIRE(pa_latent_attn_mfma_supports(rank, rot, page_size), "latent_attn_mfma: a latent of %d + %d is not a size it takes", rank, rot);
  PA_REQUIRE(n_seqs > 0 && max_q_len > 0 && nh > 0 && table_stride > 0 && window >= 0,
             "latent_attn_mfma: bad sizes seqs=%d q=%d heads=%d stride=%d window=%d", n_seqs, max_q_len, nh, table_stride, window);
  PA_REQUIRE(cache && cache_t, "latent_attn_mfma: needs the cache and its transposed copy");
  PA_REQUIRE(scale > 0.f, "latent_attn_mfma: a scale of %g is not positive", (double)scale);
  PA_REQUIRE(n_splits <= kMergeMaxSplits, "latent_attn_mfma: %d splits are more than the %d the merge takes", n_splits, kMergeMaxSplits);
  PA_REQUIRE(n_splits >= 1 && (n_splits == 1 || (split_keys > 0 && split_keys % kLmKeys == 0 && ws && max_q_len == 1)),
             "latent_attn_mfma: %d splits of %d keys need a workspace, whole blocks and sequences of one token", n_splits, split_keys);
  hipStream_t st = (hipStream_t)stream;
  if (n_splits > 1 && wave_splits) {
    // sequences of one token, many of them: a wavefront a split, operands straight from the cache, then the merge
    const int head_tiles = (nh + 15) / 16;
    PA_REQUIRE(n_seqs <= 0x7fffffff && head_tiles <= 65535, "latent_attn_mfma: %d sequences or %d heads exceed the grid", n_seqs, nh);
    dim3 grid(n_seqs, (n_splits + 3) / 4, head_tiles);
#define PA_LD(RT, QS)                                                                                                    \
  hipLaunchKernelGGL((latent_attn_decode_kernel<RT, QS>), grid, dim3(256), 0, st, (const bf16*)q, (const bf16*)cache,     \
                     (const bf16*)cache_t, block_table, table_stride, seq_ids, cu_q, context_lens, (float*)ws, nh, rank, rot, \
                     page_size, window, scale, split_keys, n_splits)
    if (rank <= 64) PA_LD(4, 4);
    else if (rank <= 128) PA_LD(8, 6);
    else if (rank <= 256) PA_LD(16, 10);
    else PA_LD(32, 18);
#undef PA_LD
    if (int e = check_launch("latent_attn_decode")) return e;
    hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(n_seqs * nh), dim3(rank >= 256 ? 256 : 64), 0, st, (const float*)ws, sink,
                       seq_ids, cu_q, (bf16*)out, nh, rank, n_splits);
    return check_launch("latent_attn_merge");
  }
  const long tiles = ((long)max_q_len * nh + kLmRows - 1) / kLmRows;
  PA_REQUIRE(tiles <= 0x7fffffffL && n_seqs <= 65535 && n_splits <= 65535, "latent_attn_mfma: the grid %ld x %d x %d is too large", tiles,
             n_seqs, n_splits);
  dim3 grid((unsigned)tiles, n_seqs, n_splits);
  const size_t lds = latent_mfma_lds(rank, rot);
  int rc;
#define PA_LM(RT, QS)                                                                                                  \
  rc = launch_latent_mfma<RT, QS>(st, grid, lds, (const bf16*)q, (const bf16*)cache, (const bf16*)cache_t, sink, block_table, table_stride,  \
                                  seq_ids, cu_q, context_lens, (bf16*)out, (float*)ws, nh, rank, rot, page_size, window, \
                                  scale, split_keys, n_splits)
  if (rank <= 64) PA_LM(4, 4);
  else if (rank <= 128) PA_LM(8, 6);
  else if (rank <= 256) PA_LM(16, 10);
  else PA_LM(32, 18);
#undef PA_LM
  if (rc) return rc;
  if (int e = check_launch("latent_attn_mfma")) return e;
  if (n_splits > 1) {
    hipLaunchKernelGGL(latent_attn_merge_kernel, dim3(n_seqs * nh), dim3(rank >= 256 ? 256 : 64), 0, st, (const float*)ws, sink,
                       seq_ids, cu_q, (bf16*)out, nh, rank, n_splits);
    return check_launch("latent_attn_merge");
  }
  return 0;
}
