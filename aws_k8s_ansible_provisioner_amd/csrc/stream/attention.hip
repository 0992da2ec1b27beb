// Paged attention with a lower-bounded causal mask (chunks and / or a sliding window), a
// per-head sink logit in the softmax denominator and a per-head sigmoid output gate, over a
// K cache [NB, G, BS, D] and a V cache [NB, G, BS/8, D, 8] of bf16 or fp32.
//
// Scores, the running softmax and the gate are fp32.  A query at position i sees the keys
// [lo(i), i] with lo(i) = max(floor(i / chunk) * chunk, i - window + 1, 0): only that range is
// read, so a chunked layer costs O(chunk) per token however long the sequence.
//
// row kernel (any D <= 256, bf16 / fp32): one wave per (token, head).  Keys go in 64-aligned
//   pieces: each lane scores one key (q broadcast from LDS, 16-byte K loads), the wave takes
//   the piece's max and sum, and lanes then own output dimensions for the P.V update, reading
//   V one 8-key group (16 bytes) at a time.  Decode rows cut [lo, i] into partitions that a
//   second launch merges together with the sink and the gate; prefill tiles give a
//   workgroup's four waves the tokens of one tile (fp32 models, head sizes the matrix kernel
//   does not take).
// matrix kernels (bf16, D in {32, 64, 128, 256}): v_mfma_f32_32x32x16_bf16 for S^T = K Q^T and
//   O^T = V^T P^T.  Prefill: one wave per 64 queries of a head (two 32-column tiles share every
//   K / V fragment load).  Decode: the columns of a tile are the query heads of one K/V head,
//   so a GQA group reads its keys and values once; the key range is split over workgroups.  With keys as the MFMA rows,
//   a query is a lane column: its softmax statistics are 16 registers and one cross-half
//   exchange, never an LDS pass.  The A rows of the K fragment are loaded in the order that
//   makes the S^T accumulator registers of a lane exactly the 8 keys of a V group, so P goes
//   from accumulator to B operand without any lane movement, and the V^T operand is one
//   16-byte load from the grouped V cache.  K / V fragments come straight from global memory
//   (L1 / L2 hits across the workgroup's four waves and the heads of a GQA group).
#include <cstdlib>

#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::wave_max;
using akap::wave_sum;

constexpr int kMaxDV = 4;  // output dimensions per lane: D <= 256

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)*p; }

struct Softmax {
  float m, l;
  float acc[kMaxDV];
};

// 8 consecutive values of one (group, dim) of the V cache, as floats
__device__ __forceinline__ void ld_group(float (&v)[8], const bf16* p) {
  const akap::bf16x8 x = *reinterpret_cast<const akap::bf16x8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (float)x[e];
}
__device__ __forceinline__ void ld_group(float (&v)[8], const float* p) {
  const akap::f32x4 a = *reinterpret_cast<const akap::f32x4*>(p);
  const akap::f32x4 b = *reinterpret_cast<const akap::f32x4*>(p + 4);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    v[e] = a[e];
    v[4 + e] = b[e];
  }
}

// q . k over D dims; 16-byte loads when the row allows (D % 8 == 0: rows are 16-byte aligned)
__device__ __forceinline__ float dot_row(const float* qs, const bf16* kr, int D) {
  float dot = 0.f;
  int d = 0;
  if ((D & 7) == 0) {
    for (; d < D; d += 8) {
      const akap::bf16x8 x = *reinterpret_cast<const akap::bf16x8*>(kr + d);
#pragma unroll
      for (int e = 0; e < 8; ++e) dot += qs[d + e] * (float)x[e];
    }
    return dot;
  }
  for (; d < D; ++d) dot += qs[d] * (float)kr[d];
  return dot;
}
__device__ __forceinline__ float dot_row(const float* qs, const float* kr, int D) {
  float dot = 0.f;
  int d = 0;
  if ((D & 3) == 0) {
    for (; d < D; d += 4) {
      const akap::f32x4 x = *reinterpret_cast<const akap::f32x4*>(kr + d);
#pragma unroll
      for (int e = 0; e < 4; ++e) dot += qs[d + e] * x[e];
    }
    return dot;
  }
  for (; d < D; ++d) dot += qs[d] * kr[d];
  return dot;
}

// Keys [lo, j1) of one sequence against one query held in `qs` (LDS, D floats, pre-scaled),
// in pieces aligned to 64 keys (so a piece is 8 whole V groups).  `ps`: 64 floats of LDS owned
// by this wave.  Every key below j1 is a cached position of the sequence (its block exists).
template <typename T>
__device__ __forceinline__ void attend_range(Softmax& st, const float* qs, float* ps,
                                             const T* __restrict__ kc, const T* __restrict__ vc,
                                             const int32_t* __restrict__ bt, int max_blocks, int NB,
                                             int G, int g, int BS, int D, int lo, int j1) {
  const int lane = threadIdx.x & 63;
  const int NG = BS >> 3;
  for (int base = lo & ~63; base < j1; base += 64) {
    const int j = base + lane;
    const bool ok = j >= lo && j < j1;
    int grow = 0;  // this lane's key's row in the [NB * G * BS/8] group view of the V cache
    float s = -INFINITY;
    if (j < j1) {
      const int bi = j / BS;
      int blk = bi < max_blocks ? bt[bi] : 0;
      if (blk < 0 || blk >= NB) blk = 0;
      const int off = j - bi * BS;
      grow = (blk * G + g) * NG + (off >> 3);
      if (ok) s = dot_row(qs, kc + ((size_t)(blk * G + g) * BS + off) * D, D);
    }
    const float mt = wave_max(s);
    const float mn = fmaxf(st.m, mt);  // finite: a piece always holds a visible key
    const float corr = expf(st.m - mn);  // first piece: exp(-inf) = 0
    const float pj = ok ? expf(s - mn) : 0.f;
    st.l = st.l * corr + wave_sum(pj);
    st.m = mn;
    ps[lane] = pj;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < kMaxDV; ++c) st.acc[c] *= corr;
    for (int gi = 0; gi < 8; ++gi) {
      const int gb = base + gi * 8;
      if (gb >= j1 || gb + 8 <= lo) continue;  // (wave-uniform) nothing visible in this group
      const int gr = __shfl(grow, gi * 8, 64);
      float pv[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) pv[e] = ps[gi * 8 + e];
#pragma unroll
      for (int c = 0; c < kMaxDV; ++c) {
        const int d = c * 64 + lane;
        if (d < D) {
          float v[8];
          ld_group(v, vc + ((size_t)gr * D + d) * 8);
#pragma unroll
          for (int e = 0; e < 8; ++e) st.acc[c] += pv[e] * v[e];
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
}

__device__ __forceinline__ int lower_bound_of(int pos, int chunk, int window) {
  int lo = 0;
  if (chunk > 0) lo = (pos / chunk) * chunk;
  if (window > 0) lo = max(lo, pos - window + 1);
  return lo;
}

template <typename T>
__device__ __forceinline__ void load_q(float* qs, const T* q, int D, float scale) {
  const int lane = threadIdx.x & 63;
  for (int d = lane; d < D; d += 64) qs[d] = ldf(q + d) * scale;
  __builtin_amdgcn_wave_barrier();
}

// sink into the denominator, normalise, gate, store
template <typename T>
__device__ __forceinline__ void finish_row(const Softmax& st, const AttnParams& p, int t, int h) {
  const int lane = threadIdx.x & 63;
  float m = st.m, l = st.l, corr = 1.f;
  if (p.sink) {
    const float sk = p.sink[h];
    m = fmaxf(st.m, sk);
    corr = expf(st.m - m);
    l = l * corr + expf(sk - m);
  }
  float gate = 1.f;
  if (p.gate) {
    const float z = ldf((const T*)p.gate + (size_t)t * p.gate_stride + h);
    gate = 1.0f / (1.0f + expf(-z));
  }
  const float f = l > 0.f ? corr * gate / l : 0.f;
  T* o = (T*)p.out + (size_t)t * p.out_stride + h * p.D;
#pragma unroll
  for (int c = 0; c < kMaxDV; ++c) {
    const int d = c * 64 + lane;
    if (d < p.D) o[d] = (T)(st.acc[c] * f);
  }
}

// grid (tiles x H, flat); 4 waves share a tile's tokens
template <typename T>
__global__ __launch_bounds__(256) void sink_attn_prefill_rows_kernel(AttnParams p) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6;
  float* qs = smem + wave * (p.D + 64);
  float* ps = qs + p.D;
  // flat grid, walked from the END of the tile map: the scheduler sorts tiles by ascending
  // causal work, so the longest tiles start first and the shortest fill the tail; the heads of
  // a tile (and of a GQA group) are neighbours and share its K / V in L2
  const int tile = p.num_tiles - 1 - (int)(blockIdx.x / p.H), h = (int)(blockIdx.x % p.H);
  const int b = p.tile_seq[tile];
  if (b < 0 || b >= p.B) return;
  const int r0 = p.tile_row[tile];
  const int qs0 = p.q_start[b];
  const int qlen = p.q_start[b + 1] - qs0;
  const int kv = p.seq_lens[b];
  const int g = h / (p.H / p.G);
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  const int rend = min(r0 + p.tile_rows, qlen);
  for (int r = r0 + wave; r < rend; r += 4) {
    const int t = qs0 + r;
    const int pos = kv - qlen + r;
    if (pos < 0) continue;
    load_q(qs, (const T*)p.q + ((size_t)t * p.H + h) * p.D, p.D, p.scale);
    Softmax st;
    st.m = -INFINITY;
    st.l = 0.f;
#pragma unroll
    for (int c = 0; c < kMaxDV; ++c) st.acc[c] = 0.f;
    attend_range<T>(st, qs, ps, (const T*)p.k_cache, (const T*)p.v_cache, bt, p.max_blocks, p.NB,
                    p.G, g, p.BS, p.D, lower_bound_of(pos, p.chunk, p.window), pos + 1);
    finish_row<T>(st, p, t, h);
  }
}

// grid (B, H, parts); one wave each
template <typename T>
__global__ __launch_bounds__(64) void sink_attn_decode_rows_kernel(AttnParams p) {
  extern __shared__ float smem[];
  float* qs = smem;
  float* ps = qs + p.D;
  const int b = blockIdx.x, h = blockIdx.y, part = blockIdx.z;
  const int lane = threadIdx.x;
  const int kv = p.seq_lens[b];
  if (kv <= 0) {  // padding row of a bucketed batch: defined output, no cache reads
    if (part == 0) {
      T* o = (T*)p.out + (size_t)b * p.out_stride + h * p.D;
      for (int d = lane; d < p.D; d += 64) o[d] = (T)0.f;
    }
    return;
  }
  const int pos = kv - 1;
  const int lo = lower_bound_of(pos, p.chunk, p.window);
  // partitions are whole 64-aligned pieces of [lo & ~63, pos]
  const int a0 = lo & ~63;
  int per = (pos + 1 - a0 + p.num_parts - 1) / p.num_parts;
  per = (per + 63) & ~63;
  const int j0 = max(lo, a0 + part * per);
  const int j1 = min(pos + 1, a0 + (part + 1) * per);
  const int g = h / (p.H / p.G);
  Softmax st;
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int c = 0; c < kMaxDV; ++c) st.acc[c] = 0.f;
  if (j0 < j1) {
    load_q(qs, (const T*)p.q + ((size_t)b * p.H + h) * p.D, p.D, p.scale);
    attend_range<T>(st, qs, ps, (const T*)p.k_cache, (const T*)p.v_cache,
                    p.block_tables + (size_t)b * p.max_blocks, p.max_blocks, p.NB, p.G, g, p.BS,
                    p.D, j0, j1);
  }
  if (p.num_parts == 1) {
    finish_row<T>(st, p, b, h);
    return;
  }
  const size_t slot = ((size_t)b * p.H + h) * p.num_parts + part;
  if (lane == 0) {
    p.ws_ml[slot * 2] = st.m;
    p.ws_ml[slot * 2 + 1] = st.l;
  }
#pragma unroll
  for (int c = 0; c < kMaxDV; ++c) {
    const int d = c * 64 + lane;
    if (d < p.D) p.ws_o[slot * p.D + d] = st.acc[c];
  }
}

// grid (B, H): merge the partitions' states, then sink, gate and store
template <typename T>
__global__ __launch_bounds__(64) void sink_attn_decode_merge_kernel(AttnParams p) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int lane = threadIdx.x;
  if (p.seq_lens[b] <= 0) return;  // the partition kernel zeroed the row
  const size_t base = ((size_t)b * p.H + h) * p.num_parts;
  float m = -INFINITY;
  for (int i = 0; i < p.num_parts; ++i) m = fmaxf(m, p.ws_ml[(base + i) * 2]);
  Softmax st;
  st.m = m;
  st.l = 0.f;
#pragma unroll
  for (int c = 0; c < kMaxDV; ++c) st.acc[c] = 0.f;
  for (int i = 0; i < p.num_parts; ++i) {
    const float mi = p.ws_ml[(base + i) * 2];
    const float li = p.ws_ml[(base + i) * 2 + 1];
    if (li <= 0.f) continue;  // an empty partition
    const float w = expf(mi - m);
    st.l += li * w;
#pragma unroll
    for (int c = 0; c < kMaxDV; ++c) {
      const int d = c * 64 + lane;
      if (d < p.D) st.acc[c] += p.ws_o[(base + i) * p.D + d] * w;
    }
  }
  finish_row<T>(st, p, b, h);
}

// swap bits 2 and 3: the A-row order of the K fragment (see the file comment)
__device__ __forceinline__ int swap23(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

// Running state of NQ tiles of 32 query columns (one column per lane & 31, both lane halves):
// O^T accumulators [D / 32 blocks][16 registers], softmax max and sum per column.
template <int DB, int NQ>
struct MfmaState {
  akap::f32x16 o[NQ][DB];
  float m[NQ], l[NQ];
};

// Softmax update of one 32-key block: masks (unless the block is visible to every column),
// moves the running max and sum (log2 domain), turns the scores of the NQ tiles into bf16 P
// operands and rescales the output accumulators if a maximum moved.
template <int DB, int NQ>
__device__ __forceinline__ void mfma_softmax(MfmaState<DB, NQ>& st, akap::f32x16 (&s)[NQ],
                                             akap::bf16x8 (&pb)[NQ][2], int j0,
                                             const int (&pos)[NQ], const int (&my_lo)[NQ],
                                             int pos_min, int lo_max, float sc2) {
  const int hf = (threadIdx.x & 63) >> 5;
  float alpha[NQ];
  // a block below every column's position and above every column's lower bound needs no
  // mask (all but the first and last blocks of a wave's range)
  const bool full = j0 + 31 <= pos_min && j0 >= lo_max;
  bool rescale = false;
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    // accumulator register i of this lane: key j0 + 16 (i >> 3) + 8 hf + (i & 7), column col
    float sv[16];
    float bmax = -INFINITY;
    if (full) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        sv[i] = s[q][i];
        bmax = fmaxf(bmax, sv[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = j0 + 16 * (i >> 3) + 8 * hf + (i & 7);
        const bool vis = key <= pos[q] && key >= my_lo[q];
        sv[i] = vis ? s[q][i] : -INFINITY;
        bmax = fmaxf(bmax, sv[i]);
      }
    }
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    // running max and exponentials in the log2 domain of the scaled scores (sc2 > 0)
    const float mn = fmaxf(st.m[q], bmax * sc2);
    const float ms = mn == -INFINITY ? 0.f : mn;  // nothing visible yet: every exp below is 0
    alpha[q] = __builtin_amdgcn_exp2f(st.m[q] - ms);
    rescale |= alpha[q] != 1.0f;
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sv[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], sc2, -ms));
      psum += sv[i];
    }
    psum += __shfl_xor(psum, 32, 64);
    st.l[q] = st.l[q] * alpha[q] + psum;
    st.m[q] = mn;
#pragma unroll
    for (int i = 0; i < 16; ++i) pb[q][i >> 3][i & 7] = (bf16)sv[i];
  }
  if (__any(rescale)) {  // (wave-uniform) the maxima settle after the first blocks
#pragma unroll
    for (int dt = 0; dt < DB; ++dt)
#pragma unroll
      for (int q = 0; q < NQ; ++q)
#pragma unroll
        for (int i = 0; i < 16; ++i) st.o[q][dt][i] *= alpha[q];
  }
}

// Keys [jb, je] (jb a multiple of 32) against the wave's query columns.  qf: the columns' Q
// fragments (B operands); pos / my_lo: each lane's query position and lowest visible key per
// tile; pos_min / lo_max: the smallest position and the largest lower bound among the wave's
// columns (an unused column computes like a used one and is never stored).  m is kept in log2
// units of the scaled scores.  Each K and V fragment is loaded once, straight from the cache,
// and feeds the MFMAs of all NQ tiles.
template <int DB, int NQ>
__device__ __forceinline__ void mfma_attend(MfmaState<DB, NQ>& st, const AttnParams& p,
                                            const int32_t* __restrict__ bt, int g,
                                            const akap::bf16x8 (&qf)[NQ][2 * DB],
                                            const int (&pos)[NQ], const int (&my_lo)[NQ], int jb,
                                            int je, int pos_min, int lo_max) {
  constexpr int D = 32 * DB, KS = 2 * DB;
  const float sc2 = p.scale * 1.44269504088896f;  // scores -> log2 units
  using akap::bf16x8;
  using akap::f32x16;
  const int lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int NG = p.BS >> 3;
  const int krow = swap23(col);
  // The next block's K fragments are requested before this block's softmax, and this block's
  // V fragments before its Q K^T MFMAs: a wave keeps its own loads in flight under its own
  // matrix and VALU work (the accumulators leave room for one or two waves per SIMD only).
  auto block_of = [&](int j0) {
    const int bi = j0 / p.BS;
    int blk = bi < p.max_blocks ? bt[bi] : 0;
    if (blk < 0 || blk >= p.NB) blk = 0;
    return (blk * p.G + g) * p.BS + (j0 - bi * p.BS);  // row of key j0 in the [.., D] K view
  };
  bf16x8 kf[KS];
  int row0 = block_of(jb);
  // one column tile per wave: the block-table entry of the block after next is requested a
  // whole iteration before the K loads that need it (no K load waits on a table load; 715 ->
  // 591 us at 8 x 2048 causal, D = 128).  With two tiles the extra live state costs the last
  // free registers (534 -> 697 us), so there the entry is looked up when it is needed.
  constexpr bool kTableAhead = NQ == 1;
  int row1 = kTableAhead && jb + 32 <= je ? block_of(jb + 32) : 0;
  {
    const bf16* kp = (const bf16*)p.k_cache + ((size_t)row0 + krow) * D + 8 * hf;
#pragma unroll
    for (int c = 0; c < KS; ++c) kf[c] = *reinterpret_cast<const bf16x8*>(kp + 16 * c);
  }
  for (int j0 = jb; j0 <= je; j0 += 32) {
    // V groups of this block: row0 is a multiple of 8 keys (blocks and j0 are multiples of 32)
    const bf16* vp = (const bf16*)p.v_cache + (((size_t)(row0 >> 3) + hf) * D + col) * 8;
    bf16x8 vf[DB][2];
#pragma unroll
    for (int dt = 0; dt < DB; ++dt)
#pragma unroll
      for (int sl = 0; sl < 2; ++sl)
        vf[dt][sl] = *reinterpret_cast<const bf16x8*>(vp + ((size_t)(2 * sl) * D + 32 * dt) * 8);
    f32x16 s[NQ];
#pragma unroll
    for (int q = 0; q < NQ; ++q) {
#pragma unroll
      for (int i = 0; i < 16; ++i) s[q][i] = 0.f;
#pragma unroll
      for (int c = 0; c < KS; ++c)
        s[q] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf[c], qf[q][c], s[q], 0, 0, 0);
    }
    if (j0 + 32 <= je) {
      row0 = kTableAhead ? row1 : block_of(j0 + 32);
      const bf16* kp = (const bf16*)p.k_cache + ((size_t)row0 + krow) * D + 8 * hf;
#pragma unroll
      for (int c = 0; c < KS; ++c) kf[c] = *reinterpret_cast<const bf16x8*>(kp + 16 * c);
      if (kTableAhead && j0 + 64 <= je) row1 = block_of(j0 + 64);
    }
    bf16x8 pb[NQ][2];
    mfma_softmax<DB, NQ>(st, s, pb, j0, pos, my_lo, pos_min, lo_max, sc2);
#pragma unroll
    for (int dt = 0; dt < DB; ++dt)
#pragma unroll
      for (int sl = 0; sl < 2; ++sl)
#pragma unroll
        for (int q = 0; q < NQ; ++q)
          st.o[q][dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf[dt][sl], pb[q][sl], st.o[q][dt],
                                                                0, 0, 0);
  }
}

template <int DB, int NQ>
__device__ __forceinline__ void mfma_init(MfmaState<DB, NQ>& st) {
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    st.m[q] = -INFINITY;
    st.l[q] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DB; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i) st.o[q][dt][i] = 0.f;
  }
}

// sink, normalise, gate and store column tile q of a lane (token row t, head h).
// Accumulator register i of o[dt]: dimension 32 dt + 8 (i >> 2) + 4 hf + (i & 3).
template <int DB, int NQ>
__device__ __forceinline__ void mfma_finish(const MfmaState<DB, NQ>& st, int q,
                                            const AttnParams& p, int t, int h) {
  constexpr int D = 32 * DB;
  const int hf = (threadIdx.x & 63) >> 5;
  float l = st.l[q], corr = 1.f;
  if (p.sink) {
    const float sk = p.sink[h];
    const float mq = st.m[q] * 0.693147180559945f;  // back from log2 units
    const float mf = fmaxf(mq, sk);
    corr = expf(mq - mf);
    l = l * corr + expf(sk - mf);
  }
  float gate = 1.f;
  if (p.gate) {
    const float z = (float)((const bf16*)p.gate)[(size_t)t * p.gate_stride + h];
    gate = 1.0f / (1.0f + expf(-z));
  }
  const float f = l > 0.f ? corr * gate / l : 0.f;
  bf16* o = (bf16*)p.out + (size_t)t * p.out_stride + h * D;
#pragma unroll
  for (int dt = 0; dt < DB; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      o[32 * dt + 8 * (i >> 2) + 4 * hf + (i & 3)] = (bf16)(st.o[q][dt][i] * f);
}

// Prefill: grid (tiles of 128 or 256 tokens x H, flat), tile / (32 NQ) waves of NQ column tiles each.
template <int DB, int NQ>
__global__ __launch_bounds__(512 / NQ) void sink_attn_prefill_mfma_kernel(AttnParams p) {
  constexpr int D = 32 * DB, KS = 2 * DB;
  using akap::bf16x8;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  // Flat grid.  Work units are (tile, K/V head) pairs, taken from the END of the tile map: the
  // scheduler sorts tiles by ascending causal work, so the longest start first and the
  // shortest fill the tail.  The hardware deals workgroup i to XCD i % 8: units are dealt
  // round-robin over the XCDs in that order (balanced), and the query heads of one unit are
  // consecutive workgroups of ONE XCD, so a GQA group's K / V crosses into a single L2.
  const int rep = p.H / p.G;
  const int xcd = blockIdx.x & 7, jx = blockIdx.x >> 3;
  const int unit = (jx / rep) * 8 + xcd;
  if (unit >= p.num_tiles * p.G) return;
  const int tile = p.num_tiles - 1 - unit / p.G;
  const int h = (unit % p.G) * rep + jx % rep;
  const int b = p.tile_seq[tile];
  if (b < 0 || b >= p.B) return;
  const int qs0 = p.q_start[b];
  const int qlen = p.q_start[b + 1] - qs0;
  const int kv = p.seq_lens[b];
  const int rend = min(p.tile_row[tile] + p.tile_rows, qlen);
  const int r0 = p.tile_row[tile] + wave * 32 * NQ;
  if (r0 >= rend || kv < qlen) return;
  const int g = h / (p.H / p.G);
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  int pos[NQ], my_lo[NQ], t[NQ];
  bool valid[NQ];
  bf16x8 qf[NQ][KS];
#pragma unroll
  for (int q = 0; q < NQ; ++q) {
    const int r = r0 + 32 * q + col;
    valid[q] = r < rend;
    t[q] = qs0 + (valid[q] ? r : r0);
    pos[q] = kv - qlen + r;
    my_lo[q] = lower_bound_of(pos[q], p.chunk, p.window);
    const bf16* qp = (const bf16*)p.q + ((size_t)t[q] * p.H + h) * D + 8 * hf;
#pragma unroll
    for (int c = 0; c < KS; ++c) qf[q][c] = *reinterpret_cast<const bf16x8*>(qp + 16 * c);
  }
  const int pos_last = kv - qlen + min(r0 + 32 * NQ - 1, rend - 1);
  const int lo_w = lower_bound_of(kv - qlen + r0, p.chunk, p.window);
  MfmaState<DB, NQ> st;
  mfma_init(st);
  // columns past the tile's end compute like real ones (positions past the last key are
  // masked by the range, never read) and are not stored
  const int pos_first = kv - qlen + r0;
  const int lo_max = lower_bound_of(kv - qlen + r0 + 32 * NQ - 1, p.chunk, p.window);
  mfma_attend<DB, NQ>(st, p, bt, g, qf, pos, my_lo, lo_w & ~31, pos_last, pos_first,
                      max(lo_w, lo_max));
#pragma unroll
  for (int q = 0; q < NQ; ++q)
    if (valid[q]) mfma_finish<DB, NQ>(st, q, p, t[q], h);
}

// Decode: grid (B, G * ceil(rep / 32), parts), one wave: the query heads of one K/V head are
// the columns of one tile, so K and V are read once per K/V head, not once per query head.
template <int DB>
__global__ __launch_bounds__(64) void sink_attn_decode_mfma_kernel(AttnParams p) {
  constexpr int D = 32 * DB, KS = 2 * DB;
  using akap::bf16x8;
  const int lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int rep = p.H / p.G;
  const int cgroups = (rep + 31) >> 5;
  const int b = blockIdx.x, g = blockIdx.y / cgroups, part = blockIdx.z;
  const int c0 = (blockIdx.y % cgroups) * 32;
  const int kv = p.seq_lens[b];
  const bool valid = c0 + col < rep;
  const int h = g * rep + (valid ? c0 + col : 0);
  if (kv <= 0) {  // padding row of a bucketed batch: defined output, no cache reads
    if (part == 0 && valid) {
      bf16* o = (bf16*)p.out + (size_t)b * p.out_stride + h * D;
      for (int d = hf; d < D; d += 2) o[d] = (bf16)0.f;
    }
    return;
  }
  const int pos1 = kv - 1;
  const int lo = lower_bound_of(pos1, p.chunk, p.window);
  const int a0 = lo & ~31;
  int per = (pos1 + 1 - a0 + p.num_parts - 1) / p.num_parts;
  per = (per + 31) & ~31;
  const int jb = a0 + part * per;
  const int je = min(pos1, jb + per - 1);
  int pos[1] = {pos1}, my_lo[1] = {lo};
  bf16x8 qf[1][KS];
  {
    const bf16* qp = (const bf16*)p.q + ((size_t)b * p.H + h) * D + 8 * hf;
#pragma unroll
    for (int c = 0; c < KS; ++c) qf[0][c] = *reinterpret_cast<const bf16x8*>(qp + 16 * c);
  }
  MfmaState<DB, 1> st;
  mfma_init(st);
  if (jb <= je)
    mfma_attend<DB, 1>(st, p, p.block_tables + (size_t)b * p.max_blocks, g, qf, pos, my_lo, jb, je,
                       pos1, lo);
  if (!valid) return;
  if (p.num_parts == 1) {
    mfma_finish<DB, 1>(st, 0, p, b, h);
    return;
  }
  const size_t slot = ((size_t)b * p.H + h) * p.num_parts + part;
  if (hf == 0) {
    p.ws_ml[slot * 2] = st.m[0] * 0.693147180559945f;  // the merge works in natural units
    p.ws_ml[slot * 2 + 1] = st.l[0];
  }
#pragma unroll
  for (int dt = 0; dt < DB; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      p.ws_o[slot * D + 32 * dt + 8 * (i >> 2) + 4 * hf + (i & 3)] = st.o[0][dt][i];
}

// the matrix kernels take bf16 and these head sizes (prefill: tiles of 128 tokens)
static bool mfma_ok(const AttnParams& p, bool f32) {
  return !f32 && (p.D == 32 || p.D == 64 || p.D == 128 || p.D == 256) && p.BS % 32 == 0 &&
         p.scale > 0.f;  // (the running max is taken on unscaled scores)
}

void launch_sink_attention_prefill(const AttnParams& p, bool f32, hipStream_t s) {
  if (p.num_tiles <= 0) return;
  const dim3 grid((unsigned)p.num_tiles * p.H);
  if (mfma_ok(p, f32) && (p.tile_rows == 128 || p.tile_rows == 256)) {
    // (tile, K/V head) units padded to a multiple of the 8 XCDs, rep workgroups each
    const dim3 grid((unsigned)((p.num_tiles * p.G + 7) / 8 * 8) * (p.H / p.G));
    const int tr = p.tile_rows;
    static const int nq = [] {  // AKAP_STREAM_NQ=1|2: column tiles per wave (A/B knob)
      const char* e = getenv("AKAP_STREAM_NQ");
      return e ? atoi(e) : 2;
    }();
    if (nq == 1 || p.D == 256) {
      switch (p.D) {
        case 32: sink_attn_prefill_mfma_kernel<1, 1><<<grid, 2 * tr, 0, s>>>(p); break;
        case 64: sink_attn_prefill_mfma_kernel<2, 1><<<grid, 2 * tr, 0, s>>>(p); break;
        case 128: sink_attn_prefill_mfma_kernel<4, 1><<<grid, 2 * tr, 0, s>>>(p); break;
        default: sink_attn_prefill_mfma_kernel<8, 1><<<grid, 2 * tr, 0, s>>>(p); break;
      }
    } else {
      switch (p.D) {
        case 32: sink_attn_prefill_mfma_kernel<1, 2><<<grid, tr, 0, s>>>(p); break;
        case 64: sink_attn_prefill_mfma_kernel<2, 2><<<grid, tr, 0, s>>>(p); break;
        default: sink_attn_prefill_mfma_kernel<4, 2><<<grid, tr, 0, s>>>(p); break;
      }
    }
    return;
  }
  const size_t sm = 4 * (p.D + 64) * sizeof(float);
  if (f32)
    sink_attn_prefill_rows_kernel<float><<<grid, 256, sm, s>>>(p);
  else
    sink_attn_prefill_rows_kernel<bf16><<<grid, 256, sm, s>>>(p);
}

void launch_sink_attention_decode(const AttnParams& p, bool f32, hipStream_t s) {
  if (p.B <= 0) return;
  const dim3 grid(p.B, p.H, p.num_parts);
  const size_t sm = (p.D + 64) * sizeof(float);
  if (mfma_ok(p, f32)) {
    const int rep = p.H / p.G;
    const dim3 mg(p.B, p.G * ((rep + 31) / 32), p.num_parts);
    switch (p.D) {
      case 32: sink_attn_decode_mfma_kernel<1><<<mg, 64, 0, s>>>(p); break;
      case 64: sink_attn_decode_mfma_kernel<2><<<mg, 64, 0, s>>>(p); break;
      case 128: sink_attn_decode_mfma_kernel<4><<<mg, 64, 0, s>>>(p); break;
      default: sink_attn_decode_mfma_kernel<8><<<mg, 64, 0, s>>>(p); break;
    }
  } else if (f32)
    sink_attn_decode_rows_kernel<float><<<grid, 64, sm, s>>>(p);
  else
    sink_attn_decode_rows_kernel<bf16><<<grid, 64, sm, s>>>(p);
  if (p.num_parts > 1) {
    const dim3 mg(p.B, p.H);
    if (f32)
      sink_attn_decode_merge_kernel<float><<<mg, 64, 0, s>>>(p);
    else
      sink_attn_decode_merge_kernel<bf16><<<mg, 64, 0, s>>>(p);
  }
}

}  // namespace akap_stream
