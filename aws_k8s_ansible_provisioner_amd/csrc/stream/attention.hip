// Paged attention with a lower-bounded causal mask (chunks and / or a sliding window), a
// per-head sink logit in the softmax denominator and a per-head sigmoid output gate, over
// K / V caches [NB, G, BS, D] of bf16 or fp32 with any head size D.
//
// Scores, the running softmax and the gate are fp32.  A query at position i sees the keys
// [lo(i), i] with lo(i) = max(floor(i / chunk) * chunk, i - window + 1, 0): only that range is
// read, so a chunked layer costs O(chunk) per token however long the sequence.
//
// row kernel (any D, bf16 / fp32): one wave per (token, head).  Per 64-key piece each lane
//   scores one key (q broadcast from LDS), the wave takes the piece's max and sum, and lanes
//   then own output dimensions for the P.V update (coalesced V rows).  Prefill tiles give a
//   workgroup's four waves the tokens of one tile; decode rows cut [lo, i] into partitions
//   that a second launch merges together with the sink and the gate.
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

// Keys [j0, j1) of one sequence against one query held in `qs` (LDS, D floats, pre-scaled).
// `ps`: 64 floats of LDS owned by this wave.
template <typename T>
__device__ __forceinline__ void attend_range(Softmax& st, const float* qs, float* ps,
                                             const T* __restrict__ kc, const T* __restrict__ vc,
                                             const int32_t* __restrict__ bt, int max_blocks, int NB,
                                             int G, int g, int BS, int D, int j0, int j1) {
  const int lane = threadIdx.x & 63;
  for (int base = j0; base < j1; base += 64) {
    const int j = base + lane;
    const bool ok = j < j1;
    int row = 0;  // row of this lane's key in the [NB * G * BS, D] view of the cache
    float s = -INFINITY;
    if (ok) {
      const int bi = j / BS;
      int blk = bi < max_blocks ? bt[bi] : 0;
      if (blk < 0 || blk >= NB) blk = 0;
      row = (blk * G + g) * BS + (j - bi * BS);
      const T* kr = kc + (size_t)row * D;
      float dot = 0.f;
      for (int d = 0; d < D; ++d) dot += qs[d] * ldf(kr + d);
      s = dot;
    }
    const float mt = wave_max(s);
    const float mn = fmaxf(st.m, mt);
    const float corr = expf(st.m - mn);  // first piece: exp(-inf) = 0
    const float pj = ok ? expf(s - mn) : 0.f;
    st.l = st.l * corr + wave_sum(pj);
    st.m = mn;
    ps[lane] = pj;
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int c = 0; c < kMaxDV; ++c) st.acc[c] *= corr;
    const int n = min(64, j1 - base);
    for (int jj = 0; jj < n; ++jj) {
      const float pv = ps[jj];
      const int r = __shfl(row, jj, 64);
      const T* vr = vc + (size_t)r * D;
#pragma unroll
      for (int c = 0; c < kMaxDV; ++c) {
        const int d = c * 64 + lane;
        if (d < D) st.acc[c] += pv * ldf(vr + d);
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

// grid (tiles, H); 4 waves share a tile's tokens
template <typename T>
__global__ __launch_bounds__(256) void sink_attn_prefill_rows_kernel(AttnParams p) {
  extern __shared__ float smem[];
  const int wave = threadIdx.x >> 6;
  float* qs = smem + wave * (p.D + 64);
  float* ps = qs + p.D;
  const int tile = blockIdx.x, h = blockIdx.y;
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
  const int n = pos + 1 - lo;
  int per = (n + p.num_parts - 1) / p.num_parts;
  per = (per + 63) & ~63;
  const int j0 = lo + part * per;
  const int j1 = min(pos + 1, j0 + per);
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

void launch_sink_attention_prefill(const AttnParams& p, bool f32, hipStream_t s) {
  if (p.num_tiles <= 0) return;
  const dim3 grid(p.num_tiles, p.H);
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
  if (f32)
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
