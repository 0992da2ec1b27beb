// Kernels of layers with grouped norms, a token shift, latent attention and routed experts:
// residual update + grouped RMS norm with two weight sets, token shift with per-sequence state,
// latent norm + rotary + paged latent-cache write, in-place rotary on query heads, attention of
// all heads against one cached row per key, sigmoid output gates, xIELU, the grouped top-k
// router and the two expert-combine helpers.
//
// One workgroup of 256 threads per token row (the attention: per token and 4 heads).  Sums of
// squares, norm scales, angles, scores, softmax, routing and the residual sum are fp32
// whatever the storage type; every size is a run-time argument.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::block_sum;
using akap::wave_max;
using akap::wave_sum;

namespace {

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

__device__ __forceinline__ float sigmoidf(float z) { return 1.0f / (1.0f + __expf(-z)); }
__device__ __forceinline__ float softplusf(float z) {
  return log1pf(__expf(-fabsf(z))) + fmaxf(z, 0.f);
}

// ------------------------------------------------------------------ residual + grouped norm
template <typename TY, typename TO>
__global__ __launch_bounds__(256) void add_group_norm_kernel(
    TO* __restrict__ out1, TO* __restrict__ out2, int out1_stride, int out2_stride,
    float* __restrict__ x, const TY* __restrict__ y, int y_stride, const float* __restrict__ y2,
    const TY* __restrict__ bias, const float* __restrict__ w1, const float* __restrict__ w2, int d,
    int groups, float eps, ShiftArgs sh) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float* xr = x + (size_t)row * d;
  const TY* yr = y ? y + (size_t)row * y_stride : nullptr;
  const float* y2r = y2 ? y2 + (size_t)row * d : nullptr;
  TO* o1 = out1 + (size_t)row * out1_stride;
  TO* o2 = out2 ? out2 + (size_t)row * out2_stride : nullptr;
  const int gs = d / groups;
  const bool add = yr || y2r || bias;
  // token shift of out1 for rows that are sequences of their own (see ShiftArgs)
  TO* st = sh.mu && sh.slot[row] >= 0 ? (TO*)sh.state + (size_t)sh.slot[row] * d : nullptr;
  const bool have = st != nullptr && sh.pos[row] > 0;
  for (int g = 0; g < groups; ++g) {
    const int c0 = g * gs, c1 = c0 + gs;
    float ss = 0.f;
    for (int c = c0 + threadIdx.x; c < c1; c += 256) {
      float f = xr[c];
      if (add) {
        // the deferred outputs of the previous layer: projection (+ bias) and routed experts
        float a = 0.f;
        if (yr) a += ldf(yr + c);
        if (bias) a += ldf(bias + c);
        if (y2r) a += y2r[c];
        f += a;
        xr[c] = f;
      }
      ss += f * f;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
    // each thread re-reads the columns it wrote itself
    for (int c = c0 + threadIdx.x; c < c1; c += 256) {
      const float n = xr[c] * inv;
      if (sh.mu) {
        const TO h = (TO)(n * w1[c]);                // the unshifted row, as stored
        const float hv = (float)h, pv = have ? ldf(st + c) : 0.f;
        stf(o1 + c, hv + (pv - hv) * sh.mu[c]);
        if (st) st[c] = h;
      } else {
        stf(o1 + c, n * w1[c]);
      }
      if (o2) stf(o2 + c, n * w2[c]);
    }
  }
}

// ------------------------------------------------------------------ token shift
__device__ __forceinline__ bool continues(const int32_t* slot, const int64_t* pos, int t) {
  return t > 0 && slot[t] >= 0 && slot[t] == slot[t - 1] && pos[t] == pos[t - 1] + 1;
}

template <typename T>
__global__ __launch_bounds__(256) void token_shift_kernel(T* __restrict__ out,
                                                          const T* __restrict__ h,
                                                          const float* __restrict__ mu,
                                                          const T* __restrict__ state,
                                                          const int32_t* __restrict__ slot,
                                                          const int64_t* __restrict__ pos, int d) {
  const int t = blockIdx.x;
  const T* hr = h + (size_t)t * d;
  const T* prev = nullptr;
  if (continues(slot, pos, t)) prev = hr - d;
  else if (slot[t] >= 0 && pos[t] > 0) prev = state + (size_t)slot[t] * d;
  T* o = out + (size_t)t * d;
  for (int c = threadIdx.x; c < d; c += 256) {
    const float v = ldf(hr + c);
    const float p = prev ? ldf(prev + c) : 0.f;
    stf(o + c, v + (p - v) * mu[c]);
  }
}

// every row is a sequence of its own (decode steps): the row's workgroup reads its state and
// replaces it, one launch
template <typename T>
__global__ __launch_bounds__(256) void token_shift_single_kernel(T* __restrict__ out,
                                                                 const T* __restrict__ h,
                                                                 const float* __restrict__ mu,
                                                                 T* __restrict__ state,
                                                                 const int32_t* __restrict__ slot,
                                                                 const int64_t* __restrict__ pos,
                                                                 int d) {
  const int t = blockIdx.x;
  const T* hr = h + (size_t)t * d;
  T* st = slot[t] >= 0 ? state + (size_t)slot[t] * d : nullptr;
  const bool have = st != nullptr && pos[t] > 0;
  T* o = out + (size_t)t * d;
  for (int c = threadIdx.x; c < d; c += 256) {
    const T raw = hr[c];
    const float v = (float)raw;
    const float pv = have ? ldf(st + c) : 0.f;
    stf(o + c, v + (pv - v) * mu[c]);
    if (st) st[c] = raw;
  }
}

// the last row of every sequence in the batch leaves its unshifted h for the next step
template <typename T>
__global__ __launch_bounds__(256) void shift_state_kernel(T* __restrict__ state,
                                                          const T* __restrict__ h,
                                                          const int32_t* __restrict__ slot,
                                                          const int64_t* __restrict__ pos, int d,
                                                          int rows) {
  const int t = blockIdx.x;
  if (slot[t] < 0) return;
  if (t + 1 < rows && continues(slot, pos, t + 1)) return;
  const T* hr = h + (size_t)t * d;
  T* s = state + (size_t)slot[t] * d;
  for (int c = threadIdx.x; c < d; c += 256) s[c] = hr[c];
}

// ------------------------------------------------------------------ latent norm + cache write
template <typename T>
__global__ __launch_bounds__(256) void latent_prep_kernel(LatentPrepParams p) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = (const T*)p.proj + (size_t)t * p.proj_stride;
  {
    const T* q = row + p.q_off;
    float ss = 0.f;
    for (int c = threadIdx.x; c < p.q_rank; c += 256) {
      const float f = ldf(q + c);
      ss += f * f;
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)p.q_rank + p.eps);
    T* o = (T*)p.cq_out + (size_t)t * p.q_rank;
    for (int c = threadIdx.x; c < p.q_rank; c += 256) stf(o + c, ldf(q + c) * inv * p.q_w[c]);
  }
  if (p.cache == nullptr) return;
  const int64_t slot = p.slots[t];
  if (slot < 0 || slot >= p.num_slots) return;      // uniform over the workgroup
  const T* kv = row + p.kv_off;
  float ss = 0.f;
  for (int c = threadIdx.x; c < p.kv_rank; c += 256) {
    const float f = ldf(kv + c);
    ss += f * f;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)p.kv_rank + p.eps);
  T* dst = (T*)p.cache + (size_t)slot * (p.kv_rank + p.rot_dim);
  // the grouped copy: 8 consecutive tokens of one dimension are 16 contiguous bytes
  T* grp = p.vgroups ? (T*)p.vgroups + (size_t)(slot >> 3) * p.kv_rank * 8 + (slot & 7) : nullptr;
  for (int c = threadIdx.x; c < p.kv_rank; c += 256) {
    const T v = (T)(ldf(kv + c) * inv * p.kv_w[c]);
    dst[c] = v;
    if (grp) grp[(size_t)c * 8] = v;
  }
  int64_t pos = p.positions[t];
  pos = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);
  const float* cs = p.cos_sin + (size_t)pos * p.rot_dim;
  const int half = p.rot_dim / 2;
  const T* kr = kv + p.kv_rank;
  for (int i = threadIdx.x; i < half; i += 256) {
    const float u = ldf(kr + 2 * i), v = ldf(kr + 2 * i + 1);
    const float c = cs[i], s = cs[half + i];
    stf(dst + p.kv_rank + 2 * i, u * c - v * s);
    stf(dst + p.kv_rank + 2 * i + 1, v * c + u * s);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void rotate_heads_kernel(T* __restrict__ q, int q_stride, int H,
                                                           int n, int offset, int dims,
                                                           const int64_t* __restrict__ positions,
                                                           const float* __restrict__ cos_sin,
                                                           int max_pos) {
  const int t = blockIdx.x;
  int64_t pos = positions[t];
  pos = pos < 0 ? 0 : (pos >= max_pos ? max_pos - 1 : pos);
  const float* cs = cos_sin + (size_t)pos * dims;
  const int half = dims / 2;
  T* row = q + (size_t)t * q_stride;
  for (int i = threadIdx.x; i < H * half; i += 256) {
    const int h = i / half, j = i % half;
    T* e = row + (size_t)h * n + offset + 2 * j;
    const float u = ldf(e), v = ldf(e + 1);
    const float c = cs[j], s = cs[half + j];
    stf(e, u * c - v * s);
    stf(e + 1, v * c + u * s);
  }
}

// ------------------------------------------------------------------ latent attention
// One wave per (token, head); the 4 waves of a workgroup take 4 heads of one token and read the
// same cached rows.  Scores: a lane per key (64 keys a piece), the query [R + r] as fp32 in
// LDS; weighted sum: a lane per latent dimension (NR per lane).
template <typename T, int NR>
__global__ __launch_bounds__(256) void latent_attention_kernel(LatentAttnParams p) {
  extern __shared__ float lds[];
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + wave;
  // the token's sequence: row t itself (one query per sequence) or a search in q_start
  int b = t;
  if (p.q_start != nullptr) {
    int lo = 0, hi = p.B - 1;
    while (lo < hi) {
      const int mid = (lo + hi + 1) >> 1;
      if (p.q_start[mid] <= t) lo = mid; else hi = mid - 1;
    }
    b = lo;
    if (t >= p.q_start[p.B]) return;
  }
  const int kv_len = p.seq_lens[b];
  if (kv_len <= 0 || head >= p.H) return;            // uniform per wave; no barriers below
  const int R = p.R, r = p.r, DK = R + r;
  int64_t pos = p.positions[t];
  const int last = (int)(pos < kv_len ? pos : kv_len - 1);   // keys 0 .. last
  float* q = lds + wave * DK;
  const T* ql = (const T*)p.q_lat + ((size_t)head * p.T + t) * R;
  const T* qr = (const T*)p.q + (size_t)t * p.q_stride + (size_t)head * p.q_head + p.rot_off;
  for (int c = lane; c < R; c += 64) q[c] = ldf(ql + c) * p.scale;
  for (int c = lane; c < r; c += 64) q[R + c] = ldf(qr + c) * p.scale;
  __builtin_amdgcn_wave_barrier();
  const int32_t* bt = p.block_tables + (size_t)b * p.max_blocks;
  const T* cache = (const T*)p.cache;
  float acc[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  for (int k0 = 0; k0 <= last; k0 += 64) {
    const int key = k0 + lane;
    const bool ok = key <= last;
    const int kk = ok ? key : last;
    const int64_t rowoff = ((int64_t)bt[kk / p.BS] * p.BS + kk % p.BS) * DK;
    const T* krow = cache + rowoff;
    float s = 0.f;
    if (p.vec) {
      constexpr int W = 16 / sizeof(T);
      for (int c = 0; c < DK; c += W) {
        float v[W];
        if constexpr (sizeof(T) == 2) {
          const akap::bf16x8 x = *reinterpret_cast<const akap::bf16x8*>(krow + c);
#pragma unroll
          for (int e = 0; e < W; ++e) v[e] = (float)x[e];
        } else {
          const akap::f32x4 x = *reinterpret_cast<const akap::f32x4*>(krow + c);
#pragma unroll
          for (int e = 0; e < W; ++e) v[e] = x[e];
        }
#pragma unroll
        for (int e = 0; e < W; ++e) s += q[c + e] * v[e];
      }
    } else {
      for (int c = 0; c < DK; ++c) s += q[c] * ldf(krow + c);
    }
    s = ok ? s : -INFINITY;
    const float mn = fmaxf(m, wave_max(s));
    const float corr = __expf(m - mn);               // first piece: exp(-inf) = 0
    const float pj = ok ? __expf(s - mn) : 0.f;
    l = l * corr + wave_sum(pj);
    m = mn;
#pragma unroll
    for (int i = 0; i < NR; ++i) acc[i] *= corr;
    const int n = min(64, last - k0 + 1);
    for (int j = 0; j < n; ++j) {
      const float w = __shfl(pj, j, 64);
      const int64_t off = __shfl(rowoff, j, 64);
      const T* vrow = cache + off;
#pragma unroll
      for (int i = 0; i < NR; ++i) {
        const int c = lane + 64 * i;
        if (c < R) acc[i] += w * ldf(vrow + c);
      }
    }
  }
  const float inv = 1.0f / l;
  T* o = (T*)p.out + ((size_t)head * p.T + t) * R;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = lane + 64 * i;
    if (c < R) stf(o + c, acc[i] * inv);
  }
}

// ------------------------------------------------------------------ gates and activations
template <typename T>
__global__ __launch_bounds__(256) void head_gate_kernel(T* __restrict__ out, int out_stride,
                                                        const T* __restrict__ o,
                                                        const T* __restrict__ gate,
                                                        int gate_stride, int per_head, int H, int V,
                                                        int rows) {
  const int t = blockIdx.x;
  const T* g = gate + (size_t)t * gate_stride;
  T* dst = out + (size_t)t * out_stride;
  for (int c = threadIdx.x; c < H * V; c += 256) {
    const int h = c / V, j = c - h * V;
    const float z = ldf(g + (per_head ? h : c));
    stf(dst + c, ldf(o + ((size_t)h * rows + t) * V + j) * sigmoidf(z));
  }
}

template <typename T>
__global__ __launch_bounds__(256) void xielu_kernel(T* __restrict__ out, int out_stride,
                                                    const T* __restrict__ x, int x_stride,
                                                    const T* __restrict__ bias,
                                                    const float* __restrict__ act, int F) {
  const int t = blockIdx.x;
  const float ap = softplusf(act[0]), aq = 0.5f + softplusf(act[1]);
  const T* xr = x + (size_t)t * x_stride;
  T* o = out + (size_t)t * out_stride;
  for (int c = threadIdx.x; c < F; c += 256) {
    const float z = ldf(xr + c) + (bias ? ldf(bias + c) : 0.f);
    const float v = z > 0.f ? ap * z * z + 0.5f * z : aq * (expm1f(z) - z) + 0.5f * z;
    stf(o + c, v);
  }
}

// ------------------------------------------------------------------ routing
// logits by the 4 waves (an output per wave and turn), softmax by wave 0, selection by thread 0
template <typename T>
__global__ __launch_bounds__(256) void moe_route_kernel(int32_t* __restrict__ ids,
                                                        float* __restrict__ wout,
                                                        const T* __restrict__ h, int h_stride,
                                                        const float* __restrict__ router,
                                                        const float* __restrict__ corr, int d,
                                                        int n, int top, int groups, int keep) {
  extern __shared__ float lds[];
  float* s = lds;           // [n] scores
  float* ch = lds + n;      // [n] choice values
  float* gs = lds + 2 * n;  // [groups]
  const int t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const T* hr = h + (size_t)t * h_stride;
  for (int e = wave; e < n; e += 4) {
    const float* wr = router + (size_t)e * d;
    float a = 0.f;
    for (int c = lane; c < d; c += 64) a += ldf(hr + c) * wr[c];
    a = wave_sum(a);
    if (lane == 0) s[e] = a;
  }
  __syncthreads();
  if (wave == 0) {
    float mx = -INFINITY;
    for (int e = lane; e < n; e += 64) mx = fmaxf(mx, s[e]);
    mx = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < n; e += 64) sum += __expf(s[e] - mx);
    sum = wave_sum(sum);
    for (int e = lane; e < n; e += 64) {
      const float v = __expf(s[e] - mx) / sum;
      s[e] = v;
      ch[e] = v + (corr ? corr[e] : 0.f);
    }
  }
  __syncthreads();
  if (threadIdx.x != 0) return;
  const int per = n / groups;
  if (groups > 1) {
    for (int g = 0; g < groups; ++g) {
      float mx = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) mx = fmaxf(mx, ch[e]);
      gs[g] = mx;
    }
    // the groups that are not kept lose their outputs: drop the (groups - keep) worst
    for (int k = 0; k < groups - keep; ++k) {
      int worst = -1;
      for (int g = groups - 1; g >= 0; --g)
        if (gs[g] != INFINITY && (worst < 0 || gs[g] < gs[worst])) worst = g;
      gs[worst] = INFINITY;                          // marks a dropped group
      for (int e = worst * per; e < (worst + 1) * per; ++e) ch[e] = -INFINITY;
    }
  }
  float total = 0.f;
  for (int k = 0; k < top; ++k) {
    int best = 0;
    float bv = -INFINITY;
    bool found = false;
    for (int e = 0; e < n; ++e) {
      const float v = ch[e];
      if (v == -INFINITY) continue;
      if (!found || v > bv) { best = e; bv = v; found = true; }
    }
    ch[best] = -INFINITY;
    ids[(size_t)t * top + k] = best;
    wout[(size_t)t * top + k] = s[best];
    total += s[best];
  }
  const float inv = 1.0f / (total + 1e-20f);
  for (int k = 0; k < top; ++k) wout[(size_t)t * top + k] *= inv;
}

template <typename T>
__global__ __launch_bounds__(256) void relu2_routed_kernel(T* __restrict__ out, int out_stride,
                                                           const T* __restrict__ up, int up_stride,
                                                           const int32_t* __restrict__ ids,
                                                           const float* __restrict__ w, int top,
                                                           int E, int F) {
  extern __shared__ float lds[];                     // [E] routing weight of every expert
  const int t = blockIdx.x;
  for (int e = threadIdx.x; e < E; e += 256) lds[e] = 0.f;
  __syncthreads();
  if (threadIdx.x < top) {
    const int e = ids[(size_t)t * top + threadIdx.x];
    if (e >= 0 && e < E) lds[e] = w[(size_t)t * top + threadIdx.x];
  }
  __syncthreads();
  const T* u = up + (size_t)t * up_stride;
  T* o = out + (size_t)t * out_stride;
  for (int c = threadIdx.x; c < E * F; c += 256) {
    const float z = fmaxf(ldf(u + c), 0.f);
    stf(o + c, z * z * lds[c / F]);
  }
}

template <typename T>
__global__ __launch_bounds__(256) void moe_combine_kernel(float* __restrict__ out,
                                                          const T* __restrict__ y,
                                                          const int32_t* __restrict__ inv,
                                                          const int32_t* __restrict__ ids,
                                                          const float* __restrict__ w,
                                                          const T* __restrict__ h, int h_stride,
                                                          int d, int top, int E, int y_rows) {
  const int t = blockIdx.x;
  const int32_t* id = ids + (size_t)t * top;
  const float* wt = w + (size_t)t * top;
  float ident = 0.f;
  for (int k = 0; k < top; ++k)
    if (id[k] >= E) ident += wt[k];
  const T* hr = h + (size_t)t * h_stride;
  for (int c = threadIdx.x; c < d; c += 256) {
    float a = 0.f;
    if (inv == nullptr) {
      a = ldf(y + (size_t)t * d + c);
    } else {
      for (int k = 0; k < top; ++k) {
        const int rrow = inv[(size_t)t * top + k];
        if (id[k] < E && rrow >= 0 && rrow < y_rows) a += wt[k] * ldf(y + (size_t)rrow * d + c);
      }
    }
    out[(size_t)t * d + c] = a + ident * ldf(hr + c);
  }
}


// ------------------------------------------------------------------ 16-byte variants
// 4 consecutive elements as floats (16 bytes of fp32, 8 of bf16); the launchers check sizes,
// strides and pointers for that alignment and fall back to the kernels above otherwise
__device__ __forceinline__ void ld4(float (&v)[4], const float* p) {
  const akap::f32x4 x = *reinterpret_cast<const akap::f32x4*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = x[e];
}
__device__ __forceinline__ void ld4(float (&v)[4], const bf16* p) {
  const akap::bf16x4 x = *reinterpret_cast<const akap::bf16x4*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = (float)x[e];
}
__device__ __forceinline__ void st4(float* p, const float (&v)[4]) {
  akap::f32x4 x;
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] = v[e];
  *reinterpret_cast<akap::f32x4*>(p) = x;
}
__device__ __forceinline__ void st4(bf16* p, const float (&v)[4]) {
  akap::bf16x4 x;
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] = (bf16)v[e];
  *reinterpret_cast<akap::bf16x4*>(p) = x;
}

// the row's group stays in registers between the sum of squares and the scaled writes when it
// has at most 1024 NR elements: x is read once and written once
template <typename TY, typename TO, int NR>
__global__ __launch_bounds__(256) void add_group_norm_vec_kernel(
    TO* __restrict__ out1, TO* __restrict__ out2, int out1_stride, int out2_stride,
    float* __restrict__ x, const TY* __restrict__ y, int y_stride, const float* __restrict__ y2,
    const TY* __restrict__ bias, const float* __restrict__ w1, const float* __restrict__ w2, int d,
    int groups, float eps, ShiftArgs sh) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float* xr = x + (size_t)row * d;
  const TY* yr = y ? y + (size_t)row * y_stride : nullptr;
  const float* y2r = y2 ? y2 + (size_t)row * d : nullptr;
  TO* o1 = out1 + (size_t)row * out1_stride;
  TO* o2 = out2 ? out2 + (size_t)row * out2_stride : nullptr;
  const int gs = d / groups;
  const bool add = yr || y2r || bias;
  TO* st = sh.mu && sh.slot[row] >= 0 ? (TO*)sh.state + (size_t)sh.slot[row] * d : nullptr;
  const bool have = st != nullptr && sh.pos[row] > 0;
  for (int g = 0; g < groups; ++g) {
    const int c0 = g * gs;
    float v[NR][4];
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int c = (i * 256 + threadIdx.x) * 4;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[i][e] = 0.f;
      if (c < gs) {
        ld4(v[i], xr + c0 + c);
        if (add) {
          float a[4];
          if (yr) {
            ld4(a, yr + c0 + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[i][e] += a[e];
          }
          if (bias) {
            ld4(a, bias + c0 + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[i][e] += a[e];
          }
          if (y2r) {
            ld4(a, y2r + c0 + c);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[i][e] += a[e];
          }
          st4(xr + c0 + c, v[i]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) ss += v[i][e] * v[i][e];
      }
    }
    ss = block_sum(ss, scratch);
    const float inv = 1.0f / sqrtf(ss / (float)gs + eps);
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int c = (i * 256 + threadIdx.x) * 4;
      if (c < gs) {
        float w[4], r[4];
        ld4(w, w1 + c0 + c);
#pragma unroll
        for (int e = 0; e < 4; ++e) r[e] = v[i][e] * inv * w[e];
        if (sh.mu) {
          float pv[4] = {0.f, 0.f, 0.f, 0.f}, m[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) r[e] = (float)(TO)r[e];   // the unshifted row, as stored
          if (have) ld4(pv, st + c0 + c);
          ld4(m, sh.mu + c0 + c);
          if (st) st4(st + c0 + c, r);
#pragma unroll
          for (int e = 0; e < 4; ++e) r[e] = r[e] + (pv[e] - r[e]) * m[e];
        }
        st4(o1 + c0 + c, r);
        if (o2) {
          ld4(w, w2 + c0 + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) r[e] = v[i][e] * inv * w[e];
          st4(o2 + c0 + c, r);
        }
      }
    }
  }
}

// grid (rows, pieces of 4096 columns): a thread takes 4 pieces of 4 columns, 1024 apart
template <typename T>
__global__ __launch_bounds__(256) void xielu_vec_kernel(T* __restrict__ out, int out_stride,
                                                        const T* __restrict__ x, int x_stride,
                                                        const T* __restrict__ bias,
                                                        const float* __restrict__ act, int F) {
  const int t = blockIdx.x;
  const float ap = softplusf(act[0]), aq = 0.5f + softplusf(act[1]);
  const T* xr = x + (size_t)t * x_stride;
  T* o = out + (size_t)t * out_stride;
  float z[4][4], b[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = blockIdx.y * 4096 + i * 1024 + threadIdx.x * 4;
    if (c < F) {
      ld4(z[i], xr + c);
      if (bias) ld4(b[i], bias + c);
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int c = blockIdx.y * 4096 + i * 1024 + threadIdx.x * 4;
    if (c < F) {
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float u = z[i][e] + (bias ? b[i][e] : 0.f);
        z[i][e] = u > 0.f ? ap * u * u + 0.5f * u : aq * (expm1f(u) - u) + 0.5f * u;
      }
      st4(o + c, z[i]);
    }
  }
}

template <typename T>
__global__ __launch_bounds__(256) void token_shift_vec_kernel(T* __restrict__ out,
                                                              const T* __restrict__ h,
                                                              const float* __restrict__ mu,
                                                              T* __restrict__ state,
                                                              const int32_t* __restrict__ slot,
                                                              const int64_t* __restrict__ pos,
                                                              int d, int single) {
  const int t = blockIdx.x;
  const T* hr = h + (size_t)t * d;
  const T* prev = nullptr;
  if (!single && continues(slot, pos, t)) prev = hr - d;
  else if (slot[t] >= 0 && pos[t] > 0) prev = state + (size_t)slot[t] * d;
  T* st = single && slot[t] >= 0 ? state + (size_t)slot[t] * d : nullptr;
  T* o = out + (size_t)t * d;
  for (int c = threadIdx.x * 4; c < d; c += 1024) {
    float v[4], pv[4] = {0.f, 0.f, 0.f, 0.f}, m[4], r[4];
    ld4(v, hr + c);
    if (prev) ld4(pv, prev + c);
    ld4(m, mu + c);
#pragma unroll
    for (int e = 0; e < 4; ++e) r[e] = v[e] + (pv[e] - v[e]) * m[e];
    st4(o + c, r);
    if (st) st4(st + c, v);       // v came from T: the round trip is exact
  }
}

// per-head gates, V % 4 == 0: 4 consecutive output entries share a head
template <typename T>
__global__ __launch_bounds__(256) void head_gate_vec_kernel(T* __restrict__ out, int out_stride,
                                                            const T* __restrict__ o,
                                                            const T* __restrict__ gate,
                                                            int gate_stride, int per_head, int H,
                                                            int V, int rows) {
  const int t = blockIdx.x;
  const T* g = gate + (size_t)t * gate_stride;
  T* dst = out + (size_t)t * out_stride;
  for (int c = threadIdx.x * 4; c < H * V; c += 1024) {
    const int h = c / V, j = c - h * V;
    float v[4], z[4];
    ld4(v, o + ((size_t)h * rows + t) * V + j);
    if (per_head) {
      const float zh = ldf(g + h);
      z[0] = z[1] = z[2] = z[3] = zh;
    } else {
      ld4(z, g + c);
    }
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] *= sigmoidf(z[e]);
    st4(dst + c, v);
  }
}

bool al(const void* p, size_t a) { return p == nullptr || ((uintptr_t)p % a) == 0; }

}  // namespace

// ------------------------------------------------------------------ launchers
void launch_add_group_norm(void* out1, void* out2, bool out_f32, int out1_stride, int out2_stride,
                           float* x, const void* y, bool y_f32, int y_stride, const float* y2,
                           const void* bias, const float* w1, const float* w2, int rows, int d,
                           int groups, float eps, const ShiftArgs& sh, hipStream_t s) {
  if (rows <= 0) return;
  // 16-byte path: every group a multiple of 4 columns that fits 4096 columns in registers
  const int gsz = d / groups;
  const size_t ob = out_f32 ? 16 : 8, yb = y_f32 ? 16 : 8;
  if (gsz % 4 == 0 && gsz <= 4096 && out1_stride % 4 == 0 && out2_stride % 4 == 0 &&
      y_stride % 4 == 0 && al(x, 16) && al(y2, 16) && al(w1, 16) && al(w2, 16) && al(out1, ob) &&
      al(out2, ob) && al(y, yb) && al(bias, yb) && al(sh.mu, 16) && al(sh.state, ob)) {
#define AGNV(TY, TO, NR)                                                                         \
  add_group_norm_vec_kernel<TY, TO, NR><<<rows, 256, 0, s>>>(                                    \
      (TO*)out1, (TO*)out2, out1_stride, out2_stride, x, (const TY*)y, y_stride, y2,             \
      (const TY*)bias, w1, w2, d, groups, eps, sh)
#define AGNT(NR)                                                                                 \
  if (y_f32 && out_f32) AGNV(float, float, NR);                                                  \
  else if (!y_f32 && out_f32) AGNV(bf16, float, NR);                                             \
  else if (y_f32) AGNV(float, bf16, NR);                                                         \
  else AGNV(bf16, bf16, NR)
    if (gsz <= 1024) { AGNT(1); }
    else if (gsz <= 2048) { AGNT(2); }
    else { AGNT(4); }
#undef AGNT
#undef AGNV
    return;
  }
#define AGN(TY, TO)                                                                              \
  add_group_norm_kernel<TY, TO><<<rows, 256, 0, s>>>((TO*)out1, (TO*)out2, out1_stride,          \
                                                     out2_stride, x, (const TY*)y, y_stride, y2, \
                                                     (const TY*)bias, w1, w2, d, groups, eps, sh)
  if (y_f32 && out_f32) AGN(float, float);
  else if (!y_f32 && out_f32) AGN(bf16, float);
  else if (y_f32) AGN(float, bf16);
  else AGN(bf16, bf16);
#undef AGN
}

void launch_token_shift(void* out, const void* h, const float* mu, void* state,
                        const int32_t* slot, const int64_t* pos, bool f32, int rows, int d,
                        bool single, hipStream_t s) {
  if (rows <= 0) return;
  const size_t eb = f32 ? 16 : 8;
  if (d % 4 == 0 && al(out, eb) && al(h, eb) && al(state, eb) && al(mu, 16)) {
    if (f32) {
      token_shift_vec_kernel<float><<<rows, 256, 0, s>>>((float*)out, (const float*)h, mu,
                                                         (float*)state, slot, pos, d, single);
      if (!single)
        shift_state_kernel<float><<<rows, 256, 0, s>>>((float*)state, (const float*)h, slot, pos,
                                                       d, rows);
    } else {
      token_shift_vec_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)out, (const bf16*)h, mu,
                                                        (bf16*)state, slot, pos, d, single);
      if (!single)
        shift_state_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)state, (const bf16*)h, slot, pos, d,
                                                      rows);
    }
    return;
  }
  if (single) {
    if (f32)
      token_shift_single_kernel<float><<<rows, 256, 0, s>>>((float*)out, (const float*)h, mu,
                                                            (float*)state, slot, pos, d);
    else
      token_shift_single_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)out, (const bf16*)h, mu,
                                                           (bf16*)state, slot, pos, d);
    return;
  }
  if (f32) {
    token_shift_kernel<float><<<rows, 256, 0, s>>>((float*)out, (const float*)h, mu,
                                                   (const float*)state, slot, pos, d);
    shift_state_kernel<float><<<rows, 256, 0, s>>>((float*)state, (const float*)h, slot, pos, d,
                                                   rows);
  } else {
    token_shift_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)out, (const bf16*)h, mu,
                                                  (const bf16*)state, slot, pos, d);
    shift_state_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)state, (const bf16*)h, slot, pos, d,
                                                  rows);
  }
}

void launch_latent_prep(const LatentPrepParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  if (f32) latent_prep_kernel<float><<<p.T, 256, 0, s>>>(p);
  else latent_prep_kernel<bf16><<<p.T, 256, 0, s>>>(p);
}

void launch_rotate_heads(void* q, int q_stride, int T, int H, int n, int offset, int dims,
                         const int64_t* positions, const float* cos_sin, int max_pos, bool f32,
                         hipStream_t s) {
  if (T <= 0) return;
  if (f32)
    rotate_heads_kernel<float><<<T, 256, 0, s>>>((float*)q, q_stride, H, n, offset, dims,
                                                 positions, cos_sin, max_pos);
  else
    rotate_heads_kernel<bf16><<<T, 256, 0, s>>>((bf16*)q, q_stride, H, n, offset, dims, positions,
                                                cos_sin, max_pos);
}

template <typename T>
static void attn_dispatch(const LatentAttnParams& p, hipStream_t s) {
  const dim3 grid(p.T, (p.H + 3) / 4);
  const size_t lds = (size_t)4 * (p.R + p.r) * sizeof(float);
  const int nr = (p.R + 63) / 64;
#define LA(N) latent_attention_kernel<T, N><<<grid, 256, lds, s>>>(p)
  if (nr <= 1) LA(1);
  else if (nr <= 2) LA(2);
  else if (nr <= 4) LA(4);
  else if (nr <= 8) LA(8);
  else LA(16);
#undef LA
}

void launch_latent_attention(const LatentAttnParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0 || p.H <= 0) return;
  if (f32) attn_dispatch<float>(p, s);
  else attn_dispatch<bf16>(p, s);
}

void launch_head_gate(void* out, int out_stride, const void* o, const void* gate, int gate_stride,
                      bool per_head, int rows, int H, int V, bool f32, hipStream_t s) {
  if (rows <= 0) return;
  const size_t eb = f32 ? 16 : 8;
  if (V % 4 == 0 && out_stride % 4 == 0 && al(out, eb) && al(o, eb) &&
      (per_head || (gate_stride % 4 == 0 && al(gate, eb)))) {
    if (f32)
      head_gate_vec_kernel<float><<<rows, 256, 0, s>>>((float*)out, out_stride, (const float*)o,
                                                       (const float*)gate, gate_stride, per_head,
                                                       H, V, rows);
    else
      head_gate_vec_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)out, out_stride, (const bf16*)o,
                                                      (const bf16*)gate, gate_stride, per_head, H,
                                                      V, rows);
    return;
  }
  if (f32)
    head_gate_kernel<float><<<rows, 256, 0, s>>>((float*)out, out_stride, (const float*)o,
                                                 (const float*)gate, gate_stride, per_head, H, V,
                                                 rows);
  else
    head_gate_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)out, out_stride, (const bf16*)o,
                                                (const bf16*)gate, gate_stride, per_head, H, V,
                                                rows);
}

void launch_xielu(void* out, int out_stride, const void* x, int x_stride, const void* bias,
                  const float* act, int rows, int F, bool f32, hipStream_t s) {
  if (rows <= 0) return;
  const size_t eb = f32 ? 16 : 8;
  if (F % 4 == 0 && out_stride % 4 == 0 && x_stride % 4 == 0 && al(out, eb) && al(x, eb) &&
      al(bias, eb) && (F + 4095) / 4096 <= 65535) {
    const dim3 grid(rows, (F + 4095) / 4096);
    if (f32)
      xielu_vec_kernel<float><<<grid, 256, 0, s>>>((float*)out, out_stride, (const float*)x,
                                                   x_stride, (const float*)bias, act, F);
    else
      xielu_vec_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out, out_stride, (const bf16*)x, x_stride,
                                                  (const bf16*)bias, act, F);
    return;
  }
  if (f32)
    xielu_kernel<float><<<rows, 256, 0, s>>>((float*)out, out_stride, (const float*)x, x_stride,
                                             (const float*)bias, act, F);
  else
    xielu_kernel<bf16><<<rows, 256, 0, s>>>((bf16*)out, out_stride, (const bf16*)x, x_stride,
                                            (const bf16*)bias, act, F);
}

void launch_moe_route(int32_t* ids, float* w, const void* h, int h_stride, const float* router,
                      const float* corr, int rows, int d, int n, int top, int groups, int keep,
                      bool f32, hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)(2 * n + groups) * sizeof(float);
  if (f32)
    moe_route_kernel<float><<<rows, 256, lds, s>>>(ids, w, (const float*)h, h_stride, router, corr,
                                                   d, n, top, groups, keep);
  else
    moe_route_kernel<bf16><<<rows, 256, lds, s>>>(ids, w, (const bf16*)h, h_stride, router, corr,
                                                  d, n, top, groups, keep);
}

void launch_relu2_routed(void* out, int out_stride, const void* up, int up_stride,
                         const int32_t* ids, const float* w, int rows, int top, int E, int F,
                         bool f32, hipStream_t s) {
  if (rows <= 0) return;
  const size_t lds = (size_t)E * sizeof(float);
  if (f32)
    relu2_routed_kernel<float><<<rows, 256, lds, s>>>((float*)out, out_stride, (const float*)up,
                                                      up_stride, ids, w, top, E, F);
  else
    relu2_routed_kernel<bf16><<<rows, 256, lds, s>>>((bf16*)out, out_stride, (const bf16*)up,
                                                     up_stride, ids, w, top, E, F);
}

void launch_moe_combine(float* out, const void* y, const int32_t* inv, const int32_t* ids,
                        const float* w, const void* h, int h_stride, int rows, int d, int top,
                        int E, int y_rows, bool f32, hipStream_t s) {
  if (rows <= 0) return;
  if (f32)
    moe_combine_kernel<float><<<rows, 256, 0, s>>>(out, (const float*)y, inv, ids, w,
                                                   (const float*)h, h_stride, d, top, E, y_rows);
  else
    moe_combine_kernel<bf16><<<rows, 256, 0, s>>>(out, (const bf16*)y, inv, ids, w,
                                                  (const bf16*)h, h_stride, d, top, E, y_rows);
}

}  // namespace akap_stream
