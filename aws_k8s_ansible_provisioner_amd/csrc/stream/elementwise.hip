// Row kernels of the fp32 residual stream: scaled embedding, residual update fused with the
// next RMS norm, squared-ReLU, and the q/k whole-projection norm + rotary + paged-cache write.
//
// All memory-bound, one workgroup per token row; sums of squares, the norm scale, angles and
// the residual sum are fp32 whatever the storage type.
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::block_sum;

template <typename T>
__device__ __forceinline__ float ldf(const T* p) { return (float)*p; }
template <typename T>
__device__ __forceinline__ void stf(T* p, float v) { *p = (T)v; }

// N consecutive elements <-> floats with the widest loads / stores (N * sizeof(T) bytes,
// the caller guarantees that alignment)
template <int N>
__device__ __forceinline__ void ldv(float (&v)[N], const float* p) {
  static_assert(N % 4 == 0, "whole 16-byte pieces");
#pragma unroll
  for (int i = 0; i < N; i += 4) {
    const akap::f32x4 x = *reinterpret_cast<const akap::f32x4*>(p + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) v[i + e] = x[e];
  }
}
__device__ __forceinline__ void ldv(float (&v)[4], const bf16* p) {
  const akap::bf16x4 x = *reinterpret_cast<const akap::bf16x4*>(p);
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = (float)x[e];
}
__device__ __forceinline__ void ldv(float (&v)[8], const bf16* p) {
  const akap::bf16x8 x = *reinterpret_cast<const akap::bf16x8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = (float)x[e];
}
template <int N>
__device__ __forceinline__ void stv(float* p, const float (&v)[N]) {
#pragma unroll
  for (int i = 0; i < N; i += 4) {
    akap::f32x4 x;
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] = v[i + e];
    *reinterpret_cast<akap::f32x4*>(p + i) = x;
  }
}
__device__ __forceinline__ void stv(bf16* p, const float (&v)[4]) {
  akap::bf16x4 x;
#pragma unroll
  for (int e = 0; e < 4; ++e) x[e] = (bf16)v[e];
  *reinterpret_cast<akap::bf16x4*>(p) = x;
}
__device__ __forceinline__ void stv(bf16* p, const float (&v)[8]) {
  akap::bf16x8 x;
#pragma unroll
  for (int e = 0; e < 8; ++e) x[e] = (bf16)v[e];
  *reinterpret_cast<akap::bf16x8*>(p) = x;
}
static bool aligned(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

template <typename T>
__global__ __launch_bounds__(256) void embed_scaled_kernel(float* __restrict__ out,
                                                           const int64_t* __restrict__ ids,
                                                           const T* __restrict__ table, int d,
                                                           int vocab, float scale) {
  const int row = blockIdx.x;
  const int64_t id = ids[row];
  const bool ok = id >= 0 && id < vocab;
  const T* src = table + (size_t)(ok ? id : 0) * d;
  float* dst = out + (size_t)row * d;
  for (int c = threadIdx.x; c < d; c += 256) dst[c] = ok ? ldf(src + c) * scale : 0.f;
}

void launch_embed_scaled(float* out, const int64_t* ids, const void* table, bool f32, int rows,
                         int d, int vocab, float scale, hipStream_t s) {
  if (rows <= 0) return;
  if (f32)
    embed_scaled_kernel<float><<<rows, 256, 0, s>>>(out, ids, (const float*)table, d, vocab, scale);
  else
    embed_scaled_kernel<bf16><<<rows, 256, 0, s>>>(out, ids, (const bf16*)table, d, vocab, scale);
}

// x += mult * y, out = x / sqrt(mean(x^2) + eps) * w.  The row stays in registers between the
// two passes when it fits (d <= 256 * NR), so x is read and written once.
template <typename TY, typename TO, int NR>
__global__ __launch_bounds__(256) void add_norm_kernel(TO* __restrict__ out, float* __restrict__ x,
                                                       const TY* __restrict__ y, int y_stride,
                                                       const TY* __restrict__ bias, float mult,
                                                       const float* __restrict__ w, int d,
                                                       int out_stride, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float* xr = x + (size_t)row * d;
  const TY* yr = y ? y + (size_t)row * y_stride : nullptr;
  float v[NR];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = i * 256 + threadIdx.x;
    v[i] = 0.f;
    if (c < d) {
      float f = xr[c];
      if (yr) {
        f += mult * (ldf(yr + c) + (bias ? ldf(bias + c) : 0.f));
        xr[c] = f;
      }
      v[i] = f;
      ss += f * f;
    }
  }
  // rows wider than the register tile: the rest streams through memory twice
  for (int c = NR * 256 + threadIdx.x; c < d; c += 256) {
    float f = xr[c];
    if (yr) {
      f += mult * (ldf(yr + c) + (bias ? ldf(bias + c) : 0.f));
      xr[c] = f;
    }
    ss += f * f;
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  TO* orow = out + (size_t)row * out_stride;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = i * 256 + threadIdx.x;
    if (c < d) stf(orow + c, v[i] * inv * w[c]);
  }
  for (int c = NR * 256 + threadIdx.x; c < d; c += 256) stf(orow + c, xr[c] * inv * w[c]);
}

// The same with 4 elements per thread and access (d, strides and pointers multiples of 4
// elements): a row of up to 1024 NR elements stays in registers.
template <typename TY, typename TO, int NR>
__global__ __launch_bounds__(256) void add_norm_vec_kernel(TO* __restrict__ out,
                                                           float* __restrict__ x,
                                                           const TY* __restrict__ y, int y_stride,
                                                           const TY* __restrict__ bias, float mult,
                                                           const float* __restrict__ w, int d,
                                                           int out_stride, float eps) {
  __shared__ float scratch[16];
  const int row = blockIdx.x;
  float* xr = x + (size_t)row * d;
  const TY* yr = y ? y + (size_t)row * y_stride : nullptr;
  float v[NR][4];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = (i * 256 + threadIdx.x) * 4;
    if (c < d) {
      ldv(v[i], xr + c);
      if (yr) {
        float yy[4];
        ldv(yy, yr + c);
        if (bias) {
          float bb[4];
          ldv(bb, bias + c);
#pragma unroll
          for (int e = 0; e < 4; ++e) yy[e] += bb[e];
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) v[i][e] += mult * yy[e];
        stv(xr + c, v[i]);
      }
#pragma unroll
      for (int e = 0; e < 4; ++e) ss += v[i][e] * v[i][e];
    }
  }
  ss = block_sum(ss, scratch);
  const float inv = 1.0f / sqrtf(ss / (float)d + eps);
  TO* orow = out + (size_t)row * out_stride;
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int c = (i * 256 + threadIdx.x) * 4;
    if (c < d) {
      float ww[4], o[4];
      ldv(ww, w + c);
#pragma unroll
      for (int e = 0; e < 4; ++e) o[e] = v[i][e] * inv * ww[e];
      stv(orow + c, o);
    }
  }
}

template <typename TY, typename TO>
static void add_norm_t(void* out, float* x, const void* y, int y_stride, const void* bias,
                       float mult, const float* w, int rows, int d, int out_stride, float eps,
                       hipStream_t s) {
  const bool vec = d % 4 == 0 && d <= 8192 && y_stride % 4 == 0 && out_stride % 4 == 0 &&
                   aligned(x, 16) && aligned(w, 16) && aligned(y, 4 * sizeof(TY)) &&
                   aligned(bias, 4 * sizeof(TY)) && aligned(out, 4 * sizeof(TO));
  if (vec) {
#define AKAP_ADD_NORM_VEC(NR)                                                                  \
  add_norm_vec_kernel<TY, TO, NR><<<rows, 256, 0, s>>>((TO*)out, x, (const TY*)y, y_stride,      \
                                                       (const TY*)bias, mult, w, d, out_stride, eps)
    if (d <= 1024) AKAP_ADD_NORM_VEC(1);
    else if (d <= 2048) AKAP_ADD_NORM_VEC(2);
    else if (d <= 4096) AKAP_ADD_NORM_VEC(4);
    else AKAP_ADD_NORM_VEC(8);
#undef AKAP_ADD_NORM_VEC
    return;
  }
  if (d <= 1024)
    add_norm_kernel<TY, TO, 4><<<rows, 256, 0, s>>>((TO*)out, x, (const TY*)y, y_stride,
                                                    (const TY*)bias, mult, w, d, out_stride, eps);
  else
    add_norm_kernel<TY, TO, 16><<<rows, 256, 0, s>>>((TO*)out, x, (const TY*)y, y_stride,
                                                     (const TY*)bias, mult, w, d, out_stride, eps);
}

void launch_add_norm(void* out, bool out_f32, float* x, const void* y, bool y_f32, int y_stride,
                     const void* bias, float mult, const float* w, int rows, int d,
                     int out_stride, float eps, hipStream_t s) {
  if (rows <= 0) return;
  if (out_f32 && y_f32)
    add_norm_t<float, float>(out, x, y, y_stride, bias, mult, w, rows, d, out_stride, eps, s);
  else if (out_f32)
    add_norm_t<bf16, float>(out, x, y, y_stride, bias, mult, w, rows, d, out_stride, eps, s);
  else if (y_f32)
    add_norm_t<float, bf16>(out, x, y, y_stride, bias, mult, w, rows, d, out_stride, eps, s);
  else
    add_norm_t<bf16, bf16>(out, x, y, y_stride, bias, mult, w, rows, d, out_stride, eps, s);
}

template <typename T>
__global__ __launch_bounds__(256) void relu2_kernel(T* __restrict__ out, const T* __restrict__ x,
                                                    int F, int x_stride, int out_stride) {
  const int row = blockIdx.y;
  const int c = blockIdx.x * 256 + threadIdx.x;
  if (c >= F) return;
  const float f = fmaxf(ldf(x + (size_t)row * x_stride + c), 0.f);
  stf(out + (size_t)row * out_stride + c, f * f);
}

// 16 bytes per thread and access
template <typename T, int V>
__global__ __launch_bounds__(256) void relu2_vec_kernel(T* __restrict__ out,
                                                        const T* __restrict__ x, int F,
                                                        int x_stride, int out_stride) {
  const int row = blockIdx.y;
  const int c = (blockIdx.x * 256 + threadIdx.x) * V;
  if (c >= F) return;
  float v[V];
  ldv(v, x + (size_t)row * x_stride + c);
#pragma unroll
  for (int e = 0; e < V; ++e) {
    const float f = fmaxf(v[e], 0.f);
    v[e] = f * f;
  }
  stv(out + (size_t)row * out_stride + c, v);
}

void launch_relu2(void* out, const void* x, bool f32, int rows, int F, int x_stride,
                  int out_stride, hipStream_t s) {
  if (rows <= 0 || F <= 0) return;
  const int V = f32 ? 4 : 8;
  if (F % V == 0 && x_stride % V == 0 && out_stride % V == 0 && aligned(x, 16) &&
      aligned(out, 16)) {
    const dim3 vgrid((F / V + 255) / 256, rows);
    if (f32)
      relu2_vec_kernel<float, 4><<<vgrid, 256, 0, s>>>((float*)out, (const float*)x, F, x_stride,
                                                       out_stride);
    else
      relu2_vec_kernel<bf16, 8><<<vgrid, 256, 0, s>>>((bf16*)out, (const bf16*)x, F, x_stride,
                                                      out_stride);
    return;
  }
  const dim3 grid((F + 255) / 256, rows);
  if (f32)
    relu2_kernel<float><<<grid, 256, 0, s>>>((float*)out, (const float*)x, F, x_stride, out_stride);
  else
    relu2_kernel<bf16><<<grid, 256, 0, s>>>((bf16*)out, (const bf16*)x, F, x_stride, out_stride);
}

// One workgroup per token: sums of squares over the WHOLE q and the WHOLE k projection, then
// every thread norms, weights and rotates element pairs (2i, 2i+1) and stores q to q_out, k to
// the K cache and the raw k to the V cache.
template <typename T>
__global__ __launch_bounds__(256) void proj_norm_rope_cache_kernel(ProjParams p) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = (const T*)p.proj + (size_t)t * p.proj_stride;
  const T* qr = row + p.q_off;
  const T* kr = row + p.k_off;
  const int HD = p.H * p.D, GD = p.G * p.D;
  const T* qb = (const T*)p.q_b;
  const T* kb = (const T*)p.k_b;
  auto qv = [&](int c) { return ldf(qr + c) + (qb ? ldf(qb + c) : 0.f); };
  auto kv = [&](int c) { return ldf(kr + c) + (kb ? ldf(kb + c) : 0.f); };
  float sq = 0.f, sk = 0.f;
  for (int c = threadIdx.x; c < HD; c += 256) {
    const float f = qv(c);
    sq += f * f;
  }
  for (int c = threadIdx.x; c < GD; c += 256) {
    const float f = kv(c);
    sk += f * f;
  }
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float iq = 1.0f / sqrtf(sq / (float)HD + p.eps);
  const float ik = 1.0f / sqrtf(sk / (float)GD + p.eps);
  int64_t pos = p.positions[t];
  if (pos < 0) pos = 0;
  if (pos >= p.max_pos) pos = p.max_pos - 1;  // (host checks the table covers the model length)
  const float* cs = p.cos_sin ? p.cos_sin + (size_t)pos * p.rot_dims : nullptr;
  const int half = p.D >> 1, rh = p.rot_dims >> 1;
  T* qo = (T*)p.q_out + (size_t)t * HD;
  for (int e = threadIdx.x; e < (HD >> 1); e += 256) {
    const int i = e % half;
    const int c = (e / half) * p.D + 2 * i;
    float u = qv(c) * iq * p.q_w[c];
    float v = qv(c + 1) * iq * p.q_w[c + 1];
    if (cs && i < rh) {
      const float co = cs[i], si = cs[rh + i];
      const float ru = u * co - v * si;
      v = v * co + u * si;
      u = ru;
    }
    stf(qo + c, u);
    stf(qo + c + 1, v);
  }
  const int64_t slot = p.slots[t];
  if (slot < 0 || slot >= p.num_slots) return;
  const int64_t blk = slot / p.BS;
  const int off = (int)(slot % p.BS);
  for (int e = threadIdx.x; e < (GD >> 1); e += 256) {
    const int i = e % half;
    const int g = e / half;
    const int c = g * p.D + 2 * i;
    const float ru = kv(c), rv = kv(c + 1);
    float u = ru * ik * p.k_w[c];
    float v = rv * ik * p.k_w[c + 1];
    if (cs && i < rh) {
      const float co = cs[i], si = cs[rh + i];
      const float nu = u * co - v * si;
      v = v * co + u * si;
      u = nu;
    }
    T* kc = (T*)p.k_cache + (((size_t)blk * p.G + g) * p.BS + off) * p.D + 2 * i;
    stf(kc, u);
    stf(kc + 1, v);
    // the values are the projected keys, untouched; V cache [NB, G, BS/8, D, 8]
    T* vc = (T*)p.v_cache +
            ((((size_t)blk * p.G + g) * (p.BS >> 3) + (off >> 3)) * p.D + 2 * i) * 8 + (off & 7);
    vc[0] = (T)ru;
    vc[8] = (T)rv;
  }
}

// The same with 8 elements (four rotation pairs) per thread and access, the token's q (up to
// 2048 NQ elements) and k (up to 2048) held in registers between the two passes.  Needs D, the
// slice offsets and the row stride to be multiples of 8 elements and 16-byte aligned pointers.
template <typename T, int NQ>
__global__ __launch_bounds__(256) void proj_norm_rope_cache_vec_kernel(ProjParams p) {
  __shared__ float scratch[16];
  const int t = blockIdx.x;
  const T* row = (const T*)p.proj + (size_t)t * p.proj_stride;
  const T* qr = row + p.q_off;
  const T* kr = row + p.k_off;
  const int HD = p.H * p.D, GD = p.G * p.D;
  float q[NQ][8], k[8];
  float sq = 0.f, sk = 0.f;
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int c = (i * 256 + threadIdx.x) * 8;
    if (c < HD) {
      ldv(q[i], qr + c);
      if (p.q_b) {
        float bb[8];
        ldv(bb, (const T*)p.q_b + c);
#pragma unroll
        for (int e = 0; e < 8; ++e) q[i][e] += bb[e];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) sq += q[i][e] * q[i][e];
    }
  }
  const int ck = threadIdx.x * 8;
  if (ck < GD) {
    ldv(k, kr + ck);
    if (p.k_b) {
      float bb[8];
      ldv(bb, (const T*)p.k_b + ck);
#pragma unroll
      for (int e = 0; e < 8; ++e) k[e] += bb[e];
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) sk += k[e] * k[e];
  }
  sq = block_sum(sq, scratch);
  sk = block_sum(sk, scratch);
  const float iq = 1.0f / sqrtf(sq / (float)HD + p.eps);
  const float ik = 1.0f / sqrtf(sk / (float)GD + p.eps);
  int64_t pos = p.positions[t];
  if (pos < 0) pos = 0;
  if (pos >= p.max_pos) pos = p.max_pos - 1;
  const float* cs = p.cos_sin ? p.cos_sin + (size_t)pos * p.rot_dims : nullptr;
  const int rh = p.rot_dims >> 1;
  // norm weight, then rotation of the pairs (2i, 2i+1) with i < rot_dims / 2
  auto finish = [&](float (&v)[8], const float* w, float inv, int c) {
    float ww[8];
    ldv(ww, w + c);
    const int i0 = (c % p.D) >> 1;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      float u = v[e] * inv * ww[e], z = v[e + 1] * inv * ww[e + 1];
      const int i = i0 + (e >> 1);
      if (cs && i < rh) {
        const float co = cs[i], si = cs[rh + i];
        const float ru = u * co - z * si;
        z = z * co + u * si;
        u = ru;
      }
      v[e] = u;
      v[e + 1] = z;
    }
  };
  T* qo = (T*)p.q_out + (size_t)t * HD;
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int c = (i * 256 + threadIdx.x) * 8;
    if (c < HD) {
      finish(q[i], p.q_w, iq, c);
      stv(qo + c, q[i]);
    }
  }
  const int64_t slot = p.slots[t];
  if (slot < 0 || slot >= p.num_slots) return;
  const int64_t blk = slot / p.BS;
  const int off = (int)(slot % p.BS);
  // raw k -> V cache [NB, G, BS/8, D, 8]: the token's element of every (dimension) group.
  // Adjacent lanes take adjacent dimensions (16 bytes apart), so a wave's store covers whole
  // cache lines; the row is re-read from the projection (an L1 / L2 hit).
  for (int c = threadIdx.x; c < GD; c += 256) {
    const int g = c / p.D, d = c - g * p.D;
    ((T*)p.v_cache)[((((size_t)blk * p.G + g) * (p.BS >> 3) + (off >> 3)) * p.D + d) * 8 +
                    (off & 7)] = (T)(ldf(kr + c) + (p.k_b ? ldf((const T*)p.k_b + c) : 0.f));
  }
  if (ck >= GD) return;
  const int g = ck / p.D, d0 = ck % p.D;
  finish(k, p.k_w, ik, ck);
  stv((T*)p.k_cache + (((size_t)blk * p.G + g) * p.BS + off) * p.D + d0, k);
}

template <typename T>
static bool proj_vec_ok(const ProjParams& p) {
  const size_t a = 8 * sizeof(T) > 16 ? 16 : 8 * sizeof(T);
  return p.D % 8 == 0 && p.q_off % 8 == 0 && p.k_off % 8 == 0 && p.proj_stride % 8 == 0 &&
         p.H * p.D <= 4096 && p.G * p.D <= 2048 && aligned(p.proj, a) && aligned(p.q_out, a) &&
         aligned(p.q_b, a) && aligned(p.k_b, a) &&
         aligned(p.k_cache, a) && aligned(p.q_w, 16) && aligned(p.k_w, 16);
}

void launch_proj_norm_rope_cache(const ProjParams& p, bool f32, hipStream_t s) {
  if (p.T <= 0) return;
  if (f32 ? proj_vec_ok<float>(p) : proj_vec_ok<bf16>(p)) {
    const bool two = p.H * p.D > 2048;
    if (f32 && two) proj_norm_rope_cache_vec_kernel<float, 2><<<p.T, 256, 0, s>>>(p);
    else if (f32) proj_norm_rope_cache_vec_kernel<float, 1><<<p.T, 256, 0, s>>>(p);
    else if (two) proj_norm_rope_cache_vec_kernel<bf16, 2><<<p.T, 256, 0, s>>>(p);
    else proj_norm_rope_cache_vec_kernel<bf16, 1><<<p.T, 256, 0, s>>>(p);
    return;
  }
  if (f32)
    proj_norm_rope_cache_kernel<float><<<p.T, 256, 0, s>>>(p);
  else
    proj_norm_rope_cache_kernel<bf16><<<p.T, 256, 0, s>>>(p);
}

}  // namespace akap_stream
