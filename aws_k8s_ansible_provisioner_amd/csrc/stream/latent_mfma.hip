// Matrix-core latent attention (bf16): every head against ONE cached row per key.
//
// A cached token is a row [c (R) | k_rot (r)] of the latent cache, and its latent c a second time
// in 8-token groups [NB BS / 8, R, 8] (dimension-major inside a group).  With the unrotated query
// already multiplied into the latent space, head h's score of key j is
// q_lat[h] . c_j + q_rot[h] . k_rot_j and its output sum_j p_j c_j: a multi-query attention with
// R + r score dimensions and R value dimensions, whatever the number of heads.
//
// v_mfma_f32_32x32x16_bf16 computes S^T = K Q^T (keys are the 32 rows, queries the 32 columns)
// and O^T = C^T P^T.  A query is a lane column, so its softmax statistics are 16 registers and
// one exchange between the lane halves.  The K rows are loaded in the order (bits 2 and 3 of
// the row swapped) that makes a lane's S^T accumulators exactly the 8 keys of one group, so P
// moves from accumulator to operand without lane traffic and the C^T operand is one 16-byte
// load from the grouped copy.  The query tile (32 columns x (R + r)) lives in LDS.  K and C
// fragments come straight from global memory (L1 / L2: the heads of a token tile are
// workgroups of one XCD).
//
// Prefill: the 32 columns are consecutive tokens of one head (causal mask only in the blocks
// that cross its positions).  Decode: the 32 columns are the heads of one token; the key range
// is cut into partitions merged by a second launch.  Narrow latents (R <= 128): one wave per
// tile.  Wide latents: four waves per tile (see below).
#include "../kernels/common.h"
#include "stream.h"

namespace akap_stream {

using akap::bf16;
using akap::bf16x8;
using akap::f32x16;

namespace {

__device__ __forceinline__ int swap23(int r) { return (r & ~12) | ((r & 4) << 1) | ((r & 8) >> 1); }

template <int NV>
struct LatentState {
  f32x16 o[NV];
  float m, l;   // m in log2 units of the scaled scores
};

// LDS row pitch of the query tile (elements): 16 bytes of padding per row
__host__ __device__ constexpr int q_pitch(int DK) { return DK + 8; }

// The wave's 32 query columns -> LDS [32][pitch]: column col is token tok[col] of head h,
// [q_lat[h, tok] (R) | q[tok, h, rot_off : rot_off + r]].
template <int NV, int NKR>
__device__ __forceinline__ void load_queries(bf16* qs, const LatentAttnParams& p, int h, int my_tok) {
  constexpr int R = 32 * NV, DK = R + 16 * NKR, CH = DK / 8, P = q_pitch(DK);
  const int lane = threadIdx.x & 63;
  for (int idx = lane; idx < 32 * CH; idx += 64) {
    const int col = idx / CH, ch = idx - col * CH;
    const int t = __shfl(my_tok, col, 64);
    const bf16* src = ch * 8 < R
        ? (const bf16*)p.q_lat + ((size_t)h * p.T + t) * R + ch * 8
        : (const bf16*)p.q + (size_t)t * p.q_stride + (size_t)h * p.q_head + p.rot_off + ch * 8 - R;
    *reinterpret_cast<bf16x8*>(qs + col * P + ch * 8) = *reinterpret_cast<const bf16x8*>(src);
  }
  __builtin_amdgcn_wave_barrier();
}

// Keys [jb, je] (jb a multiple of 32) against the wave's 32 columns; pos: this lane's column's
// position (keys above it are masked); pos_min: the smallest position among the columns.
template <int NV, int NKR>
__device__ __forceinline__ void attend(LatentState<NV>& st, const LatentAttnParams& p,
                                       const int32_t* __restrict__ bt, const bf16* qs, int pos,
                                       int pos_min, int jb, int je) {
  constexpr int R = 32 * NV, DK = R + 16 * NKR, KS = DK / 16, P = q_pitch(DK);
  const float sc2 = p.scale * 1.44269504088896f;
  const int lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int krow = swap23(col);
  const bf16* cache = (const bf16*)p.cache;
  const bf16* vg = (const bf16*)p.vgroups;
  const bf16* qcol = qs + col * P + 8 * hf;
  for (int j0 = jb; j0 <= je; j0 += 32) {
    const int bi = j0 / p.BS;
    int blk = bi < p.max_blocks ? bt[bi] : 0;
    if (blk < 0 || blk >= p.NB) blk = 0;
    const size_t row0 = (size_t)blk * p.BS + (j0 - bi * p.BS);   // a multiple of 32
    const bf16* kp = cache + (row0 + krow) * DK + 8 * hf;
    f32x16 s;
#pragma unroll
    for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
    for (int c = 0; c < KS; ++c) {
      const bf16x8 kf = *reinterpret_cast<const bf16x8*>(kp + 16 * c);
      const bf16x8 qf = *reinterpret_cast<const bf16x8*>(qcol + 16 * c);
      s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kf, qf, s, 0, 0, 0);
    }
    // accumulator register i of this lane: key j0 + 16 (i >> 3) + 8 hf + (i & 7), column col
    float sv[16];
    float bmax = -INFINITY;
    if (j0 + 31 <= pos_min) {       // (wave-uniform) visible to every column
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        sv[i] = s[i];
        bmax = fmaxf(bmax, sv[i]);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const int key = j0 + 16 * (i >> 3) + 8 * hf + (i & 7);
        sv[i] = key <= pos ? s[i] : -INFINITY;
        bmax = fmaxf(bmax, sv[i]);
      }
    }
    bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    const float mn = fmaxf(st.m, bmax * sc2);
    const float ms = mn == -INFINITY ? 0.f : mn;   // nothing visible yet: every exp below is 0
    const float alpha = __builtin_amdgcn_exp2f(st.m - ms);
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      sv[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], sc2, -ms));
      psum += sv[i];
    }
    psum += __shfl_xor(psum, 32, 64);
    st.l = st.l * alpha + psum;
    st.m = mn;
    bf16x8 pb[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) pb[i >> 3][i & 7] = (bf16)sv[i];
    if (__any(alpha != 1.0f)) {     // (wave-uniform) the maxima settle after the first blocks
#pragma unroll
      for (int dt = 0; dt < NV; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) st.o[dt][i] *= alpha;
    }
    // latent groups of this block: row0 / 8 is its first group
    const bf16* vp = vg + (((row0 >> 3) + hf) * R + col) * 8;
#pragma unroll
    for (int dt = 0; dt < NV; ++dt) {
#pragma unroll
      for (int sl = 0; sl < 2; ++sl) {
        const bf16x8 vf = *reinterpret_cast<const bf16x8*>(vp + ((size_t)(2 * sl) * R + 32 * dt) * 8);
        st.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(vf, pb[sl], st.o[dt], 0, 0, 0);
      }
    }
  }
}

template <int NV>
__device__ __forceinline__ void init(LatentState<NV>& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) st.o[dt][i] = 0.f;
}

// accumulator register i of o[dt]: dimension 32 dt + 8 (i >> 2) + 4 hf + (i & 3)
template <int NV>
__device__ __forceinline__ void store(const LatentState<NV>& st, bf16* o) {
  const int hf = (threadIdx.x & 63) >> 5;
  const float f = st.l > 0.f ? 1.0f / st.l : 0.f;
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; i += 4) {
      akap::bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16)(st.o[dt][i + e] * f);
      *reinterpret_cast<akap::bf16x4*>(o + 32 * dt + 8 * (i >> 2) + 4 * hf) = v;
    }
}

// Prefill: flat grid over (32-token sub-tile, head block) units, WPB waves (heads) per workgroup
template <int NV, int NKR, int WPB>
__global__ __launch_bounds__(64 * WPB) void latent_prefill_mfma_kernel(LatentAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int R = 32 * NV, DK = R + 16 * NKR, P = q_pitch(DK);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 31;
  // the hardware deals workgroup i to XCD i % 8: units (sub-tiles, longest first) are dealt
  // round-robin over the XCDs, and the head blocks of one unit are workgroups of ONE XCD, so
  // a token tile's cached rows cross into a single L2
  const int hblocks = (p.H + WPB - 1) / WPB;
  const int sub = p.tile_rows / 32;
  const int xcd = blockIdx.x & 7, jx = blockIdx.x >> 3;
  const int unit = (jx / hblocks) * 8 + xcd;
  if (unit >= p.num_tiles * sub) return;
  const int h = (jx % hblocks) * WPB + wave;
  if (h >= p.H) return;                          // no workgroup barriers below
  // the scheduler sorts tiles by ascending causal work: walk from the end
  const int tile = p.num_tiles - 1 - unit / sub;
  const int si = sub - 1 - unit % sub;
  const int b = p.tile_seq[tile];
  if (b < 0 || b >= p.B) return;
  const int qs0 = p.q_start[b];
  const int qlen = p.q_start[b + 1] - qs0;
  const int kv = p.seq_lens[b];
  const int rend = min(p.tile_row[tile] + p.tile_rows, qlen);
  const int r0 = p.tile_row[tile] + 32 * si;
  if (r0 >= rend || kv < qlen) return;
  const int r = r0 + col;
  const bool valid = r < rend;
  const int t = qs0 + (valid ? r : r0);
  const int pos = kv - qlen + r;
  bf16* qs = reinterpret_cast<bf16*>(smem) + (size_t)wave * 32 * P;
  load_queries<NV, NKR>(qs, p, h, t);
  LatentState<NV> st;
  init(st);
  const int pos_first = kv - qlen + r0;
  const int pos_last = kv - qlen + min(r0 + 31, rend - 1);
  attend<NV, NKR>(st, p, p.block_tables + (size_t)b * p.max_blocks, qs, pos, pos_first, 0,
                  pos_last);
  if (valid) store<NV>(st, (bf16*)p.out + ((size_t)h * p.T + t) * R);
}

// Decode: grid (B, ceil(H / 32), parts), one wave; columns are heads
template <int NV, int NKR>
__global__ __launch_bounds__(64) void latent_decode_mfma_kernel(LatentAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int R = 32 * NV;
  const int lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int b = blockIdx.x, part = blockIdx.z;
  const int c0 = blockIdx.y * 32;
  const int kv = p.seq_lens[b];
  if (kv <= 0) return;                           // a padding row: nothing read or written
  const bool valid = c0 + col < p.H;
  const int h = valid ? c0 + col : c0;
  const int pos1 = kv - 1;
  int per = (pos1 + 1 + p.num_parts - 1) / p.num_parts;
  per = (per + 31) & ~31;
  const int jb = part * per;
  const int je = min(pos1, jb + per - 1);
  bf16* qs = reinterpret_cast<bf16*>(smem);
  LatentState<NV> st;
  init(st);
  if (jb <= je) {
    // column col is head c0 + col of token b: per-column head, one token
    {
      constexpr int DK = R + 16 * NKR, CH = DK / 8, P = q_pitch(DK);
      for (int idx = lane; idx < 32 * CH; idx += 64) {
        const int cc = idx / CH, ch = idx - cc * CH;
        const int hh = c0 + cc < p.H ? c0 + cc : c0;
        const bf16* src = ch * 8 < R
            ? (const bf16*)p.q_lat + ((size_t)hh * p.T + b) * R + ch * 8
            : (const bf16*)p.q + (size_t)b * p.q_stride + (size_t)hh * p.q_head + p.rot_off +
                  ch * 8 - R;
        *reinterpret_cast<bf16x8*>(qs + cc * P + ch * 8) = *reinterpret_cast<const bf16x8*>(src);
      }
      __builtin_amdgcn_wave_barrier();
    }
    attend<NV, NKR>(st, p, p.block_tables + (size_t)b * p.max_blocks, qs, pos1, pos1, jb, je);
  }
  if (!valid) return;
  if (p.num_parts == 1) {
    store<NV>(st, (bf16*)p.out + ((size_t)h * p.T + b) * R);
    return;
  }
  const size_t slot = ((size_t)b * p.H + h) * p.num_parts + part;
  if (hf == 0) {
    p.ws_ml[slot * 2] = st.m;
    p.ws_ml[slot * 2 + 1] = st.l;
  }
#pragma unroll
  for (int dt = 0; dt < NV; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i)
      p.ws_o[slot * R + 32 * dt + 8 * (i >> 2) + 4 * hf + (i & 3)] = st.o[dt][i];
}


// ---- wide latents (R >= 256): four waves share one tile of 32 query columns -------------------
// At R = 512 a single wave's output accumulators alone are 256 registers.  Four waves split the
// work of a 128-key step instead: wave w scores keys [32 w, 32 w + 32) of the step against the
// whole query tile (S^T = K Q^T over all R + r dimensions), the waves agree on the running
// maximum through LDS, publish their bf16 P fragments there, and each wave then accumulates
// O^T for ITS quarter of the latent dimensions over all 128 keys.  No matrix product is computed
// twice, a wave holds R / 8 accumulator registers, and two or three workgroups fit a CU.
template <int NVW>
struct CoopState {
  f32x16 o[NVW];   // this wave's quarter of the latent dimensions
  float m, l;
};

template <int NV, int NKR>
struct CoopSmem {
  static constexpr int DK = 32 * NV + 16 * NKR;
  static constexpr size_t q_bytes = (size_t)32 * q_pitch(DK) * sizeof(bf16);
  static constexpr size_t p_bytes = (size_t)4 * 2 * 64 * sizeof(bf16x8);
  static constexpr size_t fixed = q_bytes + p_bytes + 2 * 4 * 32 * sizeof(float);
  // + one cache row index per 32-key block of the workgroup's key range
  static size_t bytes(const LatentAttnParams& p) {
    return fixed + (size_t)p.max_blocks * (p.BS / 32) * sizeof(int32_t);
  }
};

// The cache rows of the 32-key blocks [jb, je] of a sequence -> LDS, once: a block's row is
// then an LDS read away instead of a block-table load ahead of every fragment load (with it,
// a 128-key step was a chain of six dependent global loads, 17 us for a lone workgroup).
template <int NV, int NKR>
__device__ __forceinline__ void coop_load_rows(unsigned char* smem, const LatentAttnParams& p,
                                               const int32_t* __restrict__ bt, int jb, int je) {
  int32_t* sm_rows = reinterpret_cast<int32_t*>(smem + CoopSmem<NV, NKR>::fixed);
  const int n = (je - jb) / 32 + 1;
  for (int i = threadIdx.x; i < n; i += 256) {
    const int j0 = jb + 32 * i;
    const int bi = j0 / p.BS;
    int blk = bi < p.max_blocks ? bt[bi] : 0;
    if (blk < 0 || blk >= p.NB) blk = 0;
    sm_rows[i] = blk * p.BS + (j0 - bi * p.BS);
  }
}

template <int NV, int NKR, int KB>
__device__ __forceinline__ void coop_attend(CoopState<NV / 4>& st, const LatentAttnParams& p,
                                            const int32_t* __restrict__ bt, unsigned char* smem,
                                            int pos, int pos_min, int jb, int je) {
  constexpr int R = 32 * NV, DK = R + 16 * NKR, KS = DK / 16, P = q_pitch(DK), NVW = NV / 4;
  using SM = CoopSmem<NV, NKR>;
  const float sc2 = p.scale * 1.44269504088896f;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int krow = swap23(col);
  const bf16* cache = (const bf16*)p.cache;
  const bf16* vg = (const bf16*)p.vgroups;
  const bf16* qcol = reinterpret_cast<const bf16*>(smem) + col * P + 8 * hf;
  bf16x8* sm_p = reinterpret_cast<bf16x8*>(smem + SM::q_bytes);          // [4][2][64]
  float* sm_max = reinterpret_cast<float*>(smem + SM::q_bytes + SM::p_bytes);   // [4][32]
  float* sm_sum = sm_max + 4 * 32;                                              // [4][32]
  const int32_t* sm_rows = reinterpret_cast<const int32_t*>(smem + SM::fixed);  // coop_load_rows
  auto row_of = [&](int j0) -> size_t { return (size_t)sm_rows[(j0 - jb) >> 5]; };
  // Fragment loads are issued in batches AHEAD of the products that use them (a load issued
  // right before its product makes a 128-key step a chain of 68 memory latencies: 17 us for a
  // lone workgroup): K in double-buffered batches of KB k-steps, the latent fragments of a
  // 32-key block one block ahead, the first block's before the softmax.  (Prefill: KB = 4 and
  // two waves per SIMD; decode: KB = 12 and one.)
  constexpr int NKB = (KS + KB - 1) / KB;
  auto load_v = [&](bf16x8 (&vf)[2 * NVW], int jk) {
    const bf16* vp = vg + (((row_of(jk) >> 3) + hf) * R + 32 * (wave * NVW) + col) * 8;
#pragma unroll
    for (int dt = 0; dt < NVW; ++dt) {
      vf[2 * dt] = *reinterpret_cast<const bf16x8*>(vp + (size_t)(32 * dt) * 8);
      vf[2 * dt + 1] = *reinterpret_cast<const bf16x8*>(vp + ((size_t)2 * R + 32 * dt) * 8);
    }
  };
  // the first K batch of a step is requested a step ahead (before the previous step's softmax)
  bf16x8 ka[KB], kb2[KB];
  auto load_k0 = [&](int jw) {
    const bf16* kp = cache + (row_of(jw) + krow) * DK + 8 * hf;
#pragma unroll
    for (int c = 0; c < KB; ++c)
      if (c < KS) ka[c] = *reinterpret_cast<const bf16x8*>(kp + 16 * c);
  };
  if (jb + 32 * wave <= je) load_k0(jb + 32 * wave);
  for (int j0 = jb; j0 <= je; j0 += 128) {
    const int jw = j0 + 32 * wave;
    const bool active = jw <= je;                    // (wave-uniform)
    float sv[16];
    float bmax = -INFINITY;
    bf16x8 va[2 * NVW], vb[2 * NVW];
    if (active) {
      const bf16* kp = cache + (row_of(jw) + krow) * DK + 8 * hf;
      f32x16 s;
#pragma unroll
      for (int i = 0; i < 16; ++i) s[i] = 0.f;
#pragma unroll
      for (int b = 0; b < NKB; ++b) {
        // the next batch goes out before this batch's products
        if (b + 1 < NKB) {
#pragma unroll
          for (int c = 0; c < KB; ++c)
            if ((b + 1) * KB + c < KS) {
              const bf16x8 f = *reinterpret_cast<const bf16x8*>(kp + 16 * ((b + 1) * KB + c));
              if (b % 2 == 0) kb2[c] = f; else ka[c] = f;
            }
        } else {
          load_v(va, j0);                            // block 0 of the step: always a valid block
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int c = 0; c < KB; ++c)
          if (b * KB + c < KS) {
            const bf16x8 qf = *reinterpret_cast<const bf16x8*>(qcol + 16 * (b * KB + c));
            s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(b % 2 == 0 ? ka[c] : kb2[c], qf, s, 0, 0, 0);
          }
        __builtin_amdgcn_sched_barrier(0);
      }
      if (jw + 31 <= pos_min) {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          sv[i] = s[i];
          bmax = fmaxf(bmax, sv[i]);
        }
      } else {
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          const int key = jw + 16 * (i >> 3) + 8 * hf + (i & 7);
          sv[i] = key <= pos ? s[i] : -INFINITY;
          bmax = fmaxf(bmax, sv[i]);
        }
      }
      bmax = fmaxf(bmax, __shfl_xor(bmax, 32, 64));
    } else {
      load_v(va, j0);
    }
    if (jw + 128 <= je) load_k0(jw + 128);           // (both K buffers are free here)
    if (hf == 0) sm_max[wave * 32 + col] = bmax;
    __syncthreads();
    const float bm = fmaxf(fmaxf(sm_max[col], sm_max[32 + col]),
                           fmaxf(sm_max[64 + col], sm_max[96 + col]));
    const float mn = fmaxf(st.m, bm * sc2);
    const float ms = mn == -INFINITY ? 0.f : mn;
    const float alpha = __builtin_amdgcn_exp2f(st.m - ms);
    float psum = 0.f;
    bf16x8 pb[2];
    if (active) {
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        sv[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], sc2, -ms));
        psum += sv[i];
      }
      psum += __shfl_xor(psum, 32, 64);
#pragma unroll
      for (int i = 0; i < 16; ++i) pb[i >> 3][i & 7] = (bf16)sv[i];
      sm_p[(wave * 2 + 0) * 64 + lane] = pb[0];
      sm_p[(wave * 2 + 1) * 64 + lane] = pb[1];
    }
    if (hf == 0) sm_sum[wave * 32 + col] = psum;
    st.m = mn;
    if (__any(alpha != 1.0f)) {
#pragma unroll
      for (int dt = 0; dt < NVW; ++dt)
#pragma unroll
        for (int i = 0; i < 16; ++i) st.o[dt][i] *= alpha;
    }
    __syncthreads();
    st.l = st.l * alpha + ((sm_sum[col] + sm_sum[32 + col]) + (sm_sum[64 + col] + sm_sum[96 + col]));
#pragma unroll
    for (int kb = 0; kb < 4; ++kb) {
      const int jk = j0 + 32 * kb;
      if (jk <= je) {                                // (uniform over the workgroup)
        if (kb + 1 < 4 && jk + 32 <= je) {           // the next block's fragments go out first
          if (kb % 2 == 0) load_v(vb, jk + 32); else load_v(va, jk + 32);
        }
        const bf16x8 p0 = sm_p[(kb * 2 + 0) * 64 + lane];
        const bf16x8 p1 = sm_p[(kb * 2 + 1) * 64 + lane];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int dt = 0; dt < NVW; ++dt) {
          st.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kb % 2 == 0 ? va[2 * dt] : vb[2 * dt],
                                                             p0, st.o[dt], 0, 0, 0);
          st.o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              kb % 2 == 0 ? va[2 * dt + 1] : vb[2 * dt + 1], p1, st.o[dt], 0, 0, 0);
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  }
}

// the workgroup's query tile -> LDS: column c is (token tok(c), head head(c))
template <int NV, int NKR, typename F>
__device__ __forceinline__ void coop_load_queries(unsigned char* smem, const LatentAttnParams& p,
                                                  F col_src) {
  constexpr int R = 32 * NV, DK = R + 16 * NKR, CH = DK / 8, P = q_pitch(DK);
  bf16* qs = reinterpret_cast<bf16*>(smem);
  for (int idx = threadIdx.x; idx < 32 * CH; idx += 256) {
    const int c = idx / CH, ch = idx - c * CH;
    int t, h;
    col_src(c, t, h);
    const bf16* src = ch * 8 < R
        ? (const bf16*)p.q_lat + ((size_t)h * p.T + t) * R + ch * 8
        : (const bf16*)p.q + (size_t)t * p.q_stride + (size_t)h * p.q_head + p.rot_off + ch * 8 - R;
    *reinterpret_cast<bf16x8*>(qs + c * P + ch * 8) = *reinterpret_cast<const bf16x8*>(src);
  }
  __syncthreads();
}

template <int NVW>
__device__ __forceinline__ void coop_init(CoopState<NVW>& st) {
  st.m = -INFINITY;
  st.l = 0.f;
#pragma unroll
  for (int dt = 0; dt < NVW; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) st.o[dt][i] = 0.f;
}

// Prefill: flat grid over (32-token sub-tile, head) units, one workgroup of 4 waves each
template <int NV, int NKR>
__global__ __launch_bounds__(256, 2) void latent_prefill_coop_kernel(LatentAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int R = 32 * NV, NVW = NV / 4;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int sub = p.tile_rows / 32;
  const int xcd = blockIdx.x & 7, jx = blockIdx.x >> 3;
  const int unit = (jx / p.H) * 8 + xcd;             // every exit below is workgroup-uniform
  if (unit >= p.num_tiles * sub) return;
  const int h = jx % p.H;
  const int tile = p.num_tiles - 1 - unit / sub;
  const int si = sub - 1 - unit % sub;
  const int b = p.tile_seq[tile];
  if (b < 0 || b >= p.B) return;
  const int qs0 = p.q_start[b];
  const int qlen = p.q_start[b + 1] - qs0;
  const int kv = p.seq_lens[b];
  const int rend = min(p.tile_row[tile] + p.tile_rows, qlen);
  const int r0 = p.tile_row[tile] + 32 * si;
  if (r0 >= rend || kv < qlen) return;
  const int pos_last = kv - qlen + min(r0 + 31, rend - 1);
  coop_load_rows<NV, NKR>(smem, p, p.block_tables + (size_t)b * p.max_blocks, 0, pos_last);
  coop_load_queries<NV, NKR>(smem, p, [&](int c, int& t, int& hh) {
    t = qs0 + (r0 + c < rend ? r0 + c : r0);
    hh = h;
  });
  const int r = r0 + col;
  const bool valid = r < rend;
  const int t = qs0 + (valid ? r : r0);
  CoopState<NVW> st;
  coop_init(st);
  const int pos_first = kv - qlen + r0;
  coop_attend<NV, NKR, 4>(st, p, p.block_tables + (size_t)b * p.max_blocks, smem, kv - qlen + r,
                       pos_first, 0, pos_last);
  if (!valid) return;
  const float f = st.l > 0.f ? 1.0f / st.l : 0.f;
  bf16* o = (bf16*)p.out + ((size_t)h * p.T + t) * R + 32 * (wave * NVW);
#pragma unroll
  for (int dt = 0; dt < NVW; ++dt)
#pragma unroll
    for (int i = 0; i < 16; i += 4) {
      akap::bf16x4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (bf16)(st.o[dt][i + e] * f);
      *reinterpret_cast<akap::bf16x4*>(o + 32 * dt + 8 * (i >> 2) + 4 * hf) = v;
    }
}

// Decode: grid (B, ceil(H / 32), parts), one workgroup of 4 waves; columns are heads
template <int NV, int NKR>
__global__ __launch_bounds__(256) void latent_decode_coop_kernel(LatentAttnParams p) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  constexpr int R = 32 * NV, NVW = NV / 4;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int col = lane & 31, hf = lane >> 5;
  const int b = blockIdx.x, part = blockIdx.z;
  const int c0 = blockIdx.y * 32;
  const int kv = p.seq_lens[b];
  if (kv <= 0) return;                               // (workgroup-uniform) a padding row
  const bool valid = c0 + col < p.H;
  const int h = valid ? c0 + col : c0;
  const int pos1 = kv - 1;
  int per = (pos1 + 1 + p.num_parts - 1) / p.num_parts;
  per = (per + 127) & ~127;
  const int jb = part * per;
  const int je = min(pos1, jb + per - 1);
  CoopState<NVW> st;
  coop_init(st);
  if (jb <= je) {                                    // (workgroup-uniform)
    coop_load_rows<NV, NKR>(smem, p, p.block_tables + (size_t)b * p.max_blocks, jb, je);
    coop_load_queries<NV, NKR>(smem, p, [&](int c, int& t, int& hh) {
      t = b;
      hh = c0 + c < p.H ? c0 + c : c0;
    });
    coop_attend<NV, NKR, 12>(st, p, p.block_tables + (size_t)b * p.max_blocks, smem, pos1, pos1, jb,
                            je);
  }
  if (!valid) return;
  if (p.num_parts == 1) {
    const float f = st.l > 0.f ? 1.0f / st.l : 0.f;
    bf16* o = (bf16*)p.out + ((size_t)h * p.T + b) * R + 32 * (wave * NVW);
#pragma unroll
    for (int dt = 0; dt < NVW; ++dt)
#pragma unroll
      for (int i = 0; i < 16; ++i)
        o[32 * dt + 8 * (i >> 2) + 4 * hf + (i & 3)] = (bf16)(st.o[dt][i] * f);
    return;
  }
  const size_t slot = ((size_t)b * p.H + h) * p.num_parts + part;
  if (wave == 0 && hf == 0) {
    p.ws_ml[slot * 2] = st.m;
    p.ws_ml[slot * 2 + 1] = st.l;
  }
  float* wo = p.ws_o + slot * R + 32 * (wave * NVW);
#pragma unroll
  for (int dt = 0; dt < NVW; ++dt)
#pragma unroll
    for (int i = 0; i < 16; ++i) wo[32 * dt + 8 * (i >> 2) + 4 * hf + (i & 3)] = st.o[dt][i];
}

// grid (B, H), 128 threads: merge the partitions of one (token, head)
__global__ __launch_bounds__(128) void latent_decode_merge_kernel(LatentAttnParams p) {
  extern __shared__ float wts[];                     // [parts] weights of the partitions
  const int b = blockIdx.x, h = blockIdx.y;
  if (p.seq_lens[b] <= 0) return;                    // (workgroup-uniform)
  const size_t base = ((size_t)b * p.H + h) * p.num_parts;
  float m = -INFINITY;
  for (int i = 0; i < p.num_parts; ++i)
    if (p.ws_ml[(base + i) * 2 + 1] > 0.f) m = fmaxf(m, p.ws_ml[(base + i) * 2]);
  float l = 0.f;
  for (int i = 0; i < p.num_parts; ++i) {
    const float li = p.ws_ml[(base + i) * 2 + 1];
    const float w = li > 0.f ? __builtin_amdgcn_exp2f(p.ws_ml[(base + i) * 2] - m) : 0.f;
    l += li * w;
    if (threadIdx.x == 0) wts[i] = w;
  }
  __syncthreads();
  const float f = l > 0.f ? 1.0f / l : 0.f;
  bf16* o = (bf16*)p.out + ((size_t)h * p.T + b) * p.R;
  for (int d = threadIdx.x; d < p.R; d += 128) {
    float a = 0.f;
    for (int i = 0; i < p.num_parts; ++i)
      if (wts[i] > 0.f) a += p.ws_o[(base + i) * p.R + d] * wts[i];
    o[d] = (bf16)(a * f);
  }
}

template <int NV, int NKR>
void launch_prefill(const LatentAttnParams& p, hipStream_t s) {
  constexpr int DK = 32 * NV + 16 * NKR;
  const int units = p.num_tiles * (p.tile_rows / 32);
  const unsigned padded = (unsigned)((units + 7) / 8 * 8);
  if constexpr (NV >= 8) {
    latent_prefill_coop_kernel<NV, NKR><<<padded * p.H, 256, CoopSmem<NV, NKR>::bytes(p), s>>>(p);
  } else {
    // narrow latents: one wave per tile and head, 4 heads per workgroup
    constexpr size_t per_wave = (size_t)32 * q_pitch(DK) * sizeof(bf16);
    static_assert(4 * per_wave <= 64 * 1024, "query tiles of four heads fit the LDS");
    latent_prefill_mfma_kernel<NV, NKR, 4><<<padded * ((p.H + 3) / 4), 256, 4 * per_wave, s>>>(p);
  }
}

template <int NV, int NKR>
void launch_decode(const LatentAttnParams& p, hipStream_t s) {
  constexpr int DK = 32 * NV + 16 * NKR;
  const dim3 grid(p.B, (p.H + 31) / 32, p.num_parts);
  if constexpr (NV >= 8)
    latent_decode_coop_kernel<NV, NKR><<<grid, 256, CoopSmem<NV, NKR>::bytes(p), s>>>(p);
  else
    latent_decode_mfma_kernel<NV, NKR><<<grid, 64, (size_t)32 * q_pitch(DK) * sizeof(bf16), s>>>(p);
  if (p.num_parts > 1)
    latent_decode_merge_kernel<<<dim3(p.B, p.H), 128, p.num_parts * sizeof(float), s>>>(p);
}

// ---- per-head products of small batches ------------------------------------------------------
// out[h, t, n] = sum_k a[h, t, k] w[h, n, k] for a few rows t (decode steps): one wave per
// 32 x 32 tile of one head, both operands contiguous in k (16-byte fragment loads), k in
// batches of 8 MFMA steps whose loads go out together.  The library's batched GEMM takes
// 12-14 us for these 0.1 GFLOP products at 64 rows.
__global__ __launch_bounds__(64) void head_matmul_kernel(bf16* __restrict__ out,
                                                         const bf16* __restrict__ a, int64_t a_hs,
                                                         int64_t a_ts, const bf16* __restrict__ w,
                                                         int T, int N, int K) {
  const int lane = threadIdx.x;
  const int col = lane & 31, hf = lane >> 5;
  const int ntn = N / 32;
  const int h = blockIdx.y, nt = blockIdx.x % ntn, mt = blockIdx.x / ntn;
  const int row = min(mt * 32 + col, T - 1);
  const bf16* ap = a + (size_t)h * a_hs + (size_t)row * a_ts + 8 * hf;
  const bf16* wp = w + ((size_t)h * N + nt * 32 + col) * K + 8 * hf;
  f32x16 acc;
#pragma unroll
  for (int i = 0; i < 16; ++i) acc[i] = 0.f;
  for (int k0 = 0; k0 < K; k0 += 128) {
    bf16x8 af[8], wf[8];
#pragma unroll
    for (int c = 0; c < 8; ++c)
      if (k0 + 16 * c < K) {                         // (uniform)
        af[c] = *reinterpret_cast<const bf16x8*>(ap + k0 + 16 * c);
        wf[c] = *reinterpret_cast<const bf16x8*>(wp + k0 + 16 * c);
      }
#pragma unroll
    for (int c = 0; c < 8; ++c)
      if (k0 + 16 * c < K) acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[c], wf[c], acc, 0, 0, 0);
  }
  // accumulator register i: row 8 (i >> 2) + 4 hf + (i & 3) of the tile, column col
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = mt * 32 + 8 * (i >> 2) + 4 * hf + (i & 3);
    if (r < T) out[((size_t)h * T + r) * N + nt * 32 + col] = (bf16)acc[i];
  }
}

}  // namespace

void launch_head_matmul(void* out, const void* a, int64_t a_hs, int64_t a_ts, const void* w, int H,
                        int T, int N, int K, hipStream_t s) {
  if (H <= 0 || T <= 0) return;
  const dim3 grid((N / 32) * ((T + 31) / 32), H);
  head_matmul_kernel<<<grid, 64, 0, s>>>((bf16*)out, (const bf16*)a, a_hs, a_ts, (const bf16*)w, T,
                                         N, K);
}

// the latent / rotated sizes the matrix kernels are built for
bool latent_mfma_sizes(int R, int r) {
  const int nv = R / 32, nkr = r / 16;
  if (R % 32 || r % 16) return false;
  return (nv == 2 && nkr == 1) || (nv == 3 && nkr == 1) || (nv == 4 && (nkr == 1 || nkr == 2)) ||
         (nv == 8 && (nkr == 2 || nkr == 4)) || (nv == 16 && nkr == 4);
}

#define LATENT_SIZES(F)                                                                    \
  const int nv = p.R / 32, nkr = p.r / 16;                                                 \
  if (nv == 2 && nkr == 1) F<2, 1>(p, s);                                                  \
  else if (nv == 3 && nkr == 1) F<3, 1>(p, s);                                             \
  else if (nv == 4 && nkr == 1) F<4, 1>(p, s);                                             \
  else if (nv == 4 && nkr == 2) F<4, 2>(p, s);                                             \
  else if (nv == 8 && nkr == 2) F<8, 2>(p, s);                                             \
  else if (nv == 8 && nkr == 4) F<8, 4>(p, s);                                             \
  else if (nv == 16 && nkr == 4) F<16, 4>(p, s);

void launch_latent_prefill_mfma(const LatentAttnParams& p, hipStream_t s) {
  if (p.num_tiles <= 0 || p.H <= 0) return;
  LATENT_SIZES(launch_prefill)
}

void launch_latent_decode_mfma(const LatentAttnParams& p, hipStream_t s) {
  if (p.B <= 0 || p.H <= 0) return;
  LATENT_SIZES(launch_decode)
}

}  // namespace akap_stream
