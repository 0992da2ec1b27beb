// Launchers of the fp32-residual-stream kernels (library _C_stream.so, torch.ops.akap_stream).
//
// Activations, weights and the KV cache are bf16 or fp32 (`f32` flags below); norms, rotary
// angles, attention scores / softmax / gates and the residual sum are fp32 in both.  Every size
// (width, heads, GQA ratio, head size, block size) is a run-time argument.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace akap_stream {

void launch_embed_scaled(float* out, const int64_t* ids, const void* table, bool f32, int rows,
                         int d, int vocab, float scale, hipStream_t s);
// x (fp32, contiguous rows of d) += mult * y (y may be null); out = rmsnorm(x) * w
// (bias: d values of y's type added to every row of y, or null)
void launch_add_norm(void* out, bool out_f32, float* x, const void* y, bool y_f32, int y_stride,
                     const void* bias, float mult, const float* w, int rows, int d,
                     int out_stride, float eps, hipStream_t s);
void launch_relu2(void* out, const void* x, bool f32, int rows, int F, int x_stride,
                  int out_stride, hipStream_t s);

struct ProjParams {
  const void* proj;   // [T, N] fused projection rows
  int proj_stride;
  void* q_out;        // [T, H, D]
  void* k_cache;      // [NB, G, BS, D]
  void* v_cache;
  const int64_t* positions;
  const int64_t* slots;
  const float* cos_sin;  // [max_pos, rot_dims] = [cos | sin], or null
  int max_pos, rot_dims;
  const float* q_w;      // [H D]
  const float* k_w;      // [G D]
  const void* q_b;       // [H D] / [G D] of the projection's type, added to the q / k slices
  const void* k_b;       //   before anything else (the projection's biases), or null
  int T, H, G, D, BS, q_off, k_off;
  int64_t num_slots;     // NB * BS
  float eps;
};
void launch_proj_norm_rope_cache(const ProjParams& p, bool f32, hipStream_t s);

struct AttnParams {
  void* out;            // rows of out_stride elements; head h at columns [h D, (h+1) D)
  int out_stride;
  const void* q;        // [T, H, D]
  const void* k_cache;  // [NB, G, BS, D]
  const void* v_cache;
  const int32_t* block_tables;  // [B, max_blocks]
  int max_blocks;
  const int32_t* seq_lens;      // [B]
  const int32_t* q_start;       // [B + 1] (prefill)
  const int32_t* tile_seq;      // prefill tile map
  const int32_t* tile_row;
  int num_tiles, tile_rows;
  const void* gate;     // [T, H] logits with row stride gate_stride, or null
  int gate_stride;
  const float* sink;    // [H] or null
  float scale;
  int chunk, window;    // 0 = off
  int B, H, G, D, BS, NB;
  // decode split: partial (max, sum) [B, H, parts, 2] and outputs [B, H, parts, D]
  float* ws_ml;
  float* ws_o;
  int num_parts;
};
void launch_sink_attention_prefill(const AttnParams& p, bool f32, hipStream_t s);
void launch_sink_attention_decode(const AttnParams& p, bool f32, hipStream_t s);

}  // namespace akap_stream
