// torch custom-op registrations (namespace `akap_stream`) of the fp32-residual-stream kernels.
//
// Like the core ops: every op launches on the caller's current HIP stream, allocates nothing
// and never synchronises (hipGraph-capturable).  Operand shapes are checked here, on the host,
// against what the kernels index.
#include <torch/library.h>
#include <ATen/ATen.h>
#include <c10/hip/HIPStream.h>
#include <c10/core/DeviceGuard.h>

#include "stream.h"

namespace {

using at::Tensor;

hipStream_t cur_stream() { return c10::hip::getCurrentHIPStream().stream(); }

#define CHECK_GPU(x) TORCH_CHECK((x).is_cuda(), #x " must be a GPU tensor")
#define CHECK_LAST_CONTIG(x) TORCH_CHECK((x).stride(-1) == 1, #x " must have unit last stride")
#define CHECK_CONTIG(x) TORCH_CHECK((x).is_contiguous(), #x " must be contiguous")
#define CHECK_F32(x) TORCH_CHECK((x).scalar_type() == at::kFloat, #x " must be fp32")

// the activation type of an op: bf16 (false) or fp32 (true)
bool is_f32(const Tensor& t, const char* name) {
  TORCH_CHECK(t.scalar_type() == at::kFloat || t.scalar_type() == at::kBFloat16, name,
              " must be bf16 or fp32");
  return t.scalar_type() == at::kFloat;
}

void embed_scaled(Tensor out, Tensor ids, Tensor table, double scale) {
  CHECK_GPU(out); CHECK_GPU(ids); CHECK_GPU(table);
  CHECK_F32(out); CHECK_CONTIG(out); CHECK_CONTIG(table); CHECK_CONTIG(ids);
  TORCH_CHECK(ids.scalar_type() == at::kLong, "ids must be int64");
  TORCH_CHECK(table.dim() == 2 && out.dim() == 2 && out.size(1) == table.size(1) &&
                  out.size(0) == ids.numel(), "embed_scaled: shapes");
  const c10::DeviceGuard g(out.device());
  akap_stream::launch_embed_scaled(out.data_ptr<float>(), ids.data_ptr<int64_t>(), table.data_ptr(),
                                   is_f32(table, "table"), (int)ids.numel(), (int)table.size(1),
                                   (int)table.size(0), (float)scale, cur_stream());
}

void add_norm(Tensor out, Tensor x, std::optional<Tensor> y, double mult, Tensor w, double eps,
              std::optional<Tensor> bias) {
  CHECK_GPU(out); CHECK_GPU(x); CHECK_GPU(w);
  CHECK_F32(x); CHECK_CONTIG(x); CHECK_F32(w); CHECK_CONTIG(w); CHECK_LAST_CONTIG(out);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.sizes() == x.sizes(), "add_norm: shapes");
  const int rows = x.size(0), d = x.size(1);
  TORCH_CHECK(w.numel() == d, "add_norm: weight size");
  const void* yp = nullptr;
  bool yf = false;
  int ys = 0;
  if (y.has_value()) {
    CHECK_GPU(*y); CHECK_LAST_CONTIG(*y);
    TORCH_CHECK(y->dim() == 2 && y->sizes() == x.sizes(), "add_norm: y shape");
    yp = y->data_ptr();
    yf = is_f32(*y, "y");
    ys = y->stride(0);
  }
  const void* bp = nullptr;
  if (bias.has_value()) {
    TORCH_CHECK(y.has_value(), "add_norm: a bias needs y");
    CHECK_GPU(*bias); CHECK_CONTIG(*bias);
    TORCH_CHECK(bias->numel() == d && bias->scalar_type() == y->scalar_type(),
                "add_norm: bias must be [d] of y's dtype");
    bp = bias->data_ptr();
  }
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_add_norm(out.data_ptr(), is_f32(out, "out"), x.data_ptr<float>(), yp, yf, ys,
                               bp, (float)mult, w.data_ptr<float>(), rows, d, (int)out.stride(0),
                               (float)eps, cur_stream());
}

void relu2(Tensor out, Tensor x) {
  CHECK_GPU(out); CHECK_GPU(x); CHECK_LAST_CONTIG(out); CHECK_LAST_CONTIG(x);
  TORCH_CHECK(x.dim() == 2 && out.dim() == 2 && out.sizes() == x.sizes(), "relu2: shapes");
  TORCH_CHECK(out.scalar_type() == x.scalar_type(), "relu2: dtypes differ");
  const c10::DeviceGuard g(x.device());
  akap_stream::launch_relu2(out.data_ptr(), x.data_ptr(), is_f32(x, "x"), (int)x.size(0),
                            (int)x.size(1), (int)x.stride(0), (int)out.stride(0), cur_stream());
}

void check_cache(const Tensor& k_cache, const Tensor& v_cache, int64_t G, int64_t D) {
  CHECK_GPU(k_cache); CHECK_GPU(v_cache); CHECK_CONTIG(k_cache); CHECK_CONTIG(v_cache);
  TORCH_CHECK(k_cache.dim() == 4 && v_cache.dim() == 5 &&
                  k_cache.scalar_type() == v_cache.scalar_type(),
              "caches must be K [NB, G, BS, D] and V [NB, G, BS/8, D, 8]");
  TORCH_CHECK(k_cache.size(1) == G && k_cache.size(3) == D, "cache does not match G / D");
  TORCH_CHECK(k_cache.size(2) % 8 == 0 && v_cache.size(0) == k_cache.size(0) &&
                  v_cache.size(1) == G && v_cache.size(2) * 8 == k_cache.size(2) &&
                  v_cache.size(3) == D && v_cache.size(4) == 8, "V cache does not match K cache");
  TORCH_CHECK(k_cache.size(0) * G * k_cache.size(2) < (1LL << 31), "cache has too many rows");
}

void proj_norm_rope_cache(Tensor proj, Tensor q_out, Tensor k_cache, Tensor v_cache,
                          Tensor positions, Tensor slots, std::optional<Tensor> cos_sin,
                          Tensor q_w, Tensor k_w, int64_t H, int64_t G, int64_t D, int64_t q_off,
                          int64_t k_off, double eps, std::optional<Tensor> q_b,
                          std::optional<Tensor> k_b) {
  CHECK_GPU(proj); CHECK_LAST_CONTIG(proj); CHECK_GPU(q_out); CHECK_CONTIG(q_out);
  CHECK_GPU(positions); CHECK_GPU(slots); CHECK_GPU(q_w); CHECK_GPU(k_w);
  CHECK_F32(q_w); CHECK_F32(k_w); CHECK_CONTIG(q_w); CHECK_CONTIG(k_w);
  TORCH_CHECK(positions.scalar_type() == at::kLong && slots.scalar_type() == at::kLong,
              "positions/slots must be int64");
  CHECK_CONTIG(positions); CHECK_CONTIG(slots);
  const bool f32 = is_f32(proj, "proj");
  TORCH_CHECK(q_out.scalar_type() == proj.scalar_type() &&
                  k_cache.scalar_type() == proj.scalar_type(), "q_out / cache dtype != proj dtype");
  check_cache(k_cache, v_cache, G, D);
  TORCH_CHECK(proj.dim() == 2 && H > 0 && G > 0 && D > 0 && D % 2 == 0, "bad H / G / D");
  const int64_t T = proj.size(0);
  TORCH_CHECK(q_off >= 0 && k_off >= 0 && q_off + H * D <= proj.size(1) &&
                  k_off + G * D <= proj.size(1), "q / k slices outside the projection");
  TORCH_CHECK(q_out.numel() == T * H * D, "q_out size");
  TORCH_CHECK(positions.numel() >= T && slots.numel() >= T, "positions/slots too short");
  TORCH_CHECK(q_w.numel() == H * D && k_w.numel() == G * D, "norm weight sizes");
  akap_stream::ProjParams p{};
  if (cos_sin.has_value()) {
    CHECK_GPU(*cos_sin); CHECK_F32(*cos_sin); CHECK_CONTIG(*cos_sin);
    TORCH_CHECK(cos_sin->dim() == 2 && cos_sin->size(1) % 2 == 0 && cos_sin->size(1) <= D,
                "cos_sin must be [max_pos, rot_dims <= D]");
    p.cos_sin = cos_sin->data_ptr<float>();
    p.max_pos = cos_sin->size(0);
    p.rot_dims = cos_sin->size(1);
  }
  if (q_b.has_value()) {
    CHECK_GPU(*q_b); CHECK_CONTIG(*q_b);
    TORCH_CHECK(q_b->numel() == H * D && q_b->scalar_type() == proj.scalar_type(), "q_b: [H D]");
    p.q_b = q_b->data_ptr();
  }
  if (k_b.has_value()) {
    CHECK_GPU(*k_b); CHECK_CONTIG(*k_b);
    TORCH_CHECK(k_b->numel() == G * D && k_b->scalar_type() == proj.scalar_type(), "k_b: [G D]");
    p.k_b = k_b->data_ptr();
  }
  p.proj = proj.data_ptr();
  p.proj_stride = proj.stride(0);
  p.q_out = q_out.data_ptr();
  p.k_cache = k_cache.data_ptr();
  p.v_cache = v_cache.data_ptr();
  p.positions = positions.data_ptr<int64_t>();
  p.slots = slots.data_ptr<int64_t>();
  p.q_w = q_w.data_ptr<float>();
  p.k_w = k_w.data_ptr<float>();
  p.T = T; p.H = H; p.G = G; p.D = D; p.BS = k_cache.size(2);
  p.q_off = q_off; p.k_off = k_off;
  p.num_slots = k_cache.size(0) * k_cache.size(2);
  p.eps = (float)eps;
  const c10::DeviceGuard g(proj.device());
  akap_stream::launch_proj_norm_rope_cache(p, f32, cur_stream());
}

// fields shared by the prefill and decode attention ops
akap_stream::AttnParams attn_params(const Tensor& out, const Tensor& q, const Tensor& k_cache,
                                    const Tensor& v_cache, const Tensor& block_tables,
                                    const Tensor& seq_lens, const std::optional<Tensor>& gate,
                                    const std::optional<Tensor>& sink, double scale, int64_t chunk,
                                    int64_t window) {
  CHECK_GPU(out); CHECK_GPU(q); CHECK_GPU(block_tables); CHECK_GPU(seq_lens);
  CHECK_LAST_CONTIG(out); CHECK_CONTIG(q); CHECK_CONTIG(block_tables); CHECK_CONTIG(seq_lens);
  TORCH_CHECK(q.dim() == 3 && out.dim() == 2, "q must be [T, H, D], out [T, >= H D]");
  const int64_t T = q.size(0), H = q.size(1), D = q.size(2);
  const int64_t G = k_cache.size(1);
  check_cache(k_cache, v_cache, G, D);
  TORCH_CHECK(H % G == 0, "H must be a multiple of G");
  TORCH_CHECK(D <= 256, "head size above 256 is not supported");
  TORCH_CHECK(out.scalar_type() == q.scalar_type() && k_cache.scalar_type() == q.scalar_type(),
              "out / cache dtype != q dtype");
  TORCH_CHECK(out.size(0) == T && out.size(1) >= H * D, "out too small");
  TORCH_CHECK(block_tables.scalar_type() == at::kInt && seq_lens.scalar_type() == at::kInt &&
                  block_tables.dim() == 2 && block_tables.size(0) >= seq_lens.numel(),
              "block_tables [B, max_blocks] / seq_lens [B] must be int32");
  TORCH_CHECK(chunk >= 0 && window >= 0, "chunk / window must be >= 0");
  akap_stream::AttnParams p{};
  p.out = out.data_ptr();
  p.out_stride = out.stride(0);
  p.q = q.data_ptr();
  p.k_cache = k_cache.data_ptr();
  p.v_cache = v_cache.data_ptr();
  p.block_tables = block_tables.data_ptr<int32_t>();
  p.max_blocks = block_tables.size(1);
  p.seq_lens = seq_lens.data_ptr<int32_t>();
  p.B = seq_lens.numel();
  if (gate.has_value()) {
    CHECK_GPU(*gate); CHECK_LAST_CONTIG(*gate);
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == T && gate->size(1) == H &&
                    gate->scalar_type() == q.scalar_type(), "gate must be [T, H] of q's dtype");
    p.gate = gate->data_ptr();
    p.gate_stride = gate->stride(0);
  }
  if (sink.has_value()) {
    CHECK_GPU(*sink); CHECK_F32(*sink); CHECK_CONTIG(*sink);
    TORCH_CHECK(sink->numel() == H, "sink must be [H]");
    p.sink = sink->data_ptr<float>();
  }
  p.scale = (float)scale;
  p.chunk = chunk; p.window = window;
  p.H = H; p.G = G; p.D = D; p.BS = k_cache.size(2); p.NB = k_cache.size(0);
  p.num_parts = 1;
  return p;
}

void sink_attention_prefill(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                            Tensor block_tables, Tensor seq_lens, Tensor q_start, Tensor tile_seq,
                            Tensor tile_row, int64_t tile_rows, std::optional<Tensor> gate,
                            std::optional<Tensor> sink, double scale, int64_t chunk,
                            int64_t window) {
  auto p = attn_params(out, q, k_cache, v_cache, block_tables, seq_lens, gate, sink, scale, chunk,
                       window);
  CHECK_GPU(q_start); CHECK_GPU(tile_seq); CHECK_GPU(tile_row);
  CHECK_CONTIG(q_start); CHECK_CONTIG(tile_seq); CHECK_CONTIG(tile_row);
  TORCH_CHECK(q_start.scalar_type() == at::kInt && tile_seq.scalar_type() == at::kInt &&
                  tile_row.scalar_type() == at::kInt, "q_start / tile map must be int32");
  TORCH_CHECK(q_start.numel() >= p.B + 1 && tile_seq.numel() == tile_row.numel(),
              "q_start / tile map sizes");
  TORCH_CHECK(tile_rows > 0, "tile_rows must be positive");
  p.q_start = q_start.data_ptr<int32_t>();
  p.tile_seq = tile_seq.data_ptr<int32_t>();
  p.tile_row = tile_row.data_ptr<int32_t>();
  p.num_tiles = tile_seq.numel();
  p.tile_rows = tile_rows;
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_sink_attention_prefill(p, is_f32(q, "q"), cur_stream());
}

void sink_attention_decode(Tensor out, Tensor q, Tensor k_cache, Tensor v_cache,
                           Tensor block_tables, Tensor seq_lens, std::optional<Tensor> gate,
                           std::optional<Tensor> sink, double scale, int64_t chunk, int64_t window,
                           std::optional<Tensor> ws_ml, std::optional<Tensor> ws_o,
                           int64_t num_parts) {
  auto p = attn_params(out, q, k_cache, v_cache, block_tables, seq_lens, gate, sink, scale, chunk,
                       window);
  TORCH_CHECK(q.size(0) == p.B, "decode: one query row per sequence");
  TORCH_CHECK(num_parts >= 1 && num_parts <= 65535, "num_parts out of range");
  TORCH_CHECK(p.H <= 65535, "too many heads");
  p.num_parts = num_parts;
  if (num_parts > 1) {
    TORCH_CHECK(ws_ml.has_value() && ws_o.has_value(), "split decode needs a workspace");
    CHECK_GPU(*ws_ml); CHECK_GPU(*ws_o); CHECK_F32(*ws_ml); CHECK_F32(*ws_o);
    CHECK_CONTIG(*ws_ml); CHECK_CONTIG(*ws_o);
    const int64_t n = (int64_t)p.B * p.H * num_parts;
    TORCH_CHECK(ws_ml->numel() >= 2 * n && ws_o->numel() >= n * p.D, "decode workspace too small");
    p.ws_ml = ws_ml->data_ptr<float>();
    p.ws_o = ws_o->data_ptr<float>();
  }
  const c10::DeviceGuard g(q.device());
  akap_stream::launch_sink_attention_decode(p, is_f32(q, "q"), cur_stream());
}

}  // namespace

TORCH_LIBRARY(akap_stream, m) {
  m.def("embed_scaled(Tensor(a!) out, Tensor ids, Tensor table, float scale) -> ()");
  m.def("add_norm(Tensor(a!) out, Tensor(b!) x, Tensor? y, float mult, Tensor w, float eps, "
        "Tensor? bias=None) -> ()");
  m.def("relu2(Tensor(a!) out, Tensor x) -> ()");
  m.def(
      "proj_norm_rope_cache(Tensor proj, Tensor(a!) q_out, Tensor(b!) k_cache, Tensor(c!) v_cache, "
      "Tensor positions, Tensor slots, Tensor? cos_sin, Tensor q_w, Tensor k_w, int H, int G, "
      "int D, int q_off, int k_off, float eps, Tensor? q_b=None, Tensor? k_b=None) -> ()");
  m.def(
      "sink_attention_prefill(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
      "Tensor block_tables, Tensor seq_lens, Tensor q_start, Tensor tile_seq, Tensor tile_row, "
      "int tile_rows, Tensor? gate, Tensor? sink, float scale, int chunk, int window) -> ()");
  m.def(
      "sink_attention_decode(Tensor(a!) out, Tensor q, Tensor k_cache, Tensor v_cache, "
      "Tensor block_tables, Tensor seq_lens, Tensor? gate, Tensor? sink, float scale, int chunk, "
      "int window, Tensor(b!)? ws_ml, Tensor(c!)? ws_o, int num_parts) -> ()");
}

TORCH_LIBRARY_IMPL(akap_stream, CUDA, m) {
  m.impl("embed_scaled", &embed_scaled);
  m.impl("add_norm", &add_norm);
  m.impl("relu2", &relu2);
  m.impl("proj_norm_rope_cache", &proj_norm_rope_cache);
  m.impl("sink_attention_prefill", &sink_attention_prefill);
  m.impl("sink_attention_decode", &sink_attention_decode);
}
