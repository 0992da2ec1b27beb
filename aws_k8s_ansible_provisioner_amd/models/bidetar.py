"""Bidetar: a layered decoder over an fp32 residual stream (LayeredConfig).

Every layer is PARALLEL: one RMS norm h = norm1(x) feeds both the attention mixer and the
feed-forward, and x <- x + m (mixer(h) + ff(h)).  The mixer is grouped-query attention whose
values are the key projection itself (no value weights), with an RMS norm over the whole q and
the whole k projection, partial interleaved rotary positions with wavelength-scaled
frequencies, a chunked causal mask, a per-head sink logit in the softmax and a per-head sigmoid
output gate.  The feed-forward is down(relu(up h)^2).  A span of layers may run several times
in a row with the same weights; every pass has its own KV cache.

MI355X mapping: the parallel layer collapses to TWO GEMMs.  All projections that read h are one
weight [q | k | up | gate] and one launch; the attention output and the activated feed-forward
share one buffer [attn | act] that a single GEMM with the weight [W_o | W_down] reduces (the
sum of the two sublayers happens in the GEMM's fp32 accumulator).  Neither GEMM has a bias
epilogue -- the q / k biases are added by the kernel that norms them, the output bias by the
residual kernel -- so decode-sized batches run the per-shape tuned MFMA GEMMs and prefill-sized
ones hipBLASLt, through ops.linear like every other model.  Between the GEMMs: one kernel
norms + rotates q and k and writes the paged cache, one attention kernel (prefill tiles or
split decode) applies mask, sink and gate, one activation kernel; the residual update and the
next layer's norm are one kernel on the fp32 stream.  Seven launches per layer, all sync-free
and allocation-stable, so the runner captures decode steps in hipGraphs.
"""
from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops
from ..ops import stream as sops
from ..parallel.state import ParallelState, get_state
from .config import LayeredConfig, LayerSpec
from .transformer import AttnBatch

# tokens per tile of the prefill attention map (csrc/stream/attention.hip: one workgroup)
PREFILL_TILE_TOKENS = 128


@dataclasses.dataclass
class ParallelLayerWeights:
    spec: LayerSpec
    norm1: torch.Tensor       # fp32 [d]
    w_in: torch.Tensor        # [q | k | up | gate | pad, d]
    b_in: torch.Tensor
    q_norm: torch.Tensor      # fp32 [H D]
    k_norm: torch.Tensor      # fp32 [G D]
    sink: torch.Tensor        # fp32 [H]
    w_out: torch.Tensor       # [d, H D + ff] = [W_o | W_down]
    b_out: torch.Tensor
    cos_sin: Optional[torch.Tensor]
    k_off: int
    up_off: int
    g_off: int
    hd: int
    ff: int


class BidetarLM:
    """Weights + forward of one replica (same surface as DecoderLM for the model runner)."""

    supports_v_tail = False   # the D = 128 decode kernel's V-group tail is not used here
    # the two per-layer GEMM weights: decode-sized batches are tuned per shape like the other
    # models' projections (ops.gemm_tuner: the MFMA decode kernels against hipBLASLt); there is
    # no fused 4-GEMM decode chain and no hand-written prefill GEMM plan for this layer shape
    gemm_tunable = True
    gemm_weight_names = ("w_in", "w_out")
    fused_gemm_chain = False
    dtypes = (torch.bfloat16, torch.float32)

    def __init__(self, cfg: LayeredConfig, device: torch.device | str = "cpu",
                 dtype: torch.dtype = torch.bfloat16, seed: int = 0,
                 pstate: Optional[ParallelState] = None, max_model_len: int = 4096,
                 full_then_shard: bool = False, init_std: float = 0.02):
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError(f"Bidetar runs in bfloat16 or float32, not {dtype}")
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.ps = pstate or get_state()
        if self.ps.tp_size != 1:
            raise ValueError("Bidetar: tensor parallelism is not implemented (tp must be 1)")
        if max_model_len > cfg.max_position:
            raise ValueError(f"max_model_len {max_model_len} exceeds max_position "
                             f"{cfg.max_position}")
        self.max_model_len = max_model_len
        self.init_std = init_std
        self.runs = cfg.layer_runs()
        # what the runner sizes its buffers from: the widest layer
        self.hq, self.hkv, self.D = cfg.num_heads, cfg.num_kv_heads, cfg.head_dim
        self.ffn = cfg.intermediate_size
        self.vocab_start, self.vocab_end = 0, cfg.vocab_size
        self._tables: dict = {}
        self._ws: Optional[tuple] = None
        self._init_weights(seed)

    # ------------------------------------------------------------------ weights
    def _table(self, rot) -> Optional[torch.Tensor]:
        if rot is None or rot.dims <= 0:
            return None
        key = (rot.dims, rot.base, tuple(sorted((rot.scaling or {}).items())))
        if key not in self._tables:
            self._tables[key] = sops.rotary_table(max(self.max_model_len, 16), rot.dims, rot.base,
                                                  rot.scaling, device=self.device)
        return self._tables[key]

    def _init_weights(self, seed: int) -> None:
        cfg, d = self.cfg, self.cfg.hidden_size
        g = torch.Generator(device="cpu")
        g.manual_seed(seed)
        std = self.init_std

        def rand(*shape, s=std, mean=0.0, dt=None):
            t = torch.empty(*shape, dtype=torch.float32).normal_(mean, s, generator=g)
            # values a bf16 checkpoint can hold, whatever the compute type
            return t.to(torch.bfloat16).to(dt or self.dtype).to(self.device)

        f32 = torch.float32
        self.embed = rand(cfg.vocab_size, d)
        self.layers: list[ParallelLayerWeights] = []
        for ls in cfg.layer_specs:
            m = ls.mixer
            hd, gd = m.heads * m.dim, m.kv_heads * m.dim
            ff = ls.mlp.ff if ls.mlp is not None else 0
            n = hd + gd + ff + m.heads
            # rows padded (zeros) to the tile width of the decode GEMM kernels when that costs
            # under 5 %, else to whole 16-byte rows of the output
            npad = -(-n // 256) * 256
            if npad > 1.05 * n:
                npad = -(-n // 8) * 8
            w_in = torch.zeros(npad, d, dtype=self.dtype, device=self.device)
            b_in = torch.zeros(npad, dtype=self.dtype, device=self.device)
            w_in[:n] = rand(n, d)
            b_in[:hd + gd] = rand(hd + gd)
            self.layers.append(ParallelLayerWeights(
                spec=ls, norm1=rand(d, s=0.1, mean=1.0, dt=f32), w_in=w_in, b_in=b_in,
                q_norm=rand(hd, s=0.1, mean=1.0, dt=f32), k_norm=rand(gd, s=0.1, mean=1.0, dt=f32),
                sink=rand(m.heads, s=1.0, dt=f32), w_out=rand(d, hd + ff), b_out=rand(d),
                cos_sin=self._table(m.rot), k_off=hd, up_off=hd + gd, g_off=hd + gd + ff, hd=hd,
                ff=ff))
        self.final_norm = rand(d, s=0.1, mean=1.0, dt=f32)
        self.lm_head = rand(cfg.vocab_size, d)

    def state_dict(self) -> dict:
        """The weights under the checkpoint's names ('embed', 'l<i>.norm1', 'l<i>.mix.q' ...,
        'l<i>.mlp.up', 'final.norm', 'head'), un-fusing the two per-layer GEMM weights."""
        sd = {"embed": self.embed.clone(), "final.norm": self.final_norm.clone(),
              "head": self.lm_head.clone()}
        for i, lw in enumerate(self.layers):
            m, p = lw.spec.mixer, f"l{i}."
            sd[p + "norm1"] = lw.norm1.clone()
            sd[p + "mix.q"] = lw.w_in[:lw.hd].clone()
            sd[p + "mix.q.b"] = lw.b_in[:lw.hd].clone()
            sd[p + "mix.k"] = lw.w_in[lw.k_off:lw.up_off].clone()
            sd[p + "mix.k.b"] = lw.b_in[lw.k_off:lw.up_off].clone()
            sd[p + "mix.q.norm"] = lw.q_norm.clone()
            sd[p + "mix.k.norm"] = lw.k_norm.clone()
            sd[p + "mix.sink"] = lw.sink.clone()
            sd[p + "mix.g"] = lw.w_in[lw.g_off:lw.g_off + m.heads].clone()
            sd[p + "mix.o"] = lw.w_out[:, :lw.hd].clone()
            sd[p + "mix.o.b"] = lw.b_out.clone()
            if lw.ff:
                sd[p + "mlp.up"] = lw.w_in[lw.up_off:lw.g_off].clone()
                sd[p + "mlp.down"] = lw.w_out[:, lw.hd:].clone()
        return sd

    def load_state_dict(self, sd: dict) -> None:
        """Checkpoint tensors (bf16 safetensors) into the fused layout; shapes are checked
        against the config."""
        def cp(dst, name):
            src = sd[name]
            if tuple(src.shape) != tuple(dst.shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(src.shape)}, config wants "
                                 f"{tuple(dst.shape)}")
            dst.copy_(src.to(dst.dtype))

        cp(self.embed, "embed")
        cp(self.final_norm, "final.norm")
        cp(self.lm_head, "head")
        for i, lw in enumerate(self.layers):
            m, p = lw.spec.mixer, f"l{i}."
            cp(lw.norm1, p + "norm1")
            cp(lw.w_in[:lw.hd], p + "mix.q")
            cp(lw.b_in[:lw.hd], p + "mix.q.b")
            cp(lw.w_in[lw.k_off:lw.up_off], p + "mix.k")
            cp(lw.b_in[lw.k_off:lw.up_off], p + "mix.k.b")
            cp(lw.q_norm, p + "mix.q.norm")
            cp(lw.k_norm, p + "mix.k.norm")
            cp(lw.sink, p + "mix.sink")
            cp(lw.w_in[lw.g_off:lw.g_off + m.heads], p + "mix.g")
            cp(lw.w_out[:, :lw.hd], p + "mix.o")
            cp(lw.b_out, p + "mix.o.b")
            if lw.ff:
                cp(lw.w_in[lw.up_off:lw.g_off], p + "mlp.up")
                cp(lw.w_out[:, lw.hd:], p + "mlp.down")

    @property
    def graph_safe(self) -> bool:
        return True

    def weight_bytes(self) -> int:
        n = 0
        for t in [self.embed, self.final_norm, self.lm_head]:
            n += t.numel() * t.element_size()
        for lw in self.layers:
            for t in (lw.norm1, lw.w_in, lw.b_in, lw.q_norm, lw.k_norm, lw.sink, lw.w_out,
                      lw.b_out):
                n += t.numel() * t.element_size()
        return n

    # ------------------------------------------------------------------ kv cache
    def prefill_tile_plan(self) -> tuple:
        """(q rows per token, rows per tile, rows per tile of short steps) of the scheduler's
        prefill tile map: tiles of whole tokens; the kernel loops over the heads itself."""
        return 1, PREFILL_TILE_TOKENS, 0

    def kv_block_bytes(self, block_size: int, kv_dtype: str = "auto") -> int:
        es = torch.empty(0, dtype=self.dtype).element_size()
        return sum(2 * self.cfg.layer_specs[i].mixer.kv_heads * block_size *
                   self.cfg.layer_specs[i].mixer.dim * es for i in self.runs)

    def allocate_kv_segments(self, num_blocks: int, block_size: int, kv_dtype: str = "auto",
                             max_segment_bytes: Optional[int] = None) -> list:
        """One allocation [2, NB, G, BS, D] per layer RUN (a looped layer has a cache per
        pass; layers may differ in G and D), zero-filled, in the model's dtype.  Plane 0 is K
        (token-major), plane 1 the same bytes viewed as V's [NB, G, BS/8, D, 8] groups."""
        if kv_dtype not in ("auto", "bf16", "bfloat16"):
            raise ValueError("Bidetar: the KV cache is kept in the model's dtype (no fp8)")
        segs = []
        for i in self.runs:
            m = self.cfg.layer_specs[i].mixer
            segs.append(torch.zeros(2, num_blocks, m.kv_heads, block_size, m.dim,
                                    dtype=self.dtype, device=self.device))
        return segs

    def allocate_kv_cache(self, num_blocks: int, block_size: int, kv_dtype: str = "auto"):
        return self.allocate_kv_segments(num_blocks, block_size, kv_dtype)

    def cache_views(self, kv, block_size: int):
        segs = list(kv)
        return [s[0] for s in segs], [s[1].view(s.shape[1], s.shape[2], s.shape[3] // 8, s.shape[4], 8)
                                      for s in segs]

    # ------------------------------------------------------------------ forward
    def _decode_parts(self, rows: int, m) -> int:
        """Split of a decode row's visible key range into workgroups: static in the batch
        size, the model length and the mask (hipGraph-capturable), never in sequence lengths."""
        span = self.max_model_len
        if m.chunk > 0:
            span = min(span, m.chunk)
        if m.window > 0:
            span = min(span, m.window)
        max_parts = max(1, math.ceil(span / sops.DECODE_PART))
        # one wave per (row, K/V head, partition): ~4 waves per CU of 256 measured best
        # (64 rows x 4 K/V heads x 2112 keys: 75 us unsplit, 49 at 4 partitions, 60 at 16)
        wgs = max(1, rows * m.kv_heads)
        return 1 if wgs >= 1024 else min(max_parts, 64, math.ceil(1024 / wgs))

    def _workspace(self, rows: int, parts: int) -> tuple:
        need = rows * self.hq * parts
        if self._ws is None or self._ws[0] < need:
            # grown on eager steps only: the runner warms every bucket before capturing it,
            # largest first
            self._ws = (need, sops.decode_workspace(rows, self.hq, self.D, parts, self.device))
        return self._ws[1]

    def _linear(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """x @ w.T: bf16 goes through ops.linear (the tuned decode GEMM of this shape when the
        runner tuned one, else hipBLASLt); fp32 always to the library."""
        if self.dtype == torch.bfloat16:
            return ops.linear(x, w)
        return F.linear(x, w)

    def embed_tokens(self, ids: torch.Tensor) -> torch.Tensor:
        return sops.embed_scaled(ids, self.embed, self.cfg.embed_scale)

    def _attention(self, lw: ParallelLayerWeights, q, gate, batch: AttnBatch, kc, vc, out) -> None:
        m = lw.spec.mixer
        sink = lw.sink if m.sink else None
        nd = batch.num_decode if batch.is_prefill else q.shape[0]
        if nd:
            parts = self._decode_parts(nd, m)
            ws = self._workspace(nd, parts) if (parts > 1 and q.is_cuda) else None
            sops.sink_attention_decode(out[:nd], q[:nd], kc, vc, batch.block_tables[:nd],
                                       batch.seq_lens[:nd], gate[:nd] if gate is not None else None,
                                       sink, m.scale, m.chunk, m.window, ws, parts)
        if batch.is_prefill:
            sops.sink_attention_prefill(out, q, kc, vc, batch.block_tables, batch.seq_lens,
                                        batch.q_start, batch.tile_seq, batch.tile_row,
                                        batch.tile_rows, gate, sink, m.scale, m.chunk, m.window,
                                        first_seq=nd)

    def forward(self, input_ids: torch.Tensor, batch: AttnBatch, k_caches, v_caches
                ) -> torch.Tensor:
        cfg, dt = self.cfg, self.dtype
        T = input_ids.shape[0]
        eps, mult = cfg.rms_eps, cfg.residual_mult
        x = self.embed_tokens(input_ids)                     # fp32 [T, d]: the residual stream
        h = sops.stream_norm(x, self.layers[self.runs[0]].norm1, eps, dt)
        for r, li in enumerate(self.runs):
            lw = self.layers[li]
            m = lw.spec.mixer
            # [T, q | k | up | gate]; the q / k biases are added by the kernel that reads them
            proj = self._linear(h, lw.w_in)
            q = torch.empty(T, m.heads, m.dim, dtype=dt, device=self.device)
            sops.proj_norm_rope_cache(proj, q, k_caches[r], v_caches[r], batch.positions,
                                      batch.slots, lw.cos_sin, lw.q_norm, lw.k_norm, m.heads,
                                      m.kv_heads, m.dim, 0, lw.k_off, eps,
                                      lw.b_in[:lw.hd], lw.b_in[lw.k_off:lw.up_off])
            cat = torch.empty(T, lw.hd + lw.ff, dtype=dt, device=self.device)
            gate = proj[:, lw.g_off:lw.g_off + m.heads] if m.gate else None
            self._attention(lw, q, gate, batch, k_caches[r], v_caches[r], cat)
            if lw.ff:
                sops.relu2(proj[:, lw.up_off:lw.g_off], cat[:, lw.hd:])
            y = self._linear(cat, lw.w_out)                  # W_o attn + W_down act
            nxt = self.layers[self.runs[r + 1]].norm1 if r + 1 < len(self.runs) \
                else self.final_norm
            h = sops.stream_add_norm(x, y, mult, nxt, eps, dt, bias=lw.b_out)   # ... + b_o
        return h

    def compute_logits(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(h, self.lm_head)
