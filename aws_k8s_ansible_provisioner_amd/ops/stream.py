"""Ops of models that keep an fp32 residual stream (``_C_stream.so``, csrc/stream/).

Same dispatch rule as the rest of ``ops``: GPU tensors run the hand-written HIP kernel (and
raise if the library is missing), CPU tensors a plain PyTorch version of the same op.  The
kernels are templated on the activation type (bf16 or fp32) and take every size at run time
(any head size, head count and GQA ratio), so a model's weights and KV cache may be bf16 or
fp32; norms, rotary angles, attention scores and weights and the residual sum are fp32 in both.

KV cache layout of these ops: K [num_blocks, G, block_size, D] (token-major rows) and
V [num_blocks, G, block_size / 8, D, 8] (groups of 8 tokens, dimension-major inside a group: the
8 keys a matrix-core operand contracts over, or a decode lane accumulates, are one 16-byte load).
"""
from __future__ import annotations

import os
from typing import Optional

import torch

_PKG = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
_LIB = os.path.join(_PKG, "_C_stream.so")
_loaded = False
_load_error: Optional[str] = None


def load_native(required: bool = False) -> bool:
    """Load ``_C_stream.so`` (torch.ops.akap_stream), building it on first use."""
    global _loaded, _load_error
    if _loaded:
        return True
    from .. import build_ext

    try:
        if os.path.exists(build_ext.STREAM_SRC):
            have = build_ext.library_hash(_LIB, "akap_stream_build_hash")
            if have != build_ext.stream_tree_hash():
                if os.environ.get("AKAP_ALLOW_STALE_NATIVE") == "1" and have:
                    pass
                else:
                    build_ext.build_stream()
        torch.ops.load_library(_LIB)
        _loaded = True
    except Exception as e:  # pragma: no cover - depends on the box
        _load_error = repr(e)
    if required and not _loaded:
        raise RuntimeError("stream HIP kernels unavailable: " + str(_load_error))
    return _loaded


def _native(t: torch.Tensor) -> bool:
    if t.is_cuda:
        load_native(required=True)
        return True
    return False


# ----------------------------------------------------------------------------- embedding, norms
def embed_scaled(ids: torch.Tensor, table: torch.Tensor, scale: float,
                 out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[t] = table[ids[t]] * scale as fp32 (the residual stream)."""
    if out is None:
        out = torch.empty(ids.shape[0], table.shape[1], dtype=torch.float32, device=table.device)
    if _native(table):
        torch.ops.akap_stream.embed_scaled(out, ids, table, float(scale))
        return out
    out.copy_(table[ids.long()].float() * scale)
    return out


def _rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x * torch.rsqrt(x.pow(2).mean(dim=-1, keepdim=True) + eps)


def stream_norm(x: torch.Tensor, w: torch.Tensor, eps: float, out_dtype: torch.dtype,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """RMS norm of the fp32 stream x [T, d] with fp32 weights w, result in out_dtype."""
    if out is None:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if _native(x):
        torch.ops.akap_stream.add_norm(out, x, None, 0.0, w, float(eps))
        return out
    out.copy_((_rms(x.float(), eps) * w.float()).to(out.dtype))
    return out


def stream_add_norm(x: torch.Tensor, y: torch.Tensor, mult: float, w: torch.Tensor, eps: float,
                    out_dtype: torch.dtype, out: Optional[torch.Tensor] = None,
                    bias: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x += mult * (y + bias) in place (fp32 sum), then the RMS norm of the new x as out_dtype:
    the residual update of one layer fused with the norm that feeds the next.  bias [d] (y's
    dtype): the bias of the projection that produced y, when its GEMM has no bias epilogue."""
    if out is None:
        out = torch.empty(x.shape, dtype=out_dtype, device=x.device)
    if _native(x):
        torch.ops.akap_stream.add_norm(out, x, y, float(mult), w, float(eps), bias)
        return out
    x.add_((y.float() + (bias.float() if bias is not None else 0.0)) * mult)
    out.copy_((_rms(x, eps) * w.float()).to(out.dtype))
    return out


def relu2(x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out = relu(x)^2; x and out are [T, F] views that may be column slices of wider rows."""
    if _native(x):
        torch.ops.akap_stream.relu2(out, x)
        return out
    r = torch.relu(x.float())
    out.copy_((r * r).to(out.dtype))
    return out


# ----------------------------------------------------------------------------- rotary, cache
def rotary_table(max_pos: int, dims: int, base: float, scaling: Optional[dict] = None,
                 device=None) -> torch.Tensor:
    """fp32 [max_pos, dims] = [cos | sin] of angle p * f_i, f_i = base^(-2i/dims), with the
    wavelength rule of `scaling` = {factor, low, high, original}: frequencies whose wavelength
    is under original/high are kept, over original/low divided by factor, and blended linearly
    (in original/wavelength) between.  Angles are formed in fp64 and rounded once."""
    from . import reference as ref

    sc = None
    if scaling:
        sc = {"rope_type": "llama3", "factor": float(scaling["factor"]),
              "low_freq_factor": float(scaling["low"]), "high_freq_factor": float(scaling["high"]),
              "original_max_position_embeddings": scaling["original"]}
    return ref.rope_cos_sin(max_pos, dims, base, sc, device=device)


def proj_norm_rope_cache(proj: torch.Tensor, q_out: torch.Tensor, k_cache: torch.Tensor,
                         v_cache: torch.Tensor, positions: torch.Tensor, slots: torch.Tensor,
                         cos_sin: Optional[torch.Tensor], q_w: torch.Tensor, k_w: torch.Tensor,
                         H: int, G: int, D: int, q_off: int, k_off: int, eps: float,
                         q_b: Optional[torch.Tensor] = None,
                         k_b: Optional[torch.Tensor] = None) -> None:
    """Per token t of the fused projection proj [T, N]: q = proj[t, q_off : q_off + H D] and
    k = proj[t, k_off : k_off + G D] are each RMS-normalised over their WHOLE length (one
    mean over all heads) with weights q_w / k_w, then rotated per head on the first
    cos_sin.shape[1] dimensions, interleaved pairs (2i, 2i+1), by the angle row of
    positions[t].  q goes to q_out [T, H, D]; k to k_cache at slots[t]; the raw k (before norm
    and rotation) to v_cache at the same slot: the values are the keys' projection.  Slot -1
    writes nothing.  k_cache [NB, G, BS, D], v_cache [NB, G, BS/8, D, 8].  q_b / k_b (proj's
    dtype): the projection's biases, added to the slices first when its GEMM did not."""
    if _native(proj):
        torch.ops.akap_stream.proj_norm_rope_cache(proj, q_out, k_cache, v_cache, positions, slots,
                                                   cos_sin, q_w, k_w, H, G, D, q_off, k_off,
                                                   float(eps), q_b, k_b)
        return
    T = proj.shape[0]
    q = proj[:, q_off:q_off + H * D].float()
    k = proj[:, k_off:k_off + G * D].float()
    if q_b is not None:
        q = q + q_b.float()
    if k_b is not None:
        k = k + k_b.float()
    qn = (_rms(q, eps) * q_w.float()).view(T, H, D)
    kn = (_rms(k, eps) * k_w.float()).view(T, G, D)
    if cos_sin is not None:
        rd = cos_sin.shape[1]
        cs = cos_sin[positions.long()]
        c, s = cs[:, None, :rd // 2], cs[:, None, rd // 2:]

        def rot(x):
            u, v = x[..., 0:rd:2], x[..., 1:rd:2]
            o = x.clone()
            o[..., 0:rd:2] = u * c - v * s
            o[..., 1:rd:2] = v * c + u * s
            return o

        qn, kn = rot(qn), rot(kn)
    q_out.copy_(qn.to(q_out.dtype))
    BS = k_cache.shape[2]
    ok = slots >= 0
    sl = slots[ok].long()
    k_cache[sl // BS, :, sl % BS] = kn[ok].to(k_cache.dtype)
    v_cache[sl // BS, :, (sl % BS) // 8, :, sl % 8] = k.view(T, G, D)[ok].to(v_cache.dtype)


def v_tokens(v_cache: torch.Tensor) -> torch.Tensor:
    """The V cache [NB, G, BS/8, D, 8] as token-major rows [NB, G, BS, D] (a copy)."""
    NB, G, NG, D, _ = v_cache.shape
    return v_cache.permute(0, 1, 2, 4, 3).reshape(NB, G, NG * 8, D)


def v_from_tokens(v: torch.Tensor) -> torch.Tensor:
    """Token-major values [NB, G, BS, D] in the V cache layout [NB, G, BS/8, D, 8]."""
    NB, G, BS, D = v.shape
    return v.view(NB, G, BS // 8, 8, D).permute(0, 1, 2, 4, 3).contiguous()


# ----------------------------------------------------------------------------- attention
def _attend_rows(out, q, k_cache, v_cache, bt_row, kv_len: int, pos0: int, rows: slice,
                 gate, sink, scale: float, chunk: int, window: int) -> None:
    """CPU: the queries `rows` of one sequence (positions pos0 ...) against its cached keys."""
    n = rows.stop - rows.start
    H, D = q.shape[1], q.shape[2]
    G, BS = k_cache.shape[1], k_cache.shape[2]
    nb = -(-kv_len // BS)
    blocks = bt_row[:nb].long()
    K = k_cache[blocks].permute(1, 0, 2, 3).reshape(G, nb * BS, D)[:, :kv_len].float()
    V = v_tokens(v_cache[blocks]).permute(1, 0, 2, 3).reshape(G, nb * BS, D)[:, :kv_len].float()
    i = torch.arange(pos0, pos0 + n)[:, None]
    j = torch.arange(kv_len)[None, :]
    ok = j <= i
    if chunk > 0:
        ok &= (i // chunk) == (j // chunk)
    if window > 0:
        ok &= j > i - window
    qf = q[rows].float()
    rep = H // G
    for h in range(H):
        s = (qf[:, h] @ K[h // rep].T) * scale
        s = s.masked_fill(~ok, float("-inf"))
        m = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            m = torch.maximum(m, sink[h].float())
        e = torch.exp(s - m)
        den = e.sum(dim=-1, keepdim=True)
        if sink is not None:
            den = den + torch.exp(sink[h].float() - m)
        o = (e / den) @ V[h // rep]
        if gate is not None:
            o = o * torch.sigmoid(gate[rows, h].float())[:, None]
        out[rows, h * D:(h + 1) * D] = o.to(out.dtype)


def sink_attention_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                           v_cache: torch.Tensor, block_tables: torch.Tensor,
                           seq_lens: torch.Tensor, q_start: torch.Tensor, tile_seq: torch.Tensor,
                           tile_row: torch.Tensor, tile_rows: int, gate: Optional[torch.Tensor],
                           sink: Optional[torch.Tensor], scale: float, chunk: int = 0,
                           window: int = 0, first_seq: int = 0) -> torch.Tensor:
    """Paged causal attention of prompt chunks.  Sequence b's chunk is rows
    [q_start[b], q_start[b+1]) of q [T, H, D]; its keys are positions [0, seq_lens[b]) of its
    block-table row, the chunk's tokens being the last ones.  A query at position i sees key
    j <= i, and only if floor(i / chunk) == floor(j / chunk) (chunk > 0; chunks count from
    position 0 of the sequence) and j > i - window (window > 0).  sink [H] (fp32): exp(sink_h)
    is added to the softmax denominator (no key, no value, unscaled).  gate [T, H] (a column
    slice of the projection): head h's output is multiplied by sigmoid(gate[t, h]).  Scores,
    softmax and the gate are fp32.  out [T, >= H D] (rows may be wider: a slice of the buffer
    the output projection reads).  The tile map (tile_seq, tile_row: a sequence and the first
    chunk row of a tile of tile_rows tokens) drives the GPU grid; sequences before first_seq
    (the decode rows of a mixed step) are not in it."""
    if _native(q):
        torch.ops.akap_stream.sink_attention_prefill(out, q, k_cache, v_cache, block_tables,
                                                     seq_lens, q_start, tile_seq, tile_row,
                                                     tile_rows, gate, sink, float(scale), chunk,
                                                     window)
        return out
    B = seq_lens.numel()
    for b in range(first_seq, B):
        r0, r1 = int(q_start[b]), int(q_start[b + 1])
        if r1 > r0:
            kv = int(seq_lens[b])
            _attend_rows(out, q, k_cache, v_cache, block_tables[b], kv, kv - (r1 - r0),
                         slice(r0, r1), gate, sink, scale, chunk, window)
    return out


# fewest keys worth a decode partition of their own
DECODE_PART = 128


def decode_workspace(max_seqs: int, max_heads: int, max_dim: int, max_parts: int, device):
    """Partial softmax state of the split decode kernel: (max, sum) and the unnormalised
    output per (sequence, head, partition), fp32."""
    n = max(1, max_seqs * max_heads * max_parts)
    return (torch.empty(n * 2, dtype=torch.float32, device=device),
            torch.empty(n * max_dim, dtype=torch.float32, device=device))


def sink_attention_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor,
                          v_cache: torch.Tensor, block_tables: torch.Tensor,
                          seq_lens: torch.Tensor, gate: Optional[torch.Tensor],
                          sink: Optional[torch.Tensor], scale: float, chunk: int = 0,
                          window: int = 0, workspace=None, num_parts: int = 1) -> torch.Tensor:
    """One query per sequence, at position seq_lens[b] - 1 (seq_lens 0: a padding row, left
    unwritten); same mask, sink and gate as sink_attention_prefill.  num_parts > 1 (GPU): the
    visible key range is cut into num_parts equal partitions (whole 32- or 64-key pieces), one
    workgroup each, merged by a second launch (workspace from decode_workspace)."""
    if _native(q):
        ws_ml, ws_o = workspace if (workspace is not None and num_parts > 1) else (None, None)
        torch.ops.akap_stream.sink_attention_decode(out, q, k_cache, v_cache, block_tables,
                                                    seq_lens, gate, sink, float(scale), chunk,
                                                    window, ws_ml, ws_o, num_parts)
        return out
    for b in range(seq_lens.numel()):
        kv = int(seq_lens[b])
        if kv > 0:
            _attend_rows(out, q, k_cache, v_cache, block_tables[b], kv, kv - 1, slice(b, b + 1),
                         gate, sink, scale, chunk, window)
    return out
