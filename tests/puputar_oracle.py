"""A plain float64 implementation of the Puputar design, one function per mechanism, written
from its equations.  It shares no code with the package: tests compare the engine with it.

Notation: x is the residual stream [T, d] of ONE sequence (positions 0 .. T-1), weights are a
dict name -> tensor under the checkpoint's names, `cfg` is the config.json dictionary.
"""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def group_norm(x, w, groups, eps):
    """RMS norm in `groups` equal consecutive parts, then the weight over the whole row."""
    T, d = x.shape
    return (rms(x.reshape(T, groups, d // groups), eps).reshape(T, d)) * w


def token_shift(h, mu, prev=None):
    """h_t + (h_{t-1} - h_t) * mu with the UNSHIFTED predecessor (zeros before position 0, or
    `prev` when the rows continue a sequence).  Returns the shifted rows and the last
    unshifted row."""
    first = torch.zeros_like(h[:1]) if prev is None else prev.reshape(1, -1)
    before = torch.cat([first, h[:-1]], dim=0)
    return h + (before - h) * mu, h[-1].clone()


def rotate_pairs(v, pos, dims, base):
    """Interleaved rotary on the first `dims` entries of the last axis; pos [T], v [T, ..., n]."""
    out = v.clone()
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    a = pos.to(F64)[:, None] * f[None, :]
    shape = [v.shape[0]] + [1] * (v.dim() - 2) + [dims // 2]
    c, s = torch.cos(a).reshape(shape), torch.sin(a).reshape(shape)
    u, w = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - w * s
    out[..., 1:dims:2] = w * c + u * s
    return out


def latent_kv(h, W, p, m, eps, pos):
    """The cached pair of a layer that owns a W_dkv: the normed latent c [T, R] and the rotated
    shared key part [T, r]."""
    R, r = m["kv_rank"], m["rot_dim"]
    kv = h @ W[p + "mix.dkv"].T
    c = rms(kv[:, :R], eps) * W[p + "mix.dkv.norm"]
    kr = rotate_pairs(kv[:, R:R + r], pos, m["rot"]["dims"], m["rot"]["base"])
    return c, kr


def latent_attention(h, W, p, m, eps, c, kr, per_element_gate):
    """Causal softmax attention of queries from h against the latent c and rotated key part kr
    (whole sequence: T queries, T keys), with the sigmoid output gate and W_o."""
    T = h.shape[0]
    H, D, r, V, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    cq = rms(h @ W[p + "mix.dq"].T, eps) * W[p + "mix.dq.norm"]
    q = (cq @ W[p + "mix.uq"].T).reshape(T, H, D + r)
    qn, qr = q[..., :D], rotate_pairs(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
    k = (c @ W[p + "mix.uk"].T).reshape(T, H, D)
    v = (c @ W[p + "mix.uv"].T).reshape(T, H, V)
    s = torch.einsum("ihd,jhd->hij", qn, k) + torch.einsum("ihd,jd->hij", qr, kr)
    s = s * m["scale"]
    mask = pos[None, :] <= pos[:, None]
    s = s.masked_fill(~mask[None], float("-inf"))
    a = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhv->ihv", a, v)
    g = torch.sigmoid(h @ W[p + "mix.g"].T)
    if per_element_gate:
        o = o * g.reshape(T, H, V)
    else:
        o = o * g[:, :, None]
    return o.reshape(T, H * V) @ W[p + "mix.o"].T


def softplus(z):
    return math.log1p(math.exp(-abs(z))) + max(z, 0.0)


def xielu(z, p, q):
    ap, aq = softplus(float(p)), softplus(float(q))
    pos = ap * z * z + z / 2
    neg = (0.5 + aq) * (torch.expm1(torch.clamp(z, max=0.0)) - z) + z / 2
    return torch.where(z > 0, pos, neg)


def dense_ff(h, W, p):
    a = W[p + "mlp.act"]
    z = h @ W[p + "mlp.up"].T + W[p + "mlp.up.b"]
    return xielu(z, a[0], a[1]) @ W[p + "mlp.down"].T + W[p + "mlp.down.b"]


def route(h, Wr, corr, rt):
    """ids [T, top] (router output index; >= experts: an identity expert) and weights."""
    n = rt["experts"] + rt.get("identity", 0)
    s = torch.softmax(h @ Wr.T, dim=-1)
    choice = s + corr
    gc, keep = rt["groups"]["count"], rt["groups"]["keep"]
    per = n // gc
    gs = choice.reshape(-1, gc, per).max(dim=-1).values
    best = gs.topk(keep, dim=-1).indices
    allowed = torch.zeros_like(gs, dtype=torch.bool).scatter_(1, best, True)
    allowed = allowed[:, :, None].expand(-1, -1, per).reshape(-1, n)
    choice = choice.masked_fill(~allowed, float("-inf"))
    ids = choice.topk(rt["top"], dim=-1).indices
    w = s.gather(1, ids)
    return ids, w / (w.sum(dim=-1, keepdim=True) + 1e-20)


def moe_ff(h, W, p, ml):
    rt = ml["router"]
    ids, w = route(h, W[p + "mlp.router"], W[p + "mlp.correction"], rt)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(ids[t].tolist(), w[t]):
            if e >= rt["experts"]:
                out[t] += we * h[t]
            else:
                z = torch.relu(W[p + f"mlp.e{e}.up"] @ h[t]) ** 2
                out[t] += we * (W[p + f"mlp.e{e}.down"] @ z)
    return out


def forward(cfg, W, tokens, want_layers=False):
    """Logits [T, vocab] of one whole sequence (and the stream after every layer)."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    T = len(tokens)
    pos = torch.arange(T)
    x = group_norm(W["embed"][torch.as_tensor(tokens)], W["embed.norm"], groups, eps)
    kv = {}
    streams = []
    for i, ly in enumerate(cfg["layers"]):
        p, m = f"l{i}.", ly["mixer"]
        h, _ = token_shift(group_norm(x, W[p + "norm1"], groups, eps), W[p + "shift"])
        if "kv_from" in m and m["kv_from"] is not None:
            c, kr = kv[m["kv_from"]]
        else:
            c, kr = kv[i] = latent_kv(h, W, p, m, eps, pos)
        y = latent_attention(h, W, p, m, eps, c, kr, ly["type"] == "latent_attention_2")
        ml = ly.get("mlp")
        if ml is not None:
            h2 = group_norm(x, W[p + "norm2"], groups, eps)
            y = y + (dense_ff(h2, W, p) if ml["kind"] == "dense" else moe_ff(h2, W, p, ml))
        x = x + y
        streams.append(x.clone())
    logits = group_norm(x, W["final.norm"], groups, eps) @ W["head"].T
    return (logits, torch.stack(streams)) if want_layers else logits


# ----------------------------------------------------------------------------- test models
def make_layer(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=12, q_rank=10, base=100.0, scale=None,
               gate="head", kv_from=None, ff=20, moe=None):
    """One entry of config.json's `layers`.  moe: dict(experts, ff, top, identity, count, keep)
    for a routed feed-forward; ff None and moe None: no feed-forward."""
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank,
         "q_rank": q_rank, "rot": {"base": base, "dims": rot_dim},
         "scale": scale if scale is not None else (dim + rot_dim) ** -0.5}
    if kv_from is not None:
        m["kv_from"] = kv_from
    if moe is not None:
        mlp = {"kind": "moe", "expert": {"ff": moe["ff"]},
               "router": {"experts": moe["experts"], "top": moe["top"],
                          "identity": moe.get("identity", 0),
                          "groups": {"count": moe.get("count", 1), "keep": moe.get("keep", 1)}}}
    elif ff is not None:
        mlp = {"kind": "dense", "ff": ff}
    else:
        mlp = None
    return {"type": "latent_attention_2" if gate == "element" else "latent_attention", "mixer": m,
            "mlp": mlp}


def make_config(width=24, vocab=41, layers=None, eps=1e-5, groups=3):
    return {"architecture": "Puputar", "layers": layers, "norm": {"eps": eps, "groups": groups},
            "vocab": vocab, "width": width}


def random_weights(cfg, seed=0):
    """Random tensors under the checkpoint's names, values that bfloat16 holds exactly."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]

    def rnd(*shape, s=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * s + mean).to(torch.bfloat16)

    W = {"embed": rnd(cfg["vocab"], d), "embed.norm": rnd(d, s=0.2, mean=1.0),
         "final.norm": rnd(d, s=0.2, mean=1.0), "head": rnd(cfg["vocab"], d, s=d ** -0.5)}
    for i, ly in enumerate(cfg["layers"]):
        p, m = f"l{i}.", ly["mixer"]
        H, D, r, V, R, Q = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["q_rank"]
        W[p + "norm1"] = rnd(d, s=0.2, mean=1.0)
        W[p + "shift"] = rnd(d, s=0.3, mean=0.4)
        W[p + "mix.dq"] = rnd(Q, d, s=d ** -0.5)
        W[p + "mix.dq.norm"] = rnd(Q, s=0.2, mean=1.0)
        W[p + "mix.uq"] = rnd(H * (D + r), Q, s=2 * Q ** -0.5)
        if m.get("kv_from") is None:
            W[p + "mix.dkv"] = rnd(R + r, d, s=d ** -0.5)
            W[p + "mix.dkv.norm"] = rnd(R, s=0.2, mean=1.0)
        W[p + "mix.uk"] = rnd(H * D, R, s=2 * R ** -0.5)
        W[p + "mix.uv"] = rnd(H * V, R, s=R ** -0.5)
        W[p + "mix.g"] = rnd(H * V if ly["type"] == "latent_attention_2" else H, d, s=d ** -0.5)
        W[p + "mix.o"] = rnd(d, H * V, s=(H * V) ** -0.5)
        ml = ly["mlp"]
        if ml is None:
            continue
        W[p + "norm2"] = rnd(d, s=0.2, mean=1.0)
        if ml["kind"] == "dense":
            F_ = ml["ff"]
            W[p + "mlp.up"] = rnd(F_, d, s=d ** -0.5)
            W[p + "mlp.up.b"] = rnd(F_, s=0.3)
            W[p + "mlp.down"] = rnd(d, F_, s=F_ ** -0.5)
            W[p + "mlp.down.b"] = rnd(d, s=0.3)
            W[p + "mlp.act"] = rnd(2, s=0.7)
        else:
            rt, F_ = ml["router"], ml["expert"]["ff"]
            n = rt["experts"] + rt.get("identity", 0)
            for e in range(rt["experts"]):
                W[p + f"mlp.e{e}.up"] = rnd(F_, d, s=d ** -0.5)
                W[p + f"mlp.e{e}.down"] = rnd(d, F_, s=F_ ** -0.5)
            W[p + "mlp.router"] = rnd(n, d, s=2 * d ** -0.5)
            W[p + "mlp.correction"] = rnd(n, s=0.1)
    return W


def decode_step_by_step(cfg, W, tokens):
    """The same logits computed one token at a time from explicit caches and shift states (an
    independent check of what a sequence has to carry from step to step)."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    L = len(cfg["layers"])
    prev = [None] * L
    cache = {}
    out = []
    for t, tok in enumerate(tokens):
        pos = torch.tensor([t])
        x = group_norm(W["embed"][torch.as_tensor([tok])], W["embed.norm"], groups, eps)
        for i, ly in enumerate(cfg["layers"]):
            p, m = f"l{i}.", ly["mixer"]
            h, prev[i] = token_shift(group_norm(x, W[p + "norm1"], groups, eps), W[p + "shift"],
                                     prev[i])
            j = m.get("kv_from")
            if j is None:
                c, kr = latent_kv(h, W, p, m, eps, pos)
                old = cache.get(i)
                cache[i] = (c, kr) if old is None else (torch.cat([old[0], c]),
                                                        torch.cat([old[1], kr]))
                j = i
            c, kr = cache[j]
            H, D, r, V = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
            cq = rms(h @ W[p + "mix.dq"].T, eps) * W[p + "mix.dq.norm"]
            q = (cq @ W[p + "mix.uq"].T).reshape(1, H, D + r)
            qr = rotate_pairs(q[..., D:], pos, m["rot"]["dims"], m["rot"]["base"])
            k = (c @ W[p + "mix.uk"].T).reshape(-1, H, D)
            v = (c @ W[p + "mix.uv"].T).reshape(-1, H, V)
            s = (torch.einsum("hd,jhd->hj", q[0, :, :D], k) +
                 torch.einsum("hd,jd->hj", qr[0], kr)) * m["scale"]
            o = torch.einsum("hj,jhv->hv", torch.softmax(s, dim=-1), v)
            g = torch.sigmoid(h @ W[p + "mix.g"].T)[0]
            o = o * (g.reshape(H, V) if ly["type"] == "latent_attention_2" else g[:, None])
            y = o.reshape(1, H * V) @ W[p + "mix.o"].T
            ml = ly.get("mlp")
            if ml is not None:
                h2 = group_norm(x, W[p + "norm2"], groups, eps)
                y = y + (dense_ff(h2, W, p) if ml["kind"] == "dense" else moe_ff(h2, W, p, ml))
            x = x + y
        out.append(group_norm(x, W["final.norm"], groups, eps) @ W["head"].T)
    return torch.cat(out)
