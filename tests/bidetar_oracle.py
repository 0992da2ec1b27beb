"""A plain, slow float64 implementation of the Bidetar design, one function per mechanism,
written from its equations and sharing no code with the package: the oracle of the tests.

Notation: d model width, H query heads, G key/value heads, D head size, R rotated dimensions,
C chunk length, m residual multiplier.  Weights are a dict name -> tensor under the
checkpoint's names; the configuration is the config.json dictionary itself.
"""
import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rotary_frequencies(rot):
    """f_i = base^(-2i/R), i < R/2, rescaled by wavelength L = 2 pi / f: kept when
    L < original/high, divided by factor when L > original/low, blended in between."""
    R = rot["dims"]
    out = []
    for i in range(R // 2):
        f = rot["base"] ** (-2.0 * i / R)
        sc = rot.get("scaling")
        if sc:
            L = 2 * math.pi / f
            if L < sc["original"] / sc["high"]:
                pass
            elif L > sc["original"] / sc["low"]:
                f = f / sc["factor"]
            else:
                s = (sc["original"] / L - sc["low"]) / (sc["high"] - sc["low"])
                f = (1 - s) * f / sc["factor"] + s * f
        out.append(f)
    return out


def rotate_head(vec, pos, freqs):
    """Rotate the pairs (2i, 2i+1), i < len(freqs), of one head vector by pos * f_i."""
    out = vec.clone()
    for i, f in enumerate(freqs):
        a = pos * f
        u, v = vec[2 * i].item(), vec[2 * i + 1].item()
        out[2 * i] = u * math.cos(a) - v * math.sin(a)
        out[2 * i + 1] = v * math.cos(a) + u * math.sin(a)
    return out


def visible(i, j, chunk):
    """May the query at position i attend to the key at position j?"""
    if j > i:
        return False
    return chunk <= 0 or i // chunk == j // chunk


def sink_softmax(scores, sink):
    """Softmax weights of `scores` when exp(sink) also sits in the denominator."""
    mx = max(scores.max().item(), sink)
    e = torch.exp(scores - mx)
    return e / (e.sum() + math.exp(sink - mx))


def attention_mixer(W, p, mx, h, eps):
    """h [T, d] -> [T, d].  q = Wq h + bq, k = Wk h + bk, values = k as projected."""
    T = h.shape[0]
    H, G, D = mx["heads"], mx["kv_heads"], mx["dim"]
    q = h @ W[p + "q"].T + W[p + "q.b"]
    k = h @ W[p + "k"].T + W[p + "k.b"]
    vals = k.reshape(T, G, D)
    q = (rms_unit(q, eps) * W[p + "q.norm"]).reshape(T, H, D)
    k = (rms_unit(k, eps) * W[p + "k.norm"]).reshape(T, G, D)
    freqs = rotary_frequencies(mx["rot"])
    q = torch.stack([torch.stack([rotate_head(q[t, a], t, freqs) for a in range(H)])
                     for t in range(T)])
    k = torch.stack([torch.stack([rotate_head(k[t, a], t, freqs) for a in range(G)])
                     for t in range(T)])
    chunk = (mx.get("mask") or {}).get("size", 0)
    gates = torch.sigmoid(h @ W[p + "g"].T)
    heads = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        js = [j for j in range(T) if visible(t, j, chunk)]
        for a in range(H):
            kv = a // (H // G)
            scores = (k[js, kv] @ q[t, a]) * mx["scale"]
            wts = sink_softmax(scores, W[p + "sink"][a].item())
            heads[t, a] = (wts @ vals[js, kv]) * gates[t, a]
    return heads.reshape(T, H * D) @ W[p + "o"].T + W[p + "o.b"]


def feed_forward(W, p, h):
    return torch.relu(h @ W[p + "up"].T) ** 2 @ W[p + "down"].T


def layer_order(cfg):
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return list(range(n))
    inner = list(range(lp["start"], lp["stop"]))
    return list(range(lp["start"])) + inner * lp["times"] + list(range(lp["stop"], n))


def forward(cfg, weights, tokens):
    """Logits [T, vocab] of a whole sequence, and the stream after every layer run."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = W["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    streams = []
    for i in layer_order(cfg):
        ly = cfg["layers"][i]
        h = rms_unit(x, eps) * W[f"l{i}.norm1"]
        y = attention_mixer(W, f"l{i}.mix.", ly["mixer"], h, eps)
        if ly.get("mlp") is not None:
            y = y + feed_forward(W, f"l{i}.mlp.", h)
        x = x + m * y
        streams.append(x.clone())
    x = rms_unit(x, eps) * W["final.norm"]
    return x @ W["head"].T, streams


def random_weights(cfg, seed=0, std=0.08):
    """bf16-representable random weights under the checkpoint's names."""
    g = torch.Generator().manual_seed(seed)
    d, V = cfg["width"], cfg["vocab"]

    def r(*shape, s=std, mean=0.0):
        return (torch.randn(*shape, generator=g) * s + mean).to(torch.bfloat16)

    W = {"embed": r(V, d, s=1.0), "final.norm": r(d, s=0.2, mean=1.0), "head": r(V, d)}
    for i, ly in enumerate(cfg["layers"]):
        mx = ly["mixer"]
        H, G, D = mx["heads"], mx["kv_heads"], mx["dim"]
        p = f"l{i}."
        W[p + "norm1"] = r(d, s=0.2, mean=1.0)
        W[p + "mix.q"] = r(H * D, d)
        W[p + "mix.q.b"] = r(H * D, s=0.3)
        W[p + "mix.k"] = r(G * D, d)
        W[p + "mix.k.b"] = r(G * D, s=0.3)
        W[p + "mix.q.norm"] = r(H * D, s=0.3, mean=1.0)
        W[p + "mix.k.norm"] = r(G * D, s=0.3, mean=1.0)
        W[p + "mix.sink"] = r(H, s=1.5)
        W[p + "mix.g"] = r(H, d, s=0.3)
        W[p + "mix.o"] = r(d, H * D)
        W[p + "mix.o.b"] = r(d, s=0.3)
        if ly.get("mlp") is not None:
            W[p + "mlp.up"] = r(ly["mlp"]["ff"], d)
            W[p + "mlp.down"] = r(d, ly["mlp"]["ff"])
    return W


def make_config(width=48, vocab=61, layers=None, loop=None, eps=1e-5, mult=0.8, embed_scale=3.0):
    return {"architecture": "Bidetar", "embedding": {"scale": embed_scale}, "layers": layers,
            "loop": loop, "norm": {"eps": eps}, "residual_mult": mult, "vocab": vocab,
            "width": width}


def make_layer(heads=3, kv_heads=1, dim=8, chunk=10, rot_dims=4, base=100.0, scaling=None,
               scale=0.4, ff=40):
    return {"type": "attention",
            "mixer": {"dim": dim, "vdim": dim, "heads": heads, "kv_heads": kv_heads,
                      "mask": {"size": chunk},
                      "rot": {"base": base, "dims": rot_dims, "scaling": scaling},
                      "scale": scale},
            "mlp": None if ff is None else {"ff": ff, "kind": "dense"}}
