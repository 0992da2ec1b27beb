"""HIP kernels of ops.stream against the plain PyTorch version of the same op (the CPU branch
of each entry point, run on fp32 copies of the same inputs)."""
import math

import pytest
import torch

from aws_k8s_ansible_provisioner_amd.ops import stream as sops

pytestmark = pytest.mark.gpu
DEV = "cuda"


def tol(dt):
    return dict(rtol=2e-2, atol=2e-2) if dt == torch.bfloat16 else dict(rtol=2e-5, atol=2e-5)


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("d", [48, 192, 1024, 5120])
def test_embed_norm_relu2(dt, d):
    g = torch.Generator().manual_seed(d)
    T, V = 37, 101
    table = torch.randn(V, d, generator=g).to(dt)
    ids = torch.randint(0, V, (T,), generator=g)
    x = sops.embed_scaled(ids.to(DEV), table.to(DEV), 3.25)
    xr = sops.embed_scaled(ids, table, 3.25)
    torch.testing.assert_close(x.cpu(), xr, rtol=1e-6, atol=1e-6)
    w = 1 + 0.1 * torch.randn(d, generator=g)
    h = sops.stream_norm(x, w.to(DEV), 1e-5, dt)
    hr = sops.stream_norm(xr, w, 1e-5, dt)
    torch.testing.assert_close(h.cpu().float(), hr.float(), **tol(dt))
    y = torch.randn(T, d + 8, generator=g).to(dt)[:, 3:3 + d]  # a strided slice
    x2, xr2 = x.clone(), xr.clone()
    h2 = sops.stream_add_norm(x2, y.to(DEV)[:, :], 0.7, w.to(DEV), 1e-5, dt)
    hr2 = sops.stream_add_norm(xr2, y, 0.7, w, 1e-5, dt)
    torch.testing.assert_close(x2.cpu(), xr2, rtol=1e-6, atol=1e-6)
    torch.testing.assert_close(h2.cpu().float(), hr2.float(), **tol(dt))
    wide = torch.randn(T, d + 16, generator=g).to(dt)
    out = torch.zeros(T, d + 5, dtype=dt, device=DEV)
    outr = torch.zeros(T, d + 5, dtype=dt)
    sops.relu2(wide.to(DEV)[:, 7:7 + d], out[:, 5:])
    sops.relu2(wide[:, 7:7 + d], outr[:, 5:])
    torch.testing.assert_close(out.cpu().float(), outr.float(), **tol(dt))


def paged(B, lens, BS, G, D, dt, g, extra_blocks=3):
    """Random caches and shuffled block tables for sequences of the given lengths."""
    mb = max(-(-n // BS) for n in lens) + 1
    NB = sum(-(-n // BS) for n in lens) + extra_blocks
    perm = torch.randperm(NB, generator=g)
    bt = torch.zeros(B, mb, dtype=torch.int32)
    o = 0
    for b, n in enumerate(lens):
        nb = -(-n // BS)
        bt[b, :nb] = perm[o:o + nb].int()
        o += nb
    kc = torch.randn(NB, G, BS, D, generator=g).to(dt)
    vc = sops.v_from_tokens(torch.randn(NB, G, BS, D, generator=g)).to(dt)
    return kc, vc, bt


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("H,G,D,rd", [(4, 2, 64, 64), (6, 2, 32, 16), (8, 8, 128, 64), (3, 1, 80, 80),
                                      (2, 1, 256, 32)])
def test_proj_norm_rope_cache(dt, H, G, D, rd):
    g = torch.Generator().manual_seed(H * 100 + D)
    T, BS, NB = 45, 32, 9
    N = H * D + G * D + 24
    proj = torch.randn(T, N + 8, generator=g).to(dt)[:, :N]
    pos = torch.randint(0, 300, (T,), generator=g)
    slots = torch.randperm(NB * BS, generator=g)[:T]
    slots[5] = -1
    cs = sops.rotary_table(300, rd, 10000.0, {"factor": 8.0, "low": 1.0, "high": 4.0,
                                              "original": 64})
    qw = 1 + 0.1 * torch.randn(H * D, generator=g)
    kw = 1 + 0.1 * torch.randn(G * D, generator=g)

    def run(dev):
        q = torch.zeros(T, H, D, dtype=dt, device=dev)
        kc = torch.zeros(NB, G, BS, D, dtype=dt, device=dev)
        vc = torch.zeros(NB, G, BS // 8, D, 8, dtype=dt, device=dev)
        sops.proj_norm_rope_cache(proj.to(dev), q, kc, vc, pos.to(dev), slots.to(dev), cs.to(dev),
                                  qw.to(dev), kw.to(dev), H, G, D, 8, 8 + H * D, 1e-5)
        return q.cpu().float(), kc.cpu().float(), vc.cpu().float()

    for a, b in zip(run(DEV), run("cpu")):
        torch.testing.assert_close(a, b, **tol(dt))


CASES = [  # H, G, D, chunk, window, sink, gate
    (4, 2, 64, 120, 0, True, True),
    (4, 2, 64, 0, 0, True, True),
    (6, 3, 32, 50, 0, False, True),
    (8, 2, 128, 0, 70, True, False),
    (2, 2, 80, 64, 33, True, True),
    (3, 1, 256, 1000, 0, False, False),
    (16, 2, 128, 512, 0, True, True),
    (40, 1, 32, 90, 0, True, True),     # more query heads per K/V head than one 32-column tile
]


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("tr", [64, 128, 256])   # 128 / 256-token tiles in bf16: matrix cores
@pytest.mark.parametrize("H,G,D,chunk,window,use_sink,use_gate", CASES)
def test_sink_attention_prefill(dt, tr, H, G, D, chunk, window, use_sink, use_gate):
    g = torch.Generator().manual_seed(H + D + chunk + window)
    BS = 32
    lens = [700, 130, 65, 1, 257]       # cached tokens after the step
    qlens = [300, 130, 2, 1, 129]       # tokens of this step's chunk
    B = len(lens)
    kc, vc, bt = paged(B, lens, BS, G, D, dt, g)
    T = sum(qlens)
    q = torch.randn(T, H, D, generator=g).to(dt)
    gate = torch.randn(T, H + 3, generator=g).to(dt)[:, 1:1 + H] if use_gate else None
    sink = torch.randn(H, generator=g) if use_sink else None
    qs = torch.tensor([0] + list(torch.tensor(qlens).cumsum(0)), dtype=torch.int32)
    ts, trow = [], []
    for b, n in enumerate(qlens):
        for r in range(0, n, tr):
            ts.append(b)
            trow.append(r)
    order = torch.randperm(len(ts), generator=g)   # any tile order
    ts = torch.tensor(ts, dtype=torch.int32)[order]
    trow = torch.tensor(trow, dtype=torch.int32)[order]
    sl = torch.tensor(lens, dtype=torch.int32)
    scale = 1.0 / math.sqrt(D)

    def run(dev):
        out = torch.zeros(T, H * D + 16, dtype=dt, device=dev)
        mv = lambda t: None if t is None else t.to(dev)  # noqa: E731
        sops.sink_attention_prefill(out, q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), sl.to(dev),
                                    qs.to(dev), ts.to(dev), trow.to(dev), tr, mv(gate), mv(sink),
                                    scale, chunk, window)
        return out.cpu().float()

    torch.testing.assert_close(run(DEV), run("cpu"), **tol(dt))


@pytest.mark.parametrize("dt", [torch.bfloat16, torch.float32])
@pytest.mark.parametrize("parts", [1, 3, 8])
@pytest.mark.parametrize("H,G,D,chunk,window,use_sink,use_gate", CASES)
def test_sink_attention_decode(dt, parts, H, G, D, chunk, window, use_sink, use_gate):
    g = torch.Generator().manual_seed(H + D + chunk + window + parts)
    BS = 32
    lens = [1500, 1, 0, 64, 65, 121, 120, 513]   # 0: a padding row
    B = len(lens)
    kc, vc, bt = paged(B, [max(n, 1) for n in lens], BS, G, D, dt, g)
    q = torch.randn(B, H, D, generator=g).to(dt)
    gate = torch.randn(B, H, generator=g).to(dt) if use_gate else None
    sink = torch.randn(H, generator=g) if use_sink else None
    sl = torch.tensor(lens, dtype=torch.int32)
    scale = 1.0 / math.sqrt(D)

    def run(dev):
        out = torch.zeros(B, H * D, dtype=dt, device=dev)
        mv = lambda t: None if t is None else t.to(dev)  # noqa: E731
        ws = sops.decode_workspace(B, H, D, parts, dev) if dev != "cpu" else None
        sops.sink_attention_decode(out, q.to(dev), kc.to(dev), vc.to(dev), bt.to(dev), sl.to(dev),
                                   mv(gate), mv(sink), scale, chunk, window, ws, parts)
        return out.cpu().float()

    torch.testing.assert_close(run(DEV), run("cpu"), **tol(dt))
