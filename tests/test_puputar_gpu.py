"""Puputar on the HIP kernels: every new kernel against the PyTorch version of the same op (fp32
and bf16 storage, odd and 16-byte-aligned sizes), then the engine -- mixed steps, hipGraph
decode, a small page and slot pool -- against the float64 oracle (tests/puputar_oracle.py), and
greedy generation through LLMEngine.generate."""
import pytest
import torch

import puputar_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from test_puputar import OTHER, _latent_case, base_config
from aws_k8s_ansible_provisioner_amd.ops import stream as sops

pytestmark = pytest.mark.gpu
TOL = {"float32": 3e-4, "bfloat16": 0.08}
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}


def gen(seed):
    return torch.Generator().manual_seed(seed)


def close(a, b, dtype):
    tol = 2e-5 if dtype == "float32" else 2e-2
    torch.testing.assert_close(a.float().cpu(), b.float().cpu(), rtol=tol, atol=tol)


# ------------------------------------------------------------------ kernels against their ops
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d,groups", [(24, 4), (2048, 1), (1536, 3), (54, 9), (4100, 2), (4096, 1),
                                      (8192, 1), (8192, 4), (40, 2)])
def test_add_group_norm_kernel(dtype, d, groups):
    g, dt = gen(d), DT[dtype]
    T = 7
    x = torch.randn(T, d, generator=g)
    # y is a column slice of wider rows (16-byte aligned rows when d allows: the vector path)
    y, b = torch.randn(T, d + 4, generator=g).to(dt), torch.randn(d, generator=g).to(dt)
    y2 = torch.randn(T, d, generator=g)
    w1, w2 = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    for use in [(True, True, True, True), (True, False, False, False), (False, False, False, False),
                (False, True, True, False)]:
        xs = [x.clone(), x.clone().cuda()]
        outs = []
        for xx in xs:
            dev = xx.device
            o1 = torch.zeros(T, d, dtype=dt, device=dev)
            o2 = torch.zeros(T, d, dtype=dt, device=dev) if use[3] else None
            sops.stream_add_group_norm(xx, y[:, :d].to(dev) if use[0] else None,
                                       y2.to(dev) if use[1] else None, b.to(dev) if use[2] else None,
                                       w1.to(dev), w2.to(dev) if use[3] else None, groups, 1e-5, o1, o2)
            outs.append((o1, o2))
        close(xs[1], xs[0], "float32")
        close(outs[1][0], outs[0][0], dtype)
        if use[3]:
            close(outs[1][1], outs[0][1], dtype)
    # fp32 output from bf16-typed inputs (the normed embedding is the stream itself)
    o_c, o_g = torch.zeros(T, d), torch.zeros(T, d, device="cuda")
    sops.stream_add_group_norm(x.clone(), None, None, None, w1, None, groups, 1e-5, o_c)
    sops.stream_add_group_norm(x.clone().cuda(), None, None, None, w1.cuda(), None, groups, 1e-5, o_g)
    close(o_g, o_c, "float32")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d,groups", [(54, 9), (2048, 4), (6144, 1)])
def test_add_group_norm_with_shift_kernel(dtype, d, groups):
    """Decode steps: the token shift of the first output inside the norm kernel equals the norm
    followed by token_shift(single=True), state included."""
    g, dt = gen(d), DT[dtype]
    T = 5
    x = torch.randn(T, d, generator=g)
    y = torch.randn(T, d, generator=g).to(dt)
    w1, w2 = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    mu = torch.rand(d, generator=g)
    state = torch.randn(4, d, generator=g).to(dt)
    slot = torch.tensor([2, 0, 3, 1, -1], dtype=torch.int32)
    pos = torch.tensor([5, 0, 9, 4, 0])
    res = []
    for dev in ("cpu", "cuda"):
        xx, st = x.clone().to(dev), state.clone().to(dev)
        o1 = torch.zeros(T, d, dtype=dt, device=dev)
        o2 = torch.zeros(T, d, dtype=dt, device=dev)
        sops.stream_add_group_norm(xx, y.to(dev), None, None, w1.to(dev), w2.to(dev), groups, 1e-5,
                                   o1, o2, shift=(mu.to(dev), st, slot.to(dev), pos.to(dev)))
        res.append((xx, o1[:4], o2, st))
    close(res[1][0], res[0][0], "float32")
    for a, b in zip(res[1][1:], res[0][1:]):
        close(a, b, dtype)
    # against the two-step form on the GPU itself
    xx, st = x.clone().cuda(), state.clone().cuda()
    n1 = torch.zeros(T, d, dtype=dt, device="cuda")
    h = torch.zeros(T, d, dtype=dt, device="cuda")
    sops.stream_add_group_norm(xx, y.cuda(), None, None, w1.cuda(), None, groups, 1e-5, n1)
    sops.token_shift(n1, mu.cuda(), st, slot.cuda(), pos.cuda(), h, single=True)
    close(h[:4], res[1][1], dtype)      # (the compiler may contract the blend differently)
    assert torch.equal(st, res[1][3])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("d", [70, 72, 2048])
def test_token_shift_kernel(dtype, d):
    g, dt = gen(1), DT[dtype]
    h = torch.randn(9, d, generator=g).to(dt)
    mu = torch.rand(d, generator=g)
    state = torch.randn(4, d, generator=g).to(dt)
    slot = torch.tensor([2, 2, 2, 0, 0, 3, 1, -1, -1], dtype=torch.int32)
    pos = torch.tensor([5, 6, 7, 0, 1, 9, 4, 0, 0])
    res = []
    for dev in ("cpu", "cuda"):
        st, out = state.clone().to(dev), torch.zeros(9, d, dtype=dt, device=dev)
        sops.token_shift(h.to(dev), mu.to(dev), st, slot.to(dev), pos.to(dev), out)
        res.append((out[:7], st))
    close(res[1][0], res[0][0], dtype)
    assert torch.equal(res[1][1].cpu(), res[0][1])
    # a decode step (every row a sequence of its own): one launch reads and replaces the state
    slot1 = torch.tensor([2, 0, 3, 1, -1], dtype=torch.int32)
    pos1 = torch.tensor([5, 0, 9, 4, 0])
    res = []
    for dev in ("cpu", "cuda"):
        st, out = state.clone().to(dev), torch.zeros(5, d, dtype=dt, device=dev)
        sops.token_shift(h[:5].to(dev), mu.to(dev), st, slot1.to(dev), pos1.to(dev), out, single=True)
        res.append((out[:4], st))
    close(res[1][0], res[0][0], dtype)
    assert torch.equal(res[1][1].cpu(), res[0][1])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("Q,R,r", [(6, 10, 4), (768, 512, 64), (17, 70, 10)])
def test_latent_prep_and_rotate_kernels(dtype, Q, R, r):
    g, dt = gen(Q), DT[dtype]
    T, BS, NB, H, D = 7, 8, 4, 3, 6
    proj = torch.randn(T, 3 + Q + R + r + 2, generator=g).to(dt)
    qw, kw = 1 + 0.3 * torch.randn(Q, generator=g), 1 + 0.3 * torch.randn(R, generator=g)
    pos = torch.tensor([0, 1, 7, 8, 9, 31, 5])
    slots = torch.tensor([3, 0, 7, 8, 15, 31, -1])
    table = sops.rotary_table(32, r, 50.0)
    q = torch.randn(T, H, D + r, generator=g).to(dt)
    res = []
    for dev in ("cpu", "cuda"):
        cq = torch.zeros(T, Q, dtype=dt, device=dev)
        cache = torch.zeros(NB, BS, R + r, dtype=dt, device=dev)
        sops.latent_prep(proj.to(dev), cq, cache, pos.to(dev), slots.to(dev), table.to(dev),
                         qw.to(dev), kw.to(dev), Q, R, r, 3, 3 + Q, 1e-5)
        cq2 = torch.zeros(T, Q, dtype=dt, device=dev)
        sops.latent_prep(proj.to(dev), cq2, None, pos.to(dev), slots.to(dev), table.to(dev),
                         qw.to(dev), None, Q, R, r, 3, -1, 1e-5)
        assert torch.equal(cq, cq2)
        qq = q.clone().to(dev)
        sops.rotate_heads_(qq, pos.to(dev), table.to(dev), D)
        res.append((cq, cache, qq))
    for a, b in zip(res[1], res[0]):
        close(a, b, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H,D,r,V,R", [(3, 6, 4, 5, 10), (5, 8, 8, 8, 24), (16, 128, 64, 128, 512),
                                       (9, 5, 10, 4, 70)])
def test_latent_attention_kernel(dtype, H, D, r, V, R):
    dt, BS = DT[dtype], 32
    lens = [300, 77, 300]
    cache, bt, rows, w_uk, w_uv, q = _latent_case(H, 23, H, D, r, V, R, BS, lens)
    pos = torch.cat([torch.arange(280, 300), torch.tensor([76, 299, 0])])
    q_start = torch.tensor([0, 20, 21, 22, 23], dtype=torch.int32)
    seq_lens = torch.tensor([300, 77, 300, 0], dtype=torch.int32)
    bt = torch.cat([bt, bt[:1]])
    cache[int(bt[0, 0]), 5] *= 4.0          # a far key that matters
    q_lat = (torch.einsum("thd,hdr->htr", q[..., :D], w_uk) * R ** -0.5).contiguous()
    scale = (D + r) ** -0.5
    res = []
    for dev in ("cpu", "cuda"):
        out = torch.zeros(H, 23, R, dtype=dt, device=dev)
        sops.latent_attention(out, q_lat.to(dt).to(dev), q.to(dt).to(dev), D, cache.to(dt).to(dev),
                              bt.to(dev), seq_lens.to(dev), q_start.to(dev), pos.to(dev), scale)
        out1 = torch.zeros(H, 3, R, dtype=dt, device=dev)
        sops.latent_attention(out1, q_lat[:, 20:23].contiguous().to(dt).to(dev),
                              q[20:23].contiguous().to(dt).to(dev), D, cache.to(dt).to(dev),
                              bt[1:4].contiguous().to(dev), seq_lens[1:4].contiguous().to(dev), None,
                              pos[20:23].to(dev), scale)
        res.append((out, out1))
    close(res[1][0], res[0][0], dtype)
    close(res[1][1], res[0][1], dtype)
    close(res[1][1][:, :2], res[1][0][:, 20:22], dtype)
    assert res[1][0][:, 22].abs().max().item() == 0      # padding rows are left alone


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("V,F_", [(5, 37), (8, 40), (128, 2052)])
def test_gate_activation_and_routing_kernels(dtype, V, F_):
    g, dt = gen(4), DT[dtype]
    H, T = 3, 6
    o = torch.randn(H, T, V, generator=g).to(dt)
    wide = torch.randn(T, 4 + H * V + 4, generator=g).to(dt)
    x = (torch.randn(T, F_ + 8, generator=g) * 3).to(dt)
    b = torch.randn(F_, generator=g).to(dt)
    act = torch.tensor([-0.7, 1.3])
    n, d, E = 12, 40, 9
    h = torch.randn(T, d, generator=g).to(dt)
    router, corr = torch.randn(n, d, generator=g), torch.randn(n, generator=g) * 0.1
    up = torch.randn(T, E * F_, generator=g).to(dt)
    ys = torch.randn(T * 4, d, generator=g).to(dt)
    res = []
    for dev in ("cpu", "cuda"):
        r = []
        for cols in (H, H * V):
            out = torch.zeros(T, H * V + 4, dtype=dt, device=dev)
            sops.head_gate(o.to(dev), wide.to(dev)[:, 4:4 + cols], out[:, :H * V])
            r.append(out)
        out = torch.zeros(T, F_ + 4, dtype=dt, device=dev)
        sops.xielu(x.to(dev)[:, 4:4 + F_], b.to(dev), act.to(dev), out[:, :F_])
        r.append(out)
        for count, keep, top in [(1, 1, 4), (3, 2, 4), (4, 1, 3), (12, 5, 4)]:
            ids, w = sops.moe_route(h.to(dev), router.to(dev), corr.to(dev), top, count, keep)
            order = ids.long().argsort(dim=1)
            r += [ids.long().gather(1, order).float(), w.gather(1, order)]
        ids, w = sops.moe_route(h.to(dev), router.to(dev), corr.to(dev), 4, 3, 2)
        a = torch.zeros(T, E * F_, dtype=dt, device=dev)
        sops.relu2_routed(up.to(dev), ids, w, E, a)
        r.append(a)
        inv = torch.randperm(T * 4, generator=gen(5)).int().view(T, 4).to(dev)
        for iv, y in ((None, ys[:T]), (inv, ys)):
            c = torch.zeros(T, d, device=dev)
            sops.moe_combine(c, y.contiguous().to(dev), iv, ids, w, h.to(dev), E)
            r.append(c)
        res.append(r)
    for a, b_ in zip(res[1], res[0]):
        close(a, b_, dtype if a.dtype != torch.float32 or dtype == "float32" else "bfloat16")


# ------------------------------------------------------------------ the engine on the GPU
@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=2)
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    return cfg, W, write_model(tmp_path_factory.mktemp("puputar_gpu"), cfg, W), reqs, want


def check(got, want, dtype):
    for n in got:
        e = rel_err(got[n], want[n])
        if dtype == "bfloat16":
            # a close routing choice can flip at bf16 precision and move one position's logits
            # (and, through the cache, a little of what follows): nearly all must be close
            assert e.median().item() < 0.03 and (e > TOL[dtype]).sum().item() <= 2, \
                f"{n}: {(e > TOL[dtype]).sum().item()} positions off, worst {e.max():.2e}"
        else:
            assert e.max().item() < TOL[dtype], f"{n}: position {int(e.argmax())} off by {e.max():.2e}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("eager", [False, True])
def test_schedules(model, dtype, eager):
    _, _, path, reqs, want = model
    eng = engine(path, dtype=dtype, device="cuda", eager=eager)
    assert eager or eng.runner.graphs, "decode hipGraphs were not captured"
    one = {"a": reqs["a"]}
    check(replay(eng, reqs, [[(n, len(t))] for n, t in reqs.items()]), want, dtype)
    check(replay(eng, one, [[("a", 40)]] + [[("a", 1)]] * 35), want, dtype)
    check(replay(eng, one, [[("a", s)] for s in [3, 2, 7, 2, 19, 2, 5, 33, 2]]), want, dtype)
    sched = [[("a", 30), ("b", 2), ("c", 1)],
             [("a", 1), ("b", 20), ("c", 22), ("d", 1)],
             [("a", 1), ("b", 1), ("e", 33)],
             [("a", 1), ("b", 1)],
             [("b", 17), ("e", 1)],
             [("a", 42), ("e", 30)]]
    check(replay(eng, reqs, sched), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pool_is_used_again(model, dtype):
    _, _, path, reqs, want = model
    eng = engine(path, dtype=dtype, max_tokens=160, max_seqs=2, device="cuda")
    many = {f"{n}{i}": reqs[n] for i in range(2) for n in ("b", "c", "e")}
    many["a"] = reqs["a"]
    sched = [[("b0", 41), ("c0", 23)], [("e0", 64), ("c1", 22)], [("c1", 1)],
             [("a", 75), ("b1", 41)], [("e1", 10)], [("e1", 54)]]
    for _ in range(2):  # graphs replayed again over pages and slots that changed owners
        check(replay(eng, many, sched), {k: want[k[0]] for k in many}, dtype)
    assert eng.sched.num_free_blocks() == 5 and eng.sched.num_free_tail_slots == 2


def test_long_decode_through_graphs(tmp_path):
    cfg = oracle.make_config(width=64, vocab=37, groups=2, layers=[
        oracle.make_layer(heads=4, dim=16, rot_dim=8, vdim=16, kv_rank=24, q_rank=20),
        oracle.make_layer(heads=2, dim=8, rot_dim=8, vdim=12, kv_rank=24, q_rank=16, kv_from=0,
                          gate="element",
                          moe=dict(experts=6, ff=16, top=2, identity=2, count=4, keep=2))])
    W = oracle.random_weights(cfg, seed=5)
    toks = tokens(700, 37, 6)
    want = {"a": oracle.forward(cfg, W, toks)}
    eng = engine(write_model(tmp_path, cfg, W), dtype="float32", max_tokens=704, device="cuda")
    assert eng.runner.graphs
    check(replay(eng, {"a": toks}, [[("a", 500)]] + [[("a", 1)]] * 200), want, "float32")


def test_large_prompt_takes_the_sorted_expert_path(tmp_path):
    """A prompt portion over the small-batch threshold of the routed feed-forward."""
    from aws_k8s_ansible_provisioner_amd.models import puputar

    cfg = oracle.make_config(width=32, vocab=37, groups=1, layers=[
        oracle.make_layer(heads=2, dim=8, rot_dim=4, vdim=8, kv_rank=16, q_rank=12,
                          moe=dict(experts=5, ff=16, top=2, identity=1, count=3, keep=2))])
    W = oracle.random_weights(cfg, seed=6)
    toks = tokens(puputar.MOE_DENSE_ROWS + 70, 37, 7)
    want = {"a": oracle.forward(cfg, W, toks)}
    eng = engine(write_model(tmp_path, cfg, W), dtype="float32", max_tokens=512, device="cuda")
    n = puputar.MOE_DENSE_ROWS + 40
    check(replay(eng, {"a": toks}, [[("a", n)], [("a", 30)]]), want, "float32")


def test_greedy_generation(model):
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    cfg, W, path, _, _ = model
    eng = LLMEngine(EngineConfig(model=path, load_format="safetensors", weights_path=path,
                                 dtype="float32", max_model_len=128, max_num_seqs=4,
                                 max_num_batched_tokens=24, num_gpu_blocks=16, device="cuda",
                                 gc_freeze=False), log=lambda *a: None)
    assert eng.runner.graphs
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (30, 3, 17, 9)]
    outs = eng.generate(None, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True),
                        prompt_ids=prompts)
    assert [len(o.output_ids) for o in outs] == [12] * 4
    for p, o in zip(prompts, outs):
        logits = oracle.forward(cfg, W, p + o.output_ids)
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_configurations(tmp_path, name, dtype):
    cfg = oracle.make_config(**dict(OTHER[name]))
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W), dtype=dtype, device="cuda")
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want, dtype)


# ------------------------------------------------------------------ matrix-core attention
def _tile_map(q_start, seq_lens, first_seq, tile_rows):
    """Tiles of tile_rows chunk rows per sequence, sorted by ascending causal work like the
    scheduler's map."""
    tiles = []
    for b in range(first_seq, len(seq_lens)):
        qlen = int(q_start[b + 1] - q_start[b])
        for r0 in range(0, qlen, tile_rows):
            tiles.append((int(seq_lens[b]) - qlen + min(r0 + tile_rows, qlen), b, r0))
    tiles.sort()
    return (torch.tensor([t[1] for t in tiles], dtype=torch.int32),
            torch.tensor([t[2] for t in tiles], dtype=torch.int32))


@pytest.mark.parametrize("H,D,r,R", [(3, 8, 16, 64), (6, 32, 16, 96), (4, 16, 32, 128), (2, 24, 16, 128),
                                     (33, 8, 32, 256), (5, 16, 64, 256), (16, 128, 64, 512)])
def test_latent_attention_matrix_core_kernels(H, D, r, R):
    """Prefill tiles (a chunk that continues a cached prefix, a whole prompt, a short one) and
    split decode on the matrix cores against the PyTorch op; one far key per sequence is made
    to matter."""
    BS, dt = 32, torch.bfloat16
    lens = [700, 333, 40, 650, 129]
    chunk = [300, 333, 40]                       # sequences 0..2 bring prompt rows, 3..4 decode
    T = sum(chunk)
    cache, bt, rows, w_uk, _, q = _latent_case(R, T, H, D, r, 8, R, BS, lens)
    for b in range(len(lens)):
        cache[int(bt[b, 0]), 3] *= 3.0
    cache = cache.to(dt)
    vg = sops_groups(cache[..., :R])
    q_start = torch.tensor([0, 300, 633, 673], dtype=torch.int32)
    seq_lens = torch.tensor(lens[:3], dtype=torch.int32)
    pos = torch.cat([torch.arange(n - c, n) for n, c in zip(lens[:3], chunk)])
    q = (q * 0.5).to(dt)
    q_lat = (torch.einsum("thd,hdr->htr", q[..., :D].float(), w_uk) * 0.5).to(dt).contiguous()
    scale = (D + r) ** -0.5
    want = torch.zeros(H, T, R, dtype=dt)
    sops.latent_attention(want, q_lat, q, D, cache, bt[:3], seq_lens, q_start, pos, scale)
    tile_seq, tile_row = _tile_map(q_start, seq_lens, 0, 128)
    got = torch.zeros(H, T, R, dtype=dt, device="cuda")
    assert sops.latent_mfma_ok(cache.cuda(), vg.cuda(), R, q.cuda(), D, scale)
    sops.latent_attention_prefill(got, q_lat.cuda(), q.cuda(), D, cache.cuda(), vg.cuda(),
                                  bt[:3].cuda(), seq_lens.cuda(), q_start.cuda(), pos.cuda(),
                                  tile_seq.cuda(), tile_row.cuda(), 128, scale)
    close(got, want, "bfloat16")
    # decode rows of sequences 3, 4 and a padding row, unsplit and split
    seq_d = torch.tensor([650, 129, 0], dtype=torch.int32)
    btd = torch.cat([bt[3:5], bt[:1]])
    qd = q[:3].contiguous()
    qld = q_lat[:, :3].contiguous()
    posd = torch.tensor([649, 128, 0])
    want_d = torch.zeros(H, 3, R, dtype=dt)
    sops.latent_attention(want_d, qld, qd, D, cache, btd, seq_d, None, posd, scale)
    for parts in (1, 2, 7):
        got_d = torch.zeros(H, 3, R, dtype=dt, device="cuda")
        ws = sops.latent_decode_workspace(3, H, R, parts, "cuda")
        sops.latent_attention_decode(got_d, qld.cuda(), qd.cuda(), D, cache.cuda(), vg.cuda(),
                                     btd.cuda(), seq_d.cuda(), posd.cuda(), scale, ws, parts)
        close(got_d, want_d, "bfloat16")
        assert got_d[:, 2].abs().max().item() == 0


def sops_groups(c):
    """[NB, BS, R] token-major latents in the grouped layout [NB, BS / 8, R, 8]."""
    NB, BS, R = c.shape
    return c.view(NB, BS // 8, 8, R).permute(0, 1, 3, 2).contiguous()


@pytest.mark.parametrize("eager", [False, True])
def test_engine_on_the_matrix_core_path(tmp_path, eager):
    """Sizes the matrix-core kernels take (bf16): prompts over several tiles, portions, mixed
    steps, a small pool used twice, decoding through hipGraphs with split keys; and the fp32
    engine of the same model (row kernel) against the oracle, tightly."""
    cfg = oracle.make_config(width=64, vocab=61, groups=4, layers=[
        oracle.make_layer(heads=5, dim=16, rot_dim=16, vdim=8, kv_rank=64, q_rank=24),
        oracle.make_layer(heads=3, dim=8, rot_dim=16, vdim=24, kv_rank=96, q_rank=40,
                          gate="element", ff=None),
        oracle.make_layer(heads=6, dim=24, rot_dim=16, vdim=16, kv_rank=64, q_rank=32, kv_from=0,
                          moe=dict(experts=6, ff=32, top=2, identity=2, count=4, keep=2))])
    W = oracle.random_weights(cfg, seed=11)
    reqs = {"a": tokens(390, 61, 1), "b": tokens(200, 61, 2), "c": tokens(35, 61, 3)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    path = write_model(tmp_path, cfg, W)
    sched = [[("a", 300), ("b", 2)], [("a", 1), ("b", 150), ("c", 35)], [("a", 1), ("b", 1)],
             [("a", 60), ("b", 47)], [("a", 28)]]
    for dtype in ("bfloat16", "float32"):
        eng = engine(path, dtype=dtype, max_tokens=704, max_seqs=3, device="cuda", eager=eager)
        grouped = [g is not None for g in eng.runner.v_caches]
        assert grouped == [dtype == "bfloat16"] * 3
        for _ in range(2):
            check(replay(eng, reqs, sched), want, dtype)
        one = {"a": reqs["a"]}
        check(replay(eng, one, [[("a", 330)]] + [[("a", 1)]] * 60), want, dtype)


@pytest.mark.parametrize("H,T,K,N", [(16, 64, 128, 512), (16, 64, 512, 128), (3, 1, 32, 96),
                                     (5, 37, 48, 64), (6, 200, 96, 32), (2, 300, 64, 64), (4, 9, 20, 64)])
def test_head_matmul_kernel(H, T, K, N):
    """The per-head products of small batches (strided rows of a [T, H, n] buffer as well as
    head-major rows) against the batched library GEMM in fp32; more rows than the kernel takes
    and sizes off its grid go to the library."""
    g = gen(H * T)
    wide = (torch.randn(T, H, K + 16, generator=g) * 0.5).to(torch.bfloat16).cuda()
    w = (torch.randn(H, N, K, generator=g) * K ** -0.5).to(torch.bfloat16).cuda()
    a = wide[:, :, :K].transpose(0, 1)
    want = torch.bmm(a.float(), w.float().transpose(1, 2))
    close(sops.head_matmul(a, w), want, "bfloat16")
    close(sops.head_matmul(a.contiguous(), w), want, "bfloat16")


def test_decode_workspace_serves_layers_of_unequal_heads_and_latents(tmp_path):
    """A layer with few heads and a wide latent followed by one with many heads and a narrow
    latent: the split-decode scratch has to fit both the per-(row, head) statistics and the
    latent outputs of every layer, also in the captured graphs."""
    cfg = oracle.make_config(width=64, vocab=41, groups=2, layers=[
        oracle.make_layer(heads=4, dim=8, rot_dim=32, vdim=8, kv_rank=256, q_rank=24),
        oracle.make_layer(heads=12, dim=16, rot_dim=16, vdim=4, kv_rank=64, q_rank=24, ff=32)])
    W = oracle.random_weights(cfg, seed=4)
    reqs = {"a": tokens(300, 41, 1), "b": tokens(200, 41, 2)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W), dtype="bfloat16", max_tokens=640, device="cuda")
    assert eng.runner.graphs and all(g is not None for g in eng.runner.v_caches)
    sched = [[("a", 280), ("b", 190)]] + [[("a", 1), ("b", 1)]] * 10 + [[("a", 10)]]
    check(replay(eng, reqs, sched), want, "bfloat16")
