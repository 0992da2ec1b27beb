"""Puputar through the engine (scheduler, block manager, sequence slots, runner, ops) against
the plain float64 oracle of tests/puputar_oracle.py, on the CPU branch of the ops (the same
suite runs on the HIP kernels in test_puputar_gpu.py).  Small configurations with random
weights; fp32 runs are compared tightly (a lost shift state, a wrongly seen key or a wrong
expert moves a logit by far more than the tolerance), bf16 runs loosely."""
import pytest
import torch

import puputar_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from aws_k8s_ansible_provisioner_amd.models.config import get_config
from aws_k8s_ansible_provisioner_amd.ops import stream as sops

FP32_TOL = 2e-4
MOE = dict(experts=5, ff=9, top=3, identity=1, count=3, keep=2)


def base_config():
    """Unequal layers: both gate kinds, dense / routed / no feed-forward, a layer that reads
    another one's cache, three norm groups."""
    layers = [
        oracle.make_layer(heads=3, dim=8, rot_dim=4, vdim=6, kv_rank=12, q_rank=10, ff=20),
        oracle.make_layer(heads=2, dim=6, rot_dim=8, vdim=10, kv_rank=20, q_rank=14, base=7000.0,
                          gate="element", moe=MOE, scale=0.3),
        oracle.make_layer(heads=4, dim=4, rot_dim=2, vdim=5, kv_rank=9, q_rank=7, ff=None),
        oracle.make_layer(heads=5, dim=10, rot_dim=8, vdim=3, kv_rank=20, q_rank=11, base=7000.0,
                          gate="element", kv_from=1, ff=13),
        oracle.make_layer(heads=1, dim=8, rot_dim=4, vdim=8, kv_rank=12, q_rank=10, kv_from=0,
                          moe=dict(experts=4, ff=6, top=1)),
    ]
    return oracle.make_config(width=36, vocab=47, layers=layers, groups=3)


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=2)
    return cfg, W, write_model(tmp_path_factory.mktemp("puputar"), cfg, W)


@pytest.fixture(scope="module")
def reference(model):
    cfg, W, _ = model
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    return reqs, {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}


def check(got, want, names=None, tol=FP32_TOL):
    for n in names or got:
        e = rel_err(got[n], want[n])
        assert e.max().item() < tol, f"{n}: position {int(e.argmax())} off by {e.max().item():.2e}"


# ------------------------------------------------------------------ configuration, weights
def test_config_reader(model):
    _, _, path = model
    c = get_config(path)
    assert c.arch == "puputar" and c.num_layers == 5 and c.norm_groups == 3
    assert c.hidden_size == 36 and c.vocab_size == 47
    assert [ls.mixer.gate for ls in c.layer_specs] == ["head", "element", "head", "element", "head"]
    assert [ls.mixer.kv_from for ls in c.layer_specs] == [None, None, None, 1, 0]
    assert c.layer_specs[2].mlp is None and c.layer_specs[1].mlp.router.identity == 1
    assert c.layer_specs[1].mlp.router.groups == 3 and c.layer_specs[4].mlp.router.top == 1
    assert c.num_heads == 5 and c.head_dim == 28
    # three layers own a cache row of kv_rank + rot_dim entries
    assert c.kv_bytes_per_token() == (16 + 28 + 11) * 2


def test_config_reader_refuses_bad_sharing(model):
    from aws_k8s_ansible_provisioner_amd.models.config import puputar_config

    cfg = base_config()
    cfg["layers"][3]["mixer"]["kv_from"] = 0     # layer 0 has another latent size
    with pytest.raises(ValueError):
        puputar_config("x", cfg)
    cfg = base_config()
    cfg["layers"][4]["mixer"]["kv_from"] = 3     # layer 3 has no cache of its own
    with pytest.raises(ValueError):
        puputar_config("x", cfg)


def test_weights_round_trip(model):
    from aws_k8s_ansible_provisioner_amd.models.puputar import PuputarLM

    _, W, path = model
    m = PuputarLM(get_config(path), dtype=torch.float32, max_model_len=64)
    m.load_state_dict(W)
    sd = m.state_dict()
    assert set(sd) == set(W)
    for k, v in W.items():
        assert torch.equal(sd[k].float(), v.float()), k
    bad = dict(W)
    bad["l1.mix.uk"] = W["l1.mix.uk"][:-1]
    with pytest.raises(ValueError):
        m.load_state_dict(bad)
    del bad["l1.mix.uk"]
    with pytest.raises(KeyError):
        m.load_state_dict(bad)


# ------------------------------------------------------------------ each mechanism alone
def test_group_norm_and_deferred_sum():
    """Each part is divided by its OWN root mean square (one part is made 40x larger, which a
    norm over the whole row would spread), both weight sets read the same normalised row, and
    the deferred outputs (projection, bias, routed experts) enter the stream first."""
    g = torch.Generator().manual_seed(0)
    T, d, G = 5, 24, 4
    x0 = torch.randn(T, d, generator=g)
    x0[:, 6:12] *= 40.0
    y, y2, b = torch.randn(T, d, generator=g), torch.randn(T, d, generator=g), torch.randn(d, generator=g)
    w1, w2 = 1 + 0.3 * torch.randn(d, generator=g), 1 + 0.3 * torch.randn(d, generator=g)
    x = x0.clone()
    o1, o2 = torch.empty(T, d), torch.empty(T, d)
    sops.stream_add_group_norm(x, y, y2, b, w1, w2, G, 1e-5, o1, o2)
    s = (x0 + y + y2 + b).double()
    torch.testing.assert_close(x.double(), s, rtol=0, atol=1e-5)
    torch.testing.assert_close(o1.double(), oracle.group_norm(s, w1.double(), G, 1e-5), rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(o2.double(), oracle.group_norm(s, w2.double(), G, 1e-5), rtol=1e-5, atol=1e-5)
    whole = oracle.group_norm(s, w1.double(), 1, 1e-5)
    assert (o1.double() - whole).abs().max() > 0.5
    x = x0.clone()
    sops.stream_add_group_norm(x, None, None, None, w1, None, G, 1e-5, o1)   # nothing added
    assert torch.equal(x, x0)


def test_token_shift_rows_state_and_first_tokens():
    """A batch of three sequences: one continues from its state, one starts at position 0
    (zeros, whatever the slot held), one is a single decoded token; every last row is saved
    unshifted."""
    g = torch.Generator().manual_seed(1)
    d = 10
    h = torch.randn(8, d, generator=g)
    mu = torch.rand(d, generator=g)
    state = torch.randn(4, d, generator=g)
    state0 = state.clone()
    slot = torch.tensor([2, 2, 2, 0, 0, 3, -1, -1], dtype=torch.int32)
    pos = torch.tensor([5, 6, 7, 0, 1, 9, 0, 0])
    out = torch.empty(8, d)
    sops.token_shift(h, mu, state, slot, pos, out)
    want_a, last_a = oracle.token_shift(h[0:3].double(), mu.double(), state0[2].double())
    want_b, last_b = oracle.token_shift(h[3:5].double(), mu.double())
    want_c, last_c = oracle.token_shift(h[5:6].double(), mu.double(), state0[3].double())
    torch.testing.assert_close(out[:6].double(), torch.cat([want_a, want_b, want_c]), rtol=0, atol=1e-6)
    assert torch.equal(state[2], h[2]) and torch.equal(state[0], h[4]) and torch.equal(state[3], h[5])
    assert torch.equal(state[1], state0[1])   # an unused slot keeps its row
    # rows of the same slot that do not follow each other (a sequence's position jumped) are
    # not neighbours
    out2 = torch.empty(2, d)
    st = state0.clone()
    sops.token_shift(h[:2], mu, st, torch.tensor([1, 1], dtype=torch.int32), torch.tensor([4, 9]), out2)
    want, _ = oracle.token_shift(h[1:2].double(), mu.double(), state0[1].double())
    torch.testing.assert_close(out2[1:].double(), want, rtol=0, atol=1e-6)


def test_latent_prep_norms_rotation_and_cache_rows():
    """The query latent and the key/value latent are normed separately (the rotated part is NOT
    part of the key/value norm: it is made 30x larger), pairs (2i, 2i+1) rotate by the position,
    and a cached row is [latent | rotated key]; slot -1 writes nothing."""
    g = torch.Generator().manual_seed(2)
    T, Q, R, r, BS, NB = 7, 6, 10, 4, 8, 3
    proj = torch.randn(T, 3 + Q + R + r + 2, generator=g)
    proj[:, 3 + Q + R:3 + Q + R + r] *= 30.0
    qw, kw = 1 + 0.3 * torch.randn(Q, generator=g), 1 + 0.3 * torch.randn(R, generator=g)
    pos = torch.tensor([0, 1, 7, 8, 9, 23, 5])
    slots = torch.tensor([3, 0, 7, 8, 15, 23, -1])
    cq = torch.zeros(T, Q)
    cache = torch.zeros(NB, BS, R + r)
    sops.latent_prep(proj, cq, cache, pos, slots, sops.rotary_table(32, r, 50.0), qw, kw, Q, R, r,
                     3, 3 + Q, 1e-5)
    p64 = proj.double()
    torch.testing.assert_close(cq.double(), oracle.rms(p64[:, 3:3 + Q], 1e-5) * qw.double(),
                               rtol=1e-5, atol=1e-5)
    c = oracle.rms(p64[:, 3 + Q:3 + Q + R], 1e-5) * kw.double()
    kr = oracle.rotate_pairs(p64[:, 3 + Q + R:3 + Q + R + r], pos, r, 50.0)
    rows = cache.view(NB * BS, R + r).double()
    for t in range(T - 1):
        torch.testing.assert_close(rows[slots[t]], torch.cat([c[t], kr[t]]), rtol=1e-5, atol=1e-4)
    written = torch.zeros(NB * BS, dtype=torch.bool)
    written[slots[:-1]] = True
    assert rows[~written].abs().max() == 0
    cq2 = torch.zeros(T, Q)
    sops.latent_prep(proj, cq2, None, pos, slots, sops.rotary_table(32, r, 50.0), qw, None, Q, R, r,
                     3, -1, 1e-5)             # a layer without a latent of its own
    assert torch.equal(cq, cq2)


def test_rotate_heads_in_place():
    g = torch.Generator().manual_seed(3)
    T, H, D, r = 5, 3, 6, 4
    q = torch.randn(T, H, D + r, generator=g)
    q0 = q.clone()
    pos = torch.tensor([0, 3, 17, 1, 30])
    sops.rotate_heads_(q, pos, sops.rotary_table(32, r, 11.0), D)
    assert torch.equal(q[..., :D], q0[..., :D])
    torch.testing.assert_close(q[..., D:].double(), oracle.rotate_pairs(q0[..., D:].double(), pos, r, 11.0),
                               rtol=1e-5, atol=1e-5)
    assert torch.equal(q[0], q0[0])          # position 0 rotates by nothing


def _latent_case(seed, T, H, D, r, V, R, BS, lens):
    """Random per-head weights and a paged latent cache for sequences of `lens` tokens whose
    pages are scattered; returns everything latent_attention and the oracle need."""
    g = torch.Generator().manual_seed(seed)
    nb = [-(-n // BS) for n in lens]
    NB = sum(nb) + 2
    perm = torch.randperm(NB, generator=g).tolist()
    bt = torch.zeros(len(lens), max(nb) + 1, dtype=torch.int32)
    cache = torch.randn(NB, BS, R + r, generator=g)
    rows = []
    for b, n in enumerate(lens):
        ids = [perm.pop() for _ in range(nb[b])]
        bt[b, :nb[b]] = torch.tensor(ids, dtype=torch.int32)
        rows.append(cache[ids].reshape(-1, R + r)[:n])
    w_uk = torch.randn(H, D, R, generator=g) * R ** -0.5
    w_uv = torch.randn(H, R, V, generator=g) * R ** -0.5
    q = torch.randn(T, H, D + r, generator=g)
    return cache, bt, rows, w_uk, w_uv, q


def _oracle_heads(q, rows, pos, w_uk, w_uv, scale):
    """Per-head keys and values expanded from the cached rows (the textbook form)."""
    H, D, R = w_uk.shape
    c, kr = rows[:, :R].double(), rows[:, R:].double()
    k = torch.einsum("jr,hdr->jhd", c, w_uk.double())
    v = torch.einsum("jr,hrv->jhv", c, w_uv.double())
    s = (torch.einsum("ihd,jhd->hij", q[..., :D].double(), k) +
         torch.einsum("ihd,jd->hij", q[..., D:].double(), kr)) * scale
    ok = torch.arange(rows.shape[0])[None, :] <= pos[:, None]
    a = torch.softmax(s.masked_fill(~ok[None], float("-inf")), dim=-1)
    return torch.einsum("hij,jhv->hiv", a, v)


@pytest.mark.parametrize("far", [0, 5, 31, 32, 200, 255, 256, 299])
def test_latent_attention_sees_one_dominant_key(far):
    """Prompt rows and single decoded rows in one call; one cached key (first token, page
    borders, far back, the last visible one) is scaled so that it takes nearly all the weight of
    the query that is scaled with it: missing it, or seeing it from a query before it, changes
    the output completely."""
    H, D, r, V, R, BS = 3, 6, 4, 5, 10, 32
    lens = [300, 77, 300]
    cache, bt, rows, w_uk, w_uv, q = _latent_case(far, 23, H, D, r, V, R, BS, lens)
    # sequence 0: 20 prompt rows at positions 280 .. 299; sequences 1, 2: one decoded row each,
    # and one padding row at the end
    pos = torch.cat([torch.arange(280, 300), torch.tensor([76, 299, 0])])
    q_start = torch.tensor([0, 20, 21, 22, 23], dtype=torch.int32)
    seq_lens = torch.tensor([300, 77, 300, 0], dtype=torch.int32)
    bt = torch.cat([bt, bt[:1]])
    for b in (0, 2):
        blk, off = int(bt[b, far // BS]), far % BS
        cache[blk, off] *= 6.0
        rows[b][far] *= 6.0
    q[19] *= 3.0
    q[21] *= 3.0
    scale = 0.37
    q_lat = torch.einsum("thd,hdr->htr", q[..., :D], w_uk).contiguous()
    out = torch.zeros(H, 23, R)
    sops.latent_attention(out, q_lat, q, D, cache, bt, seq_lens, q_start, pos, scale)
    o = torch.einsum("htr,hrv->htv", out.double(), w_uv.double())
    for b, (r0, r1) in enumerate([(0, 20), (20, 21), (21, 22)]):
        want = _oracle_heads(q[r0:r1], rows[b], pos[r0:r1], w_uk, w_uv, scale)
        torch.testing.assert_close(o[:, r0:r1], want, rtol=1e-4, atol=1e-4)
    assert out[:, 22].abs().max() == 0       # the padding row is left alone
    # the same decoded rows through the one-query-per-sequence form
    out1 = torch.zeros(H, 2, R)
    sops.latent_attention(out1, q_lat[:, 20:22].contiguous(), q[20:22].contiguous(), D, cache,
                          bt[1:3].contiguous(), seq_lens[1:3].contiguous(), None, pos[20:22], scale)
    torch.testing.assert_close(out1, out[:, 20:22], rtol=1e-5, atol=1e-5)


def test_latent_attention_does_not_see_the_future():
    """A key just after a query's position is made dominant: causal rows must not notice."""
    H, D, r, V, R, BS = 2, 4, 2, 3, 6, 32
    cache, bt, rows, w_uk, w_uv, q = _latent_case(9, 4, H, D, r, V, R, BS, [70])
    pos = torch.tensor([30, 31, 32, 63])
    q_start = torch.tensor([0, 4], dtype=torch.int32)
    seq_lens = torch.tensor([70], dtype=torch.int32)
    q_lat = torch.einsum("thd,hdr->htr", q[..., :D], w_uk).contiguous()
    out = torch.zeros(H, 4, R)
    sops.latent_attention(out, q_lat, q, D, cache, bt, seq_lens, q_start, pos, 0.5)
    for t, p in enumerate(pos.tolist()):
        blk, off = int(bt[0, (p + 1) // BS]), (p + 1) % BS
        keep = cache[blk, off].clone()
        cache[blk, off] *= 50.0
        out2 = torch.zeros(H, 4, R)
        sops.latent_attention(out2, q_lat, q, D, cache, bt, seq_lens, q_start, pos, 0.5)
        assert torch.equal(out2[:, t], out[:, t]), f"position {p} saw key {p + 1}"
        cache[blk, off] = keep


def test_head_gate_kinds():
    g = torch.Generator().manual_seed(4)
    H, T, V = 3, 4, 5
    o = torch.randn(H, T, V, generator=g)
    wide = torch.randn(T, 2 + H * V + 1, generator=g)
    out = torch.zeros(T, H * V + 3)
    sops.head_gate(o, wide[:, 2:2 + H], out[:, :H * V])
    want = o.permute(1, 0, 2).double() * torch.sigmoid(wide[:, 2:2 + H].double())[:, :, None]
    torch.testing.assert_close(out[:, :H * V].double(), want.reshape(T, H * V), rtol=1e-5, atol=1e-6)
    assert out[:, H * V:].abs().max() == 0
    sops.head_gate(o, wide[:, 2:2 + H * V], out[:, :H * V])
    want = o.permute(1, 0, 2).double() * torch.sigmoid(wide[:, 2:2 + H * V].double()).view(T, H, V)
    torch.testing.assert_close(out[:, :H * V].double(), want.reshape(T, H * V), rtol=1e-5, atol=1e-6)


def test_xielu_both_branches():
    g = torch.Generator().manual_seed(5)
    x = torch.randn(6, 11, generator=g) * 3
    x[0, :3] = torch.tensor([0.0, -1e-4, 1e-4])
    b = torch.randn(11, generator=g)
    act = torch.tensor([-0.7, 1.3])
    out = torch.empty(6, 11)
    sops.xielu(x, b, act, out)
    want = oracle.xielu(x.double() + b.double(), act[0], act[1])
    torch.testing.assert_close(out.double(), want, rtol=1e-5, atol=1e-5)
    assert (x + b > 0).any() and (x + b < 0).any()
    sops.xielu(x, None, act, out)
    torch.testing.assert_close(out.double(), oracle.xielu(x.double(), act[0], act[1]), rtol=1e-5, atol=1e-5)


def test_router_groups_correction_and_weights():
    """Constructed scores: the correction changes who is chosen but not the weights; an output
    with a larger choice value in a dropped group loses; choice values can be negative (a
    dropped output must not win as a zero); ties do not occur."""
    n, d = 8, 8
    router = torch.eye(n, d) * 4.0
    h = torch.tensor([[1.0, 0.9, 0.1, 0.0, 0.8, 0.0, 0.0, 0.7],
                      [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 1.0, 0.9]])
    corr = torch.tensor([-0.9, -0.95, -0.8, -0.85, -0.7, -0.99, -0.98, -0.6])
    rt = {"experts": 6, "identity": 2, "top": 3, "groups": {"count": 4, "keep": 2}}
    ids, w = sops.moe_route(h, router, corr, 3, 4, 2)
    oid, ow = oracle.route(h.double(), router.double(), corr.double(), rt)
    assert torch.equal(ids.long().sort(dim=1).values, oid.sort(dim=1).values)
    torch.testing.assert_close(w.double().sort(dim=1).values, ow.sort(dim=1).values, rtol=1e-5, atol=1e-6)
    assert (torch.softmax(h @ router.T, -1) + corr < 0).all()      # all choice values negative
    # without groups and correction the plain top-k of the scores
    ids2, w2 = sops.moe_route(h, router, None, 2, 1, 1)
    assert ids2.sort(dim=1).values.tolist() == [[0, 1], [6, 7]]
    torch.testing.assert_close(w2.sum(dim=1), torch.ones(2))
    # random scores against the oracle
    g = torch.Generator().manual_seed(6)
    h = torch.randn(64, 12, generator=g)
    router = torch.randn(12, 12, generator=g)
    corr = torch.randn(12, generator=g) * 0.1
    for count, keep, top in [(1, 1, 4), (3, 2, 5), (4, 1, 3), (6, 6, 1), (12, 5, 5)]:
        rt = {"experts": 9, "identity": 3, "top": top, "groups": {"count": count, "keep": keep}}
        ids, w = sops.moe_route(h, router, corr, top, count, keep)
        oid, ow = oracle.route(h.double(), router.double(), corr.double(), rt)
        assert torch.equal(ids.long().sort(dim=1).values, oid.sort(dim=1).values), (count, keep, top)
        torch.testing.assert_close(w.double().sum(dim=1), torch.ones(64, dtype=torch.float64))


@pytest.mark.parametrize("small", [True, False])
def test_routed_feed_forward_paths(model, small):
    """Both expert paths (all experts in one GEMM pair; sorted rows per expert) against the
    oracle, identity outputs included."""
    from aws_k8s_ansible_provisioner_amd.models.puputar import PuputarLM

    cfg, W, path = model
    m = PuputarLM(get_config(path), dtype=torch.float32, max_model_len=64)
    m.load_state_dict(W)
    h = torch.randn(40, cfg["width"], generator=torch.Generator().manual_seed(7))
    got = m._routed(m.layers[1], h, small)
    want = oracle.moe_ff(h.double(), {k: v.double() for k, v in W.items()}, "l1.", cfg["layers"][1]["mlp"])
    ids, _ = oracle.route(h.double(), W["l1.mlp.router"].double(), W["l1.mlp.correction"].double(),
                          cfg["layers"][1]["mlp"]["router"])
    assert (ids >= 5).any() and (ids < 5).any()
    torch.testing.assert_close(got.double(), want, rtol=1e-4, atol=1e-4)


# ------------------------------------------------------------------ whole model, schedules
def test_oracle_step_by_step(model, reference):
    """The oracle itself: whole-sequence and token-by-token forms agree."""
    cfg, W, _ = model
    reqs, want = reference
    torch.testing.assert_close(oracle.decode_step_by_step(cfg, W, reqs["c"]), want["c"],
                               rtol=1e-9, atol=1e-9)


def test_whole_prompts(model, reference):
    reqs, want = reference
    eng = engine(model[2])
    got = replay(eng, reqs, [[(n, len(t))] for n, t in reqs.items()])
    check(got, want)


def test_prefill_against_token_by_token(model, reference):
    reqs, want = reference
    eng = engine(model[2])
    one = {"a": reqs["a"]}
    check(replay(eng, one, [[("a", 1)]] * 75), want)            # every token decoded alone
    check(replay(eng, one, [[("a", 40)]] + [[("a", 1)]] * 35), want)


@pytest.mark.parametrize("sizes", [[2] * 37 + [1], [3, 2, 7, 2, 19, 2, 5, 33, 2],
                                   [31, 1, 1, 30, 2, 2, 8], [32, 32, 11]])
def test_portions(model, reference, sizes):
    """Portions of several sizes down to two tokens, cut before, on and after page borders: the
    shift state and the cache carry over every cut."""
    reqs, want = reference
    assert sum(sizes) == 75
    eng = engine(model[2])
    check(replay(eng, {"a": reqs["a"]}, [[("a", s)] for s in sizes]), want)


def test_batches_of_unequal_requests(model, reference):
    reqs, want = reference
    eng = engine(model[2])
    sched = [[("a", 30), ("b", 2), ("c", 1)],
             [("a", 1), ("b", 20), ("c", 22), ("d", 1)],
             [("a", 1), ("b", 1), ("e", 33)],
             [("a", 1), ("b", 1)],                      # a pure decode step of two
             [("b", 17), ("e", 1)],                     # a is left out of a step
             [("a", 42), ("e", 30)]]
    check(replay(eng, reqs, sched), want)


def test_pages_and_slots_are_used_again(model, reference):
    """A pool of 5 pages and 2 sequence slots serves 7 requests one after another and side by
    side: every later request lives in pages and in a state slot that an earlier one gave back
    (its shift state must start from zeros, not from the slot's last owner)."""
    reqs, want = reference
    eng = engine(model[2], max_tokens=160, max_seqs=2)
    assert eng.runner.num_blocks == 5 and eng.runner.model.state.shape[1] == 2
    many = {f"{n}{i}": reqs[n] for i in range(2) for n in ("b", "c", "e")}
    many["a"] = reqs["a"]
    sched = [[("b0", 41), ("c0", 23)], [("e0", 64), ("c1", 22)], [("c1", 1)],
             [("a", 75), ("b1", 41)], [("e1", 10)], [("e1", 54)]]
    got = replay(eng, many, sched)
    check(got, {k: want[k[0]] for k in many})
    assert eng.sched.num_free_blocks() == 5 and eng.sched.num_running == 0
    assert eng.sched.num_free_tail_slots == 2


def test_first_tokens(model, reference):
    """Position 0 alone, as a prompt of one token and as the first of a portion, in a batch."""
    reqs, want = reference
    eng = engine(model[2])
    got = replay(eng, {"d": reqs["d"], "c": reqs["c"], "b": reqs["b"]},
                 [[("d", 1), ("c", 1), ("b", 2)], [("c", 2), ("b", 39)], [("c", 20)]])
    check(got, want, ["d", "c", "b"])


def test_long_decoding(tmp_path):
    cfg = oracle.make_config(width=32, vocab=37, groups=2, layers=[
        oracle.make_layer(heads=2, dim=8, rot_dim=8, vdim=8, kv_rank=16, q_rank=12),
        oracle.make_layer(heads=2, dim=6, rot_dim=8, vdim=4, kv_rank=16, q_rank=12, kv_from=0,
                          gate="element", moe=dict(experts=3, ff=8, top=2, identity=1, count=2, keep=1))])
    W = oracle.random_weights(cfg, seed=8)
    toks = tokens(230, 37, 9)
    want = {"a": oracle.forward(cfg, W, toks)}
    eng = engine(write_model(tmp_path, cfg, W))
    check(replay(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 225), want)


OTHER = {
    "one_head_one_group_no_identity": dict(width=16, groups=1, layers=[
        oracle.make_layer(heads=1, dim=4, rot_dim=2, vdim=4, kv_rank=6, q_rank=5,
                          moe=dict(experts=4, ff=8, top=1)),
        oracle.make_layer(heads=1, dim=4, rot_dim=2, vdim=1, kv_rank=6, q_rank=5, gate="element",
                          kv_from=0, ff=4)]),
    "every_output_kept_top_all": dict(width=24, groups=24, layers=[
        oracle.make_layer(moe=dict(experts=2, ff=5, top=4, identity=2, count=2, keep=2)),
        oracle.make_layer(gate="element", ff=None)]),
    "equal_sizes": dict(width=32, groups=2, layers=[
        oracle.make_layer(heads=4, dim=8, rot_dim=8, vdim=8, kv_rank=8, q_rank=8, ff=32)] * 3),
    "odd_sizes": dict(width=54, vocab=19, groups=9, eps=1e-3, layers=[
        oracle.make_layer(heads=5, dim=7, rot_dim=6, vdim=9, kv_rank=13, q_rank=17, ff=7),
        oracle.make_layer(heads=7, dim=3, rot_dim=10, vdim=2, kv_rank=70, q_rank=3, gate="element",
                          moe=dict(experts=7, ff=11, top=3, identity=2, count=3, keep=2)),
        oracle.make_layer(heads=9, dim=5, rot_dim=10, vdim=4, kv_rank=70, q_rank=9, kv_from=1,
                          ff=100)]),
}


@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_configurations(tmp_path, name):
    cfg = oracle.make_config(**dict(OTHER[name]))
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    want = {n: oracle.forward(cfg, W, t) for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W))
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want)


# ------------------------------------------------------------------ bf16, generation, CLI
def test_bfloat16_engine(model, reference):
    reqs, want = reference
    eng = engine(model[2], dtype="bfloat16")
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 39)], [("a", 44)]]
    got = replay(eng, {"a": reqs["a"], "b": reqs["b"]}, sched)
    for n in ("a", "b"):
        assert rel_err(got[n], want[n]).median().item() < 0.05


def test_prefix_caching_is_turned_off(model):
    """A cached prefix would hold keys but not the shift state at its end."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    lines = []
    LLMEngine(EngineConfig(model=model[2], load_format="safetensors", weights_path=model[2],
                           dtype="float32", max_model_len=64, max_num_seqs=2,
                           max_num_batched_tokens=64, num_gpu_blocks=4, device="cpu",
                           enable_prefix_caching=True, gc_freeze=False),
              log=lambda *a: lines.append(" ".join(map(str, a))))
    assert any("prefix caching is off" in ln for ln in lines)


def test_greedy_generation_through_the_engine(model):
    """LLMEngine.generate (its own scheduler: admission, chunked prefill, mixed steps, decode)
    picks, token by token, the oracle's argmax for the sequence generated so far; two prompts
    share a long prefix, which must not be served from a prefix cache."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    cfg, W, path = model
    eng = LLMEngine(EngineConfig(model=path, load_format="safetensors", weights_path=path,
                                 dtype="float32", max_model_len=128, max_num_seqs=3,
                                 max_num_batched_tokens=24, num_gpu_blocks=12, device="cpu",
                                 gc_freeze=False), log=lambda *a: None)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (30, 3, 17, 9)]
    prompts.append(prompts[0][:28] + [1, 2, 3])
    outs = eng.generate(None, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True),
                        prompt_ids=prompts)
    assert [len(o.output_ids) for o in outs] == [12] * 5
    for p, o in zip(prompts, outs):
        logits = oracle.forward(cfg, W, p + o.output_ids)
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))


def test_registry_model_runs():
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    eng = LLMEngine(EngineConfig(model="tiny-puputar", dtype="float32", max_model_len=64,
                                 max_num_seqs=2, max_num_batched_tokens=32, num_gpu_blocks=4,
                                 device="cpu", gc_freeze=False), log=lambda *a: None)
    outs = eng.generate(None, SamplingParams(max_tokens=4, temperature=0.0, ignore_eos=True),
                        prompt_ids=[[5, 6, 7], [9] * 20])
    assert [len(o.output_ids) for o in outs] == [4, 4]


def test_trace_run_command_line(model, reference, tmp_path):
    import json
    import os
    import subprocess
    import sys

    import numpy as np

    cfg, _, path = model
    reqs, want = reference
    a, c = reqs["a"], reqs["c"]
    steps = [
        {"step": 0, "entries": [{"id": "x", "tokens": a[:40], "want": [39, 0, 7]},
                                {"id": "y", "tokens": c[:1], "want": [0]}], "end": []},
        {"step": 1, "entries": [{"id": "y", "tokens": c[1:], "want": []}], "end": ["y"]},
        {"step": 2, "entries": [{"id": "x", "tokens": a[40:41], "want": [0]}], "end": []},
        {"step": 3, "entries": [{"id": "x", "tokens": a[41:], "want": [33]},
                                {"id": "z", "tokens": c, "want": [22, 21]}], "end": ["x", "z"]},
    ]
    repo = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(repo, "bin", "trace_run"), "--model", path,
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "192",
                        "--device", "cpu"],
                       input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True,
                       text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == \
        [f"done {i}" for i in range(4)]
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32", "3.f32"]
    V = cfg["vocab"]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)).double()
    exp0 = torch.stack([want["a"][39], want["a"][0], want["a"][7], want["c"][0]])
    assert rel_err(got0, exp0).max().item() < FP32_TOL
    got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V)).double()
    exp3 = torch.stack([want["a"][74], want["c"][22], want["c"][21]])
    assert rel_err(got3, exp3).max().item() < FP32_TOL
