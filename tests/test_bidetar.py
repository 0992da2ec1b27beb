"""Bidetar through the engine (scheduler, block manager, runner, ops) against the plain
float64 oracle of tests/bidetar_oracle.py, on the CPU branch of the ops (the same suite runs on
the HIP kernels in test_bidetar_gpu.py).  Small configurations with random weights; fp32 runs
are compared tightly (one wrongly seen or missed key among a few hundred moves a logit by far
more than the tolerance), bf16 runs loosely."""
import math

import pytest
import torch

import bidetar_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from aws_k8s_ansible_provisioner_amd.models.config import get_config
from aws_k8s_ansible_provisioner_amd.ops import stream as sops

SCALING = {"factor": 4.0, "low": 1.0, "high": 4.0, "original": 64}
FP32_TOL = 2e-4


def base_config():
    """Layers of unequal sizes, one without a feed-forward, a looped span, partial rotary."""
    layers = [
        oracle.make_layer(heads=4, kv_heads=2, dim=8, chunk=20, rot_dims=4, scaling=SCALING),
        oracle.make_layer(heads=3, kv_heads=1, dim=16, chunk=12, rot_dims=16, base=50.0, ff=24,
                          scale=0.2),
        oracle.make_layer(heads=2, kv_heads=2, dim=8, chunk=20, rot_dims=8, scaling=SCALING,
                          ff=None),
    ]
    return oracle.make_config(width=40, vocab=53, layers=layers,
                              loop={"start": 1, "stop": 3, "times": 2})


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=3)
    return cfg, W, write_model(tmp_path_factory.mktemp("bidetar"), cfg, W)


@pytest.fixture(scope="module")
def reference(model):
    cfg, W, _ = model
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    return reqs, {n: oracle.forward(cfg, W, t)[0] for n, t in reqs.items()}


def check(got, want, names=None, tol=FP32_TOL):
    for n in names or got:
        e = rel_err(got[n], want[n])
        assert e.max().item() < tol, f"{n}: position {int(e.argmax())} off by {e.max().item():.2e}"


# ------------------------------------------------------------------ configuration, weights
def test_config_reader(model):
    cfg, _, path = model
    c = get_config(path)
    assert c.arch == "bidetar" and c.layer_runs() == [0, 1, 2, 1, 2] and c.num_layers == 5
    assert c.hidden_size == 40 and c.vocab_size == 53 and c.residual_mult == 0.8
    assert [ls.mixer.chunk for ls in c.layer_specs] == [20, 12, 20]
    assert c.layer_specs[2].mlp is None and c.layer_specs[1].mixer.rot.scaling is None
    assert c.num_heads == 4 and c.head_dim == 16 and c.intermediate_size == 40


def test_weights_round_trip(model):
    from aws_k8s_ansible_provisioner_amd.models.bidetar import BidetarLM

    cfg, W, path = model
    m = BidetarLM(get_config(path), dtype=torch.float32, max_model_len=64)
    m.load_state_dict(W)
    sd = m.state_dict()
    assert set(sd) == set(W)
    for k, v in W.items():
        assert torch.equal(sd[k].float(), v.float()), k
    bad = dict(W)
    bad["l1.mix.q"] = W["l1.mix.q"][:-1]
    with pytest.raises(ValueError):
        m.load_state_dict(bad)


# ------------------------------------------------------------------ each mechanism alone
def test_rotary_bands_and_rotation():
    rot = {"dims": 12, "base": 300.0, "scaling": SCALING}
    f = oracle.rotary_frequencies(rot)
    plain = [300.0 ** (-2.0 * i / 12) for i in range(6)]
    kinds = {"kept": 0, "divided": 0, "blended": 0}
    for a, b in zip(f, plain):
        kinds["kept" if a == b else "divided" if abs(a - b / 4) < 1e-15 else "blended"] += 1
    assert all(kinds.values()), kinds  # the configuration exercises all three bands
    table = sops.rotary_table(90, 12, 300.0, SCALING)
    pos = torch.tensor([0, 1, 17, 89])
    want = torch.tensor([[math.cos(p * x) for x in f] + [math.sin(p * x) for x in f]
                         for p in pos.tolist()], dtype=torch.float64)
    torch.testing.assert_close(table[pos].double(), want, rtol=0, atol=1e-6)


def test_projection_norm_rotation_and_value_cache():
    """The q / k norms run over the whole projection (one head is made 50x larger, which a
    per-head norm would hide), rotation touches the first R dims of every head in pairs
    (2i, 2i+1), the K cache gets the normed + rotated keys and the V cache the raw ones."""
    g = torch.Generator().manual_seed(0)
    T, H, G, D, R, BS, NB = 9, 3, 2, 8, 4, 32, 2
    proj = torch.randn(T, 5 + H * D + G * D, generator=g)
    proj[:, 5:5 + D] *= 50.0
    qw, kw = 1 + 0.3 * torch.randn(H * D, generator=g), 1 + 0.3 * torch.randn(G * D, generator=g)
    pos = torch.tensor([0, 1, 2, 31, 32, 33, 40, 63, 7])
    slots = torch.tensor([3, 0, 9, 31, 32, 63, 12, 40, -1])
    rot = {"dims": R, "base": 20.0, "scaling": None}
    q = torch.zeros(T, H, D)
    kc, vc = torch.zeros(NB, G, BS, D), torch.zeros(NB, G, BS // 8, D, 8)
    sops.proj_norm_rope_cache(proj, q, kc, vc, pos, slots, sops.rotary_table(64, R, 20.0), qw, kw,
                              H, G, D, 5, 5 + H * D, 1e-5)
    f = oracle.rotary_frequencies(rot)
    p64 = proj.double()
    vc = sops.v_tokens(vc)  # the V cache keeps 8-token groups; compare token-major
    for t in range(T):
        qn = (oracle.rms_unit(p64[t, 5:5 + H * D], 1e-5) * qw.double()).reshape(H, D)
        kraw = p64[t, 5 + H * D:].reshape(G, D)
        kn = (oracle.rms_unit(p64[t, 5 + H * D:], 1e-5) * kw.double()).reshape(G, D)
        for a in range(H):
            torch.testing.assert_close(q[t, a].double(), oracle.rotate_head(qn[a], int(pos[t]), f),
                                       rtol=1e-5, atol=1e-5)
        s = int(slots[t])
        if s < 0:
            continue
        for a in range(G):
            torch.testing.assert_close(kc[s // BS, a, s % BS].double(),
                                       oracle.rotate_head(kn[a], int(pos[t]), f),
                                       rtol=1e-5, atol=1e-5)
            torch.testing.assert_close(vc[s // BS, a, s % BS].double(), kraw[a], rtol=1e-6,
                                       atol=1e-6)
    assert kc[0, :, 1].abs().sum() == 0 and vc.abs().sum() > 0  # slot -1 wrote nothing anywhere


def spike_case(chunk, n, q_pos, key_pos, BS=32):
    """One sequence of n cached tokens whose key at key_pos has an enormous score for the query
    at q_pos; the value at key_pos is a marker.  Returns the marker's share of the output."""
    g = torch.Generator().manual_seed(n + q_pos)
    D = 8
    nb = -(-n // BS)
    bt = torch.randperm(nb + 2, generator=g)[:nb].int().view(1, nb)
    kc = 0.1 * torch.randn(nb + 2, 1, BS, D, generator=g)
    vc = torch.zeros(nb + 2, 1, BS, D)
    q = 0.1 * torch.randn(1, 1, D, generator=g)
    q[0, 0, 0] = 30.0
    kc[bt[0, key_pos // BS], 0, key_pos % BS, 0] = 30.0
    vc[bt[0, key_pos // BS], 0, key_pos % BS, :] = 1.0
    return q, kc, sops.v_from_tokens(vc), bt


@pytest.mark.parametrize("chunk,n,q_pos,key_pos,seen", [
    (0, 400, 399, 0, True),        # a far key among hundreds, full causal
    (0, 400, 399, 31, True),       # ... at the end of the first page
    (0, 400, 399, 32, True),       # ... at the start of the second
    (100, 400, 399, 300, True),    # first key of the query's chunk
    (100, 400, 399, 299, False),   # last key of the chunk before
    (100, 301, 300, 300, True),    # a chunk's first token sees itself
    (100, 301, 300, 299, False),   # ... and nothing earlier
    (100, 300, 299, 200, True),    # a chunk's last token still sees its first
    (64, 200, 130, 128, True),     # chunk border on a page border
    (64, 200, 130, 127, False),
    (7, 40, 20, 14, True),         # chunks shorter than a page
    (7, 40, 20, 13, False),
    (0, 400, 200, 201, False),     # a later key is never seen (decode rows see kv_len = pos + 1)
])
def test_attention_sees_exactly_its_range(chunk, n, q_pos, key_pos, seen):
    q, kc, vc, bt = spike_case(chunk, n, q_pos, key_pos)
    kv = q_pos + 1
    for mode in ("decode", "prefill"):
        out = torch.zeros(1, 8)
        if mode == "decode":
            sops.sink_attention_decode(out, q, kc, vc, bt, torch.tensor([kv], dtype=torch.int32),
                                       None, None, 1.0, chunk)
        else:
            sops.sink_attention_prefill(out, q, kc, vc, bt, torch.tensor([kv], dtype=torch.int32),
                                        torch.tensor([0, 1], dtype=torch.int32),
                                        torch.tensor([0], dtype=torch.int32),
                                        torch.tensor([0], dtype=torch.int32), 64, None, None, 1.0,
                                        chunk)
        share = out[0, 1].item()
        assert (share > 0.99) if seen else (share < 1e-6), (mode, share)


def test_sink_counts_once_unscaled_and_gate():
    """With every score 0 over n keys the weights are 1 / (n + exp(sink)), whatever the score
    scale; the gate multiplies the head's output by sigmoid(z)."""
    n, D, BS = 5, 4, 32
    kc = torch.zeros(1, 1, BS, D)
    vc = torch.ones(1, 1, BS // 8, D, 8)
    q = torch.zeros(1, 2, D)
    bt = torch.zeros(1, 1, dtype=torch.int32)
    sink = torch.tensor([math.log(3.0), -40.0])
    gate = torch.tensor([[0.0, 1.5]])
    out = torch.zeros(1, 2 * D)
    sops.sink_attention_decode(out, q, kc, vc, bt, torch.tensor([n], dtype=torch.int32), gate,
                               sink, 7.0, 0)
    assert abs(out[0, 0].item() - (n / (n + 3.0)) * 0.5) < 1e-6
    assert abs(out[0, D].item() - 1.0 / (1 + math.exp(-1.5))) < 1e-6
    w = oracle.sink_softmax(torch.zeros(n, dtype=torch.float64), math.log(3.0))
    assert abs(w.sum().item() - n / (n + 3.0)) < 1e-12


def test_stream_ops_alone():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(6, 40, generator=g)
    y = torch.randn(6, 40, generator=g)
    w = 1 + 0.2 * torch.randn(40, generator=g)
    x0 = x.clone()
    h = sops.stream_add_norm(x, y, 0.7, w, 1e-5, torch.float32)
    torch.testing.assert_close(x, x0 + 0.7 * y)
    torch.testing.assert_close(h.double(), oracle.rms_unit((x0 + 0.7 * y).double(), 1e-5)
                               * w.double(), rtol=1e-5, atol=1e-5)
    out = torch.zeros(6, 40)
    sops.relu2(y, out)
    torch.testing.assert_close(out, torch.relu(y) ** 2)
    table = torch.randn(9, 40, generator=g)
    e = sops.embed_scaled(torch.tensor([8, 0, 3]), table, 2.5)
    torch.testing.assert_close(e, table[[8, 0, 3]] * 2.5)


# ------------------------------------------------------------------ through the engine, fp32
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
                                   [19, 1, 1, 20, 1, 31, 2], [12, 12, 12, 12, 12, 12, 3]])
def test_portions(model, reference, sizes):
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
             [("a", 42), ("b", 17), ("e", 1)],
             [("e", 30)]]
    check(replay(eng, reqs, sched), want)


def test_pages_and_slots_are_used_again(model, reference):
    """A pool of 5 pages and 2 sequence slots serves 7 requests one after another and side by
    side; every later request lives in pages (and a slot) that an earlier one gave back."""
    reqs, want = reference
    eng = engine(model[2], max_tokens=160, max_seqs=2)
    assert eng.runner.num_blocks == 5
    many = {f"{n}{i}": reqs[n] for i in range(2) for n in ("b", "c", "e")}
    many["a"] = reqs["a"]
    sched = [[("b0", 41), ("c0", 23)], [("e0", 64), ("c1", 22)], [("c1", 1)],
             [("a", 75), ("b1", 41)], [("e1", 10)], [("e1", 54)]]
    got = replay(eng, many, sched)
    check(got, {k: want[k[0]] for k in many})
    assert eng.sched.num_free_blocks() == 5 and eng.sched.num_running == 0
    with pytest.raises(RuntimeError):   # the pool is really that small
        replay(eng, {"x": reqs["a"], "y": reqs["a"], "z": reqs["a"]}, [[("x", 75), ("y", 75)],
                                                                       [("z", 75)]])


def test_chunk_edges_in_prompts_and_decoding(model, reference):
    """Portions that end one token before, on and after the edges of both chunk lengths (12 and
    20) and of a 32-token page, then single tokens across the next edges."""
    reqs, want = reference
    eng = engine(model[2])
    sizes = [11, 1, 1, 6, 1, 1, 3, 7, 1, 1, 1, 2, 3, 1, 1, 1]
    sizes += [1] * (75 - sum(sizes))
    check(replay(eng, {"a": reqs["a"]}, [[("a", s)] for s in sizes]), want)


def test_long_decoding(tmp_path):
    cfg = oracle.make_config(width=32, vocab=37, layers=[
        oracle.make_layer(heads=2, kv_heads=1, dim=8, chunk=70, rot_dims=8, scaling=SCALING),
        oracle.make_layer(heads=2, kv_heads=2, dim=8, chunk=0, rot_dims=2)])
    W = oracle.random_weights(cfg, seed=8)
    toks = tokens(230, 37, 9)
    want = {"a": oracle.forward(cfg, W, toks)[0]}
    eng = engine(write_model(tmp_path, cfg, W))
    check(replay(eng, {"a": toks}, [[("a", 5)]] + [[("a", 1)]] * 225), want)


OTHER = {
    "mha_full_rotary_one_layer": dict(layers=[oracle.make_layer(heads=4, kv_heads=4, dim=8, chunk=9,
                                                                rot_dims=8)], loop=None),
    "one_head_chunk_longer_than_prompt": dict(layers=[oracle.make_layer(heads=1, kv_heads=1, dim=16,
                                                                        chunk=500, rot_dims=6,
                                                                        scaling=SCALING)] * 2,
                                              loop={"start": 0, "stop": 2, "times": 3}),
    "chunk_of_one_and_two": dict(layers=[oracle.make_layer(chunk=1, ff=None),
                                         oracle.make_layer(chunk=2, heads=6, kv_heads=2)],
                                 loop={"start": 1, "stop": 2, "times": 1}),
    "loop_over_everything": dict(layers=[oracle.make_layer(heads=2, kv_heads=1, dim=24, chunk=33,
                                                           rot_dims=24, scale=1.0)],
                                 loop={"start": 0, "stop": 1, "times": 4}, mult=1.0,
                                 embed_scale=1.0),
    "odd_sizes": dict(width=56, vocab=19, layers=[oracle.make_layer(heads=5, kv_heads=5, dim=6,
                                                                    chunk=13, rot_dims=2, ff=7),
                                                  oracle.make_layer(heads=9, kv_heads=3, dim=10,
                                                                    chunk=31, rot_dims=10, ff=100)],
                      loop=None, eps=1e-3, mult=0.3),
}


@pytest.mark.parametrize("name", sorted(OTHER))
def test_other_configurations(tmp_path, name):
    kw = dict(OTHER[name])
    cfg = oracle.make_config(**kw)
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    want = {n: oracle.forward(cfg, W, t)[0] for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W))
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want)


def test_first_tokens(model, reference):
    """Position 0 alone, as a prompt of one token and as the first of a portion, in a batch."""
    reqs, want = reference
    eng = engine(model[2])
    got = replay(eng, {"d": reqs["d"], "c": reqs["c"], "b": reqs["b"]},
                 [[("d", 1), ("c", 1), ("b", 2)], [("c", 2), ("b", 39)], [("c", 20)]])
    check(got, want, ["d", "c", "b"])


# ------------------------------------------------------------------ bf16, generation
def test_bfloat16_engine(model, reference):
    reqs, want = reference
    eng = engine(model[2], dtype="bfloat16")
    sched = [[("a", 30), ("b", 2)], [("a", 1), ("b", 39)], [("a", 44)]]
    got = replay(eng, {"a": reqs["a"], "b": reqs["b"]}, sched)
    for n in ("a", "b"):
        assert rel_err(got[n], want[n]).max().item() < 0.08


def test_greedy_generation_through_the_engine(model):
    """LLMEngine.generate (its own scheduler: admission, chunked prefill, mixed steps, decode)
    picks, token by token, the oracle's argmax for the sequence generated so far."""
    from aws_k8s_ansible_provisioner_amd.engine.config import EngineConfig, SamplingParams
    from aws_k8s_ansible_provisioner_amd.engine.llm_engine import LLMEngine

    cfg, W, path = model
    eng = LLMEngine(EngineConfig(model=path, load_format="safetensors", weights_path=path,
                                 dtype="float32", max_model_len=128, max_num_seqs=3,
                                 max_num_batched_tokens=24, num_gpu_blocks=12, device="cpu",
                                 gc_freeze=False), log=lambda *a: None)
    prompts = [tokens(n, cfg["vocab"], 20 + n) for n in (30, 3, 17, 9)]
    outs = eng.generate(None, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True),
                        prompt_ids=prompts)
    assert [len(o.output_ids) for o in outs] == [12] * 4
    for p, o in zip(prompts, outs):
        logits = oracle.forward(cfg, W, p + o.output_ids)[0]
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))


def test_trace_run_command_line(model, reference, tmp_path):
    """bin/trace_run: JSON steps on stdin, one `done <step>` line per step, `<step>.f32` with
    the logits of the wanted places (entries' order, then each entry's `want` order)."""
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
    assert sorted(os.listdir(out)) == ["0.f32", "2.f32", "3.f32"]   # nothing wanted in step 1
    V = cfg["vocab"]
    got0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V)).double()
    exp0 = torch.stack([want["a"][39], want["a"][0], want["a"][7], want["c"][0]])
    assert rel_err(got0, exp0).max().item() < FP32_TOL
    got3 = torch.from_numpy(np.fromfile(out / "3.f32", dtype="<f4").reshape(-1, V)).double()
    exp3 = torch.stack([want["a"][74], want["c"][22], want["c"][21]])
    assert rel_err(got3, exp3).max().item() < FP32_TOL
