"""Bidetar on the HIP kernels through the engine -- prefill tiles, mixed steps, hipGraph decode,
a small page pool -- against the float64 oracle (tests/bidetar_oracle.py), in fp32 (tight) and
bf16 (loose), and greedy generation through LLMEngine.generate."""
import pytest
import torch

import bidetar_oracle as oracle
from bidetar_harness import engine, rel_err, replay, tokens, write_model
from test_bidetar import SCALING, base_config

pytestmark = pytest.mark.gpu
TOL = {"float32": 3e-4, "bfloat16": 0.08}


@pytest.fixture(scope="module")
def model(tmp_path_factory):
    cfg = base_config()
    W = oracle.random_weights(cfg, seed=3)
    reqs = {"a": tokens(75, cfg["vocab"], 1), "b": tokens(41, cfg["vocab"], 2),
            "c": tokens(23, cfg["vocab"], 3), "d": tokens(1, cfg["vocab"], 4),
            "e": tokens(64, cfg["vocab"], 5)}
    want = {n: oracle.forward(cfg, W, t)[0] for n, t in reqs.items()}
    return cfg, W, write_model(tmp_path_factory.mktemp("bidetar_gpu"), cfg, W), reqs, want


def check(got, want, dtype):
    for n in got:
        e = rel_err(got[n], want[n])
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
             [("a", 42), ("b", 17), ("e", 1)],
             [("e", 30)]]
    check(replay(eng, reqs, sched), want, dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_small_pool_is_used_again(model, dtype):
    _, _, path, reqs, want = model
    eng = engine(path, dtype=dtype, max_tokens=160, max_seqs=2, device="cuda")
    many = {f"{n}{i}": reqs[n] for i in range(2) for n in ("b", "c", "e")}
    many["a"] = reqs["a"]
    sched = [[("b0", 41), ("c0", 23)], [("e0", 64), ("c1", 22)], [("c1", 1)],
             [("a", 75), ("b1", 41)], [("e1", 10)], [("e1", 54)]]
    for _ in range(2):  # graphs replayed again over pages that changed owners
        check(replay(eng, many, sched), {k: want[k[0]] for k in many}, dtype)
    assert eng.sched.num_free_blocks() == 5


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decode_through_graphs_and_split_partitions(tmp_path, dtype):
    """Decode over a key range that the split decode kernel cuts into several partitions, over a full-
    causal layer and a chunked one, checked at every step against the oracle."""
    cfg = oracle.make_config(width=64, vocab=37, layers=[
        oracle.make_layer(heads=4, kv_heads=2, dim=32, chunk=0, rot_dims=16, scaling=SCALING),
        oracle.make_layer(heads=2, kv_heads=1, dim=64, chunk=600, rot_dims=64, ff=96)])
    W = oracle.random_weights(cfg, seed=5)
    toks = tokens(1300, 37, 6)
    want = {"a": oracle.forward(cfg, W, toks)[0]}
    eng = engine(write_model(tmp_path, cfg, W), dtype=dtype, max_tokens=1344, device="cuda")
    assert eng.runner.graphs
    got = replay(eng, {"a": toks}, [[("a", 1100)]] + [[("a", 1)]] * 200)
    check(got, want, dtype)


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
        logits = oracle.forward(cfg, W, p + o.output_ids)[0]
        for i, tok in enumerate(o.output_ids):
            row = logits[len(p) - 1 + i]
            assert row[tok] >= row.max() - 1e-3 * row.std(), (i, tok, int(row.argmax()))
    assert torch.cuda.is_available()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", sorted(__import__("test_bidetar").OTHER))
def test_other_configurations(tmp_path, name, dtype):
    """Sizes that leave the 16-byte and matrix-core paths (odd widths, head sizes 6 / 10 / 24,
    a 7-wide feed-forward, chunk 1): the scalar and row kernels, in mixed steps and decode."""
    from test_bidetar import OTHER

    cfg = oracle.make_config(**dict(OTHER[name]))
    W = oracle.random_weights(cfg, seed=len(name))
    reqs = {"p": tokens(45, cfg["vocab"], 11), "q": tokens(38, cfg["vocab"], 12)}
    want = {n: oracle.forward(cfg, W, t)[0] for n, t in reqs.items()}
    eng = engine(write_model(tmp_path, cfg, W), dtype=dtype, device="cuda")
    sched = [[("p", 17), ("q", 2)], [("p", 1), ("q", 30)], [("p", 27), ("q", 1)],
             [("q", 1)], [("q", 4)]]
    check(replay(eng, reqs, sched), want, dtype)
