"""Helpers of the Bidetar tests: write a model folder, start an engine on it, replay a schedule."""
import json
import os

import numpy as np
import torch

from aws_k8s_ansible_provisioner_amd.engine.trace_replay import build_engine


def write_model(path, cfg, weights):
    from safetensors.torch import save_file

    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()},
              os.path.join(path, "model.safetensors"))
    return str(path)


def engine(path, dtype="float32", max_tokens=512, max_seqs=4, block_size=32, device="cpu",
           eager=False):
    return build_engine(path, dtype, max_tokens, max_seqs, block_size, device, eager,
                        log=lambda *a: None)


def replay(eng, requests, schedule):
    """requests: name -> token list; schedule: list of steps, each a list of (name, count).
    Every position's logits are asked for.  Returns name -> [T, vocab] float64; a request ends
    (its blocks return to the pool) with the step that brings its last token."""
    at = {n: 0 for n in requests}
    got = {n: [] for n in requests}
    for step in schedule:
        entries, end = [], []
        for name, count in step:
            lo, hi = at[name], at[name] + count
            entries.append((name, requests[name][lo:hi], list(range(count))))
            at[name] = hi
            if hi == len(requests[name]):
                end.append(name)
        out = eng.replay_step(entries, end)
        o = 0
        for name, count in step:
            got[name].append(np.array(out[o:o + count], dtype=np.float64))
            o += count
        assert o == out.shape[0]
    for n in requests:
        assert at[n] == len(requests[n]), f"schedule does not finish {n}"
    return {n: torch.from_numpy(np.concatenate(v)) for n, v in got.items()}


def rel_err(got, want):
    """Per position: rms of the mean-free logit difference over the rms of the mean-free
    expected logits."""
    d = got - want
    d = d - d.mean(dim=-1, keepdim=True)
    w = want - want.mean(dim=-1, keepdim=True)
    return (d.pow(2).mean(dim=-1).sqrt() / w.pow(2).mean().sqrt())


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()
