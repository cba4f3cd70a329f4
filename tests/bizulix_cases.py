"""Bizulix test bodies, shared by the CPU tests (torch twin of the executor: host logic) and the GPU tests
(HIP kernels). Every case builds its own small configuration with random weights, runs it through the
engine (`StackRunner`, its block pool, state slots and step function) and compares with the plain float64
implementation in `bizulix_oracle.py`."""
from __future__ import annotations

import json
import os

import numpy as np
import torch

import bizulix_oracle as oracle
from ollama_operator_amd.engine.safetensors_io import SafetensorsFile
from ollama_operator_amd.engine.stack_runner import StackRunner
from ollama_operator_amd.models.config import (MIX_ATTENTION, MIX_RETENTION, LayerSpec, MixerSpec, MoESpec, StackConfig)
from ollama_operator_amd.models.random_init import write_random_stack


def attn(heads=4, kv_heads=2, dim=16, vdim=24, scale=0.25, softcap=20.0, coef=0.4, every=8):
    return MixerSpec(kind=MIX_ATTENTION, heads=heads, kv_heads=kv_heads, dim=dim, vdim=vdim, scale=scale, softcap=softcap,
                     qtemp_coef=coef, qtemp_every=every)


def ret(heads=2, dim=16, vdim=32, decay=(0.9, 0.998), rot_dims=8, base=100.0):
    return MixerSpec(kind=MIX_RETENTION, heads=heads, kv_heads=heads, dim=dim, vdim=vdim, decay=tuple(decay),
                     rot_dims=rot_dims, rot_base=base)


def moe(experts=6, top=3, ff=24, shared_ff=40):
    return MoESpec(experts=experts, top=top, ff=ff, shared_ff=shared_ff)


def config(layers, width=64, vocab=96, loop=(0, 0, 0), mult=0.6, cap=12.0, eps=1e-5):
    return StackConfig(n_vocab=vocab, n_embd=width, layers=[LayerSpec(mixer=m, mlp=f) for m, f in layers],
                       loop_start=loop[0], loop_stop=loop[1], loop_times=loop[2], norm_eps=eps, residual_mult=mult,
                       logit_softcap=cap)


def standard():
    """retention, then (attention, attention) twice over, then attention and a last retention without a
    feed-forward: every mechanism, a repeated span, sizes that differ from one another."""
    return config([(ret(), moe(experts=4, top=4, ff=16, shared_ff=8)), (attn(), moe()),
                   (attn(heads=6, kv_heads=1, dim=8, vdim=8, every=5), moe(top=2, shared_ff=0)),
                   (attn(heads=2, kv_heads=2, dim=32, vdim=16), None), (ret(heads=1, dim=8, vdim=16, decay=(0.95,), rot_dims=4), None)],
                  loop=(1, 3, 2))


class Model:
    """A random model on disk + its oracle inputs."""

    def __init__(self, tmp, cfg, seed=0, name="m"):
        self.cfg = cfg
        self.path = os.path.join(str(tmp), f"{name}_{seed}")
        write_random_stack(self.path, cfg, seed=seed)
        with open(os.path.join(self.path, "config.json")) as f:
            self.json = json.load(f)
        st = SafetensorsFile(os.path.join(self.path, "model.safetensors"))
        self.tensors = {n: st.tensor(n) for n in st.names()}

    def oracle(self, tokens):
        z, trail = oracle.forward(self.json, self.tensors, tokens)
        return z.numpy(), trail.numpy()

    def runner(self, device, dtype="float32", **kw):
        kw.setdefault("max_batch", 64)
        kw.setdefault("max_seqs", 4)
        kw.setdefault("kv_tokens", 512)
        kw.setdefault("use_graphs", False)
        return StackRunner(self.path, device=device, dtype=dtype, **kw)

    def set_tensor(self, name, value):
        """Overwrite one tensor on disk (and in the oracle's copy)."""
        from ollama_operator_amd.engine.safetensors_io import write_safetensors
        self.tensors[name] = value.to(torch.bfloat16)
        write_safetensors(os.path.join(self.path, "model.safetensors"), self.tensors)


def tokens(n, vocab, seed=0):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def rel_err(got, want):
    """Root mean square of the difference over that of the expected logits (means taken off), per row."""
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    w = want - want.mean(-1, keepdims=True)
    return np.sqrt((d ** 2).mean(-1)) / np.sqrt((w ** 2).mean(-1) + 1e-30)


TOL = {"float32": 3e-4, "bfloat16": 6e-2}


def check(got, want, dtype, what=""):
    """float32: every row within 3e-4 of the logits' spread. bfloat16: rounding moves a row by ~5e-3 and,
    where a router's choice or a sharp softmax sits on a close call, by several percent: the median row within
    2e-2, at most one row in ten over 6e-2, none over 0.3."""
    e = rel_err(got, want)
    assert np.isfinite(np.asarray(got)).all(), f"{what}: non-finite logits"
    worst = f"{what}: worst row {int(e.argmax())} off by {e.max():.3g}"
    if dtype == "float32":
        assert e.max() < TOL[dtype], f"{worst} (limit {TOL[dtype]})"
    else:
        assert np.median(e) < 2e-2 and e.max() < 0.3 and (e > TOL[dtype]).sum() <= max(2, len(e) // 10), \
            f"{worst}, median {np.median(e):.3g}, {(e > TOL[dtype]).sum()} of {len(e)} rows over {TOL[dtype]}"


def run_cuts(r, toks, cuts, sid=None):
    """Feed `toks` in portions ending at `cuts`; logits of every position."""
    own = sid is None
    if own:
        sid = r.new_sequence()
    outs, a = [], 0
    for b in cuts:
        outs.append(r.step_entries([(sid, toks[a:b], list(range(b - a)))]).float().cpu().numpy())
        a = b
    if own:
        r.free_sequence(sid)
    return np.concatenate(outs)


def layer_trail(r, toks):
    """Residual stream after every layer run for a whole prompt, through the executor's stages."""
    sid = r.new_sequence()
    n = len(toks)
    r.kv.reserve(sid, n)
    r._sync_block_table(sid)
    s = r.kv.seqs[sid]
    pos = np.arange(n, dtype=np.int32)
    slots = np.array([r.kv.slot(sid, int(p)) for p in pos], np.int32)
    arr = np.stack([pos, slots, pos + 1, np.full(n, s.row, np.int32), np.zeros(n, np.int32)]).astype(np.int32)
    r._upload(arr, np.asarray(toks, np.int32))
    r.exe.run("embed", 0, n)
    out = []
    for ri in range(len(r.runs)):
        r.exe.run("run", ri, n)
        out.append(r.resid[:n].float().cpu().numpy().copy())
    r.free_sequence(sid)
    return np.stack(out)
