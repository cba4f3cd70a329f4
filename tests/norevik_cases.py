"""Norevik test bodies, shared by the CPU tests (torch twin of the executor: host logic) and the GPU tests (HIP
kernels). Every case builds its own small configuration with random weights, runs it through the engine
(`StackRunner`, its block pool, state slots and step function) and compares with the plain float64
implementation in `norevik_oracle.py`."""
from __future__ import annotations

import numpy as np

import norevik_oracle as oracle
from bizulix_cases import Model as _Model
from bizulix_cases import layer_trail, rel_err, run_cuts, tokens  # noqa: F401  (re-exported for the tests)
from ollama_operator_amd.models.config import (BLOCK_POSTNORM, FF_DENSE, FF_MOE, MIX_LATENT, MIX_MAMBA2, MIX_MLSTM,
                                               ROUTE_SCORE_GROUPS, LayerSpec, MixerSpec, MoESpec, StackConfig)


def latent(heads=3, dim=16, rot_dim=8, vdim=12, kv_rank=24, scale=0.3, rot_dims=None, base=100.0):
    return MixerSpec(kind=MIX_LATENT, heads=heads, kv_heads=1, dim=dim, vdim=vdim, scale=scale, rot_dim=rot_dim,
                     kv_rank=kv_rank, rot_dims=rot_dim if rot_dims is None else rot_dims, rot_base=base)


def mlstm(heads=2, dim=8, vdim=20, cap=6.0):
    return MixerSpec(kind=MIX_MLSTM, heads=heads, kv_heads=heads, dim=dim, vdim=vdim, gate_cap=cap)


def mamba(heads=4, vdim=8, state=16, groups=2, conv=4, norm_groups=1):
    return MixerSpec(kind=MIX_MAMBA2, heads=heads, kv_heads=groups, dim=state, vdim=vdim, state=state, groups=groups,
                     conv=conv, norm_groups=norm_groups)


def dense(ff=40):
    return MoESpec(kind=FF_DENSE, ff=ff)


def moe(experts=7, top=3, ff=24, shared_ff=40, identity=2, groups=(3, 2)):
    return MoESpec(kind=FF_MOE, route=ROUTE_SCORE_GROUPS, experts=experts, top=top, ff=ff, shared_ff=shared_ff,
                   identity=identity, group_count=groups[0], group_keep=groups[1], shared_gate=False)


def config(layers, width=64, vocab=96, eps=1e-5, embed_scale=5.0):
    return StackConfig(arch="norevik", n_vocab=vocab, n_embd=width, layers=[LayerSpec(mixer=m, mlp=f) for m, f in layers],
                       norm_eps=eps, block=BLOCK_POSTNORM, embed_scale=embed_scale)


def standard():
    """Every mixer and every feed-forward, sizes that differ from one another: Mamba-2 first (a state layer as
    layer 0), a latent attention with a partly rotated key part, an mLSTM without feed-forward, a second latent
    attention with other sizes, a Mamba-2 whose norm groups differ from its B / C groups."""
    return config([(mamba(), dense()), (latent(rot_dim=12, rot_dims=8), moe()), (mlstm(), None),
                   (latent(heads=2, dim=8, rot_dim=4, vdim=16, kv_rank=20, scale=0.5), moe(experts=4, top=2, ff=16, shared_ff=0,
                                                                                          identity=0, groups=(1, 1))),
                   (mamba(heads=2, vdim=16, state=8, groups=1, conv=2, norm_groups=4), moe(experts=5, top=1, ff=8, identity=1,
                                                                                          groups=(2, 2))),
                   (mlstm(heads=3, dim=12, vdim=4, cap=15.0), dense(24))])


def check(got, want, dtype, what=""):
    """float32: the typical row within 5e-5 of the logits' spread and every row within 2e-3 (the mLSTM divides by a
    normaliser that passes through zero, so a single row can answer rounding with a hundred times as much; the
    torch twin and the HIP kernels show the same rows). bfloat16: for the same reason, and because a layer norm
    sits on every sublayer's output and rescales whatever it gets, single rows move by tens of percent; the
    typical row must stay within 0.12 and nine in ten within 0.6. The sharp comparisons are the float32 ones,
    on the same kernels."""
    e = rel_err(got, want)
    assert np.isfinite(np.asarray(got)).all(), f"{what}: non-finite logits"
    if dtype == "float32":
        assert np.median(e) < 5e-5 and e.max() < 2e-3, \
            f"{what}: median row off by {np.median(e):.3g}, worst row {int(e.argmax())} by {e.max():.3g}"
    else:
        assert np.median(e) < 0.12 and np.quantile(e, 0.9) < 0.6, \
            f"{what}: median row off by {np.median(e):.3g}, nine in ten within {np.quantile(e, 0.9):.3g}"


def random_config(rng):
    """A configuration drawn at the scale of a small real model: 4-7 layers of any mixer in any order, widths 128-320,
    head counts, ranks, rotated parts, taps, groups and routers of many shapes (rng: random.Random)."""
    width = rng.choice([128, 160, 224, 256, 320])

    def lat():
        R = rng.choice([0, 8, 16, 24, 32])
        return latent(heads=rng.choice([2, 4, 5, 8]), dim=rng.choice([32, 48, 64, 96]), rot_dim=R, vdim=rng.choice([32, 48, 64, 80]),
                      kv_rank=rng.choice([48, 64, 80, 128, 160]), scale=rng.choice([0.08, 0.15, 0.3]),
                      rot_dims=(rng.choice([R, max(0, R - 8)]) if R else 0), base=rng.choice([1e4, 1e6]))

    def ml():
        return mlstm(heads=rng.choice([2, 3, 4, 8]), dim=rng.choice([16, 32, 48, 64]), vdim=rng.choice([24, 32, 64, 96]),
                     cap=rng.choice([8.0, 12.0, 20.0]))

    def mb():
        G = rng.choice([1, 2, 4])
        H = G * rng.choice([1, 2, 4])
        return mamba(heads=H, vdim=rng.choice([16, 32, 64]), state=rng.choice([16, 32, 64, 128]), groups=G,
                     conv=rng.choice([2, 3, 4]), norm_groups=rng.choice([1, G, H]))

    def ff():
        k = rng.random()
        if k < 0.2:
            return None
        if k < 0.4:
            return dense(rng.choice([256, 384, 512]))
        gc, per = rng.choice([1, 2, 3, 4]), rng.choice([2, 3, 4])
        nr = gc * per
        ident = rng.choice([0, 1, 2]) if nr > 3 else 0
        keep = rng.randint(1, gc)
        return moe(experts=nr - ident, top=rng.randint(1, min(4, keep * per)), ff=rng.choice([64, 96, 128]),
                   shared_ff=rng.choice([0, 128, 192]), identity=ident, groups=(gc, keep))

    layers = [(rng.choice([lat, ml, mb])(), ff()) for _ in range(rng.randint(4, 7))]
    return config(layers, width=width, vocab=rng.choice([500, 777, 1024]), eps=rng.choice([1e-5, 1e-6]), embed_scale=width ** 0.5)


class Model(_Model):
    def oracle(self, toks):
        z, trail = oracle.forward(self.json, self.tensors, toks)
        return z.numpy(), trail.numpy()
