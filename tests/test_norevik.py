"""The Norevik design in the layer-list engine against its plain float64 implementation (norevik_oracle.py):
every mechanism alone, prefill against token-by-token decoding, portions, mixed batches, reused blocks and
slots, far keys and sinks, long decoding, odd sizes, generation through the engine's own entry points.
Every case runs on the CPU (torch twin of the executor: host logic) and, marked gpu, on the HIP kernels."""
from __future__ import annotations

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import norevik_cases as nc
import norevik_oracle as oracle
from ollama_operator_amd.engine.sampling import SamplingOptions
from ollama_operator_amd.engine.scheduler import BatchScheduler
from ollama_operator_amd.models.config import StackConfig, UnsupportedArchitecture, load_stack_config

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BOTH = ["float32", "bfloat16"]
GREEDY = SamplingOptions(temperature=0.0, repeat_penalty=1.0)


@pytest.fixture(scope="module")
def std(tmp_path_factory):
    return nc.Model(tmp_path_factory.mktemp("norevik"), nc.standard(), seed=3)


# ------------------------------------------------------------------ configuration
def test_config_roundtrip(std):
    cfg = load_stack_config(std.path)
    assert cfg == nc.standard() and cfg.has_state and cfg.embed_scale == 5.0
    assert StackConfig.from_norevik(cfg.to_norevik()) == cfg
    assert [s.mixer.state_floats for s in cfg.layers][:3] == [4 * 16 * 8 + 3 * (32 + 2 * 2 * 16), 0, 2 * (8 * 20 + 8 + 1)]


def test_unknown_parts_are_refused():
    c = nc.standard().to_norevik()
    for path, val in ((("layers", 0, "type"), "conv_mixer"), (("layers", 0, "mlp", "kind"), "glu")):
        d = json.loads(json.dumps(c))
        node = d
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = val
        with pytest.raises(UnsupportedArchitecture):
            StackConfig.from_norevik(d)
    d = json.loads(json.dumps(c))
    d["layers"][1]["mlp"]["router"]["groups"] = dict(count=4, keep=1)   # 9 router outputs in 4 groups
    with pytest.raises(UnsupportedArchitecture):
        StackConfig.from_norevik(d)


# ------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "latent_all_rotated": [(nc.latent(), None)],
    "latent_part_rotated_one_head": [(nc.latent(heads=1, dim=24, rot_dim=10, vdim=7, kv_rank=13, rot_dims=6), None)],
    "latent_no_rotation": [(nc.latent(rot_dim=4, rot_dims=0), None)],
    "latent_no_shared_key_part": [(nc.latent(heads=2, dim=16, rot_dim=0, vdim=8, kv_rank=16), None)],
    "mlstm": [(nc.mlstm(), None)],
    "mlstm_tight_cap_one_head": [(nc.mlstm(heads=1, dim=20, vdim=3, cap=1.5), None)],
    "mamba2": [(nc.mamba(), None)],
    "mamba2_one_tap_group_per_head": [(nc.mamba(heads=3, vdim=5, state=7, groups=3, conv=1, norm_groups=3), None)],
    "mamba2_two_taps_one_group": [(nc.mamba(heads=2, vdim=12, state=24, groups=1, conv=2, norm_groups=2), None)],
    "dense_ff": [(nc.mlstm(), nc.dense())],
    "moe_groups_identity_shared": [(nc.mlstm(), nc.moe())],
    "moe_plain_top1": [(nc.mlstm(), nc.moe(experts=5, top=1, identity=0, groups=(1, 1), shared_ff=0))],
    "moe_all_groups_kept_identity_only_group": [(nc.mlstm(), nc.moe(experts=6, top=4, identity=3, groups=(3, 3), shared_ff=8))],
    "moe_one_group_kept": [(nc.mlstm(), nc.moe(experts=8, top=2, identity=0, groups=(4, 1)))],
    "moe_more_choices_than_real_experts": [(nc.mlstm(), nc.moe(experts=2, top=4, identity=4, groups=(1, 1), shared_ff=16))],
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    m = nc.Model(tmp_path, nc.config(MECHANISMS[name], width=48, vocab=64), seed=11)
    toks = nc.tokens(45, 64, seed=1)
    want, trail = m.oracle(toks)
    r = m.runner(device)
    got_trail = nc.layer_trail(r, toks)
    assert np.abs(got_trail - trail).max() < 2e-3 * max(1.0, np.abs(trail).max()), "residual after the layer"
    nc.check(nc.run_cuts(r, toks, [len(toks)]), want, "float32", name)
    nc.check(nc.run_cuts(r, toks, [20, 21, 23, 45]), want, "float32", name + " in portions")


def test_router_oracle_by_hand():
    """The router on numbers worked out by hand: two groups of three, the correction moves the choice but not the
    weight, a negative corrected score inside the kept group still beats everything outside it."""
    f = dict(router=dict(experts=4, identity=2, top=2, groups=dict(count=2, keep=1)))
    W = dict(router=torch.eye(6, dtype=torch.float64), correction=torch.tensor([0.0, -5.0, -5.0, 0.5, 0.0, 0.0], dtype=torch.float64))
    h = torch.log(torch.tensor([[0.4, 0.3, 0.1, 0.05, 0.1, 0.05]], dtype=torch.float64))
    ids, wt = oracle.route(h, W, f)
    # corrected: [0.4, -4.7, -4.9 | 0.55, 0.1, 0.05]: the second group wins; its best two are 3 and 4
    assert ids.tolist() == [[3, 4]] and np.allclose(wt.numpy(), [[0.05, 0.1]])
    W["correction"][3] = 0.0   # now the first group wins, and its second choice has a negative corrected score
    ids, wt = oracle.route(h, W, f)
    assert ids.tolist() == [[0, 1]] and np.allclose(wt.numpy(), [[0.4, 0.3]])


# ------------------------------------------------------------------ whole prompts, decoding, portions
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_whole_prompt_and_layers(std, device, dtype):
    toks = nc.tokens(60, 96, seed=2)
    want, trail = std.oracle(toks)
    r = std.runner(device, dtype)
    got_trail = nc.layer_trail(r, toks)
    for i in range(trail.shape[0]):
        if dtype == "float32":
            assert np.abs(got_trail[i] - trail[i]).max() < 2e-3 * max(1.0, np.abs(trail[i]).max()), f"residual after layer {i}"
        else:  # rounding is amplified from layer to layer (see nc.check): the typical row decides
            e = np.sqrt(((got_trail[i] - trail[i]) ** 2).mean(-1)) / np.sqrt((trail[i] ** 2).mean(-1))
            assert np.median(e) < 0.02 * (i + 1), f"residual after layer {i}: median row off by {np.median(e):.3g}"
    nc.check(nc.run_cuts(r, toks, [len(toks)]), want, dtype, "whole prompt")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_prefill_then_token_by_token(std, device, dtype):
    toks = nc.tokens(80, 96, seed=4)
    want, _ = std.oracle(toks)
    r = std.runner(device, dtype)
    nc.check(nc.run_cuts(r, toks, [40] + list(range(41, 81))), want, dtype, "prefill 40, then one by one")


@pytest.mark.parametrize("device", DEVICES)
def test_every_token_alone_from_the_start(std, device):
    toks = nc.tokens(37, 96, seed=5)
    nc.check(nc.run_cuts(std.runner(device), toks, list(range(1, 38))), std.oracle(toks)[0], "float32", "one by one from 0")


@pytest.mark.parametrize("device", DEVICES)
def test_portions_of_many_sizes(std, device):
    """Portions of 2, 3, 1, 17, ... tokens across block borders (16) and shorter than the convolution's window;
    more rows than one forward holds (max_batch 32), so a portion is also cut by the engine."""
    toks = nc.tokens(150, 96, seed=6)
    want, _ = std.oracle(toks)
    r = std.runner(device, max_batch=32)
    cuts = [2, 5, 6, 8, 10, 27, 31, 32, 33, 35, 64, 66, 127, 129, 131, 150]
    nc.check(nc.run_cuts(r, toks, cuts), want, "float32", "portions")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_mixed_batch_equals_each_alone(std, device, dtype):
    """Five requests on four slots and a ten-block pool: portions of some beside single tokens of others, one
    sitting out a step, one ending early and its slot and blocks taken by a newcomer."""
    V = 96
    reqs = {k: nc.tokens(n, V, seed=30 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 21), ("e", 40)])}
    want = {k: std.oracle(t)[0] for k, t in reqs.items()}
    r = std.runner(device, dtype, kv_tokens=160, max_seqs=4)
    plan = [[("a", 20), ("b", 2)], [("a", 1), ("b", 5), ("c", 17)], [("a", 1), ("c", 1), ("d", 16)],
            [("c", 15), ("d", 5)], [("a", 28), ("e", 3)], [("e", 30)], [("e", 1)], [("e", 6)]]
    at = {k: 0 for k in reqs}
    sid, got = {}, {k: [] for k in reqs}
    for step in plan:
        entries = []
        for k, n in step:
            if k not in sid:
                sid[k] = r.new_sequence()
            entries.append((sid[k], reqs[k][at[k]:at[k] + n], list(range(n))))
        out = r.step_entries(entries).float().cpu().numpy()
        o = 0
        for k, n in step:
            got[k].append(out[o:o + n])
            o += n
            at[k] += n
            if at[k] == len(reqs[k]):
                r.free_sequence(sid.pop(k))
    assert all(at[k] == len(reqs[k]) for k in reqs)
    for k in reqs:
        nc.check(np.concatenate(got[k]), want[k], dtype, f"request {k} in the mixed batch")


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_and_slots_are_clean(std, device):
    """One slot and a pool for one request: the next request gets the previous one's blocks, matrix memories,
    state space states and convolution window and must see nothing of them."""
    r = std.runner(device, kv_tokens=64, max_seqs=1)
    for seed in (40, 41, 42):
        toks = nc.tokens(60, 96, seed=seed)
        nc.check(nc.run_cuts(r, toks, [33, 34, 60]), std.oracle(toks)[0], "float32", f"request {seed} on reused blocks")
    assert r.kv.alloc.n_free == r.kv.alloc.n_blocks and len(r.kv.rows_free) == 1


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(std, device):
    for n in (1, 2, 3):
        toks = nc.tokens(n, 96, seed=50 + n)
        nc.check(nc.run_cuts(std.runner(device), toks, [n]), std.oracle(toks)[0], "float32", f"{n} token prompt")


# ------------------------------------------------------------------ far keys, sinks, gates
@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_block_borders_and_sinks(tmp_path, device):
    """Sharp latent attention (a large score scale): most queries put their weight on ONE key, often far back, so
    a lost or misplaced cache row shows. One head's sink is huge (it takes most of the denominator), one is
    negligible, one is of the size of the scores. Portions and single tokens end just before, at and just after
    block borders."""
    layers = [(nc.latent(heads=3, dim=16, rot_dim=8, vdim=16, kv_rank=32, scale=3.0, base=30.0), None),
              (nc.latent(heads=2, dim=8, rot_dim=16, vdim=8, kv_rank=16, scale=2.0, rot_dims=12, base=1e4), nc.dense())]
    m = nc.Model(tmp_path, nc.config(layers, width=64, vocab=80), seed=5)
    m.set_tensor("l0.mix.sink", torch.tensor([30.0, -40.0, 6.0]))
    toks = nc.tokens(300, 80, seed=6)
    want, _ = m.oracle(toks)
    no_sink = {**m.tensors, "l0.mix.sink": torch.full((3,), -1e4)}
    assert nc.rel_err(oracle.forward(m.json, no_sink, toks)[0].numpy(), want).max() > 0.05, "the sinks must matter here"
    r = m.runner(device, max_batch=128, kv_tokens=320)
    cuts = [15, 16, 17, 31, 33, 47, 48, 49, 200, 255, 256, 257, 271, 272, 273] + list(range(274, 301))
    nc.check(nc.run_cuts(r, toks, cuts), want, "float32", "far keys")


@pytest.mark.parametrize("device", DEVICES)
def test_one_key_stands_out(tmp_path, device):
    """All the weight on the FIRST token, 251 positions back. With no rotated part in play (its query rows are
    zero) the score of key s is q_plain . W_uk c_s; the query matrix is rebuilt so that the last token's plain
    query is a large multiple of W_uk c_first in every head. A cache that lost that row answers with other keys."""
    mx = nc.latent(heads=2, dim=16, rot_dim=4, vdim=16, kv_rank=24, scale=1.0)
    m = nc.Model(tmp_path, nc.config([(mx, None)], width=32, vocab=50, embed_scale=1.0), seed=9)
    A, B = 7, 11
    T = {k: v.double() for k, v in m.tensors.items()}
    xa, xb = T["embed"][A], T["embed"][B]
    dkv = T["l0.mix.dkv"] @ xa
    ca = oracle.unit_rms(dkv[:24], 1e-5) * T["l0.mix.dkv.norm"]
    ka = (T["l0.mix.uk"] @ ca).view(2, 16)                     # token A's plain key per head
    Wq = torch.zeros(2, 20, 32, dtype=torch.float64)
    Wq[:, :16] = 4.0 * ka[:, :, None] * xb[None, None, :] / (xb @ xb)   # q_plain(B) = 4 k_A; rotated rows stay zero
    m.set_tensor("l0.mix.q", Wq.view(40, 32).float())
    body = [t for t in nc.tokens(300, 49, seed=8) if t not in (A, B)][:250]
    toks = [A] + body + [B]
    want, _ = m.oracle(toks)
    without = m.oracle([body[0]] + body + [B])[0][-1]
    assert nc.rel_err(want[-1], without) > 0.2, "the far key must matter in this construction"
    r = m.runner(device, max_batch=64, kv_tokens=320)
    n = len(toks)
    nc.check(nc.run_cuts(r, toks, [n - 1, n])[-1:], want[-1:], "float32", "decoded token asking for a far key")
    nc.check(nc.run_cuts(r, toks, [100, n])[-1:], want[-1:], "float32", "prompt portion asking for a far key")


@pytest.mark.parametrize("device", DEVICES)
def test_long_context_decode(tmp_path, device):
    """Single tokens after 1300 cached rows: on a GPU the decode attention then shares a row's keys among several
    blocks and merges their partial sums (the sink joins once, after the merge); a long row beside short ones."""
    layers = [(nc.latent(heads=4, dim=16, rot_dim=8, vdim=24, kv_rank=40, scale=1.5, base=1e4), None)]
    m = nc.Model(tmp_path, nc.config(layers, width=32, vocab=60), seed=21)
    m.set_tensor("l0.mix.sink", torch.tensor([8.0, 0.0, -30.0, 3.0]))
    toks = nc.tokens(1306, 60, seed=22)
    want, _ = m.oracle(toks)
    r = m.runner(device, max_batch=512, kv_tokens=1400)
    cuts = [1300] + list(range(1301, 1307))
    got = nc.run_cuts(r, toks, cuts)
    rows = list(range(1300, 1306))
    nc.check(got[rows], want[rows], "float32", "decoded after a long context")
    short = nc.tokens(9, 60, seed=23)
    ws = m.oracle(short)[0]
    a, b = r.new_sequence(), r.new_sequence()
    r.step_entries([(a, toks[:1200], []), (b, short[:5], [])])
    out = r.step_entries([(a, toks[1200:1201], [0]), (b, short[5:7], [0, 1])]).float().cpu().numpy()
    nc.check(out[:1], want[1200:1201], "float32", "long row of a mixed step")
    nc.check(out[1:], ws[5:7], "float32", "short rows of a mixed step")


@pytest.mark.parametrize("device", DEVICES)
def test_memories_that_last_and_gates_at_their_limits(tmp_path, device):
    """mLSTM heads with a forget gate that hardly forgets and an input gate pushed to both ends of its cap (a
    running maximum that climbs, and one that stays at its starting value 0 while exp(-m) bounds the
    denominator); Mamba-2 heads whose decay spans 'gone in a token' to 'kept for thousands'. 400 tokens, then
    single tokens: what the first tokens wrote must still be there."""
    layers = [(nc.mlstm(heads=3, dim=8, vdim=8, cap=4.0), None), (nc.mamba(heads=4, vdim=8, state=8, groups=2, conv=3), None)]
    m = nc.Model(tmp_path, nc.config(layers, width=32, vocab=40), seed=13)
    m.set_tensor("l0.mix.f.b", torch.tensor([9.0, 9.0, 0.0]))
    m.set_tensor("l0.mix.i.b", torch.tensor([7.0, -7.0, 0.0]))
    m.set_tensor("l1.mix.A_log", torch.tensor([-9.0, -3.0, 0.0, 3.0]))
    m.set_tensor("l1.mix.dt_bias", torch.tensor([-1.0, 0.0, 1.0, 4.0]))
    toks = nc.tokens(420, 40, seed=14)
    want, _ = m.oracle(toks)
    changed = m.oracle([(toks[0] + 1) % 40] + toks[1:])[0][-1]
    assert nc.rel_err(changed, want[-1]) > 1e-3, "the first token must still matter at the end"
    r = m.runner(device, max_batch=128, kv_tokens=512)
    nc.check(nc.run_cuts(r, toks, [400] + list(range(401, 421))), want, "float32", "long memories")


# ------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_other_sizes(tmp_path, device, dtype):
    """A width, head sizes and expert sizes that are not multiples of 8 (no vector loads), more rows than one
    tile, a vocabulary wider than a tile, eps and embedding scale of their own, every group kept, top 4."""
    layers = [(nc.latent(heads=5, dim=12, rot_dim=6, vdim=10, kv_rank=18, scale=0.4, rot_dims=4),
               nc.moe(experts=9, top=4, ff=20, shared_ff=12, identity=1, groups=(5, 3))),
              (nc.mamba(heads=6, vdim=6, state=10, groups=3, conv=5, norm_groups=2), nc.dense(36)),
              (nc.mlstm(heads=5, dim=6, vdim=14, cap=9.0), nc.moe(experts=3, top=3, ff=12, shared_ff=0, identity=0, groups=(1, 1))),
              (nc.latent(heads=2, dim=64, rot_dim=32, vdim=64, kv_rank=96, scale=0.1),
               nc.moe(experts=16, top=2, ff=64, shared_ff=64, identity=0, groups=(4, 2)))]
    m = nc.Model(tmp_path, nc.config(layers, width=52, vocab=300, eps=1e-3, embed_scale=0.7), seed=17)
    toks = nc.tokens(90, 300, seed=18)
    want, _ = m.oracle(toks)
    r = m.runner(device, dtype, max_batch=128)
    nc.check(nc.run_cuts(r, toks, [70, 71, 72, 90]), want, dtype, "odd sizes")


@pytest.mark.parametrize("device", DEVICES)
def test_matrix_core_sizes(tmp_path, device):
    """Sizes the matrix-core products and vector loads take (multiples of 64), in bfloat16, with enough rows for the
    grouped routed feed-forward; prompt portion, then single tokens."""
    layers = [(nc.latent(heads=4, dim=64, rot_dim=32, vdim=64, kv_rank=96, scale=0.1),
               nc.moe(experts=6, top=2, ff=64, shared_ff=128, identity=2, groups=(2, 1))),
              (nc.mamba(heads=4, vdim=32, state=32, groups=1, conv=4, norm_groups=2), nc.dense(256)),
              (nc.mlstm(heads=2, dim=32, vdim=64, cap=10.0), nc.moe(experts=4, top=2, ff=128, shared_ff=64, identity=0, groups=(1, 1)))]
    m = nc.Model(tmp_path, nc.config(layers, width=128, vocab=256), seed=19)
    toks = nc.tokens(200, 256, seed=20)
    want, _ = m.oracle(toks)
    for dtype in BOTH:
        r = m.runner(device, dtype, max_batch=256)
        nc.check(nc.run_cuts(r, toks, [190] + list(range(191, 201))), want, dtype, "matrix-core sizes")


# ------------------------------------------------------------------ generation through the engine's entry points
def greedy_oracle(m, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(m.oracle(toks)[0][-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generate_and_long_decode(std, device):
    """`Runner.generate` (prefill, the on-device sampler, the decode graph on a GPU) produces the oracle's greedy
    continuation over several block borders; the next turn extends the cached sequence (its states are kept
    whole), a prompt that shares only a part starts over."""
    prompt = nc.tokens(12, 96, seed=60)
    want = greedy_oracle(std, prompt, 40)
    r = std.runner(device, use_graphs=None)
    sid = r.new_sequence()
    got = list(r.generate(sid, prompt, GREEDY, max_tokens=40))
    assert got == want
    more = list(r.generate(sid, prompt + got + [5, 6], GREEDY, max_tokens=4))
    assert more == greedy_oracle(std, prompt + got + [5, 6], 4)
    other = prompt[:6] + [1, 2, 3]
    assert list(r.generate(sid, other, GREEDY, max_tokens=3)) == greedy_oracle(std, other, 3)


@pytest.mark.parametrize("device", DEVICES)
def test_scheduler_batches_requests(std, device):
    r = std.runner(device, max_seqs=5, kv_tokens=1024, use_graphs=None)
    sch = BatchScheduler(r, max_parallel=3)
    try:
        prompts = [nc.tokens(n, 96, seed=70 + i) for i, n in enumerate((9, 20, 14))]
        lens = (12, 5, 9)
        its = [sch.submit(p, GREEDY, max_tokens=k) for p, k in zip(prompts, lens)]
        got = [list(it) for it in its]
        for p, k, g in zip(prompts, lens, got):
            assert g == greedy_oracle(std, p, k)
    finally:
        sch.close()


def test_command_line_generates_token_ids(std, capsys):
    from ollama_operator_amd import cli
    prompt = nc.tokens(9, 96, seed=90)
    cli.main(["tokens", std.path, "--ids", " ".join(map(str, prompt)), "--num-predict", "5", "--device", "cpu",
              "--dtype", "float32"])
    out = capsys.readouterr().out.strip().splitlines()[-1]
    assert [int(t) for t in out.split()] == greedy_oracle(std, prompt, 5)


def test_trace_replay_program(std, tmp_path):
    """bin/trace_run on the CPU twin: a request that sits out a step, one that ends and gives its slot back."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = nc.tokens(30, 96, seed=91), nc.tokens(12, 96, seed=92)
    steps = [dict(step=0, entries=[dict(id="a", tokens=a[:20], want=[0, 19])], end=[]),
             dict(step=1, entries=[dict(id="b", tokens=b, want=[11])], end=["b"]),
             dict(step=2, entries=[dict(id="a", tokens=a[20:], want=[9]), dict(id="c", tokens=b[:2], want=[])], end=["a", "c"])]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", std.path, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "64", "--device", "cpu"], input="".join(json.dumps(x) + "\n" for x in steps),
                       capture_output=True, text=True, timeout=300, env={**os.environ, "PYTHON": sys.executable})
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(3)]
    wa, wb = std.oracle(a)[0], std.oracle(b)[0]
    nc.check(np.fromfile(out / "0.f32", "<f4").reshape(2, 96), wa[[0, 19]], "float32", "step 0")
    nc.check(np.fromfile(out / "1.f32", "<f4").reshape(1, 96), wb[[11]], "float32", "step 1")
    nc.check(np.fromfile(out / "2.f32", "<f4").reshape(1, 96), wa[[29]], "float32", "step 2")


# ------------------------------------------------------------------ the HIP executor against its twin
@pytest.mark.gpu
def test_gpu_matches_twin_layer_by_layer(std):
    toks = nc.tokens(50, 96, seed=95)
    for dtype, tol in (("float32", 1e-4), ("bfloat16", 0.05)):
        a = nc.layer_trail(std.runner("cpu", dtype), toks)
        b = nc.layer_trail(std.runner("cuda", dtype), toks)
        for i in range(a.shape[0]):
            assert np.abs(a[i] - b[i]).max() < tol * max(1.0, np.abs(a[i]).max()), f"{dtype}: layer run {i}"


@pytest.mark.gpu
@pytest.mark.parametrize("rank,rot", [(96, 32), (128, 16)])
def test_matrix_core_attention_matches_twin(tmp_path, rank, rot):
    """Latent attention of prompt portions on the matrix cores (bfloat16): one layer, so rounding is not amplified and
    the comparison is sharp; sinks from dominant to negligible; a portion that starts in the middle of the cache."""
    m = nc.Model(tmp_path, nc.config([(nc.latent(heads=4, dim=48, rot_dim=rot, vdim=40, kv_rank=rank, scale=0.6), None)],
                                     width=128, vocab=128), seed=23)
    m.set_tensor("l0.mix.sink", torch.tensor([12.0, -30.0, 2.0, 5.0]))
    toks = nc.tokens(230, 128, seed=24)
    want, _ = m.oracle(toks)
    a = nc.run_cuts(m.runner("cpu", "bfloat16", max_batch=256), toks, [70, 230])
    b = nc.run_cuts(m.runner("cuda", "bfloat16", max_batch=256), toks, [70, 230])
    e = nc.rel_err(b, a)
    assert np.median(e) < 5e-3 and e.max() < 3e-2, f"HIP against twin: median {np.median(e):.3g}, worst {e.max():.3g}"
    e = nc.rel_err(b, want)
    assert np.median(e) < 2e-2 and e.max() < 0.1, f"HIP against the plain implementation: median {np.median(e):.3g}, worst {e.max():.3g}"


@pytest.mark.gpu
@pytest.mark.parametrize("seed", [0, 1, 2, 3])
def test_random_configurations(tmp_path, seed):
    """Configurations drawn at the scale of a small real model, a prompt of 700 tokens in portions of 64 and a tail of
    single tokens against the whole prompt in one step and against the plain implementation, float32; bfloat16 against
    the twin (the same rounding points: the two must be much closer to each other than either is to float64)."""
    import random
    cfg = nc.random_config(random.Random(100 + seed))
    m = nc.Model(tmp_path, cfg, seed=seed)
    n = 700
    toks = nc.tokens(n, cfg.n_vocab, seed=seed)
    want, _ = m.oracle(toks)
    r = m.runner("cuda", "float32", max_batch=512, kv_tokens=1536)
    cuts = list(range(64, n - 40, 64)) + [n - 37] + list(range(n - 36, n + 1))
    for what, got in (("portions", nc.run_cuts(r, toks, cuts)), ("whole", nc.run_cuts(r, toks, [n]))):
        e = nc.rel_err(got, want)  # stacks of up to seven layers: the odd ill-conditioned row may reach 1e-2
        assert np.isfinite(got).all() and np.median(e) < 5e-5 and np.quantile(e, 0.99) < 1e-3 and e.max() < 2e-2, \
            f"{what}: median {np.median(e):.3g}, 99 in 100 within {np.quantile(e, 0.99):.3g}, worst row {int(e.argmax())} by {e.max():.3g}"
    short = toks[:300]
    a = nc.run_cuts(m.runner("cpu", "bfloat16", max_batch=512, kv_tokens=512), short, [300])
    b = nc.run_cuts(m.runner("cuda", "bfloat16", max_batch=512, kv_tokens=512), short, [64, 128, 192, 256, 298, 299, 300])
    e = nc.rel_err(b, a)
    assert np.isfinite(b).all() and np.median(e) < 0.04 and np.quantile(e, 0.9) < 0.2, \
        f"bfloat16 HIP against twin: median {np.median(e):.3g}, nine in ten within {np.quantile(e, 0.9):.3g}"
