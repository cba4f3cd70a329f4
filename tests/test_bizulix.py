"""Bizulix through the engine against the plain float64 implementation (tests/bizulix_oracle.py).

Every test runs twice: on the CPU (the torch twin of the stack executor: block pool, state slots, batching and
scheduling logic) and, marked `gpu`, on the HIP kernels. float32 runs are held to 3e-4 of the logits' spread,
bfloat16 runs to 6e-2."""
from __future__ import annotations

import numpy as np
import pytest
import torch

import bizulix_cases as bc
import bizulix_oracle as oracle
from ollama_operator_amd.engine.sampling import SamplingOptions
from ollama_operator_amd.engine.scheduler import BatchScheduler
from ollama_operator_amd.models.config import StackConfig, load_stack_config

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
BOTH = ["float32", "bfloat16"]


@pytest.fixture(scope="module")
def std(tmp_path_factory):
    return bc.Model(tmp_path_factory.mktemp("bizulix"), bc.standard(), seed=3)


# ------------------------------------------------------------------ configuration and files
def test_config_roundtrip_and_run_order(std):
    cfg = load_stack_config(std.path)
    assert cfg == std.cfg and StackConfig.from_bizulix(cfg.to_bizulix()) == cfg
    assert [(i, p) for i, p, _ in cfg.runs()] == [(0, 0), (1, 0), (2, 0), (1, 1), (2, 1), (3, 0), (4, 0)]
    assert [o for _, _, o in cfg.runs()] == [False, True, False, True, False, False, False]
    assert cfg.has_state
    assert [i for i, _, _ in bc.config([(bc.attn(), None)] * 3).runs()] == [0, 1, 2]


def test_unknown_architecture_is_refused(tmp_path):
    import json
    from ollama_operator_amd.models.config import UnsupportedArchitecture
    (tmp_path / "config.json").write_text(json.dumps({"architecture": "Nope"}))
    with pytest.raises(UnsupportedArchitecture):
        load_stack_config(str(tmp_path))


# ------------------------------------------------------------------ each mechanism alone
MECHANISMS = {
    "attention": [(bc.attn(), None)],
    "attention_plain": [(bc.attn(heads=3, kv_heads=3, dim=16, vdim=16, softcap=0.0, coef=0.0), None)],
    "attention_mqa_wide_v": [(bc.attn(heads=5, kv_heads=1, dim=8, vdim=40, every=3), None)],
    "retention": [(bc.ret(), None)],
    "retention_full_rot": [(bc.ret(heads=3, dim=8, vdim=8, decay=(0.5, 0.97, 0.9995), rot_dims=8), None)],
    "retention_no_rot": [(bc.ret(heads=1, dim=24, vdim=72, decay=(0.99,), rot_dims=0), None)],
    "retention_wide_heads": [(bc.ret(heads=1, dim=72, vdim=264, decay=(0.98,), rot_dims=36), None)],
    "moe": [(bc.attn(heads=1, kv_heads=1, dim=8, vdim=8), bc.moe())],
    "moe_top1_no_shared": [(bc.attn(heads=1, kv_heads=1, dim=8, vdim=8), bc.moe(experts=5, top=1, ff=12, shared_ff=0))],
    "moe_all_experts": [(bc.ret(heads=1, dim=8, vdim=8, decay=(0.9,)), bc.moe(experts=3, top=3, ff=8, shared_ff=8))],
}


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", sorted(MECHANISMS))
def test_mechanism_alone(tmp_path, device, name):
    m = bc.Model(tmp_path, bc.config(MECHANISMS[name], width=48, vocab=64, mult=1.0, cap=0.0), seed=11)
    toks = bc.tokens(45, 64, seed=1)
    want, trail = m.oracle(toks)
    r = m.runner(device)
    got_trail = bc.layer_trail(r, toks)
    assert np.abs(got_trail - trail).max() < 2e-3 * max(1.0, np.abs(trail).max()), "residual after the layer"
    bc.check(bc.run_cuts(r, toks, [len(toks)]), want, "float32", name)


@pytest.mark.parametrize("device", DEVICES)
def test_loop_passes_have_their_own_cache(tmp_path, device):
    """A span that runs twice over the same weights: the second pass must not read the first one's keys or
    state. Also a loop over all layers, and one of a single pass."""
    for k, loop in enumerate([(0, 2, 2), (1, 2, 3), (0, 1, 1)]):
        m = bc.Model(tmp_path, bc.config([(bc.attn(), None), (bc.ret(), bc.moe())], loop=loop), seed=20 + k, name=f"loop{k}")
        toks = bc.tokens(40, 96, seed=k)
        want, trail = m.oracle(toks)
        r = m.runner(device)
        assert np.abs(bc.layer_trail(r, toks) - trail).max() < 2e-3 * max(1.0, np.abs(trail).max())
        bc.check(bc.run_cuts(r, toks, [25, 26, 27, 40]), want, "float32", f"loop {loop}")


# ------------------------------------------------------------------ whole prompt, portions, decoding
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_whole_prompt_and_layers(std, device, dtype):
    toks = bc.tokens(70, 96, seed=2)
    want, trail = std.oracle(toks)
    r = std.runner(device, dtype, max_batch=128)
    got = bc.layer_trail(r, toks)
    lim = (2e-3 if dtype == "float32" else 0.15) * np.abs(trail).max()
    for ri in range(len(trail)):
        assert np.abs(got[ri] - trail[ri]).max() < lim, f"residual after layer run {ri}"
    bc.check(bc.run_cuts(r, toks, [len(toks)]), want, dtype, "whole prompt")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_prefill_then_token_by_token(std, device, dtype):
    """Most of the prompt at once, then single tokens through the cache and the state, across block borders."""
    toks = bc.tokens(90, 96, seed=3)
    want, _ = std.oracle(toks)
    r = std.runner(device, dtype)
    bc.check(bc.run_cuts(r, toks, [45] + list(range(46, 91))), want, dtype, "prefill + decode")


@pytest.mark.parametrize("device", DEVICES)
def test_every_token_alone_from_the_start(std, device):
    toks = bc.tokens(40, 96, seed=4)
    want, _ = std.oracle(toks)
    bc.check(bc.run_cuts(std.runner(device), toks, list(range(1, 41))), want, "float32", "token by token")


@pytest.mark.parametrize("device", DEVICES)
def test_portions_of_many_sizes(std, device):
    toks = bc.tokens(120, 96, seed=5)
    want, _ = std.oracle(toks)
    r = std.runner(device, max_batch=32)  # portions longer than the step's rows run as several forwards
    for cuts in ([2, 4, 7, 16, 17, 32, 33, 64, 120], [15, 31, 33, 47, 49, 50, 52, 100, 118, 120], [50, 120]):
        bc.check(bc.run_cuts(r, toks, cuts), want, "float32", f"portions {cuts}")


# ------------------------------------------------------------------ batches, pages, slots
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", BOTH)
def test_mixed_batch_equals_each_alone(std, device, dtype):
    """Four requests of unequal length advance together: portions of some beside single tokens of others, one
    sitting out a step, one ending early and its slot and blocks taken by a newcomer."""
    V = 96
    reqs = {k: bc.tokens(n, V, seed=30 + i) for i, (k, n) in enumerate([("a", 50), ("b", 7), ("c", 33), ("d", 21), ("e", 40)])}
    want = {k: std.oracle(t)[0] for k, t in reqs.items()}
    r = std.runner(device, dtype, kv_tokens=160, max_seqs=4)  # 10 blocks of 16: reuse is forced
    plan = [  # per step: (request, tokens)
        [("a", 20), ("b", 2)], [("a", 1), ("b", 5), ("c", 17)], [("a", 1), ("c", 1), ("d", 16)],
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
        bc.check(np.concatenate(got[k]), want[k], dtype, f"request {k} in the mixed batch")


@pytest.mark.parametrize("device", DEVICES)
def test_freed_blocks_and_slots_are_clean(std, device):
    """The pool holds one request at a time and there is one slot: the second request gets the first one's
    blocks and state slot and must not see anything of it."""
    r = std.runner(device, kv_tokens=64, max_seqs=1)
    for seed in (40, 41, 42):
        toks = bc.tokens(60, 96, seed=seed)
        bc.check(bc.run_cuts(r, toks, [33, 34, 60]), std.oracle(toks)[0], "float32", f"request {seed} on reused blocks")
    assert r.kv.alloc.n_free == r.kv.alloc.n_blocks and len(r.kv.rows_free) == 1


@pytest.mark.parametrize("device", DEVICES)
def test_pool_exhaustion_is_an_error(std, device):
    from ollama_operator_amd.engine.kv_cache import OutOfBlocks
    r = std.runner(device, kv_tokens=32, max_seqs=2)
    a, b = r.new_sequence(), r.new_sequence()
    r.step_entries([(a, bc.tokens(20, 96), [])])
    with pytest.raises(OutOfBlocks):
        r.step_entries([(b, bc.tokens(20, 96), [])])


# ------------------------------------------------------------------ far keys, borders, first tokens
@pytest.mark.parametrize("device", DEVICES)
def test_far_keys_and_borders(tmp_path, device):
    """Sharp attention (scores of spread ~8, a high cap): most queries put their weight on ONE key, often far
    back, so a lost or misplaced key shows. The temperature steps every 16 positions, blocks are 16 tokens,
    and prompt portions and single tokens end just before, at and just after both kinds of border. One
    retention head forgets within a few tokens, the other hardly at all."""
    layers = [(bc.attn(heads=4, kv_heads=2, dim=16, vdim=16, scale=2.0, softcap=50.0, coef=1.0, every=16), None),
              (bc.ret(heads=2, dim=16, vdim=16, decay=(0.6, 0.9998), rot_dims=16, base=50.0), None),
              (bc.attn(heads=2, kv_heads=1, dim=32, vdim=8, scale=1.5, softcap=40.0, coef=0.25, every=7), bc.moe())]
    m = bc.Model(tmp_path, bc.config(layers, width=64, vocab=80, mult=1.0), seed=5)
    toks = bc.tokens(300, 80, seed=6)
    want, _ = m.oracle(toks)
    r = m.runner(device, max_batch=128, kv_tokens=320)
    cuts = [15, 16, 17, 31, 33, 47, 48, 49, 200, 255, 256, 257, 271, 272, 273] + list(range(274, 301))
    bc.check(bc.run_cuts(r, toks, cuts), want, "float32", "far keys")


@pytest.mark.parametrize("device", DEVICES)
def test_one_key_stands_out(tmp_path, device):
    """The query projection of an attention layer is rebuilt from its key projection so that the LAST token's
    query is three times the key of the FIRST token, 251 positions back: almost all of its weight must land
    there. The oracle says what comes out; a cache that lost that key answers with the other keys instead."""
    m = bc.Model(tmp_path, bc.config([(bc.attn(heads=2, kv_heads=2, dim=16, vdim=16, scale=1.0, softcap=0.0, coef=0.0), None)],
                                     width=32, vocab=50, mult=1.0, cap=0.0), seed=9)
    A, B = 7, 11  # the far token and the last one
    T = {k: v.double() for k, v in m.tensors.items()}
    hA, hB = (oracle.layer_norm(T["embed"][t], T["l0.norm1"], T["l0.norm1.b"], 1e-5) for t in (A, B))
    # W_q = 3 W_k (I + (hA - hB) hB^T / |hB|^2): token B's query is 3 x token A's key in every head
    m.set_tensor("l0.mix.q", (3.0 * T["l0.mix.k"] @ (torch.eye(32, dtype=torch.float64) + torch.outer(hA - hB, hB) / (hB @ hB))).float())
    body = [t for t in bc.tokens(300, 49, seed=8) if t not in (A, B)][:250]
    toks = [A] + body + [B]
    want, _ = m.oracle(toks)
    without = m.oracle([body[0]] + body + [B])[0][-1]
    assert bc.rel_err(want[-1], without) > 0.2, "the far key must matter in this construction"
    r = m.runner(device, max_batch=64, kv_tokens=320)
    n = len(toks)
    bc.check(bc.run_cuts(r, toks, [n - 1, n])[-1:], want[-1:], "float32", "decoded token asking for a far key")
    bc.check(bc.run_cuts(r, toks, [100, n])[-1:], want[-1:], "float32", "prompt portion asking for a far key")


@pytest.mark.parametrize("device", DEVICES)
def test_long_context_decode(tmp_path, device):
    """Single tokens after 1300 and after 2300 cached keys: on a GPU the decode attention then shares a row's keys
    among several blocks and merges their partial softmax sums; sharp scores make single far keys matter."""
    layers = [(bc.attn(heads=4, kv_heads=2, dim=16, vdim=24, scale=1.5, softcap=40.0, coef=0.5, every=512), None),
              (bc.attn(heads=2, kv_heads=1, dim=64, vdim=64, scale=0.4, softcap=0.0, coef=0.0), None)]
    m = bc.Model(tmp_path, bc.config(layers, width=32, vocab=60, mult=1.0, cap=0.0), seed=21)
    toks = bc.tokens(2306, 60, seed=22)
    want, _ = m.oracle(toks)
    r = m.runner(device, max_batch=512, kv_tokens=2400)
    cuts = [1300, 1301, 1302, 1303, 2300] + list(range(2301, 2307))
    got = bc.run_cuts(r, toks, cuts)
    rows = [1300, 1301, 1302] + list(range(2300, 2306))
    bc.check(got[rows], want[rows], "float32", "decoded after a long context")
    # a long sequence's single token beside a short sequence's two: the short rows' extra blocks have no keys
    short = bc.tokens(9, 60, seed=23)
    ws = m.oracle(short)[0]
    a, b = r.new_sequence(), r.new_sequence()
    r.step_entries([(a, toks[:2200], []), (b, short[:5], [])])
    out = r.step_entries([(a, toks[2200:2201], [0]), (b, short[5:7], [0, 1])]).float().cpu().numpy()
    bc.check(out[:1], want[2200:2201], "float32", "long row of a mixed step")
    bc.check(out[1:], ws[5:7], "float32", "short rows of a mixed step")
    r2 = m.runner(device, "bfloat16", max_batch=512, kv_tokens=2400, use_graphs=None)
    sid = r2.new_sequence()
    out = list(r2.generate(sid, toks[:1100], SamplingOptions(temperature=0.0, repeat_penalty=1.0), max_tokens=3))
    assert len(out) == 3  # the batch-1 decode graph of a split bucket runs


@pytest.mark.parametrize("device", DEVICES)
def test_first_tokens(std, device):
    for n in (1, 2, 3):
        toks = bc.tokens(n, 96, seed=50 + n)
        bc.check(bc.run_cuts(std.runner(device), toks, [n]), std.oracle(toks)[0], "float32", f"{n} token prompt")


# ------------------------------------------------------------------ other sizes
@pytest.mark.parametrize("device", DEVICES)
def test_other_sizes(tmp_path, device):
    """Sizes off the beaten track: a width and head sizes that are not multiples of 8 (no vector loads), one
    query head per key/value head, more rows than one tile, a wide vocabulary, no caps, residual factor 1."""
    layers = [(bc.attn(heads=3, kv_heads=3, dim=10, vdim=6, scale=0.3, softcap=0.0, coef=0.0),
               bc.moe(experts=3, top=2, ff=10, shared_ff=6)),
              (bc.ret(heads=2, dim=10, vdim=14, decay=(0.8, 0.95), rot_dims=4), None),
              (bc.attn(heads=8, kv_heads=2, dim=64, vdim=64, every=1), bc.moe(experts=9, top=4, ff=64, shared_ff=128))]
    m = bc.Model(tmp_path, bc.config(layers, width=52, vocab=203, mult=1.0, cap=0.0, eps=1e-3), seed=13)
    toks = bc.tokens(150, 203, seed=14)
    want, _ = m.oracle(toks)
    for dtype in BOTH:
        r = m.runner(device, dtype, max_batch=160)
        bc.check(bc.run_cuts(r, toks, [150]), want, dtype, "whole")
        bc.check(bc.run_cuts(r, toks, [140] + list(range(141, 151))), want, dtype, "decode")


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dim", [64, 96, 128])
def test_matrix_core_head_sizes(tmp_path, device, dim):
    """Head sizes that the matrix-core kernels take on a GPU (bfloat16 prompt portions: query tiles of 32 rows,
    keys by 32), grouped and ungrouped heads, a retention layer between: whole prompt, portions that end inside
    a tile, single tokens, and two sequences in one step."""
    layers = [(bc.attn(heads=4, kv_heads=2, dim=dim, vdim=dim, scale=dim ** -0.5, softcap=25.0, coef=0.3, every=32),
               bc.moe(ff=32, shared_ff=32)),
              (bc.ret(heads=2, dim=64, vdim=128, decay=(0.97, 0.999), rot_dims=64, base=1e4), None),
              (bc.attn(heads=2, kv_heads=2, dim=dim, vdim=dim, scale=2.0 * dim ** -0.5, softcap=0.0, coef=0.0), None)]
    m = bc.Model(tmp_path, bc.config(layers, width=128, vocab=120, mult=0.5), seed=dim)
    a, b = bc.tokens(170, 120, seed=1), bc.tokens(75, 120, seed=2)
    wa, wb = m.oracle(a)[0], m.oracle(b)[0]
    for dtype in BOTH:
        r = m.runner(device, dtype, max_batch=256, kv_tokens=512)
        bc.check(bc.run_cuts(r, a, [170]), wa, dtype, "whole")
        bc.check(bc.run_cuts(r, a, [33, 100, 131, 132, 170]), wa, dtype, "portions")
        sa, sb = r.new_sequence(), r.new_sequence()
        o1 = r.step_entries([(sa, a[:90], list(range(90))), (sb, b[:40], list(range(40)))]).float().cpu().numpy()
        o2 = r.step_entries([(sa, a[90:], list(range(80))), (sb, b[40:], list(range(35)))]).float().cpu().numpy()
        bc.check(np.concatenate([o1[:90], o2[:80]]), wa, dtype, "first of two sequences")
        bc.check(np.concatenate([o1[90:], o2[80:]]), wb, dtype, "second of two sequences")


# ------------------------------------------------------------------ generation through the engine's entry points
def greedy_oracle(m, prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(int(np.argmax(m.oracle(toks)[0][-1])))
    return toks[len(prompt):]


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generate_and_long_decode(std, device):
    """`Runner.generate` (prefill, the on-device sampler, the decode graph on a GPU) produces the oracle's
    greedy continuation, over several block borders."""
    prompt = bc.tokens(12, 96, seed=60)
    want = greedy_oracle(std, prompt, 40)
    r = std.runner(device, use_graphs=None)
    sid = r.new_sequence()
    got = list(r.generate(sid, prompt, SamplingOptions(temperature=0.0, repeat_penalty=1.0), max_tokens=40))
    assert got == want
    # the same sequence continues: its cached prefix is kept whole (it has state), the next turn extends it
    more = list(r.generate(sid, prompt + got + [5, 6], SamplingOptions(temperature=0.0, repeat_penalty=1.0), max_tokens=4))
    assert more == greedy_oracle(std, prompt + got + [5, 6], 4)
    # a prompt that shares only part of the cached tokens starts over (a state cannot be cut back)
    other = prompt[:6] + [1, 2, 3]
    assert list(r.generate(sid, other, SamplingOptions(temperature=0.0, repeat_penalty=1.0), max_tokens=3)) == \
        greedy_oracle(std, other, 3)


@pytest.mark.parametrize("device", DEVICES)
def test_scheduler_batches_requests(std, device):
    """Three clients through the continuous-batching scheduler: batched admission, batched decode steps,
    rows that finish at different times; each gets its own greedy continuation."""
    r = std.runner(device, max_seqs=5, kv_tokens=1024, use_graphs=None)
    sch = BatchScheduler(r, max_parallel=3)
    try:
        prompts = [bc.tokens(n, 96, seed=70 + i) for i, n in enumerate((9, 20, 14))]
        lens = (12, 5, 9)
        o = SamplingOptions(temperature=0.0, repeat_penalty=1.0)
        its = [sch.submit(p, o, max_tokens=k) for p, k in zip(prompts, lens)]
        got = [list(it) for it in its]
        for p, k, g in zip(prompts, lens, got):
            assert g == greedy_oracle(std, p, k)
    finally:
        sch.close()


def test_command_line_generates_token_ids(std, capsys):
    """`ollama tokens MODEL --ids ...`: the command line picks the runner class by the model and generates
    through `Runner.generate`."""
    from ollama_operator_amd import cli
    prompt = bc.tokens(9, 96, seed=90)
    cli.main(["tokens", std.path, "--ids", " ".join(map(str, prompt)), "--num-predict", "5", "--device", "cpu",
              "--dtype", "float32"])
    out = capsys.readouterr().out.strip().splitlines()[-1]
    assert [int(t) for t in out.split()] == greedy_oracle(std, prompt, 5)


def test_trace_replay_program(std, tmp_path):
    """bin/trace_run on the CPU twin: steps on standard input, logits files and `done` lines out; a request
    that sits out a step, one that ends and gives its slot back."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    a, b = bc.tokens(30, 96, seed=91), bc.tokens(12, 96, seed=92)
    steps = [dict(step=0, entries=[dict(id="a", tokens=a[:20], want=[0, 19])], end=[]),
             dict(step=1, entries=[dict(id="b", tokens=b, want=[11])], end=["b"]),
             dict(step=2, entries=[dict(id="a", tokens=a[20:], want=[9])], end=["a"]),
             dict(step=3, entries=[dict(id="c", tokens=b[:2], want=[])], end=["c"])]
    out = tmp_path / "out"
    p = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", std.path, "--dtype", "float32", "--out", str(out),
                        "--max-tokens", "64", "--device", "cpu"], input="".join(json.dumps(x) + "\n" for x in steps),
                       capture_output=True, text=True, timeout=300, env={**os.environ, "PYTHON": sys.executable})
    assert p.returncode == 0, p.stderr[-2000:]
    assert [ln for ln in p.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = std.oracle(a)[0], std.oracle(b)[0]
    got0 = np.fromfile(out / "0.f32", "<f4").reshape(2, 96)
    got1 = np.fromfile(out / "1.f32", "<f4").reshape(1, 96)
    got2 = np.fromfile(out / "2.f32", "<f4").reshape(1, 96)
    bc.check(got0, wa[[0, 19]], "float32", "step 0")
    bc.check(got1, wb[[11]], "float32", "step 1")
    bc.check(got2, wa[[29]], "float32", "step 2")
    assert not (out / "3.f32").exists()


# ------------------------------------------------------------------ kernels on their own (GPU)
@pytest.mark.gpu
def test_gemm_kernels_against_torch():
    from ollama_operator_amd.ops import stack_native
    C = stack_native()
    dev = "cuda"
    g = torch.Generator(device="cpu").manual_seed(0)
    s = torch.cuda.current_stream().cuda_stream
    for f32 in (0, 1):
        T = torch.float32 if f32 else torch.bfloat16
        for M, N, K in [(1, 7, 40), (3, 130, 64), (8, 33, 13), (9, 64, 64), (70, 100, 96), (130, 257, 72), (64, 64, 50),
                        (300, 1030, 256)]:
            a = torch.randn(M, K, generator=g).to(T).to(dev)
            w = torch.randn(N, K, generator=g).to(T).to(dev)
            ref = a.double() @ w.double().T
            for mfma in (1, 0):
                C.set_gemm_mfma(mfma)
                out = torch.zeros(M, N, device=dev)
                C.gemm(dict(A=a.data_ptr(), lda=K, W=w.data_ptr(), M=M, N=N, K=K, C=out.data_ptr(), ldc=N, epi=0, f32=f32), s)
                torch.cuda.synchronize()
                err = float((out.double() - ref).abs().max() / ref.abs().max())
                assert err < 1e-5, f"gemm {M}x{N}x{K} f32={f32} path {C.gemm_path(M, N, K, f32)}: {err}"
            C.set_gemm_mfma(1)
            # residual and capped epilogues
            res = torch.randn(M, N, generator=g).to(dev)
            add = torch.randn(M, N, generator=g).to(dev)
            out = res.clone()
            C.gemm(dict(A=a.data_ptr(), lda=K, W=w.data_ptr(), M=M, N=N, K=K, C=out.data_ptr(), ldc=N, epi=1, mult=0.5,
                        add=add.data_ptr(), f32=f32), s)
            want = res.double() + 0.5 * (ref + add.double())
            assert float((out.double() - want).abs().max() / want.abs().max()) < 1e-5
            C.gemm(dict(A=a.data_ptr(), lda=K, W=w.data_ptr(), M=M, N=N, K=K, C=out.data_ptr(), ldc=N, epi=2, cap=5.0, f32=f32), s)
            want = 5.0 * torch.tanh(ref / 5.0)
            assert float((out.double() - want).abs().max()) < 1e-4


@pytest.mark.gpu
def test_gpu_matches_twin_layer_by_layer(std):
    """The HIP executor against its torch twin, residual after every layer run, both number formats."""
    toks = bc.tokens(100, 96, seed=80)
    for dtype, lim in (("float32", 1e-4), ("bfloat16", 3e-2)):
        a = bc.layer_trail(std.runner("cuda", dtype, max_batch=128), toks)
        b = bc.layer_trail(std.runner("cpu", dtype, max_batch=128), toks)
        for ri in range(len(a)):
            assert np.abs(a[ri] - b[ri]).max() < lim * np.abs(b).max(), f"{dtype}: layer run {ri}"
