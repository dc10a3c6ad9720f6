"""Lovapel through the serving engine (loader, paged sink-window attention cache with pages per
layer run, scheduler, batching, sampling) and its mechanisms alone, against the slow oracle in
tests/lovapel_oracle.py.

The engine runs on the CPU reference ops here and on the HIP kernels in the GPU tier (same
tests, ``device`` parameter).  Configurations are small and irregular on purpose: windows that
end inside pages, rotation on part of the head, a looped span in the middle of the stack, expert
groups of several sizes with identity experts in the last group, layers without feed-forward.
"""
import json
import math

import numpy as np
import pytest
import torch
from safetensors.torch import save_file

import lovapel_oracle as oracle
from agentic_traffic_testing_amd.config import EngineConfig, LovapelConfig
from agentic_traffic_testing_amd.engine.llm_engine import LLMEngine
from agentic_traffic_testing_amd.engine.sequence import SamplingParams
from agentic_traffic_testing_amd.models.lovapel import LovapelModel
from agentic_traffic_testing_amd.ops import mixers as mx

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]

ATT = {"heads": 4, "kv_heads": 2, "dim": 32, "vdim": 24, "scale": 0.21, "mask": {"size": 21},
       "rot": {"dims": 12, "base": 3000.0}}
MOE = {"kind": "moe", "expert": {"ff": 24},
       "router": {"experts": 7, "identity": 2, "top": 3, "groups": {"count": 3, "keep": 2}},
       "shared": {"ff": 20}}


def make_cfg(order="ded-", width=48, vocab=97, att=None, moe=None, ff=40, loop=(1, 3, 2),
             scale=0.4, cap=9.0):
    """One letter per layer for its feed-forward: d dense, e experts, - none."""
    layers = []
    for ch in order:
        mlp = {"d": {"kind": "dense", "ff": ff}, "e": dict(moe or MOE), "-": None}[ch]
        layers.append({"type": "attention", "mixer": dict(att or ATT), "mlp": mlp})
    cfg = {"architecture": "Lovapel", "vocab": vocab, "width": width, "norm": {"eps": 3e-6},
           "layers": layers, "logit_scale": scale}
    if cap:
        cfg["logit_softcap"] = cap
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_params(cfg, seed=0):
    shapes = LovapelModel(LovapelConfig.from_dict(cfg), torch.float32, "cpu").tensor_shapes()
    g = torch.Generator().manual_seed(seed)
    p = {}
    for name, shape in shapes.items():
        r = torch.randn(shape, generator=g)
        leaf = name.split(".")[-1]
        if name == "embed":
            t = r
        elif leaf.startswith("norm"):
            t = 1.1 + 0.3 * r
        elif leaf == "sink":
            t = 1.5 * r
        elif leaf == "correction":
            t = 0.08 * r          # the order of the scores of about 1 / experts changes with it
        elif leaf == "router":
            t = r * (6.0 / math.sqrt(shape[-1]))
        else:
            t = r * (1.5 / math.sqrt(shape[-1]))
        p[name] = t.to(torch.bfloat16).contiguous()
    return p


@pytest.fixture(scope="module")
def model_dir(tmp_path_factory):
    made = {}

    def get(key="default", **kw):
        if key not in made:
            d = tmp_path_factory.mktemp("lovapel_" + key)
            cfg = make_cfg(**kw)
            params = make_params(cfg, seed=len(made))
            (d / "config.json").write_text(json.dumps(cfg))
            save_file(params, str(d / "model.safetensors"))
            made[key] = (str(d), cfg, params)
        return made[key]

    return get


def engine(path, device, dtype="float32", pool_tokens=512, max_seqs=4, block_size=16):
    cfg = EngineConfig(model=path, device=device, dtype=dtype, block_size=block_size,
                       max_model_len=pool_tokens, max_num_seqs=max_seqs,
                       max_num_batched_tokens=max(512, pool_tokens),
                       num_kv_blocks=pool_tokens // block_size, use_graphs=False,
                       async_decode=False, startup_warmup=False, gemm_tuning="")
    return LLMEngine(cfg)


def close(got, want, dtype="float32"):
    got, want = np.asarray(got, dtype=np.float64), np.asarray(want, dtype=np.float64)
    d = got - want
    d = d - d.mean(-1, keepdims=True)
    err = np.sqrt((d ** 2).mean(-1)) / max(1e-9, float(np.sqrt((want ** 2).mean())))
    if dtype != "float32":   # bf16 rounding: small on average, a few times that at single rows
        assert err.mean() < 2e-2, f"mean relative logit error {err.mean():.3g}"
    lim = 2e-4 if dtype == "float32" else 0.12
    assert err.max() < lim, f"relative logit error {err.max():.3g} at row {int(err.argmax())}"


def replay(eng, rid, toks, cuts):
    """Feed ``toks`` of request ``rid`` in portions of the sizes ``cuts`` (cycled); all logits."""
    out, i, k = [], 0, 0
    while i < len(toks):
        n = min(cuts[k % len(cuts)], len(toks) - i)
        out.append(eng.replay_step([(rid, toks[i:i + n], list(range(n)))]))
        i += n
        k += 1
    return np.concatenate(out)


def tokens(n, vocab, seed):
    return np.random.default_rng(seed).integers(0, vocab, n).tolist()


def want_logits(cfg, params, toks, layers=None):
    return oracle.forward(cfg, params, toks, layers).numpy()


def decided_rows(cfg, params, toks, gap=0.02):
    """Rows whose routing is no close call in any layer run: 16-bit rounding of a router's input
    can choose another expert where two scores nearly tie, which is no fault of the engine."""
    margins = []
    oracle.forward(cfg, params, toks, None, margins)
    per_row = np.asarray(margins).reshape(-1, len(toks)) if margins else np.ones((1, len(toks)))
    keep = (per_row > gap).all(0)
    assert keep.mean() > 0.3
    return keep


# ---- whole prompts, decoding, portions ----------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_whole_prompt_matches_oracle(model_dir, device):
    path, cfg, params = model_dir()
    toks = tokens(75, cfg["vocab"], 1)
    layers = []
    want = want_logits(cfg, params, toks, layers)
    eng = engine(path, device)
    close(eng.replay_step([("a", toks, list(range(len(toks))))]), want)
    eng.finish_request("a")
    # the residual stream after every layer run (the looped span counts every pass)
    from agentic_traffic_testing_amd.engine.scheduler import Batch
    from agentic_traffic_testing_amd.engine.sequence import Sequence

    seq = Sequence("b", toks, SamplingParams())
    assert eng.scheduler.admit(seq, len(toks))
    lo = []
    eng.runner.execute_logits(Batch([seq], [0], [len(toks)], 0), [0], layer_out=lo)
    assert len(lo) == len(layers) == 6
    for i, x in enumerate(lo):
        assert torch.allclose(x.cpu().double(), layers[i], atol=3e-3, rtol=3e-4), i


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("order", ["-", "d", "e"])
def test_each_mechanism_alone(model_dir, device, order):
    """One-layer models without a loop: the mixer alone, then with each kind of feed-forward."""
    path, cfg, params = model_dir("only_" + order, order=order, loop=None)
    toks = tokens(45, cfg["vocab"], 7)
    close(replay(engine(path, device), "a", toks, [28, 1, 1, 2, 6]), want_logits(cfg, params, toks))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_prefill_then_token_by_token(model_dir, device, dtype):
    """The window (21 keys) passes over the border between the prompt and the decoded tokens."""
    path, cfg, params = model_dir()
    toks = tokens(90, cfg["vocab"], 2)
    got = replay(engine(path, device, dtype), "a", toks, [37] + [1] * 60)
    keep = decided_rows(cfg, params, toks) if dtype != "float32" else slice(None)
    close(got[keep], want_logits(cfg, params, toks)[keep], dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("cuts", [[2], [3, 2, 17, 1, 2, 5], [16, 15, 1, 33], [1], [21, 22, 20]])
def test_portions_of_any_size(model_dir, device, cuts):
    path, cfg, params = model_dir()
    toks = tokens(70, cfg["vocab"], 3)
    close(replay(engine(path, device), "a", toks, cuts), want_logits(cfg, params, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding(model_dir, device):
    """Hundreds of single-token steps: the window leaves whole pages and decode partitions
    behind in every pass of the loop."""
    path, cfg, params = model_dir("long", order="de", loop=(0, 2, 2),
                                  att=dict(ATT, mask={"size": 150}))
    toks = tokens(330, cfg["vocab"], 4)
    close(replay(engine(path, device), "a", toks, [3] + [1] * 400), want_logits(cfg, params, toks))


@pytest.mark.parametrize("device", DEVICES)
def test_other_sizes(model_dir, device):
    """Values a model may happen to make equal or 1: one key / value head and as many as query
    heads; rotation of the whole head and none; no window and a window of one key; one group and
    groups of one expert; every route chosen and a single one; no identity experts, no shared
    expert; only identity experts besides one; no loop, a loop over everything, a loop that
    runs once; no soft cap; widths that are not multiples of 8, odd head widths."""
    variants = {
        "one": dict(order="-e-", width=40, loop=(0, 3, 3), cap=0.0, scale=1.0,
                    att={"heads": 3, "kv_heads": 1, "dim": 16, "vdim": 16, "scale": 0.3,
                         "rot": {"dims": 16, "base": 100.0}},
                    moe={"kind": "moe", "expert": {"ff": 16},
                         "router": {"experts": 3, "top": 3}}),
        "mha": dict(order="ded", width=36, ff=20, loop=None,
                    att={"heads": 3, "kv_heads": 3, "dim": 10, "vdim": 14, "scale": 0.5,
                         "mask": {"size": 1}},
                    moe={"kind": "moe", "expert": {"ff": 9},
                         "router": {"experts": 5, "identity": 1, "top": 1,
                                    "groups": {"count": 6, "keep": 2}}}),
        "ident": dict(order="e", width=32, loop=(0, 1, 1),
                      att={"heads": 2, "kv_heads": 1, "dim": 8, "vdim": 8, "scale": 0.4,
                           "mask": {"size": 5}, "rot": {"dims": 4, "base": 10.0}},
                      moe={"kind": "moe", "expert": {"ff": 12},
                           "router": {"experts": 1, "identity": 3, "top": 2,
                                      "groups": {"count": 2, "keep": 1}},
                           "shared": {"ff": 7}}),
        "odd": dict(order="d", width=30, ff=11, loop=None,
                    att={"heads": 2, "kv_heads": 1, "dim": 9, "vdim": 5, "scale": 0.3,
                         "mask": {"size": 40}, "rot": {"dims": 4, "base": 50.0}}),
        "wide": dict(order="ed", width=64, ff=72, loop=(1, 2, 2),
                     att={"heads": 8, "kv_heads": 2, "dim": 64, "vdim": 64, "scale": 0.11,
                          "mask": {"size": 64}, "rot": {"dims": 64, "base": 15000.0}},
                     moe={"kind": "moe", "expert": {"ff": 32},
                          "router": {"experts": 6, "identity": 2, "top": 2,
                                     "groups": {"count": 4, "keep": 3}},
                          "shared": {"ff": 48}}),
    }
    for key, kw in variants.items():
        path, cfg, params = model_dir(key, **kw)
        toks = tokens(83, cfg["vocab"], 5)
        close(replay(engine(path, device), "a", toks, [65, 1, 1, 2, 7]),
              want_logits(cfg, params, toks))


@pytest.mark.gpu
def test_matrix_core_paths_in_bfloat16(model_dir):
    """bf16 on the GPU with widths the matrix-core attention and expert kernels take."""
    path, cfg, params = model_dir("wide")  # made above (or here, with defaults that differ)
    toks = tokens(200, cfg["vocab"], 6)
    got = replay(engine(path, "cuda", "bfloat16"), "a", toks, [130, 3] + [1] * 80)
    keep = decided_rows(cfg, params, toks)
    close(got[keep], want_logits(cfg, params, toks)[keep], "bfloat16")
    # a 150-key window over a 200-token portion, then decode rows whose window crosses the
    # 128- and 256-key partition borders
    path, cfg, params = model_dir("long", order="de", loop=(0, 2, 2),
                                  att=dict(ATT, mask={"size": 150}))
    toks = tokens(330, cfg["vocab"], 8)
    got = replay(engine(path, "cuda", "bfloat16"), "b", toks, [200] + [1] * 130)
    keep = decided_rows(cfg, params, toks)
    close(got[keep], want_logits(cfg, params, toks)[keep], "bfloat16")


# ---- batches and pages ----------------------------------------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_mixed_batches_equal_each_alone(model_dir, device):
    path, cfg, params = model_dir()
    V = cfg["vocab"]
    reqs = {"a": tokens(61, V, 10), "b": tokens(1, V, 11), "c": tokens(34, V, 12),
            "d": tokens(50, V, 13), "e": tokens(23, V, 14)}
    want = {k: want_logits(cfg, params, t) for k, t in reqs.items()}
    # four live requests at most; 'e' arrives after 'b' and 'c' ended and reuses a slot and
    # pages (the pool holds 10 pages of 16 tokens: everything is used again)
    plan = [[("a", 17), ("b", 1)], [("a", 2), ("c", 30), ("d", 1)], [("a", 1), ("c", 1), ("d", 16)],
            [("a", 1), ("c", 3), ("d", 2), ("e", 5)], [("a", 40), ("d", 31), ("e", 1)],
            [("e", 17)]]
    ends = {0: ["b"], 3: ["c"], 4: ["a", "d"], 5: ["e"]}
    eng = engine(path, device, pool_tokens=160, max_seqs=4)
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    for i, step in enumerate(plan):
        portions = []
        for rid, n in step:
            portions.append((rid, reqs[rid][at[rid]:at[rid] + n], list(range(n))))
            at[rid] += n
        out = eng.replay_step(portions)
        r = 0
        for rid, n in step:
            got[rid].append(out[r:r + n])
            r += n
        for rid in ends.get(i, []):
            eng.finish_request(rid)
    assert eng.runner.bm.num_free_state_slots() == 4
    assert eng.runner.bm.num_free_blocks() == 10
    for k in reqs:
        assert at[k] == len(reqs[k])
        close(np.concatenate(got[k]), want[k])


@pytest.mark.parametrize("device", DEVICES)
def test_freed_pages_start_clean(model_dir, device):
    """One slot, pages for one request: the next request inherits the pages with the keys of the
    one before still in them, in every pass of the loop."""
    path, cfg, params = model_dir()
    eng = engine(path, device, pool_tokens=64, max_seqs=1)
    for seed, n, cuts in ((20, 60, [60]), (21, 7, [1, 1, 5]), (22, 33, [2, 31]), (23, 1, [1])):
        toks = tokens(n, cfg["vocab"], seed)
        got = replay(eng, f"r{seed}", toks, cuts)
        eng.finish_request(f"r{seed}")
        close(got, want_logits(cfg, params, toks))


def test_cache_layout(model_dir):
    """A layer inside the looped span owns pages per pass; nothing else is kept per sequence."""
    path, cfg, _ = model_dir()
    eng = engine(path, "cpu")
    layers = eng.runner.cache.layers
    assert len(layers) == 6 and eng.model_cfg.runs == (0, 1, 2, 1, 2, 3)
    ptrs = {lc.k.data_ptr() for lc in layers} | {lc.v.data_ptr() for lc in layers}
    assert len(ptrs) == 12
    for lc in layers:
        assert lc.k.shape[1:] == (ATT["kv_heads"], 16, ATT["dim"])
        assert lc.v.shape[1:] == (ATT["kv_heads"], ATT["vdim"], 16)
        assert lc.state is None and lc.conv is None and lc.shift is None


# ---- generation through the engine's own entry point ----------------------------------------
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation(model_dir, device):
    path, cfg, params = model_dir()
    prompts = [tokens(19, cfg["vocab"], 30), tokens(3, cfg["vocab"], 31), tokens(33, cfg["vocab"], 32)]
    eng = engine(path, device)
    sp = SamplingParams(temperature=0.0, max_tokens=12, ignore_eos=True)
    outs = eng.generate(prompts, sp)
    for p, o in zip(prompts, outs):
        ids = list(p)
        for tok in o.token_ids:
            lg = oracle.forward(cfg, params, ids)[-1]
            top2 = torch.topk(lg, 2).values
            if float(top2[0] - top2[1]) > 1e-3:   # skip numerically tied steps
                assert tok == int(lg.argmax())
            ids.append(tok)
        assert len(o.token_ids) == 12
    assert eng.runner.bm.num_free_state_slots() == eng.runner.bm.num_state_slots()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
def test_graph_replayed_decode_equals_eager(model_dir, dtype):
    """Decode steps replayed from captured hipGraphs (several buckets, many replays with eager
    prefill steps between them) give the tokens of the eager engine: routing, the expert plan
    and the combine run on the device, so the routed layers are part of the graph."""
    path, cfg, params = model_dir()
    prompts = [tokens(n, cfg["vocab"], 40 + n) for n in (21, 2, 40)]
    sp = SamplingParams(temperature=0.0, max_tokens=40, ignore_eos=True)
    outs = {}
    for graphs in (False, True):
        c = EngineConfig(model=path, device="cuda", dtype=dtype, max_model_len=512,
                         max_num_seqs=4, max_num_batched_tokens=512, num_kv_blocks=64,
                         use_graphs=graphs, graph_batch_sizes=(1, 2, 4), startup_warmup=False,
                         gemm_tuning="")
        eng = LLMEngine(c)
        first = eng.generate(prompts, sp)
        again = eng.generate(prompts[:2], sp)          # pages reused, graphs replayed
        outs[graphs] = [o.token_ids for o in first + again]
        assert (eng.runner.graph_steps > 0) == graphs
    if dtype == "float32":
        assert outs[True] == outs[False]
    assert outs[True][:2] == outs[True][3:]            # same prompts, same tokens the second time


def test_registry_and_config_reader(model_dir):
    path, cfg, _ = model_dir()
    eng = engine(path, "cpu")
    assert type(eng.runner.model).__name__ == "LovapelModel"
    mc = eng.model_cfg
    assert mc.hidden_size == cfg["width"] and mc.vocab_size == cfg["vocab"]
    assert mc.norm_eps == 3e-6 and mc.logit_scale == 0.4 and mc.logit_softcap == 9.0
    assert (mc.loop_start, mc.loop_stop, mc.loop_times) == (1, 3, 2) and mc.num_layers == 6
    a = mc.layers[0].mixer
    assert (a.heads, a.kv_heads, a.dim, a.vdim, a.window, a.rot_dims) == (4, 2, 32, 24, 21, 12)
    assert a.rot_base == 3000.0 and a.scale == 0.21
    assert mc.layers[0].ff == 40 and mc.layers[0].moe is None and mc.layers[3].ff == 0
    m = mc.layers[1].moe
    assert (m.experts, m.identity, m.top, m.ff, m.groups, m.keep, m.shared_ff) == \
        (7, 2, 3, 24, 3, 2, 20) and mc.layers[1].ff == 0
    plain = LovapelConfig.from_dict(make_cfg(order="e", loop=None, cap=0.0, moe={
        "kind": "moe", "expert": {"ff": 8}, "router": {"experts": 4, "top": 2}}))
    assert plain.runs == (0,) and plain.logit_softcap == 0.0
    m = plain.layers[0].moe
    assert (m.identity, m.groups, m.keep, m.shared_ff) == (0, 1, 1, 0)
    for path_, value in ((("layers", 1, "mlp", "router", "top"), 7),           # > kept experts
                         (("layers", 1, "mlp", "router", "groups", "count"), 4),   # 9 % 4
                         (("layers", 0, "mixer", "kv_heads"), 3),
                         (("layers", 0, "mixer", "rot", "dims"), 34),
                         (("loop", "stop"), 5)):
        bad = json.loads(json.dumps(cfg))
        node = bad
        for k in path_[:-1]:
            node = node[k]
        node[path_[-1]] = value
        with pytest.raises(ValueError):
            LovapelConfig.from_dict(bad)


@pytest.mark.parametrize("device", DEVICES)
def test_preempted_sequence_recomputes(model_dir, device):
    path, cfg, _ = model_dir()
    prompts = [tokens(20, cfg["vocab"], 70), tokens(18, cfg["vocab"], 71)]
    sp = SamplingParams(temperature=0.0, max_tokens=30, ignore_eos=True)
    want = [o.token_ids for o in engine(path, device, pool_tokens=512).generate(prompts, sp)]
    small = engine(path, device, pool_tokens=80, max_seqs=2)
    got = [o.token_ids for o in small.generate(prompts, sp)]
    assert small.scheduler.num_preemptions > 0
    assert got == want


def test_trace_replay_command_line(model_dir, tmp_path):
    import os
    import subprocess
    import sys

    path, cfg, params = model_dir()
    V = cfg["vocab"]
    a, b = tokens(30, V, 50), tokens(9, V, 51)
    steps = [
        {"step": 0, "entries": [{"id": "a", "tokens": a[:11], "want": [0, 10]}], "end": []},
        {"step": 1, "entries": [{"id": "b", "tokens": b[:8], "want": [7]},
                                {"id": "a", "tokens": a[11:12], "want": [0]}], "end": []},
        {"step": 2, "entries": [{"id": "b", "tokens": b[8:], "want": []}], "end": ["b"]},
        {"step": 3, "entries": [{"id": "a", "tokens": a[12:], "want": [17]}], "end": ["a"]},
    ]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    r = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path,
                        "--dtype", "float32", "--out", str(out), "--max-tokens", "128",
                        "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", text=True,
                       capture_output=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == \
        [f"done {i}" for i in range(4)]
    wa, wb = want_logits(cfg, params, a), want_logits(cfg, params, b)
    got = {i: np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V) for i in (0, 1, 3)}
    assert not (out / "2.f32").exists()
    close(got[0], wa[[0, 10]])
    close(got[1], np.stack([wb[7], wa[11]]))
    close(got[3], wa[[29]])


# ---- mechanisms alone, made so that a fault shows ---------------------------------------------
def i32(a, device):
    return torch.tensor(a, dtype=torch.int32, device=device)


def paged(k, v, bs, device, seed=0):
    """k [T, G, d], v [T, G, dv] of one sequence -> shuffled pages, block table [1, n]."""
    T, G, d = k.shape
    dv = v.shape[2]
    n = (T + bs - 1) // bs
    perm = torch.randperm(n + 3, generator=torch.Generator().manual_seed(seed))[:n]
    kc = torch.randn(n + 3, G, bs, d, dtype=k.dtype) * 50        # stale keys everywhere else
    vc = torch.randn(n + 3, G, dv, bs, dtype=k.dtype) * 50
    for j in range(T):
        kc[perm[j // bs], :, j % bs] = k[j]
        vc[perm[j // bs], :, :, j % bs] = v[j]
    return kc.to(device), vc.to(device), perm.to(torch.int32).view(1, n).to(device)


def attend(q, kc, vc, bt, T, n, window, scale, sink, device, decode=False):
    """The last ``n`` rows of a sequence of T cached tokens as one portion (or one decode row)."""
    H = q.shape[1]
    nt = 0 if decode else (n + mx.ATTN_TILE_TOKENS - 1) // mx.ATTN_TILE_TOKENS
    return mx.sink_attention(
        q.to(device), kc, vc, bt, i32([T], device), i32([0, n], device),
        i32([0] * nt, device), i32([j * mx.ATTN_TILE_TOKENS for j in range(nt)], device), scale,
        True, 1 if decode else 0, T if decode else 0,
        sink_values=sink.to(device), window=window).cpu().view(n, H, -1)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", [torch.float32, pytest.param(torch.bfloat16, marks=pytest.mark.gpu)])
@pytest.mark.parametrize("T,window", [(300, 75), (129, 128), (200, 17), (64, 200), (700, 0),
                                      (700, 690)])
def test_window_edge_and_sink(device, dtype, T, window):
    """One key stands out by its score: it decides the output while it is the oldest key of the
    window and is gone one row later, in prompts and in decoding, across page and partition
    borders.  The sink's share of the denominator is checked through the output's size."""
    if dtype == torch.bfloat16 and device == "cpu":
        pytest.skip("bf16 attention is checked on the GPU kernels")
    g = torch.Generator().manual_seed(T + window)
    H, G, d, dv, bs = 4, 2, 32, 32, 16
    k = 0.05 * torch.randn(T, G, d, generator=g)
    v = torch.randn(T, G, dv, generator=g)
    q = 0.05 * torch.randn(T, H, d, generator=g)
    # the marked key: three rows before the last window begins; with no window or a long one it
    # lies hundreds of keys back, on the first page
    j = max(0, T - window - 3) if 0 < window < 600 else 5
    k[j] = 0.0
    k[j, :, 0] = 9.0
    q[:, :, 0] = 3.0                                # score 27 against the marked key, ~0 otherwise
    v[j] = 100.0
    sink = torch.tensor([-30.0, 0.0, 27.0, 3.0])    # head 2: the sink weighs as much as the key
    k, v, q = k.to(dtype), v.to(dtype), q.to(dtype)
    kc, vc, bt = paged(k, v, bs, device)
    want = oracle.sink_window_attention(q.double(), k.double(), v.double(), 1.0, window,
                                        sink.double())
    n = min(T, 90)
    got = attend(q[T - n:], kc, vc, bt, T, n, window, 1.0, sink, device)
    tol = dict(atol=2e-3, rtol=2e-3) if dtype == torch.float32 else dict(atol=0.6, rtol=3e-2)
    assert torch.allclose(got.double(), want[T - n:], **tol)
    last_in = j + window - 1 if window else T - 1   # the last row that still sees the marked key
    if last_in < T:
        assert got[last_in - (T - n), 1].mean() > 90 and got[last_in - (T - n), 2].mean() < 60
        if last_in + 1 < T:
            assert got[last_in + 1 - (T - n)].abs().mean() < 5
    # the same rows decoded alone, each against the cache as it was at its step
    for row in {last_in, last_in + 1, T - 1}:
        if 0 <= row < T:
            one = attend(q[row:row + 1], kc, vc, bt, row + 1, 1, window, 1.0, sink, device, True)
            assert torch.allclose(one[0].double(), want[row], **tol), row


@pytest.mark.parametrize("device", DEVICES)
def test_whole_projection_norm_and_partial_rotation(device):
    """The norm runs over all heads at once (one head is made large: a per-head norm would hide
    it), with one weight per row of the projection; only the leading channels turn."""
    g = torch.Generator().manual_seed(5)
    T, H, G, d, dv, bs, rd = 9, 3, 1, 16, 8, 4, 6
    qx, kx, vx = (torch.randn(T, n, generator=g) for n in (H * d, G * d, G * dv))
    qx[:, :d] *= 30.0
    qw, kw = torch.rand(H * d, generator=g) + 0.5, torch.rand(G * d, generator=g) + 0.5
    pos = torch.tensor([0, 1, 2, 3, 4, 1000, 1001, 50000, 50001], dtype=torch.int32)
    slots = torch.arange(T, dtype=torch.int32)
    kc = torch.zeros(3, G, bs, d)
    vc = torch.zeros(3, G, dv, bs)
    dev = torch.device(device)
    tab = mx.rotary_table(pos.to(dev), mx.inv_freq(rd, 777.0, dev))
    kc_d, vc_d = kc.to(dev), vc.to(dev)
    q = mx.qk_norm_rope_cache(qx.to(dev), kx.to(dev), vx.to(dev), qw.to(dev), kw.to(dev), 1e-5,
                              pos.to(dev), slots.to(dev), tab, kc_d, vc_d, H, G, d, dv,
                              rotate_half_pairs=True, whole_norm=True).cpu()
    wq = oracle.rotate(oracle.rms_norm(qx.double(), qw, 1e-5).view(T, H, d), pos, rd, 777.0)
    wk = oracle.rotate(oracle.rms_norm(kx.double(), kw, 1e-5).view(T, G, d), pos, rd, 777.0)
    assert torch.allclose(q.double(), wq, atol=2e-3, rtol=1e-4)   # angles of 50000 rad in fp32
    got_k = kc_d.cpu().permute(0, 2, 1, 3).reshape(-1, G, d)[:T]
    assert torch.allclose(got_k.double(), wk, atol=2e-3, rtol=1e-4)
    plain = oracle.rms_norm(qx.double(), qw, 1e-5).view(T, H, d)
    assert torch.allclose(q[..., rd:].double(), plain[..., rd:], atol=1e-5, rtol=1e-5)
    assert not torch.allclose(q[5:, :, :rd].double(), plain[5:, :, :rd], atol=1e-2)
    got_v = vc_d.cpu().permute(0, 3, 1, 2).reshape(-1, G, dv)[:T]
    assert torch.equal(got_v, vx.view(T, G, dv))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("W", [48, 250, 4096, 33000])
def test_sandwich_norm_boundary(device, W):
    """Mean and variance matter: rows with a large common offset, where an RMS norm (no mean) or
    a one-pass variance would be far off; widths for the vector and the plain kernel."""
    g = torch.Generator().manual_seed(W)
    T = 5
    x = torch.randn(T, W, generator=g) + 40.0
    y = 3.0 * torch.randn(T, W, generator=g) - 700.0
    wp, wn = torch.rand(W, generator=g) + 0.5, torch.rand(W, generator=g) + 0.5
    dev = torch.device(device)
    xd = x.clone().to(dev)
    h = mx.norm_add_norm(xd, y.to(dev), wp.to(dev), wn.to(dev), 1e-5, "layer", torch.float32)
    wx = x.double() + oracle.layer_norm(y.double(), wp, 1e-5)
    assert torch.allclose(xd.cpu().double(), wx, atol=1e-3, rtol=1e-5)
    assert torch.allclose(h.cpu().double(), oracle.layer_norm(wx, wn, 1e-5), atol=2e-3, rtol=1e-4)
    # the first norm of a step and the norm before the head: nothing is added
    x2 = x.clone().to(dev)
    h2 = mx.norm_add_norm(x2, None, None, wn.to(dev), 1e-5, "layer", torch.float32)
    assert torch.equal(x2.cpu(), x)
    assert torch.allclose(h2.cpu().double(), oracle.layer_norm(x.double(), wn, 1e-5), atol=2e-3,
                          rtol=1e-4)
    # the last layer: no next norm; and the RMS kind of the same boundary
    x3 = x.clone().to(dev)
    assert mx.norm_add_norm(x3, y.to(dev), wp.to(dev), None, 1e-5, "layer") is None
    assert torch.allclose(x3.cpu().double(), wx, atol=1e-3, rtol=1e-5)
    x4 = x.clone().to(dev)
    h4 = mx.norm_add_norm(x4, y.to(dev), wp.to(dev), wn.to(dev), 1e-5, "rms", torch.float32)
    w4 = x.double() + oracle.rms_norm(y.double(), wp, 1e-5)
    assert torch.allclose(x4.cpu().double(), w4, atol=1e-3, rtol=1e-5)
    assert torch.allclose(h4.cpu().double(), oracle.rms_norm(w4, wn, 1e-5), atol=2e-3, rtol=1e-4)


@pytest.mark.parametrize("device", DEVICES)
def test_router_choice_and_weights(device):
    """Logits made so that every rule decides a row.  12 routes in 4 groups of 3 neighbours, the
    2 best groups are kept, 3 routes are chosen."""
    E, groups, keep, top = 12, 4, 2, 3
    base = -4.0 - 0.05 * torch.arange(E)            # no two scores tie; lower index = larger
    plain = base.clone()
    plain[[7, 2, 10]] = torch.tensor([3.0, 2.0, 1.0])
    best = base.clone()                             # group 3 has the largest sum, not the best
    best[[4, 0, 9, 10, 11]] = torch.tensor([3.0, 2.6, 2.5, 2.4, 2.3])
    big6 = base.clone()
    big6[[6, 1, 2, 0, 9]] = torch.tensor([3.0, 1.2, 1.1, 1.0, 0.5])
    none = torch.zeros(E)
    minus6 = none.clone()
    minus6[6] = -0.9
    plus10 = none.clone()
    plus10[10] = 0.5
    cases = [
        # the third best score (route 10) lies outside the kept groups 2 and 0
        (plain, none, {7, 2, 0}),
        # a group is kept for its best route: groups 1 and 0, not group 3
        (best, none, {4, 0, 1}),
        # the correction takes route 6 (by far the largest score) out of the choice ...
        (big6, minus6, {1, 2, 0}),
        (big6, none, {6, 1, 2}),
        # ... or brings route 10 and its group in; its weight stays its small plain score
        (plain, plus10, {7, 10, 6}),
        # all choice scores negative: a route outside the kept groups still never wins
        (plain, none - 1.0, {7, 2, 0}),
    ]
    dev = torch.device(device)
    for z, corr, chosen in cases:
        rows = z.repeat(5, 1)                       # several rows per launch, one of them last
        idx, w = mx.moe_route(rows.to(dev), top, "softmax", corr.to(dev), groups, keep, renorm=True)
        idx, w = idx.cpu().long(), w.cpu().double()
        wi, ww, _ = oracle.route(z.double(), corr.double(), top, groups, keep)
        assert set(wi.tolist()) == chosen
        for t in range(rows.shape[0]):
            assert set(idx[t].tolist()) == chosen, (chosen, idx[t])
            assert torch.allclose(w[t][torch.argsort(idx[t])], ww[torch.argsort(wi)], atol=1e-6)
            assert abs(float(w[t].sum()) - 1.0) < 1e-5
    s = torch.softmax(plain.double(), 0)
    idx, w = mx.moe_route(plain.view(1, E).to(dev), top, "softmax", plus10.to(dev), groups, keep,
                          renorm=True)
    got10 = float(w.cpu()[0][idx.cpu()[0].tolist().index(10)])
    assert abs(got10 - float(s[10] / (s[7] + s[10] + s[6]))) < 1e-6 and got10 < 0.2
    # without groups, correction and renormalisation: the sigmoid scores themselves, best first
    i2, w2 = mx.moe_route(plain.view(1, E).to(dev), 2, "sigmoid")
    assert i2.cpu()[0].tolist() == [7, 2]
    assert torch.allclose(w2.cpu()[0], torch.sigmoid(torch.tensor([3.0, 2.0])), atol=1e-6)
    # one group per route, all kept; every route chosen
    i3, w3 = mx.moe_route(plain.view(1, E).to(dev), E, "softmax", None, E, E, renorm=True)
    assert sorted(i3.cpu()[0].tolist()) == list(range(E))
    assert torch.allclose(w3.cpu()[0][torch.argsort(i3.cpu()[0])].double(), s, atol=1e-6)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype,T,W,ff", [
    (torch.float32, 37, 40, 24), (torch.float32, 3, 36, 9),
    pytest.param(torch.bfloat16, 70, 64, 32, marks=pytest.mark.gpu),
    pytest.param(torch.bfloat16, 2, 64, 512, marks=pytest.mark.gpu),       # split down product
    pytest.param(torch.bfloat16, 700, 64, 64, marks=pytest.mark.gpu)])     # large tiles
def test_experts_weight_the_output_and_identity_experts(device, dtype, T, W, ff):
    """The router weight multiplies the expert's output (a SiLU GLU is not homogeneous: weighting
    the input instead gives other numbers); an identity expert returns the row itself; the
    shared expert's rows are added once."""
    if dtype == torch.bfloat16 and device == "cpu":
        pytest.skip("bf16 grouped products are checked on the GPU kernels")
    g = torch.Generator().manual_seed(T)
    E, ident, top = 5, 2, 3
    h = torch.randn(T, W, generator=g).to(dtype)
    w_gu = (torch.randn(E, 2 * ff, W, generator=g) / math.sqrt(W)).to(dtype)
    w_down = (torch.randn(E, W, ff, generator=g) / math.sqrt(ff)).to(dtype)
    idx = torch.stack([torch.randperm(E + ident, generator=g)[:top] for _ in range(T)]).int()
    wts = torch.rand(T, top, generator=g) + 0.2
    add = torch.randn(T, W, generator=g).to(dtype)
    dev = torch.device(device)
    got = mx.moe_experts(h.to(dev), idx.to(dev), wts.to(dev), w_gu.to(dev), w_down.to(dev),
                         glu="silu", addend=add.to(dev)).cpu().double()
    st = {}
    for e in range(E):
        st[f"e{e}.gate"], st[f"e{e}.up"], st[f"e{e}.down"] = w_gu[e, :ff], w_gu[e, ff:], w_down[e]
    want = add.double().clone()
    for t in range(T):
        for e, w in zip(idx[t].tolist(), wts[t].double()):
            want[t] += w * (h[t].double() if e >= E else oracle.glu(h[t].double(), st, f"e{e}.", oracle.silu))
    tol = dict(atol=2e-4, rtol=2e-4) if dtype == torch.float32 else dict(atol=0.08, rtol=3e-2)
    assert torch.allclose(got, want, **tol)


@pytest.mark.parametrize("device", DEVICES)
def test_glu_activations_and_logit_cap(device):
    g = torch.Generator().manual_seed(3)
    dev = torch.device(device)
    P = (4.0 * torch.randn(6, 48, generator=g)).to(dev)      # fused [gate | pad | up] rows
    for act, f in (("gelu_tanh", oracle.gelu_tanh), ("silu", oracle.silu)):
        got = mx.gate_mul(P[:, 24:44], P[:, :20], act).cpu().double()
        want = f(P[:, :20].cpu().double()) * P[:, 24:44].cpu().double()
        assert torch.allclose(got, want, atol=1e-5, rtol=1e-5)
    z = (30.0 * torch.randn(5, 33, generator=g)).to(dev)
    got = mx.scale_softcap(z, 0.25, 7.0).cpu().double()
    assert torch.allclose(got, 7.0 * torch.tanh(z.cpu().double() * 0.25 / 7.0), atol=1e-5)
    assert got.abs().max() <= 7.0 and got.abs().max() > 5.0
    assert torch.allclose(mx.scale_softcap(z, 0.5, 0.0).cpu(), z.cpu() * 0.5)
