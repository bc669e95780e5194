"""Revitar through the framework (loader, window rings, slot scheduler, ragged batches, generate loop) against the plain float64
statement of the design in tests/revitar_oracle.py.  Every scenario runs on the CPU (the modules' torch graph: cache, slot and
batching logic) and, marked gpu, on the HIP kernels of libgbx_mixers.so.  Configurations and weights are made here; sizes differ
between layers of one model and include the corners: one kv head per query head, a single expert choice, all experts chosen, a
window longer than any sequence, a window of 1, no soft cap, no feed-forward, multipliers of 1."""
import math

import pytest
import torch

import revitar_oracle as O
from gbx_lm_amd.batching import BatchScheduler, StepBatch
from gbx_lm_amd.utils import generate_step, load_model

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
# worst row's rms difference relative to the reference row's rms
TOL = {torch.float32: 2e-5, torch.bfloat16: 4e-2}
# the same arithmetic through another schedule: fp32 sums are reordered at most
SAME = {torch.float32: 1e-5, torch.bfloat16: 4e-2}

MIXED = O.make_config([
    O.attention_layer(4, 2, 32, 32, window=5, mlp=O.moe(5, 2, 32)),
    O.attention_layer(2, 2, 16, 48, window=300, softcap=None, mlp=None),                 # one kv head per head, window > sequence
    O.attention_layer(4, 1, 64, 64, window=17, scale=0.21, softcap=3.0, mlp=O.moe(3, 1, 48)),
    O.attention_layer(3, 1, 20, 7, window=1, mlp=O.moe(4, 4, 16)),                        # sees itself only; every expert chosen; odd sizes
], vocab=61, width=64, residual_mult=0.5, embed_scale=2.0)
PLAIN = O.make_config([
    O.attention_layer(2, 1, 64, 128, window=130, mlp=O.moe(8, 2, 64)),                    # a window that ends inside a second query tile
    O.attention_layer(8, 2, 32, 32, window=33, mlp=None),
    O.attention_layer(6, 3, 12, 10, window=9, mlp=O.moe(3, 2, 20)),                       # nothing a multiple of 8
], vocab=40, width=136, eps=1e-6, residual_mult=1.0, embed_scale=1.0)


@pytest.fixture(scope="module")
def checkpoints(tmp_path_factory):
    out = {}
    for name, cfg, seed in (("mixed", MIXED, 3), ("plain", PLAIN, 5)):
        for wide in (False, True):             # bf16 runs use the checkpoint whose router margins are wide by construction
            w = O.make_weights(cfg, seed, wide_margins=wide)
            key = name + ("_wide" if wide else "")
            out[key] = (O.save_checkpoint(str(tmp_path_factory.mktemp(key)), cfg, w), cfg, w)
    return out


def pick(name, dtype):
    return name + ("_wide" if dtype == torch.bfloat16 else "")


_loaded = {}


def model_for(checkpoints, name, device, dtype):
    key = (name, device, dtype)
    if key not in _loaded:
        _loaded[key] = load_model(checkpoints[name][0], device=device, dtype=dtype)[0]
    return _loaded[key]


_memo = {}


def oracle_logits(cfg, w, toks):
    key = (id(w), tuple(toks))
    if key not in _memo:
        _memo[key] = O.forward(toks, cfg, w)
    return _memo[key]


def tokens_for(cfg, n, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, cfg["vocab"], (n,), generator=g).tolist()


def all_places(n):
    return list(range(n))


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("mixed", 40), ("plain", 150)])
def test_whole_prompt_and_layers(checkpoints, device, dtype, name, n):
    name = pick(name, dtype)
    _, cfg, w = checkpoints[name]
    model = model_for(checkpoints, name, device, dtype)
    toks = tokens_for(cfg, n, 1)
    streams = []
    want = O.forward(toks, cfg, w, streams)
    model.trace_layers = []
    try:
        got = BatchScheduler(model).step([("a", toks)], [all_places(n)])
        layers = list(model.trace_layers)
    finally:
        model.trace_layers = None
    for i, (x, ref) in enumerate(zip(layers, streams)):
        assert O.rel_err(x, ref) < TOL[dtype], f"stream after layer {i}"
    assert O.rel_err(got, want) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_prefill_then_token_by_token(checkpoints, device, dtype):
    """Most of a prompt in one step, the rest one token a step through the rings: windows of 5 and 17 pass over decoded tokens, the
    window of 300 never fills; 60 decode steps."""
    _, cfg, w = checkpoints[pick("mixed", dtype)]
    model = model_for(checkpoints, pick("mixed", dtype), device, dtype)
    toks = tokens_for(cfg, 90, 2)
    want = oracle_logits(cfg, w, toks)
    eng = BatchScheduler(model)
    got = [eng.step([("a", toks[:30])], [all_places(30)])]
    for t in toks[30:]:
        got.append(eng.step([("a", [t])]))
    assert O.rel_err(torch.cat(got), want) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("portion", [2, 3, 16, 64])
def test_portions(checkpoints, device, dtype, portion):
    """A prompt cut into portions of one size (down to two tokens): the portion's first tokens read the ring, its later ones the
    portion itself; a portion longer than a window overwrites ring rows its own first queries still needed."""
    _, cfg, w = checkpoints[pick("mixed", dtype)]
    model = model_for(checkpoints, pick("mixed", dtype), device, dtype)
    toks = tokens_for(cfg, 75, 4)
    want = oracle_logits(cfg, w, toks)
    eng, got = BatchScheduler(model), []
    for lo in range(0, len(toks), portion):
        part = toks[lo:lo + portion]
        got.append(eng.step([("a", part)], [all_places(len(part))]))
    assert O.rel_err(torch.cat(got), want) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "plain"])
def test_unequal_batch_against_each_alone(checkpoints, device, dtype, name):
    """Requests of 1, 7, 33 and 140 tokens start together and are decoded together; the short ones leave first.  Every row must
    agree with the oracle and with the same request run alone."""
    name = pick(name, dtype)
    _, cfg, w = checkpoints[name]
    model = model_for(checkpoints, name, device, dtype)
    lens, extra = [1, 7, 33, 140], [3, 12, 6, 9]
    seqs = [tokens_for(cfg, n + e, 10 + i) for i, (n, e) in enumerate(zip(lens, extra))]
    eng = BatchScheduler(model)
    got = {i: [] for i in range(4)}
    out = eng.step([(i, seqs[i][:lens[i]]) for i in range(4)], [all_places(lens[i]) for i in range(4)])
    r0 = 0
    for i in range(4):
        got[i].append(out[r0:r0 + lens[i]])
        r0 += lens[i]
    for step in range(max(extra)):
        live = [i for i in range(4) if step < extra[i]]
        out = eng.step([(i, [seqs[i][lens[i] + step]]) for i in live])
        for r, i in enumerate(live):
            got[i].append(out[r:r + 1])
        for i in live:
            if step == extra[i] - 1:
                eng.release(i)
    assert eng.slots.live_tokens() == 0
    for i in range(4):
        mine = torch.cat(got[i])
        assert O.rel_err(mine, oracle_logits(cfg, w, seqs[i])) < TOL[dtype], f"request {i} against the oracle"
        alone = BatchScheduler(model).step([("x", seqs[i])], [all_places(len(seqs[i]))])
        assert O.rel_err(mine, alone) < SAME[dtype], f"request {i} in the batch against itself alone"


@pytest.mark.parametrize("device", DEVICES)
def test_slots_are_reused(checkpoints, device):
    """A finished request's slot goes to the next one; what the old owner left in the rings must not reach the new one (its first
    tokens see only themselves), also while a neighbour keeps decoding."""
    _, cfg, w = checkpoints["mixed"]
    model = model_for(checkpoints, "mixed", device, torch.float32)
    a, b, c = tokens_for(cfg, 50, 20), tokens_for(cfg, 64, 21), tokens_for(cfg, 9, 22)
    eng = BatchScheduler(model)
    eng.step([("a", a), ("b", b[:40])])
    slot_a = eng.slot_of["a"]
    eng.release("a")
    out = eng.step([("b", b[40:41]), ("c", c[:4])], [[0], all_places(4)])
    assert eng.slot_of["c"] == slot_a
    got_c = [out[1:]]
    got_b = [out[:1]]
    for i in range(4, 9):
        out = eng.step([("c", [c[i]]), ("b", [b[37 + i]])])
        got_c.append(out[:1])
        got_b.append(out[1:])
    assert O.rel_err(torch.cat(got_c), O.forward(c, cfg, w)) < TOL[torch.float32]
    assert O.rel_err(torch.cat(got_b), O.forward(b[:46], cfg, w)[40:46]) < TOL[torch.float32]
    eng.release("b"); eng.release("c")
    # more sequences than slots exist: the rings grow (and keep what they hold) while "d" is in the middle of its sequence
    d = tokens_for(cfg, 30, 23)
    others = [tokens_for(cfg, 5 + i, 24 + i) for i in range(4)]
    got_d = [eng.step([("d", d[:12])], [all_places(12)])]
    before = eng.caches[0].keys.shape[0]
    out = eng.step([("d", d[12:20])] + [(("o", i), o) for i, o in enumerate(others)], [all_places(8)] + [[len(o) - 1] for o in others])
    assert eng.caches[0].keys.shape[0] > before
    got_d.append(out[:8])
    got_d.append(eng.step([("d", d[20:])], [all_places(10)]))
    assert O.rel_err(torch.cat(got_d), O.forward(d, cfg, w)) < TOL[torch.float32]
    for i, o in enumerate(others):
        assert O.rel_err(out[8 + i][None], O.forward(o, cfg, w)[-1:]) < TOL[torch.float32]
    with pytest.raises(KeyError):
        eng.release("c")
    tight = BatchScheduler(model, max_tokens=10)
    with pytest.raises(RuntimeError):
        tight.step([("z", a[:11])])


def _edge_module(device, dtype, window, heads=2, kv_heads=1, dim=32, vdim=32):
    """An attention module whose projections pass q | k | v through unchanged and whose gate is ~1 only for a key whose code
    matches the query's in both halves: a window that is one token off adds or loses a whole value row."""
    from gbx_lm_amd.models.window_attention import GatedWindowAttention
    n = heads * dim + kv_heads * (dim + vdim)
    m = GatedWindowAttention(n, heads, kv_heads, dim, vdim, window, scale=24.0 / dim, softcap=0.0, eps=1e-6)
    m.qkv.weight.copy_(torch.eye(n))
    m.o.weight.copy_(torch.eye(n, heads * vdim))
    m.gate_bias.fill_(-18.0)
    m.dist_mul.fill_(0.5)
    m.dist_rate.fill_(0.25)
    m.to(device)
    m.qkv.to(dtype)
    m.o.to(dtype)
    return m


def _edge_oracle(q, k, v, m):
    T = q.shape[0]
    qn = O.rms(q.to(O.F64), torch.ones(q.shape[1], dtype=O.F64), m.eps).view(T, m.heads, m.dim)
    kn = O.rms(k.to(O.F64), torch.ones(k.shape[1], dtype=O.F64), m.eps).view(T, m.kv_heads, m.dim)
    vv = v.to(O.F64).view(T, m.kv_heads, m.vdim)
    spec = {"mask": {"size": m.window}, "scale": m.scale, "softcap": 0.0}
    P = {"r1": m.dist_mul.tolist(), "r2": m.dist_rate.tolist(), "pb": m.gate_bias.tolist()}
    out = torch.zeros((T, m.heads, m.vdim), dtype=O.F64)
    for h in range(m.heads):
        g = h // (m.heads // m.kv_heads)
        out[:, h] = O.attention_gates(qn[:, h], kn[:, g], spec, P, h) @ vv[:, g]
    return out.reshape(T, m.heads * m.vdim)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,n,cut", [(7, 40, None), (7, 40, 25), (128, 300, None), (128, 300, 260), (129, 300, 131), (64, 200, 199)])
def test_window_edge_stands_out(device, dtype, window, n, cut):
    """Position j's key carries code j % (window + 1) as two one-hot halves; head 0 of query i asks for the code at distance
    window - 1 (the last key it sees), head 1 for the code at distance window (the first it does not see).  A full match scores +24
    against a bias of -18, a half match +12, anything else 0: head 0 returns (nearly) one value row, head 1 (nearly) nothing.
    ``cut``: rows after it are decoded one by one, so the edge is met inside a prompt's portion, across the ring, and in decoding;
    windows of 128 / 129 put it on both sides of a query tile's border."""
    heads, kv_heads, dim, vdim = 2, 1, 32, 32
    m = _edge_module(device, dtype, window, heads, kv_heads, dim, vdim)
    g = torch.Generator().manual_seed(7)

    def code(c):
        e = torch.zeros(dim)
        e[c // 16] = 1.0
        e[16 + c % 16] = 1.0
        return e

    q = torch.zeros((n, heads * dim)); k = torch.zeros((n, kv_heads * dim))
    v = torch.randn((n, kv_heads * vdim), generator=g)
    for i in range(n):
        k[i] = code(i % (window + 1))
        for h in range(heads):
            q[i, h * dim:(h + 1) * dim] = code((i - (window - 1 + h)) % (window + 1))
    h_in = torch.cat([q, k, v], dim=1).to(dtype)
    nq, nk = heads * dim, kv_heads * dim
    ref = _edge_oracle(h_in[:, :nq].float(), h_in[:, nq:nq + nk].float(), h_in[:, nq + nk:].float(), m)
    from gbx_lm_amd.models.cache import SequenceSlots
    slots = SequenceSlots(1)
    slots.length[0] = 0
    cache = m.make_cache(slots)
    steps = [(0, n)] if cut is None else [(0, cut)] + [(i, i + 1) for i in range(cut, n)]
    outs = []
    with torch.no_grad():
        for lo, hi in steps:
            batch = StepBatch.build([0], [lo], [hi - lo], device)
            outs.append(m(h_in[lo:hi].to(device), batch, cache)[:, :heads * vdim])
            slots.length[0] = hi
    got = torch.cat(outs).float().cpu()
    err = (got.to(O.F64) - ref).abs().max().item()
    assert err < (1e-4 if dtype == torch.float32 else 3e-2), err
    assert ref[window:, :vdim].abs().max() > 0.5 and ref[:, vdim:].abs().max() < 0.05     # the scenario is what it claims to be


@pytest.mark.parametrize("device", DEVICES)
def test_router_mechanism(device):
    """Top-k of the softmax over all experts, ties to the lower index, weights not renormalised (and renormalised on request)."""
    from gbx_lm_amd.models.switch_layers import DenseRoutedGLU
    for experts, top, k in ((7, 3, 48), (64, 8, 32), (2, 2, 16), (130, 1, 64)):
        m = DenseRoutedGLU(k, 16, experts, top)
        m.router.copy_(torch.randn(experts, k))
        m.router[1] = m.router[0]                                        # an exact tie between experts 0 and 1
        m = m.to(device)
        h = torch.randn(9, k)
        prob = torch.softmax(h.to(O.F64) @ m.router.cpu().to(O.F64).T, -1)
        idx, w = m.route(h.to(device))
        for t in range(h.shape[0]):
            order = sorted(range(experts), key=lambda e: (-float(prob[t, e]), e))[:top]
            assert sorted(idx[t].tolist()) == sorted(order)
            got = dict(zip(idx[t].tolist(), w[t].tolist()))
            assert all(abs(got[e] - float(prob[t, e])) < 1e-5 for e in order)
            if 0 in got or 1 in got:
                assert 0 in got                                           # of two equal experts the lower index goes first
        m.renormalize = True
        _, wn = m.route(h.to(device))
        assert torch.allclose(wn.sum(-1).cpu(), torch.ones(9), atol=1e-5)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows,k,f,experts,top", [(5, 64, 32, 6, 2), (300, 64, 96, 5, 3), (200, 160, 32, 3, 2), (40, 48, 20, 4, 1)])
def test_expert_mechanism(device, dtype, rows, k, f, experts, top):
    """Routed gated MLPs with GIVEN choices (so rounding cannot change them): few rows (one workgroup per row and choice), many rows
    (grouped products, some experts unused, one expert with more than a tile of rows), sizes off the tile grid."""
    from gbx_lm_amd.models.switch_layers import DenseRoutedGLU
    g = torch.Generator().manual_seed(rows)
    m = DenseRoutedGLU(k, f, experts, top)
    m.gate_up.copy_(torch.randn((experts, 2 * f, k), generator=g) / math.sqrt(k))
    m.down.copy_(torch.randn((experts, k, f), generator=g) / math.sqrt(f))
    m.to(device)
    m._buffers["gate_up"], m._buffers["down"] = m.gate_up.to(dtype), m.down.to(dtype)
    h = torch.randn((rows, k), generator=g).to(dtype)
    idx = torch.stack([torch.randperm(experts - 1, generator=g)[:top] for _ in range(rows)]).to(torch.int32)   # the last expert stays unused
    idx[: rows // 2, 0] = 0 if top == 1 else idx[: rows // 2, 0]
    if device == "cuda":
        from gbx_lm_amd import mixer_ops as M, _lib
        grouped = _lib.mixers().gbxm_expert_glu_grouped(rows, k, f, experts, top, _lib.GBXM_BF16 if dtype == torch.bfloat16 else _lib.GBXM_F32) == 1
        assert grouped == (dtype == torch.bfloat16 and rows * top >= 256 and k % 32 == 0 and f % 32 == 0)
        y = M.expert_glu(h.to(device), m.gate_up, m.down, idx.to(device))
    else:
        m.route = lambda _h: (idx, torch.ones((rows, top)))
        y, _ = m(h)
    gu, dn, hd = m.gate_up.cpu().to(O.F64), m.down.cpu().to(O.F64), h.to(O.F64)
    for t in range(0, rows, max(1, rows // 25)):
        for s_ in range(top):
            e = int(idx[t, s_])
            z = gu[e, :f] @ hd[t]
            ref = dn[e] @ (z / (1 + torch.exp(-z)) * (gu[e, f:] @ hd[t]))
            assert O.rel_err(y[t, s_][None], ref[None]) < (1e-5 if dtype == torch.float32 else 2e-2), (t, s_, e)


@pytest.mark.gpu
def test_prompt_portions_run_on_the_matrix_cores():
    from gbx_lm_amd import _lib
    L = _lib.mixers()
    assert L.gbxm_window_attention_tiled(64, 128, _lib.GBXM_BF16, 0) == 1 and L.gbxm_window_attention_tiled(32, 32, _lib.GBXM_BF16, 0) == 1
    assert L.gbxm_window_attention_tiled(64, 128, _lib.GBXM_BF16, 1) == 0 and L.gbxm_window_attention_tiled(64, 128, _lib.GBXM_F32, 0) == 0
    assert L.gbxm_window_attention_tiled(24, 8, _lib.GBXM_BF16, 0) == 0


@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_through_the_entry_points(checkpoints, device):
    """generate_step (the one-sequence loop) and BatchScheduler.generate (several prompts, ragged) produce the oracle's greedy
    continuation; a stop token ends one request while the others go on."""
    _, cfg, w = checkpoints["mixed"]
    model = model_for(checkpoints, "mixed", device, torch.float32)
    prompts = [tokens_for(cfg, n, 30 + n) for n in (3, 11, 26)]

    def oracle_greedy(p, n):
        seq, out = list(p), []
        for _ in range(n):
            out.append(int(torch.argmax(O.forward(seq, cfg, w)[-1])))
            seq.append(out[-1])
        return out

    want = [oracle_greedy(p, 8) for p in prompts]
    got1 = [t for t, _, _ in generate_step(torch.tensor(prompts[1]), model, max_tokens=8)]
    assert got1 == want[1]
    assert [t for t, _, _ in generate_step(torch.tensor(prompts[2]), model, max_tokens=8, prefill_step_size=7)] == want[2]
    got = BatchScheduler(model).generate(prompts, max_tokens=8)
    assert got == want
    stop = want[0][2]
    cut = BatchScheduler(model).generate(prompts, max_tokens=8, stop_tokens=[stop])
    for g, wnt in zip(cut, want):
        n = wnt.index(stop) + 1 if stop in wnt else len(wnt)
        assert g == wnt[:n]


def test_loader_reads_every_size_from_the_config(checkpoints, tmp_path):
    path, cfg, w = checkpoints["mixed"]
    model, conf = load_model(path, device="cpu")
    assert type(model).__module__.endswith("revitar") and conf["architecture"] == "Revitar"
    at = model.layers[2].mixer
    assert (at.heads, at.kv_heads, at.dim, at.vdim, at.window, at.softcap) == (4, 1, 64, 64, 17, 3.0) and abs(at.scale - 0.21) < 1e-12
    assert model.layers[1].mlp is None and model.layers[1].norm2 is None and model.layers[1].mixer.softcap == 0.0
    assert model.layers[3].mlp.top == 4 and model.layers[0].mlp.router.dtype == torch.float32
    assert (model.layers[3].mixer.dim, model.layers[3].mixer.vdim, model.layers[3].mixer.window) == (20, 7, 1)
    assert model.model.embed_tokens.weight.dtype == torch.bfloat16 and model.layers[0].norm1.weight.dtype == torch.float32
    broken = dict(w)
    del broken["l2.mix.pb"]
    with pytest.raises((KeyError, ValueError)):
        load_model(O.save_checkpoint(str(tmp_path / "broken"), cfg, broken), device="cpu")
    odd = O.make_config([{"type": "convolution", "mixer": {}, "mlp": None}])
    with pytest.raises(ValueError):
        load_model(O.save_checkpoint(str(tmp_path / "odd"), odd, {"embed": torch.zeros(1)}), device="cpu")


def test_command_line_and_samplers(checkpoints, capsys):
    """``python -m gbx_lm_amd.cli``: one prompt through generate_step, several through the scheduler; greedy output equals the
    loops' own; the temperature / top-p sampler is reproducible from its seed and never leaves the nucleus."""
    import json
    from gbx_lm_amd import cli as G
    path, cfg, w = checkpoints["mixed"]
    p1, p2 = tokens_for(cfg, 6, 70), tokens_for(cfg, 13, 71)
    ids = lambda p: ",".join(map(str, p))
    assert G.main(["--model", path, "--prompt-ids", ids(p1), "--max-tokens", "5", "--dtype", "float32"]) == 0
    one = json.loads(capsys.readouterr().out.strip().splitlines()[-1])
    assert G.main(["--model", path, "--prompt-ids", ids(p1), "--prompt-ids", ids(p2), "--max-tokens", "5", "--dtype", "float32"]) == 0
    two = [json.loads(l) for l in capsys.readouterr().out.strip().splitlines()[-2:]]
    assert one["tokens"] == two[0]["tokens"] and len(two[1]["tokens"]) == 5 and two[1]["prompt_tokens"] == 13
    lp = torch.log_softmax(torch.tensor([[4.0, 3.0, 0.0, -1.0, -9.0]]), -1).repeat(200, 1)
    s1, s2 = G.make_sampler(0.8, 0.9, seed=4)(lp), G.make_sampler(0.8, 0.9, seed=4)(lp)
    assert torch.equal(s1, s2) and set(s1.tolist()) <= {0, 1} and len(set(s1.tolist())) == 2
    assert G.make_sampler(0.0) is None
    model = model_for(checkpoints, "mixed", "cpu", torch.float32)
    sampled = BatchScheduler(model).generate([p1, p2], max_tokens=4, sampler=G.make_sampler(1.0, 0.95, seed=1))
    assert [len(o) for o in sampled] == [4, 4] and all(0 <= t < cfg["vocab"] for o in sampled for t in o)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("width", [24, 136, 4500])
def test_norm_residual_and_embedding_mechanisms(device, dtype, width):
    """The stream update x += m * N(branch) * w alone (plain branch, and top candidate rows mixed by fp32 weights), the last norm,
    the whole-segment norms of q | k rows and the scaled embedding; rows wider than one pass of a workgroup included."""
    from gbx_lm_amd.models.residual import BranchNormResidual, StreamRMSNorm
    g = torch.Generator().manual_seed(width)
    rows, top, eps, mult = 5, 3, 1e-5, 0.7
    tol = 1e-5 if dtype == torch.float32 else 1e-2
    x0 = torch.randn((rows, width), generator=g)
    w = torch.rand((width,), generator=g) + 0.5
    for mix in (None, torch.rand((rows, top), generator=g)):
        branch = torch.randn((rows, width) if mix is None else (rows, top, width), generator=g).to(dtype)
        m = BranchNormResidual(width, eps, mult)
        m.weight.copy_(w)
        m.to(device)
        x = x0.clone().to(device)
        h = m(x, branch.to(device), None if mix is None else mix.to(device), dtype)
        z = branch.to(O.F64) if mix is None else (branch.to(O.F64) * mix.to(O.F64)[..., None]).sum(1)
        ref = x0.to(O.F64) + mult * O.rms(z, w.to(O.F64), eps)
        assert O.rel_err(x, ref) < 1e-5 and h.dtype == dtype and O.rel_err(h, ref) < tol
    n = StreamRMSNorm(width, eps)
    n.weight.copy_(w)
    n.to(device)
    assert O.rel_err(n(x0.to(device), dtype), O.rms(x0.to(O.F64), w.to(O.F64), eps)) < tol
    # segment norms: q (2/3 of the row) and k (1/6) normalised each over its whole segment, v untouched
    if device == "cuda":
        from gbx_lm_amd import mixer_ops as M
        n0, n1 = 4 * (width // 6), width // 6
        qkv = torch.randn((rows, width), generator=g).to(dtype)
        w0, w1 = torch.rand((n0,), generator=g) + 0.5, torch.rand((n1,), generator=g) + 0.5
        out = qkv.clone().to(device)
        M.segment_rmsnorm_(out, n0, n1, w0.to(device), w1.to(device), eps)
        assert O.rel_err(out[:, :n0], O.rms(qkv[:, :n0].to(O.F64), w0.to(O.F64), eps)) < tol
        assert O.rel_err(out[:, n0:n0 + n1], O.rms(qkv[:, n0:n0 + n1].to(O.F64), w1.to(O.F64), eps)) < tol
        assert torch.equal(out[:, n0 + n1:].cpu(), qkv[:, n0 + n1:])
        table = torch.randn((11, width), generator=g).to(dtype)
        toks = torch.tensor([3, 0, 10, 3])
        xe, he = M.embed_scaled(table.to(device), toks.to(device), 0.37)
        assert O.rel_err(xe, table[toks].to(O.F64) * 0.37) < 1e-6 and he.dtype == dtype


@pytest.mark.gpu
def test_decode_steps_are_replayed_from_a_graph(checkpoints):
    """From its third occurrence a decode-only step of the same slots runs as one HIP-graph replay; replays (with eager prompt steps
    of other sequences between them, and the rings re-allocated once) must keep agreeing with the oracle."""
    _, cfg, w = checkpoints["mixed"]
    model = model_for(checkpoints, "mixed", "cuda", torch.float32)
    a, b = tokens_for(cfg, 40, 90), tokens_for(cfg, 12, 91)
    eng = BatchScheduler(model)
    got = [eng.step([("a", a[:10])], [all_places(10)])]
    for i in range(10, 25):
        got.append(eng.step([("a", [a[i]])]))
    assert eng._graphs and all(gr.graph is not None for gr in eng._graphs.values())
    other = eng.step([("b", b)], [all_places(len(b))])                    # a second slot: the rings grow, captured pointers are stale
    for i in range(25, 40):
        got.append(eng.step([("a", [a[i]])]))
    assert O.rel_err(torch.cat(got), O.forward(a, cfg, w)) < TOL[torch.float32]
    assert O.rel_err(other, O.forward(b, cfg, w)) < TOL[torch.float32]
