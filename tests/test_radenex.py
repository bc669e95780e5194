"""Radenex through the framework (loader, slot tables, slot scheduler, ragged batches, generate loop) against the plain float64
statement of the design in tests/radenex_oracle.py.  Every scenario runs on the CPU (the modules' torch graph: cache, slot and
batching logic) and, marked gpu, on the HIP kernels of libgbx_mixers.so.  Configurations and weights are made here; sizes differ
between layers of one model and include the corners: one kv head per query head, no kept tokens, more kept tokens than the window,
a window of 1, a window longer than any sequence, rotation over a part of the head and over all of it, odd head sizes, no
feed-forward, loops of one layer and of several, no loop."""
import json
import math
import subprocess
import sys

import pytest
import torch

import radenex_oracle as O
from gbx_lm_amd.batching import BatchScheduler, StepBatch
from gbx_lm_amd.models import sink_attention as SA
from gbx_lm_amd.models.cache import SequenceSlots, SlotKVCache
from gbx_lm_amd.utils import generate_step, load_model

DEVICES = ["cpu", pytest.param("cuda", marks=pytest.mark.gpu)]
DTYPES = [torch.float32, torch.bfloat16]
TOL = {torch.float32: 2e-5, torch.bfloat16: 4e-2}      # worst row's rms difference relative to the reference row's rms
SAME = {torch.float32: 1e-5, torch.bfloat16: 4e-2}     # the same arithmetic through another schedule

YARN = {"factor": 8.0, "original": 64, "fast": 16.0, "slow": 2.0}
MIXED = O.make_config([
    O.latent_layer(4, 16, 8, 24, 32, base=5000.0, scaling=YARN, ff=96),
    O.attention_layer(4, 2, 32, 32, 16, window=7, keep_first=2, factor=2.0, ff=80),
    O.latent_layer(2, 24, 16, 16, 40, ff=None),                                           # no scaling, no feed-forward
    O.attention_layer(3, 3, 20, 10, 20, window=1, keep_first=0, base=300.0, ff=48),       # sees itself only; one kv head per head; odd sizes
    O.attention_layer(2, 1, 16, 48, 8, window=3, keep_first=9, scale=0.4, ff=None),       # more kept tokens than the window
], vocab=61, width=64, loop=(1, 3, 2))
PLAIN = O.make_config([
    O.attention_layer(2, 1, 64, 64, 32, window=130, keep_first=5, factor=4.0, ff=160),    # a window that ends inside a second query tile
    O.latent_layer(4, 32, 32, 64, 96, base=100000.0, scaling={"factor": 2.0, "original": 32, "fast": 8.0, "slow": 1.0}, ff=72),
    O.attention_layer(6, 3, 12, 10, 6, window=400, keep_first=3, ff=40),                  # nothing a multiple of 8; window > sequence
    O.latent_layer(3, 8, 4, 20, 12, ff=24),                                               # head sizes off every tile
], vocab=40, width=136, eps=1e-6, loop=(3, 4, 1))
SINGLE = O.make_config([O.latent_layer(2, 16, 16, 16, 24, ff=32), O.attention_layer(2, 2, 16, 16, 16, window=5, keep_first=1, ff=32)],
                       vocab=33, width=32, loop=(0, 2, 2))                                # the loop spans the whole stack


@pytest.fixture(scope="module")
def checkpoints(tmp_path_factory):
    out = {}
    for name, cfg, seed in (("mixed", MIXED, 3), ("plain", PLAIN, 5), ("single", SINGLE, 8)):
        w = O.make_weights(cfg, seed)
        out[name] = (O.save_checkpoint(str(tmp_path_factory.mktemp(name)), cfg, w), cfg, w)
    return out


_loaded, _memo = {}, {}


def model_for(checkpoints, name, device, dtype):
    key = (name, device, dtype)
    if key not in _loaded:
        _loaded[key] = load_model(checkpoints[name][0], device=device, dtype=dtype)[0]
    return _loaded[key]


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


# ------------------------------------------------------------------------------------------------ mechanisms alone
def test_rotary_tables():
    from gbx_lm_amd.models.rope_utils import rotary_table
    for rot in ({"base": 10000.0, "dims": 16}, {"base": 500.0, "dims": 6, "scaling": {"factor": 4.0}},
                {"base": 250000.0, "dims": 32, "scaling": {"factor": 40.0, "original": 4096, "fast": 32.0, "slow": 1.0}},
                {"base": 5000.0, "dims": 8, "scaling": YARN}):
        want, mult = O.scaled_frequencies(rot)
        got, gmult = rotary_table(rot["base"], rot["dims"], rot.get("scaling"))
        assert torch.allclose(got.double(), want, rtol=1e-6, atol=0) and abs(gmult - mult) < 1e-12
    f, _ = O.scaled_frequencies({"base": 5000.0, "dims": 8, "scaling": YARN})
    plain = O.plain_frequencies(5000.0, 8)
    assert 0.1 < float(f[-1] / plain[-1]) < 0.2 and float(f[0] / plain[0]) == 1.0          # the ramp spans both ends in this table


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_rotate_norm_heads(device, dtype):
    """Rotation of a part of each head at any offset, unit norm, weighted norm, turning back, several segments of one row."""
    g = torch.Generator().manual_seed(1)
    t, eps = 11, 1e-5
    pos = torch.tensor([0, 1, 2, 3, 900, 901, 17, 4000, 5, 6, 70000], dtype=torch.int32)
    segs = [(0, 3, 24, 8, 16, 1.3, 1.0, SA.NORM_NONE), (72, 2, 20, 0, 20, 1.0, 1.0, SA.NORM_UNIT), (112, 1, 70, 0, 0, 1.0, 1.0, SA.NORM_WEIGHT),
            (182, 2, 130, 0, 130, 1.0, -1.0, SA.NORM_NONE)]
    width = 182 + 260 + 3
    rows = torch.randn((t, width), generator=g).to(dtype)
    want = rows.to(O.F64).clone()
    made = []
    for off, heads, hd, ro, rd, mult, sign, norm in segs:
        freq = O.plain_frequencies(777.0, rd) if rd else None
        wgt = torch.rand(hd, generator=g) + 0.5 if norm == SA.NORM_WEIGHT else None
        v = want[:, off:off + heads * hd].view(t, heads, hd).clone()
        if rd:
            f32_angles = (pos.float()[:, None] * freq.float()[None, :]).double()            # angles are formed in 32-bit
            a = sign * f32_angles
            cos, sin = (torch.cos(a) * mult)[:, None], (torch.sin(a) * mult)[:, None]
            u, w2 = v[..., ro:ro + rd // 2], v[..., ro + rd // 2:ro + rd]
            v = torch.cat([v[..., :ro], u * cos - w2 * sin, w2 * cos + u * sin, v[..., ro + rd:]], dim=-1)
        if norm != SA.NORM_NONE:
            v = O.rms(v, eps, None if wgt is None else wgt.double())
        want[:, off:off + heads * hd] = v.reshape(t, heads * hd)
        made.append(SA.HeadSegment(off, heads, hd, ro, rd, None if freq is None else freq.float().to(device), mult, sign, False, norm,
                                   None if wgt is None else wgt.to(device)))
    got = rows.clone().to(device)
    SA.rotate_norm_heads_(got, pos.to(device), made, eps)
    assert torch.equal(got[:, -3:].cpu(), rows[:, -3:])                                     # what no segment covers stays
    err = (got.cpu().double() - want).abs().max().item()
    assert err < (2e-5 if dtype == torch.float32 else 4e-2), err
    # interleaved pairs
    rows2 = torch.randn((t, 16), generator=g).to(dtype)
    freq = O.plain_frequencies(50.0, 16)
    a = (pos.float()[:, None] * freq.float()[None, :]).double()
    r64 = rows2.double()
    want2 = torch.stack([r64[:, 0::2] * torch.cos(a) - r64[:, 1::2] * torch.sin(a), r64[:, 1::2] * torch.cos(a) + r64[:, 0::2] * torch.sin(a)], -1).flatten(-2)
    got2 = rows2.clone().to(device)
    SA.rotate_norm_heads_(got2, pos.to(device), [SA.HeadSegment(0, 1, 16, 0, 16, freq.float().to(device), interleaved=True)], eps)
    assert (got2.cpu().double() - want2).abs().max().item() < (2e-5 if dtype == torch.float32 else 4e-2)


def _attend_oracle(q, k, v, scale, window, keep, sink, gate):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv] float64 of one sequence -> [T, H * dv]."""
    T, H, G = q.shape[0], q.shape[1], k.shape[1]
    seen = O.causal(T) if window is None else O.window_keep_first(T, window, keep)
    out = torch.zeros((T, H, v.shape[2]), dtype=O.F64)
    for h in range(H):
        g = h // (H // G)
        p = O.sink_softmax_rows((q[:, h] @ k[:, g].T) * scale, seen, None if sink is None else float(sink[h]))
        out[:, h] = p @ v[:, g]
        if gate is not None:
            out[:, h] = out[:, h] / (1.0 + torch.exp(-gate[:, h:h + 1]))
    return out.reshape(T, -1)


def _run_attend(q, k, v, steps, device, dtype, scale, window, keep, sink, gate, slot=0, n_slots=1):
    """The same rows through ``sink_attend`` and a slot table, cut into ``steps`` = [(lo, hi), ...]."""
    slots = SequenceSlots(n_slots)
    slots.length[slot] = 0
    T, H, dk = q.shape
    G, dv = v.shape[1], v.shape[2]
    cache = SlotKVCache(G * dk, G * dv, window, keep, slots, first_capacity=64)
    qd, kd, vd = (x.to(dtype).to(device) for x in (q, k, v))
    gd = None if gate is None else gate.to(dtype).to(device)
    sd = None if sink is None else sink.float().to(device)
    outs = []
    for lo, hi in steps:
        batch = StepBatch.build([slot], [lo], [hi - lo], device)
        cache.reserve(hi, dtype, torch.device(device))
        outs.append(SA.sink_attend(qd[lo:hi], kd[lo:hi], vd[lo:hi], cache, batch, scale, window, keep, sd, None if gd is None else gd[lo:hi]))
        SA.cache_append(cache, kd[lo:hi].reshape(hi - lo, -1), vd[lo:hi].reshape(hi - lo, -1), batch)
        slots.length[slot] = hi
    return torch.cat(outs).float().cpu()


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H,G,dk,dv,window,keep,sinked,gated", [
    (4, 2, 32, 32, None, 0, True, True), (2, 2, 16, 24, 9, 3, True, False), (3, 1, 20, 10, 4, 0, False, False),
    (2, 1, 64, 64, 40, 50, True, True), (8, 1, 40, 32, None, 0, False, True), (1, 1, 8, 8, 1, 0, True, False), (12, 1, 24, 16, 33, 2, True, False)])
def test_sink_attention_alone(device, dtype, H, G, dk, dv, window, keep, sinked, gated):
    """Random rows through the core alone: whole, in portions, and token by token; with and without sink, gate, window, kept tokens."""
    g = torch.Generator().manual_seed(H * 100 + dk)
    T = 150
    q, k, v = torch.randn((T, H, dk), generator=g), torch.randn((T, G, dk), generator=g), torch.randn((T, G, dv), generator=g)
    q, k, v = (x.to(dtype).float() for x in (q, k, v))
    sink = torch.randn(H, generator=g) * 2 if sinked else None
    gate = torch.randn((T, H), generator=g).to(dtype).float() if gated else None
    scale = 1.7 / math.sqrt(dk)
    want = _attend_oracle(q.double(), k.double(), v.double(), scale, window, keep, sink, None if gate is None else gate.double())
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    for steps in ([(0, T)], [(0, 70), (70, 72), (72, 139), (139, T)], [(0, 100)] + [(i, i + 1) for i in range(100, T)]):
        got = _run_attend(q, k, v, steps, device, dtype, scale, window, keep, sink, gate)
        err = (got.double() - want).abs().max().item()
        assert err < tol, (steps[:2], err)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("window,keep,n,cut", [(None, 0, 700, None), (None, 0, 700, 640), (7, 3, 60, None), (7, 3, 60, 30), (128, 4, 300, None),
                                               (128, 4, 300, 250), (129, 32, 300, 140), (64, 1, 200, 199), (33, 40, 120, 50)])
def test_one_key_stands_out(device, dtype, window, keep, n, cut):
    """Keys are nearly orthogonal codes and each query asks for ONE position with a score far above the rest, so its output is
    (nearly) that position's value row if the mask shows it and (nearly) nothing -- the sink takes the weight -- if not.  Head by
    head the asked position is: the farthest the window shows (i - window + 1), the first it hides (i - window), the last kept
    token (keep - 1), the first that is not kept (keep), position 0, and a key hundreds of tokens back.  ``cut``: rows after it
    are decoded one by one, so every edge is met inside a prompt, across the table's ring, and in decoding; windows of 128 / 129
    put it on both sides of a query tile's border.  Without a window every asked key is seen, however far."""
    dim, vdim = 64, 16
    g = torch.Generator().manual_seed(11)
    codes = torch.randn((n, dim), generator=g)
    codes = codes / codes.norm(dim=-1, keepdim=True)
    w = window if window is not None else 10 ** 6
    asks = [lambda i: i - w + 1, lambda i: i - w, lambda i: keep - 1, lambda i: keep, lambda i: 0, lambda i: i - 500]
    H = len(asks)
    q = torch.zeros((n, H, dim))
    for i in range(n):
        for h, ask in enumerate(asks):
            j = ask(i)
            if window is None:
                j = max(j, 0)                                                               # no window: ask for far keys that exist
            q[i, h] = codes[j] if 0 <= j <= i else codes[i] * 0.0
    k = codes[:, None, :].clone()
    v = torch.randn((n, 1, vdim), generator=g)
    q, k, v = (x.to(dtype).float() for x in (q, k, v))
    sink = torch.full((H,), 14.0)
    scale = 24.0                                                                            # a match scores 24, the sink 14, others about +-3
    want = _attend_oracle(q.double(), k.double(), v.double(), scale, window, keep, sink, None)
    steps = [(0, n)] if cut is None else [(0, cut)] + [(i, i + 1) for i in range(cut, n)]
    got = _run_attend(q, k, v, steps, device, dtype, scale, window, keep, sink, None)
    err = (got.double() - want).abs().max().item()
    assert err < (1e-4 if dtype == torch.float32 else 3e-2), err
    if window is not None and n > window + keep + 1:                                        # the scenario is what it claims to be
        i = n - 1
        ref = want.view(n, H, vdim)
        assert (ref[i, 0] - v[i - w + 1, 0].double()).abs().max() < 0.1 and ref[i, 1].abs().max() < 0.1
        if keep:
            assert (ref[i, 2] - v[keep - 1, 0].double()).abs().max() < 0.1
        assert ref[i, 3].abs().max() < 0.1


@pytest.mark.parametrize("device", DEVICES)
def test_slot_table_rows(device):
    """Where a position lives: kept rows first, then the ring; a portion longer than the ring leaves its last rows; a table without
    a window grows and keeps what it holds; another slot's rows are not touched."""
    slots = SequenceSlots(3)
    slots.length[1] = 0
    c = SlotKVCache(4, 2, window=5, keep=2, slots=slots)
    c.reserve(40, torch.float32, torch.device(device))
    rows = torch.arange(40, dtype=torch.float32)[:, None].to(device)
    batch = StepBatch.build([1], [0], [23], device)
    SA.cache_append(c, rows[:23].expand(23, 4).contiguous(), rows[:23].expand(23, 2).contiguous(), batch)
    held = c.keys[1, :, 0].cpu().tolist()
    assert held[:2] == [0.0, 1.0] and sorted(held[2:]) == [18.0, 19.0, 20.0, 21.0, 22.0]
    assert all(held[2 + (p - 2) % 5] == float(p) for p in range(18, 23))
    assert c.stored(23).tolist() == [0, 1, 18, 19, 20, 21, 22]
    assert float(c.keys[0].abs().sum()) == 0.0 and float(c.keys[2].abs().sum()) == 0.0
    grow = SlotKVCache(4, 0, window=None, slots=SequenceSlots(1), first_capacity=8)
    grow.slots.length[0] = 0
    grow.reserve(6, torch.float32, torch.device(device))
    SA.cache_append(grow, rows[:6].expand(6, 4).contiguous(), None, StepBatch.build([0], [0], [6], device))
    grow.reserve(30, torch.float32, torch.device(device))
    assert grow.ring == 32 and grow.keys[0, :6, 0].cpu().tolist() == [0.0, 1.0, 2.0, 3.0, 4.0, 5.0] and grow.values is grow.keys
    SA.cache_append(grow, rows[6:30].expand(24, 4).contiguous(), None, StepBatch.build([0], [6], [24], device))
    assert grow.keys[0, :30, 3].cpu().tolist() == [float(i) for i in range(30)]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
def test_feed_forward_and_stream_update(device, dtype):
    from gbx_lm_amd.models.feed_forward import DenseFeedForward, activate_
    from gbx_lm_amd.models.residual import stream_add_
    g = torch.Generator().manual_seed(2)
    m = DenseFeedForward(48, 100, "relu2")
    m.up.weight.copy_(torch.randn((100, 48), generator=g) / 7)
    m.down.weight.copy_(torch.randn((48, 100), generator=g) / 10)
    m = m.to(device).to(dtype)
    h = torch.randn((37, 48), generator=g).to(dtype)
    want = O.dense_ff(h.double(), {"up": m.up.weight.cpu().double(), "down": m.down.weight.cpu().double()})
    assert O.rel_err(m(h.to(device)).float(), want) < (1e-5 if dtype == torch.float32 else 2e-2)
    z = torch.randn((5, 1000), generator=g).to(dtype)
    ref = z.double()
    ref = 0.5 * ref * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (ref + 0.044715 * ref ** 3)))
    assert (activate_(z.clone().to(device), "gelu_tanh").cpu().double() - ref).abs().max() < (1e-5 if dtype == torch.float32 else 2e-2)
    odd = z[:, :999].contiguous()                                                          # a length off the 16-byte grid
    assert (activate_(odd.clone().to(device), "relu2").cpu().double() - torch.relu(odd.double()) ** 2).abs().max() < (1e-5 if dtype == torch.float32 else 6e-2)
    x = torch.randn((9, 300), generator=g)
    a, b = torch.randn((9, 300), generator=g).to(dtype), torch.randn((9, 300), generator=g).to(dtype)
    got = stream_add_(x.clone().to(device), a.to(device), b.to(device)).cpu()
    assert torch.allclose(got, x + (a.float() + b.float()), atol=1e-6)
    got = stream_add_(x.clone().to(device), a.to(device), None).cpu()
    assert torch.allclose(got, x + a.float(), atol=1e-6)
    from gbx_lm_amd.models.residual import StreamRMSNorm, stream_add_norm_
    norm = StreamRMSNorm(300, 1e-5)
    norm.weight.copy_(torch.rand(300, generator=g) + 0.5)
    norm = norm.to(device)
    xs = x.clone().to(device)
    h = stream_add_norm_(xs, a.to(device), b.to(device), norm)
    want_x = x.double() + (a.double() + b.double())
    assert torch.allclose(xs.cpu().double(), want_x, atol=1e-6) and h.dtype == dtype
    assert O.rel_err(h.float(), O.rms(want_x, 1e-5, norm.weight.cpu().double())) < (1e-6 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("rows", [1, 7, 40])
def test_head_project(device, dtype, rows):
    """Every head's own matrix on the head's leading channels, the rest copied through (few rows: one launch; more: batched product)."""
    g = torch.Generator().manual_seed(rows)
    heads, n_in, n_out, tail = 5, 37, 300, 6
    x = torch.randn((rows, heads * (n_in + tail) + 3), generator=g).to(dtype)[:, :heads * (n_in + tail)].view(rows, heads, n_in + tail)   # strided rows
    w = (torch.randn((heads, n_in, n_out), generator=g) / 6).to(dtype)
    want = torch.cat([torch.einsum("thi,hio->tho", x[..., :n_in].double(), w.double()), x[..., n_in:].double()], dim=-1)
    got = SA.head_project(x.to(device), w.to(device), tail)
    assert got.shape == want.shape and O.rel_err(got.float().reshape(rows, -1), want.reshape(rows, -1)) < (1e-6 if dtype == torch.float32 else 1e-2)
    got = SA.head_project(x[..., :n_in].to(device), w.to(device))
    assert O.rel_err(got.float().reshape(rows, -1), want[..., :n_out].reshape(rows, -1)) < (1e-6 if dtype == torch.float32 else 1e-2)
    w2 = (torch.randn((heads, n_in, 2600), generator=g) / 6).to(dtype)                    # 16-byte rows of w, more outputs than one pass
    got = SA.head_project(x.to(device), w2.to(device), tail)
    want2 = torch.einsum("thi,hio->tho", x[..., :n_in].double(), w2.double())
    assert O.rel_err(got[..., :2600].float().reshape(rows, -1), want2.reshape(rows, -1)) < (1e-6 if dtype == torch.float32 else 1e-2)
    assert torch.equal(got[..., 2600:].cpu(), x[..., n_in:])


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("kind", ["latent", "attention", "latent_odd", "attention_wide", "latent_wide", "latent_many_heads"])
def test_mixers_alone(device, dtype, kind):
    """One mixer module with random weights: a whole prompt (keys and values formed per head), then token by token and in portions
    (the latent mixer attends over its cached rows directly there)."""
    g = torch.Generator().manual_seed(4)
    W, T, eps = 72, 90, 1e-5
    layer = {"latent": O.latent_layer(4, 16, 8, 24, 32, scaling=YARN), "latent_odd": O.latent_layer(3, 10, 6, 14, 18, base=77.0),
             "latent_wide": O.latent_layer(16, 64, 32, 64, 256),                          # one latent row of 288 channels for 16 heads
             "latent_many_heads": O.latent_layer(40, 16, 16, 8, 48, scaling=YARN),        # more heads than one group of query rows
             "attention": O.attention_layer(4, 2, 32, 32, 16, window=20, keep_first=3, factor=3.0),
             "attention_wide": O.attention_layer(2, 1, 128, 128, 128, window=64, keep_first=0)}[kind]
    cfg = O.make_config([layer], vocab=8, width=W, eps=eps)
    w = O.make_weights(cfg, 6)
    P = O.sub(w, "l0.mix.")
    m = layer["mixer"]
    if layer["type"] == "latent_attention":
        mod = SA.LatentAttention(W, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["rot"]["base"], m["rot"].get("scaling"), m["scale"], eps)
        fused = mod.fuse_weights(w["l0.mix.q"], w["l0.mix.dkv"], w["l0.mix.g"], w["l0.mix.uk"], w["l0.mix.uv"])
        state = {**fused, "o.weight": w["l0.mix.o"], "latent_norm": w["l0.mix.dkv.norm"].float(), "sink": w["l0.mix.sink"].float()}
        ref = lambda h: O.latent_attention(h, m, P, eps)
    else:
        mod = SA.RotatedValueWindowAttention(W, m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["rot"]["dims"], m["rot"]["base"],
                                             m["rot"].get("scaling"), m["mask"]["size"], m["mask"]["keep_first"], m["scale"], eps)
        state = {"qkv.weight": torch.cat([w["l0.mix.q"], w["l0.mix.k"], w["l0.mix.v"]]), "o.weight": w["l0.mix.o"]}
        ref = lambda h: O.attention(h, m, P, eps)
    mod.load_state_dict(state, strict=False)
    for name in ("inp", "up", "o", "qkv"):
        if hasattr(mod, name):
            getattr(mod, name).to(dtype)
    for name in ("uk_heads", "uv_heads_t"):
        if hasattr(mod, name):
            mod._buffers[name] = mod._buffers[name].to(dtype)
    mod.to(device)
    h = torch.randn((T, W), generator=g).to(dtype)
    want = ref(h.double())
    for steps in ([(0, T)], [(0, 33), (33, 35), (35, 60)] + [(i, i + 1) for i in range(60, T)]):
        slots = SequenceSlots(1)
        slots.length[0] = 0
        cache, outs = mod.make_cache(slots), []
        with torch.no_grad():
            for lo, hi in steps:
                outs.append(mod(h[lo:hi].to(device), StepBatch.build([0], [lo], [hi - lo], device), cache))
                slots.length[0] = hi
        assert O.rel_err(torch.cat(outs).float(), want) < (2e-5 if dtype == torch.float32 else 3e-2), steps[:2]


# ------------------------------------------------------------------------------------------------ whole models
@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name,n", [("mixed", 40), ("plain", 150), ("single", 20)])
def test_whole_prompt_and_layers(checkpoints, device, dtype, name, n):
    _, cfg, w = checkpoints[name]
    model = model_for(checkpoints, name, device, dtype)
    toks = tokens_for(cfg, n, 1)
    streams = []
    want = O.forward(toks, cfg, w, streams)
    assert len(streams) == len(O.layer_runs(cfg)) == len(model.layers)
    model.trace_layers = []
    try:
        got = BatchScheduler(model).step([("a", toks)], [all_places(n)])
        layers = list(model.trace_layers)
    finally:
        model.trace_layers = None
    for i, (x, ref) in enumerate(zip(layers, streams)):
        assert O.rel_err(x, ref) < TOL[dtype], f"stream after layer run {i}"
    assert O.rel_err(got, want) < TOL[dtype]
    one = BatchScheduler(model).step([("a", toks[:1])], [[0]])                             # a sequence of one token
    assert O.rel_err(one, want[:1]) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("name", ["mixed", "plain"])
def test_prefill_then_token_by_token(checkpoints, device, dtype, name):
    """Most of a prompt in one step, the rest one token a step through the tables: the windows of 7, 3 and 1 pass over decoded
    tokens, kept tokens stay, the windows of 400 / 130 never fill or fill in the prompt; 60 decode steps (graph replays on the GPU)."""
    _, cfg, w = checkpoints[name]
    model = model_for(checkpoints, name, device, dtype)
    first = 30 if name == "mixed" else 140
    toks = tokens_for(cfg, first + 60, 2)
    want = oracle_logits(cfg, w, toks)
    eng = BatchScheduler(model)
    got = [eng.step([("a", toks[:first])], [all_places(first)])]
    for t in toks[first:]:
        got.append(eng.step([("a", [t])]))
    assert O.rel_err(torch.cat(got), want) < TOL[dtype]


@pytest.mark.parametrize("device", DEVICES)
def test_long_decoding_grows_tables(checkpoints, device):
    """Token by token from the first token past two doublings of the latent tables (capacity 256), far keys included."""
    _, cfg, w = checkpoints["single"]
    model = model_for(checkpoints, "single", device, torch.float32)
    toks = tokens_for(cfg, 530, 9)
    want = oracle_logits(cfg, w, toks)
    eng = BatchScheduler(model)
    got = [eng.step([("a", [t])]) for t in toks]
    assert eng.caches[0].ring == 1024
    assert O.rel_err(torch.cat(got), want) < TOL[torch.float32]


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("portion", [2, 3, 16, 64])
def test_portions(checkpoints, device, dtype, portion):
    """A prompt cut into portions of one size (down to two tokens): a portion's first tokens read the tables, its later ones the
    portion itself; a portion longer than a window overwrites ring rows its own first queries still needed."""
    _, cfg, w = checkpoints["mixed"]
    model = model_for(checkpoints, "mixed", device, dtype)
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
    """A finished request's slot goes to the next one; what the old owner left in the tables (kept rows included) must not reach
    the new one, also while a neighbour keeps decoding; more sequences than slots make the tables grow in the middle of one."""
    _, cfg, w = checkpoints["mixed"]
    model = model_for(checkpoints, "mixed", device, torch.float32)
    a, b, c = tokens_for(cfg, 50, 20), tokens_for(cfg, 64, 21), tokens_for(cfg, 9, 22)
    eng = BatchScheduler(model)
    eng.step([("a", a), ("b", b[:40])])
    slot_a = eng.slot_of["a"]
    eng.release("a")
    out = eng.step([("b", b[40:41]), ("c", c[:4])], [[0], all_places(4)])
    assert eng.slot_of["c"] == slot_a
    got_c, got_b = [out[1:]], [out[:1]]
    for i in range(4, 9):
        out = eng.step([("c", [c[i]]), ("b", [b[37 + i]])])
        got_c.append(out[:1])
        got_b.append(out[1:])
    assert O.rel_err(torch.cat(got_c), O.forward(c, cfg, w)) < TOL[torch.float32]
    assert O.rel_err(torch.cat(got_b), O.forward(b[:46], cfg, w)[40:46]) < TOL[torch.float32]
    eng.release("b"); eng.release("c")
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


@pytest.mark.gpu
def test_decode_graph_replays_match_eager(checkpoints):
    """Decode steps replayed from a HIP graph (captured at the third step) against eager launches, step by step, across a growth of
    the latent tables (every captured pointer is stale then) and after a one-token sequence took the same slot."""
    import os
    _, cfg, w = checkpoints["single"]
    model = model_for(checkpoints, "single", "cuda", torch.float32)
    toks = tokens_for(cfg, 300, 30)
    os.environ["GBX_STEP_GRAPH"] = "0"
    try:
        eager = BatchScheduler(model)
        ref = [eager.step([("a", toks[:200])])] + [eager.step([("a", [t])]) for t in toks[200:]]
    finally:
        os.environ.pop("GBX_STEP_GRAPH")
    eng = BatchScheduler(model)
    for t in toks[:3]:                                   # three one-token sequences in slot 0: the step that gets captured starts at 0
        eng.step([("s", [t])])
        eng.release("s")
    got = [eng.step([("a", toks[:200])])] + [eng.step([("a", [t])]) for t in toks[200:]]
    assert eng._graphs and eng.caches[0].ring == 512
    for i, (x, y) in enumerate(zip(got, ref)):
        assert O.rel_err(x, y) < 1e-5, f"step {i}"


# ------------------------------------------------------------------------------------------------ generation
@pytest.mark.parametrize("device", DEVICES)
def test_greedy_generation_entry_points(checkpoints, device):
    """generate_step (one sequence), BatchScheduler.generate (several) and the command line give the oracle's greedy tokens."""
    folder, cfg, w = checkpoints["mixed"]
    model = model_for(checkpoints, "mixed", device, torch.float32)
    prompts = [tokens_for(cfg, 12, 40), tokens_for(cfg, 5, 41), tokens_for(cfg, 21, 42)]

    def oracle_greedy(p, n):
        seq, out = list(p), []
        for _ in range(n):
            lg = O.forward(seq, cfg, w)[-1]
            top2 = torch.topk(lg, 2).values
            assert float(top2[0] - top2[1]) > 1e-3, "the reference's choice is a close call: pick another prompt"
            out.append(int(torch.argmax(lg)))
            seq.append(out[-1])
        return out

    want = [oracle_greedy(p, 8) for p in prompts]
    got = [tok for tok, _, _ in generate_step(torch.tensor(prompts[0]), model, max_tokens=8)]
    assert got == want[0]
    assert BatchScheduler(model).generate(prompts, max_tokens=8) == want
    if device == "cpu":
        cmd = [sys.executable, "-m", "gbx_lm_amd.cli", "--model", folder, "--dtype", "float32", "--max-tokens", "8"]
        for p in prompts[:2]:
            cmd += ["--prompt-ids", ",".join(map(str, p))]
        lines = subprocess.run(cmd, capture_output=True, text=True, check=True, cwd=str(__import__("pathlib").Path(__file__).parent.parent)).stdout.strip().splitlines()
        assert [json.loads(l)["tokens"] for l in lines] == want[:2]


def test_trace_replay_program(checkpoints, tmp_path):
    """bin/trace_run: steps on standard input, logits files out, slots given back at 'end'."""
    import numpy as np
    folder, cfg, w = checkpoints["single"]
    a, b = tokens_for(cfg, 9, 50), tokens_for(cfg, 4, 51)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:6], "want": [0, 5]}, {"id": "b", "tokens": b[:3], "want": []}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[6:7], "want": [0]}, {"id": "b", "tokens": b[3:4], "want": [0]}], "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[7:8], "want": []}], "end": []},
             {"step": 3, "entries": [{"id": "a", "tokens": a[8:9], "want": [0]}], "end": ["a"]}]
    root = __import__("pathlib").Path(__file__).parent.parent
    r = subprocess.run([sys.executable, str(root / "bin" / "trace_run"), "--model", folder, "--dtype", "float32", "--out", str(tmp_path), "--max-tokens", "64"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, cwd=str(root))
    assert r.returncode == 0, r.stderr[-2000:]
    assert [l for l in r.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2", "done 3"]
    la, lb = O.forward(a, cfg, w), O.forward(b, cfg, w)
    read = lambda n: torch.from_numpy(np.fromfile(str(tmp_path / f"{n}.f32"), dtype="<f4").reshape(-1, cfg["vocab"]))
    assert O.rel_err(read(0), la[[0, 5]]) < 2e-5
    assert O.rel_err(read(1), torch.stack([la[6], lb[3]])) < 2e-5
    assert not (tmp_path / "2.f32").exists()
    assert O.rel_err(read(3), la[8:9]) < 2e-5
