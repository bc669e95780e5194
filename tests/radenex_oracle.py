"""Plain, slow statement of the Radenex design in float64, one function per mechanism, sharing no code with gbx_lm_amd.  A whole
sequence at a time: no cache, no batching, no absorbed products, every (query, key) pair written out.

Notation: x is the residual stream [T, W].  A layer run does  h = N(x) = x / sqrt(mean(x^2) + eps) * w,  x += mixer(h) + ff(h)
(both sublayers read the same h); config 'loop' repeats a span of layers with the same weights; logits = head . N_final(x).
Also here: a random checkpoint writer (config.json + model.safetensors in the design's tensor names), so that tests go through
the framework's own loader.
"""
import json
import math
import os

import torch

F64 = torch.float64


def rms(y, eps, w=None):
    y = y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


# ------------------------------------------------------------------------------------------------ rotations
def plain_frequencies(base, dims):
    return torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F64)


def scaled_frequencies(rot):
    """(frequencies [dims/2], multiplier of cos and sin) of a 'rot' entry: no scaling, linear (factor only), or the ramp between
    scaled and unscaled frequencies (factor, original, fast, slow)."""
    base, dims, sc = rot["base"], rot["dims"], rot.get("scaling")
    f = plain_frequencies(base, dims)
    if not sc:
        return f, 1.0
    if "original" not in sc:
        return f / sc["factor"], 1.0

    def turn_dim(t):
        return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))

    lo = max(math.floor(turn_dim(sc["fast"])), 0)
    hi = min(math.ceil(turn_dim(sc["slow"])), dims - 1)
    out = f.clone()
    for i in range(dims // 2):
        ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out[i] = f[i] / sc["factor"] * ramp + f[i] * (1 - ramp)
    return out, 0.1 * math.log(sc["factor"]) + 1.0


def rotate_halves(v, positions, freq, mult=1.0, sign=1.0):
    """v [T, n, D] with D = 2 * len(freq): pair (i, i + D/2) of row t turns by sign * positions[t] * freq[i]."""
    half = freq.shape[0]
    a = sign * positions.to(F64)[:, None] * freq[None, :]
    cos, sin = (torch.cos(a) * mult)[:, None, :], (torch.sin(a) * mult)[:, None, :]
    u, w = v[..., :half], v[..., half:]
    return torch.cat([u * cos - w * sin, w * cos + u * sin], dim=-1)


# ------------------------------------------------------------------------------------------------ softmax with a sink
def sink_softmax_rows(scores, seen, sink):
    """scores, seen [T, T]; sink: a number (its exponential joins the denominator, it has no value) or None."""
    s = torch.where(seen, scores, torch.full((), -math.inf, dtype=F64))
    top = s.max(-1, keepdim=True).values
    if sink is not None:
        top = top.clamp(min=float(sink))
    e = torch.exp(s - top)                                                   # unseen keys: exp(-inf) = 0
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(float(sink) - top)
    return e / den


def causal(T):
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return j <= i


def window_keep_first(T, size, keep):
    i, j = torch.arange(T)[:, None], torch.arange(T)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep))


# ------------------------------------------------------------------------------------------------ mixers
def latent_attention(h, m, P, eps):
    """P: q, dkv, dkv.norm, uk, uv, sink, g, o."""
    T = h.shape[0]
    H, d, r, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T)
    freq, mult = scaled_frequencies(m["rot"])
    q = (h @ P["q"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate_halves(q[..., d:], pos, freq, mult)
    low = h @ P["dkv"].T
    c = rms(low[:, :R], eps, P["dkv.norm"])
    k_rot = rotate_halves(low[:, None, R:], pos, freq, mult)[:, 0]           # one rotated key part for all heads
    k_plain = (c @ P["uk"].T).view(T, H, d)
    v = (c @ P["uv"].T).view(T, H, dv)
    gate = 1.0 / (1.0 + torch.exp(-(h @ P["g"].T)))                          # [T, H]
    out = torch.zeros((T, H, dv), dtype=F64)
    seen = causal(T)
    for head in range(H):
        s = (q_plain[:, head] @ k_plain[:, head].T + q_rot[:, head] @ k_rot.T) * m["scale"]
        out[:, head] = (sink_softmax_rows(s, seen, float(P["sink"][head])) @ v[:, head]) * gate[:, head:head + 1]
    return out.reshape(T, H * dv) @ P["o"].T


def attention(h, m, P, eps):
    """P: q, k, v, o."""
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    freq, mult = scaled_frequencies(m["rot"])
    n = m["rot"]["dims"]

    def turned(t):
        return torch.cat([rotate_halves(t[..., :n], pos, freq, mult), t[..., n:]], dim=-1)

    q = rms(turned((h @ P["q"].T).view(T, H, d)), eps)                       # unit root mean square per head, after the rotation
    k = rms(turned((h @ P["k"].T).view(T, G, d)), eps)
    vfreq = plain_frequencies(m["rot"]["base"], dv)
    v = rotate_halves((h @ P["v"].T).view(T, G, dv), pos, vfreq)             # values turn by their own position ...
    seen = window_keep_first(T, m["mask"]["size"], m["mask"].get("keep_first", 0))
    out = torch.zeros((T, H, dv), dtype=F64)
    for head in range(H):
        g = head // (H // G)
        s = (q[:, head] @ k[:, g].T) * m["scale"]
        out[:, head] = sink_softmax_rows(s, seen, 0.0) @ v[:, g]             # one added to the denominator
    out = rotate_halves(out, pos, vfreq, sign=-1.0)                          # ... and the sum turns back by the query's
    return out.reshape(T, H * dv) @ P["o"].T


def dense_ff(h, P):
    z = torch.relu(h @ P["up"].T)
    return (z * z) @ P["down"].T


# ------------------------------------------------------------------------------------------------ the stack
def layer_runs(cfg):
    n, loop = len(cfg["layers"]), cfg.get("loop")
    if not loop:
        return list(range(n))
    span = list(range(loop["start"], loop["stop"]))
    return list(range(loop["start"])) + span * loop["times"] + list(range(loop["stop"], n))


def sub(weights, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in weights.items() if k.startswith(prefix)}


def forward(tokens, cfg, weights, streams=None):
    """tokens: list of ids -> logits float64 [T, vocab]; ``streams`` (a list) receives x after every layer run."""
    eps = cfg["norm"]["eps"]
    x = weights["embed"].to(F64)[torch.tensor(tokens)]
    for i in layer_runs(cfg):
        layer = cfg["layers"][i]
        h = rms(x, eps, weights[f"l{i}.norm1"].to(F64))
        mix = {"latent_attention": latent_attention, "attention": attention}[layer["type"]]
        y = mix(h, layer["mixer"], sub(weights, f"l{i}.mix."), eps)
        if layer.get("mlp") is not None:
            assert layer["mlp"]["kind"] == "dense"
            y = y + dense_ff(h, sub(weights, f"l{i}.mlp."))
        x = x + y
        if streams is not None:
            streams.append(x.clone())
    return rms(x, eps, weights["final.norm"].to(F64)) @ weights["head"].to(F64).T


# ------------------------------------------------------------------------------------------------ random checkpoints
def latent_layer(heads, dim, rot_dim, vdim, kv_rank, base=10000.0, scaling=None, scale=None, ff=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling:
        rot["scaling"] = scaling
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot,
                      "scale": scale if scale is not None else 1.0 / math.sqrt(dim + rot_dim)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def attention_layer(heads, kv_heads, dim, vdim, rot_dims, window, keep_first, base=10000.0, factor=None, scale=None, ff=None):
    rot = {"base": base, "dims": rot_dims}
    if factor:
        rot["scaling"] = {"factor": factor}
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot,
                      "mask": {"size": window, "keep_first": keep_first}, "scale": scale if scale is not None else 1.0 / math.sqrt(dim)},
            "mlp": {"kind": "dense", "ff": ff} if ff else None}


def make_config(layers, vocab=61, width=64, eps=1e-5, loop=None):
    cfg = {"architecture": "Radenex", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps}}
    if loop:
        cfg["loop"] = {"start": loop[0], "stop": loop[1], "times": loop[2]}
    return cfg


def make_weights(cfg, seed=0):
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=1.0):
        return (torch.randn((o, i), generator=gen) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, lo, hi):
        return (torch.rand((n,), generator=gen) * (hi - lo) + lo).to(torch.bfloat16)

    w = {"embed": torch.randn((cfg["vocab"], W), generator=gen).to(torch.bfloat16), "final.norm": vec(W, 0.5, 1.5), "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        w[p + "norm1"] = vec(W, 0.5, 1.5)
        H = m["heads"]
        if layer["type"] == "latent_attention":
            d, r, dv, R = m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
            w[p + "mix.q"], w[p + "mix.dkv"], w[p + "mix.dkv.norm"] = mat(H * (d + r), W, 2.0), mat(R + r, W, 2.0), vec(R, 0.5, 1.5)
            w[p + "mix.uk"], w[p + "mix.uv"] = mat(H * d, R, 2.0), mat(H * dv, R)
            w[p + "mix.sink"], w[p + "mix.g"], w[p + "mix.o"] = vec(H, -1.0, 2.0), mat(H, W, 2.0), mat(W, H * dv, 0.5)
        else:
            G, d, dv = m["kv_heads"], m["dim"], m["vdim"]
            w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = mat(H * d, W), mat(G * d, W), mat(G * dv, W)
            w[p + "mix.o"] = mat(W, H * dv, 0.5)
        if layer.get("mlp") is not None:
            ff = layer["mlp"]["ff"]
            w[p + "mlp.up"], w[p + "mlp.down"] = mat(ff, W, 1.5), mat(W, ff, 0.5)
    return w


def save_checkpoint(folder, cfg, weights):
    from safetensors.torch import save_file
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(cfg, f)
    save_file({k: v.contiguous() for k, v in weights.items()}, os.path.join(folder, "model.safetensors"))
    return folder


def rel_err(got, want):
    """Root mean square of the difference over that of the reference, per row, worst row."""
    got, want = got.to(F64).cpu(), want.to(F64).cpu()
    return float(((got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean(-1).sqrt().clamp_min(1e-12)).max())
