"""Plain, slow statement of the Revitar design in float64, one function per mechanism, written from the design's equations and
sharing no code with gbx_lm_amd.  A whole sequence at a time, no cache, no batching: what the framework computes step by step
through rings, slots and ragged batches must agree with this.

Notation: x is the residual stream [T, W]; a layer does  x += m * N1(mixer(x)),  x += m * N2(ff(x))  with
N(y) = y / sqrt(mean(y^2) + eps) * w;  logits = head . N_final(x).
Also here: a random checkpoint writer (config.json + model.safetensors with the design's tensor names) so that tests go through
the framework's own loader.
"""
import json
import math
import os

import torch

F64 = torch.float64


def rms(y, w, eps):
    return y / torch.sqrt((y * y).mean(-1, keepdim=True) + eps) * w


def attention_gates(q, k, spec, P, head):
    """Gate matrix [T, T] of one query head: sigmoid(softcapped score - distance penalty + bias) inside the window, 0 outside."""
    T = q.shape[0]
    a, b, c = float(P["r1"][head]), float(P["r2"][head]), float(P["pb"][head])
    cap = spec.get("softcap") or 0.0
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    dist = (i - j).to(F64)
    seen = (i - j >= 0) & (i - j < spec["mask"]["size"])
    s = (q @ k.T) * spec["scale"]
    if cap > 0:
        s = cap * torch.tanh(s / cap)
    s = s - a * torch.log(1.0 + b * dist.clamp(min=0))
    return torch.where(seen, 1.0 / (1.0 + torch.exp(-(s + c))), torch.zeros((), dtype=F64))


def attention(h, spec, P, eps):
    """P: q, k, v, o matrices [out, in]; q.norm, k.norm; r1, r2, pb per head."""
    T = h.shape[0]
    H, G, dk, dv = spec["heads"], spec["kv_heads"], spec["dim"], spec["vdim"]
    q = rms(h @ P["q"].T, P["q.norm"], eps).view(T, H, dk)          # the norm spans all heads' channels
    k = rms(h @ P["k"].T, P["k.norm"], eps).view(T, G, dk)
    v = (h @ P["v"].T).view(T, G, dv)
    out = torch.zeros((T, H, dv), dtype=F64)
    for head in range(H):
        kv = head // (H // G)
        out[:, head] = attention_gates(q[:, head], k[:, kv], spec, P, head) @ v[:, kv]
    return out.reshape(T, H * dv) @ P["o"].T


def routed_experts(h, spec, P):
    """P: router [E, W]; e<i>.gate / up [F, W], e<i>.down [W, F]."""
    E, top = spec["router"]["experts"], spec["router"]["top"]
    prob = torch.softmax(h @ P["router"].T, dim=-1)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(prob[t, e]), e))[:top]
        for e in order:
            z = P[f"e{e}.gate"] @ h[t]
            act = z / (1.0 + torch.exp(-z)) * (P[f"e{e}.up"] @ h[t])
            out[t] += prob[t, e] * (P[f"e{e}.down"] @ act)           # the chosen probabilities as they are, not renormalised
    return out


def sub(weights, prefix):
    return {k[len(prefix):]: v.to(F64) for k, v in weights.items() if k.startswith(prefix)}


def forward(tokens, cfg, weights, streams=None):
    """tokens: list of ids -> logits float64 [T, vocab]; ``streams`` (a list) receives x after every layer."""
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    x = weights["embed"].to(F64)[torch.tensor(tokens)] * cfg["embedding"]["scale"]
    for i, layer in enumerate(cfg["layers"]):
        assert layer["type"] == "attention"
        x = x + m * rms(attention(x, layer["mixer"], sub(weights, f"l{i}.mix."), eps), weights[f"l{i}.norm1"].to(F64), eps)
        if layer["mlp"] is not None:
            assert layer["mlp"]["kind"] == "moe"
            x = x + m * rms(routed_experts(x, layer["mlp"], sub(weights, f"l{i}.mlp.")), weights[f"l{i}.norm2"].to(F64), eps)
        if streams is not None:
            streams.append(x.clone())
    return rms(x, weights["final.norm"].to(F64), eps) @ weights["head"].to(F64).T


# ------------------------------------------------------------------------------------------------ random checkpoints
def attention_layer(heads, kv_heads, dim, vdim, window, scale=None, softcap=30.0, mlp=None):
    mixer = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "mask": {"size": window},
             "scale": scale if scale is not None else 1.0 / math.sqrt(dim)}
    if softcap is not None:
        mixer["softcap"] = softcap
    return {"type": "attention", "mixer": mixer, "mlp": mlp}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def make_config(layers, vocab=61, width=64, eps=1e-5, residual_mult=0.5, embed_scale=2.0):
    return {"architecture": "Revitar", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "residual_mult": residual_mult, "embedding": {"scale": embed_scale}}


def make_weights(cfg, seed=0, wide_margins=False):
    """Random bf16 checkpoint in the design's tensor names.  ``wide_margins``: every embedding row gets a common component along one
    direction and the routers read mostly that component, with a different gain per expert: router logits are then about one unit
    apart for every token, so rounding to bf16 upstream never changes which experts are chosen (the choice is still made by the
    router, it is just not a close call), while the probabilities stay spread (about 0.6 / 0.2 / 0.1 ...)."""
    gen = torch.Generator().manual_seed(seed)
    W = cfg["width"]

    def mat(o, i, s=1.0):
        return (torch.randn((o, i), generator=gen) * s / math.sqrt(i)).to(torch.bfloat16)

    def vec(n, lo, hi):
        return (torch.rand((n,), generator=gen) * (hi - lo) + lo).to(torch.bfloat16)

    common = torch.ones(W) / math.sqrt(W)
    emb = torch.randn((cfg["vocab"], W), generator=gen)
    if wide_margins:
        emb = emb + 5.0 * common
    w = {"embed": emb.to(torch.bfloat16), "final.norm": vec(W, 0.5, 1.5), "head": mat(cfg["vocab"], W)}
    for i, layer in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", layer["mixer"]
        H, G, dk, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
        w[p + "norm1"] = vec(W, 0.5, 1.5)
        w[p + "mix.q"], w[p + "mix.k"], w[p + "mix.v"] = mat(H * dk, W), mat(G * dk, W), mat(G * dv, W)
        w[p + "mix.q.norm"], w[p + "mix.k.norm"] = vec(H * dk, 0.5, 2.0), vec(G * dk, 0.5, 2.0)
        w[p + "mix.r1"], w[p + "mix.r2"], w[p + "mix.pb"] = vec(H, 0.1, 1.0), vec(H, 0.05, 2.0), vec(H, -2.0, 0.5)
        w[p + "mix.o"] = mat(W, H * dv)
        if layer["mlp"] is not None:
            ff, E = layer["mlp"]["expert"]["ff"], layer["mlp"]["router"]["experts"]
            w[p + "norm2"] = vec(W, 0.5, 1.5)
            w[p + "mlp.router"] = mat(E, W, 4.0)
            if wide_margins:
                gain = torch.arange(E, 0, -1, dtype=torch.float32) / (5.0 * cfg["embedding"]["scale"])
                w[p + "mlp.router"] = (gain[:, None] * common[None, :] + 0.02 * torch.randn((E, W), generator=gen) / math.sqrt(W)).to(torch.bfloat16)
            for e in range(E):
                w[p + f"mlp.e{e}.gate"], w[p + f"mlp.e{e}.up"], w[p + f"mlp.e{e}.down"] = mat(ff, W, 2.0), mat(ff, W, 2.0), mat(W, ff, 2.0)
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
