"""Plain, slow restatement of the Kagalorn layers in float64, one function per mechanism, whole
sequences at a time (no cache, no state carried between calls, no batching). Test infrastructure
only: it shares no code with the package and is what the engine's results are compared with."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def grouped_rms_norm(x, w, groups, eps):
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * w


def streams_read(xs, read):
    """xs [S, T, W] -> sum_s read[s] xs[s]."""
    return sum(read[s] * xs[s] for s in range(xs.shape[0]))


def streams_write(xs, y, mix, write):
    """new[t] = sum_s mix[s, t] xs[s] + write[t] y, all from the old streams."""
    S = xs.shape[0]
    return torch.stack([sum(mix[s, t] * xs[s] for s in range(S)) + write[t] * y for t in range(S)])


def short_conv_silu(x, w):
    """x [T, C], w [C, taps], last tap on the current token, zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for i in range(taps):
            src = t - (taps - 1 - i)
            if src >= 0:
                out[t] += w[:, i] * x[src]
    return out * torch.sigmoid(out)


def unit(x, eps):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + eps)


def delta_rule(q, k, v, beta, g):
    """One head: q, k [T, D], v [T, Dv], beta, g [T]. Returns o [T, Dv]."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=F64)
    o = []
    for t in range(T):
        S = g[t] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o.append(S.T @ q[t])
    return torch.stack(o)


def delta_mixer(h, W, p, m, norm_eps, unit_eps=1e-6):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, G, D)
    k = short_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, D)
    v = short_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, H, Dv)
    q = unit(q, unit_eps) * D ** -0.5
    k = unit(k, unit_eps)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) * torch.nn.functional.softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    rep = H // G
    o = torch.stack([delta_rule(q[:, hh // rep], k[:, hh // rep], v[:, hh], beta[:, hh], g[:, hh]) for hh in range(H)], 1)
    o = o / torch.sqrt((o * o).mean(-1, keepdim=True) + norm_eps) * W[p + "norm"]
    gate = (h @ W[p + "g"].T)
    gate = (gate * torch.sigmoid(gate)).view(T, H, Dv)
    return (o * gate).reshape(T, H * Dv) @ W[p + "o"].T


def window_pool_softmax_attention(q, k, v, window, pool, scale, sink=True):
    """One query head against its key/value head: q [T, D], k [T, D], v [T, Dv]."""
    T = q.shape[0]
    out = []
    for i in range(T):
        ks = [k[j] for j in range(T) if 0 <= i - j < window]
        vs = [v[j] for j in range(T) if 0 <= i - j < window]
        b = 0
        while pool > 0 and b * pool + pool - 1 <= i - window:
            ks.append(k[b * pool:(b + 1) * pool].mean(0))
            vs.append(v[b * pool:(b + 1) * pool].mean(0))
            b += 1
        s = torch.stack(ks) @ q[i] * scale
        e = torch.exp(s)
        out.append((e / ((1.0 if sink else 0.0) + e.sum())) @ torch.stack(vs))
    return torch.stack(out)


def attention_mixer(h, W, p, m, norm_eps, cache_round=None):
    """cache_round: optional function applied to keys and values where a cache would hold them."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q, k, v = h @ W[p + "q"].T, h @ W[p + "k"].T, h @ W[p + "v"].T
    q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + norm_eps) * W[p + "q.norm"]
    k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + norm_eps) * W[p + "k.norm"]
    if cache_round is not None:
        q, k, v = cache_round(q), cache_round(k), cache_round(v)
    q, k, v = q.view(T, H, D), k.view(T, G, D), v.view(T, G, Dv)
    rep = H // G
    o = torch.stack([window_pool_softmax_attention(q[:, hh], k[:, hh // rep], v[:, hh // rep], m["mask"]["size"],
                                                   m["mask"].get("pool", 0), m["scale"]) for hh in range(H)], 1)
    gate = torch.sigmoid(h @ W[p + "g"].T)
    return (o.reshape(T, H * Dv) * gate) @ W[p + "o"].T


def clamped_glu_ff(h, W, p, limit, alpha=1.702):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(alpha * g) * (u + 1)) @ W[p + "down"].T


def forward(cfg: dict, weights: dict, tokens, layer_outputs=None):
    """Logits [T, vocab] of one sequence. weights: name -> tensor (any float dtype)."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps, groups, S = cfg["norm"]["eps"], cfg["norm"].get("groups", 1), cfg.get("streams", 1)
    x = W["embed"][torch.tensor(tokens)]
    xs = torch.stack([x] * S)
    for i, L in enumerate(cfg["layers"]):
        p = f"l{i}."
        for qn in (1, 2):
            if qn == 2 and L["mlp"] is None:
                continue
            h = grouped_rms_norm(streams_read(xs, W[p + f"hc{qn}.in"]), W[p + f"norm{qn}"], groups, eps)
            if qn == 2:
                y = clamped_glu_ff(h, W, p + "mlp.", L["mlp"]["limit"])
            elif L["type"] == "delta":
                y = delta_mixer(h, W, p + "mix.", L["mixer"], eps)
            else:
                y = attention_mixer(h, W, p + "mix.", L["mixer"], eps)
            xs = streams_write(xs, y, W[p + f"hc{qn}.mix"], W[p + f"hc{qn}.out"])
        if layer_outputs is not None:
            layer_outputs.append(xs.sum(0))
    return grouped_rms_norm(xs.sum(0), W["final.norm"], groups, eps) @ W["head"].T


def tensor_shapes(cfg: dict) -> dict:
    """name -> shape of every checkpoint tensor of a configuration."""
    W, S = cfg["width"], cfg.get("streams", 1)
    t = {"embed": (cfg["vocab"], W), "head": (cfg["vocab"], W), "final.norm": (W,)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        t[p + "norm1"] = (W,)
        for q in (1, 2) if L["mlp"] is not None else (1,):
            t[p + f"hc{q}.in"], t[p + f"hc{q}.out"], t[p + f"hc{q}.mix"] = (S,), (S,), (S, S)
        if L["type"] == "delta":
            for nm, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                t[p + "mix." + nm] = (rows, W)
                t[p + f"mix.{nm}.conv"] = (rows, m["conv"])
            t[p + "mix.b"], t[p + "mix.a"] = (H, W), (H, W)
            t[p + "mix.A_log"], t[p + "mix.dt_bias"], t[p + "mix.norm"] = (H,), (H,), (Dv,)
        else:
            t[p + "mix.q"], t[p + "mix.k"], t[p + "mix.v"] = (H * D, W), (G * D, W), (G * Dv, W)
            t[p + "mix.q.norm"], t[p + "mix.k.norm"] = (H * D,), (G * D,)
        t[p + "mix.g"], t[p + "mix.o"] = (H * Dv, W), (W, H * Dv)
        if L["mlp"] is not None:
            ff = L["mlp"]["ff"]
            t[p + "norm2"] = (W,)
            t[p + "mlp.gate"], t[p + "mlp.up"], t[p + "mlp.down"] = (ff, W), (ff, W), (W, ff)
    return t


def random_weights(cfg: dict, seed: int) -> dict:
    """Seeded bf16-representable weights that keep activations of order one."""
    g = torch.Generator().manual_seed(seed)
    S = cfg.get("streams", 1)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(*shape, generator=g)
        if "norm" in leaf:
            w = 1.0 + 0.2 * r
        elif ".hc" in name and leaf == "mix":
            w = 0.7 * torch.eye(S) + 0.2 * r
        elif ".hc" in name:
            w = (1.0 / S if leaf == "in" else 0.8) + 0.2 * r
        elif leaf in ("conv", "A_log", "dt_bias"):
            w = 0.6 * r
        elif len(shape) == 2:
            w = r / math.sqrt(shape[1])
        else:
            w = 0.5 * r
        out[name] = w.to(torch.bfloat16).to(torch.float32)
    return out
