"""Plain, slow restatement of the Bokulorn layers in float64, one function per mechanism, whole
sequences at a time (no cache, no state carried between calls, no batching, no absorbed matrices:
every head's keys and values are written out). Test infrastructure only: it shares no code with the
package and is what the engine's results are compared with."""
from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * w


def offset_rms_norm(x, w, eps):
    """Norm whose weight is an offset from one."""
    return rms_norm(x, 1.0 + w, eps)


def rotate(x, positions, dims, base):
    """x [T, d]: entry i of the first `dims` and entry i + dims/2 form a pair, which is turned by
    position * base^(-2i/dims); entries from `dims` on pass unchanged."""
    out = x.clone()
    half = dims // 2
    for t in range(x.shape[0]):
        for i in range(half):
            a = float(positions[t]) * base ** (-2.0 * i / dims)
            u, v = x[t, i], x[t, i + half]
            out[t, i] = u * math.cos(a) - v * math.sin(a)
            out[t, i + half] = v * math.cos(a) + u * math.sin(a)
    return out


def causal_softmax_attention(q, k, v, scale):
    """One head: q [T, D], k [T, D], v [T, Dv]; causal mask (keys up to and including the query's own position)."""
    out = []
    for i in range(q.shape[0]):
        s = k[:i + 1] @ q[i] * scale
        e = torch.exp(s - s.max())
        out.append((e / e.sum()) @ v[:i + 1])
    return torch.stack(out)


def latent_attention_mixer(h, W, p, m, norm_eps, positional: bool, cache_round=None):
    """positional: the rotated part and a gate per head; otherwise no positions and a gate per channel.
    cache_round: optional function applied to what a cache would hold (latent and rotated key part)."""
    T = h.shape[0]
    H, Dn, Dv, R = m["heads"], m["dim"], m["vdim"], m["kv_rank"]
    Dr = int(m.get("rot_dim", 0)) if positional else 0
    pos = list(range(T))
    cq = rms_norm(h @ W[p + "dq"].T, W[p + "dq.norm"], norm_eps)
    q = (cq @ W[p + "uq"].T).view(T, H, Dn + Dr)
    down = h @ W[p + "dkv"].T
    c = rms_norm(down[:, :R], W[p + "dkv.norm"], norm_eps)
    kr = rotate(down[:, R:], pos, m["rot"]["dims"], m["rot"]["base"]) if Dr else None
    if cache_round is not None:
        c = cache_round(c)
        kr = cache_round(kr) if Dr else None
    k = (c @ W[p + "uk"].T).view(T, H, Dn)
    v = (c @ W[p + "uv"].T).view(T, H, Dv)
    heads = []
    for hh in range(H):
        qh, kh = q[:, hh, :Dn], k[:, hh]
        if Dr:
            qh = torch.cat([qh, rotate(q[:, hh, Dn:], pos, m["rot"]["dims"], m["rot"]["base"])], -1)
            kh = torch.cat([kh, kr], -1)
        heads.append(causal_softmax_attention(qh, kh, v[:, hh], m["scale"]))
    o = torch.stack(heads, 1)                                   # [T, H, Dv]
    gate = torch.sigmoid(h @ W[p + "g"].T)
    o = o * gate[:, :, None] if positional else o * gate.view(T, H, Dv)
    return o.reshape(T, H * Dv) @ W[p + "o"].T


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


def channel_delta_rule(q, k, v, beta, g):
    """One head: q, k [T, D], v [T, Dv], beta [T], g [T, D] (one decay per key channel = row of S)."""
    T, D = q.shape
    S = torch.zeros(D, v.shape[1], dtype=F64)
    o = []
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        o.append(S.T @ q[t])
    return torch.stack(o)


def channel_delta_mixer(h, W, p, m, norm_eps, unit_eps=1e-6):
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, G, D)
    k = short_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, D)
    v = short_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, H, Dv)
    q = unit(q, unit_eps) * D ** -0.5
    k = unit(k, unit_eps)
    beta = torch.sigmoid(h @ W[p + "b"].T)
    a = (h @ W[p + "a1"].T) @ W[p + "a2"].T + W[p + "dt_bias"]
    g = torch.exp(-torch.exp(W[p + "A_log"])[None, :, None] * torch.nn.functional.softplus(a).view(T, H, D))
    rep = H // G
    o = torch.stack([channel_delta_rule(q[:, hh // rep], k[:, hh // rep], v[:, hh], beta[:, hh], g[:, hh])
                     for hh in range(H)], 1)
    o = rms_norm(o, W[p + "norm"], norm_eps)
    gate = torch.sigmoid((h @ W[p + "g1"].T) @ W[p + "g2"].T).view(T, H, Dv)
    return (o * gate).reshape(T, H * Dv) @ W[p + "o"].T


def route(z, correction, top, groups=1, keep=1, margin=None):
    """z [E] router logits of one token -> (chosen experts, their weights), both lists in order of choice.
    margin: a list that receives by how much the choice was decided (last chosen against first left out,
    for groups and for experts): a small number marks a token whose choice rounding may turn."""
    E = z.shape[0]
    s = [1.0 / (1.0 + math.exp(-float(x))) for x in z]
    c = [s[e] + float(correction[e]) for e in range(E)]
    allowed = set(range(E))
    if groups > 1:
        size = E // groups
        scores = []
        for gi in range(groups):
            best = sorted((c[e] for e in range(gi * size, (gi + 1) * size)), reverse=True)
            scores.append(sum(best[:2]))
        ranked = sorted(range(groups), key=lambda gi: (-scores[gi], gi))
        order = ranked[:keep]
        if margin is not None and keep < groups:
            margin.append(scores[ranked[keep - 1]] - scores[ranked[keep]])
        allowed = {e for gi in order for e in range(gi * size, (gi + 1) * size)}
    ranked = sorted(allowed, key=lambda e: (-c[e], e))
    chosen = ranked[:top]
    if margin is not None and top < len(ranked):
        margin.append(c[ranked[top - 1]] - c[ranked[top]])
    total = sum(s[e] for e in chosen) + 1e-20
    return chosen, [s[e] / total for e in chosen]


def moe_ff(h, W, p, mlp, margins=None):
    """margins: optional list of per-token lists, see route."""
    r = mlp["router"]
    gr = r.get("groups") or {}
    groups = int(gr.get("count", 1))
    keep = int(gr.get("keep", groups))
    z = h @ W[p + "router"].T
    rows = []
    for t in range(h.shape[0]):
        chosen, weights = route(z[t], W[p + "correction"], r["top"], groups, keep,
                                margins[t] if margins is not None else None)
        y = torch.zeros(h.shape[1], dtype=F64)
        for e, w in zip(chosen, weights):
            y = y + w * (W[p + f"e{e}.down"] @ torch.relu(W[p + f"e{e}.up"] @ h[t]) ** 2)
        rows.append(y)
    return torch.stack(rows)


def source_of(cfg: dict, i: int) -> int:
    while cfg["layers"][i].get("weights_of") is not None:
        i = cfg["layers"][i]["weights_of"]
    return i


def forward(cfg: dict, weights: dict, tokens, layer_outputs=None, margins=None):
    """Logits [T, vocab] of one sequence. weights: name -> tensor (any float dtype). margins: a list that
    receives, per token, the smallest margin by which any router decided (see route)."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)] * cfg.get("embedding", {}).get("scale", 1.0)
    per_token = [[] for _ in tokens]
    for i, L in enumerate(cfg["layers"]):
        p = f"l{source_of(cfg, i)}."
        h = offset_rms_norm(x, W[p + "norm1"], eps)
        if L["type"] == "channel_delta":
            y = channel_delta_mixer(h, W, p + "mix.", L["mixer"], eps)
        else:
            y = latent_attention_mixer(h, W, p + "mix.", L["mixer"], eps, L["type"] == "latent_attention")
        if L["mlp"] is not None:
            y = y + moe_ff(h, W, p + "mlp.", L["mlp"], per_token)
        x = x + y
        if layer_outputs is not None:
            layer_outputs.append(x.clone())
    if margins is not None:
        margins.extend(min(m) if m else math.inf for m in per_token)
    return offset_rms_norm(x, W["final.norm"], eps) @ W["head"].T


def tensor_shapes(cfg: dict) -> dict:
    """name -> shape of every checkpoint tensor of a configuration (layers that borrow weights have none)."""
    W = cfg["width"]
    t = {"embed": (cfg["vocab"], W), "head": (cfg["vocab"], W), "final.norm": (W,)}
    for i, L in enumerate(cfg["layers"]):
        if L.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", L["mixer"]
        t[p + "norm1"] = (W,)
        if L["type"] == "channel_delta":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            for nm, rows in (("q", G * D), ("k", G * D), ("v", H * Dv)):
                t[p + "mix." + nm] = (rows, W)
                t[p + f"mix.{nm}.conv"] = (rows, m["conv"])
            t[p + "mix.b"] = (H, W)
            t[p + "mix.a1"], t[p + "mix.a2"] = (m["decay_rank"], W), (H * D, m["decay_rank"])
            t[p + "mix.g1"], t[p + "mix.g2"] = (m["gate_rank"], W), (H * Dv, m["gate_rank"])
            t[p + "mix.A_log"], t[p + "mix.dt_bias"], t[p + "mix.norm"] = (H,), (H * D,), (Dv,)
            t[p + "mix.o"] = (W, H * Dv)
        else:
            H, Dn, Dv, R, Rq = m["heads"], m["dim"], m["vdim"], m["kv_rank"], m["q_rank"]
            Dr = int(m.get("rot_dim", 0)) if L["type"] == "latent_attention" else 0
            t[p + "mix.dq"], t[p + "mix.dq.norm"], t[p + "mix.uq"] = (Rq, W), (Rq,), (H * (Dn + Dr), Rq)
            t[p + "mix.dkv"], t[p + "mix.dkv.norm"] = (R + Dr, W), (R,)
            t[p + "mix.uk"], t[p + "mix.uv"] = (H * Dn, R), (H * Dv, R)
            t[p + "mix.g"] = (H if L["type"] == "latent_attention" else H * Dv, W)
            t[p + "mix.o"] = (W, H * Dv)
        if L["mlp"] is not None:
            ff, E = L["mlp"]["expert"]["ff"], L["mlp"]["router"]["experts"]
            for e in range(E):
                t[p + f"mlp.e{e}.up"], t[p + f"mlp.e{e}.down"] = (ff, W), (W, ff)
            t[p + "mlp.router"], t[p + "mlp.correction"] = (E, W), (E,)
    return t


def random_weights(cfg: dict, seed: int) -> dict:
    """Seeded bf16-representable weights that keep activations of order one."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        leaf = name.rsplit(".", 1)[-1]
        r = torch.randn(*shape, generator=g)
        if name.endswith("dq.norm") or name.endswith("dkv.norm") or name.endswith("mix.norm"):
            w = 1.0 + 0.2 * r
        elif "norm" in leaf:
            w = 0.2 * r                       # an offset from one
        elif leaf in ("conv", "A_log", "dt_bias"):
            w = 0.6 * r
        elif leaf == "correction":
            w = 0.3 * r
        elif leaf == "router":
            w = 2.0 * r / math.sqrt(shape[1])
        elif len(shape) == 2:
            w = r / math.sqrt(shape[1])
        else:
            w = 0.5 * r
        out[name] = w.to(torch.bfloat16).to(torch.float32)
    return out
