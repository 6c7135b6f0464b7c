"""Plain float64 implementation of the Medilix design, one function per
mechanism, token-by-token loops where the design is recurrent. It shares no
code with kllms_amd: tests compare the engine against it.

A model is (config, weights): ``config`` is the checkpoint's config.json as a
dict, ``weights`` maps checkpoint tensor names to torch tensors.
"""

from __future__ import annotations

import math
from typing import Dict, List

import torch

F64 = torch.float64


def _w(weights, name):
    return weights[name].to(F64)


def group_rms(x: torch.Tensor, w: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Split the last dim into ``groups`` runs, divide each by its own
    sqrt(mean square + eps), scale the whole by w."""
    shp = x.shape
    xg = x.reshape(*shp[:-1], groups, shp[-1] // groups)
    xg = xg / torch.sqrt((xg * xg).mean(-1, keepdim=True) + eps)
    return xg.reshape(shp) * w


def rms_plain(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def embed_tokens(tokens: List[int], weights, cfg) -> torch.Tensor:
    e = cfg["embedding"]
    bg = e["bigram"]
    table, big = _w(weights, "embed"), _w(weights, "bigram")
    rows = []
    for t, tok in enumerate(tokens):
        x = table[tok] * e["scale"]
        if t == 0:
            x = x + big[bg["buckets"]]
        else:
            x = x + big[(tokens[t - 1] * bg["mul_prev"] + tok * bg["mul_cur"]) % bg["buckets"]]
        rows.append(x)
    return torch.stack(rows)


def attention(h: torch.Tensor, weights, pre: str, m: dict, eps: float) -> torch.Tensor:
    """Softmax attention with a sliding window that keeps the first tokens,
    a sink in the denominator, q/k norm, elementwise output gate."""
    T = h.shape[0]
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size, keep = m["mask"]["size"], m["mask"]["keep_first"]
    q = (h @ _w(weights, pre + "q").T).reshape(T, H, D)
    k = (h @ _w(weights, pre + "k").T).reshape(T, G, D)
    v = (h @ _w(weights, pre + "v").T).reshape(T, G, Dv)
    q = rms_plain(q, eps) * _w(weights, pre + "q.norm")
    k = rms_plain(k, eps) * _w(weights, pre + "k.norm")
    out = torch.zeros(T, H, Dv, dtype=F64)
    for i in range(T):
        js = [j for j in range(i + 1) if (i - j < size or j < keep)]
        for hh in range(H):
            g = hh // (H // G)
            s = (k[js, g] @ q[i, hh]) * m["scale"]
            e = torch.exp(s)
            p = e / (1.0 + e.sum())
            out[i, hh] = p @ v[js, g]
    gate = torch.sigmoid(h @ _w(weights, pre + "g").T)
    return (out.reshape(T, -1) * gate) @ _w(weights, pre + "o").T


def wkv(h: torch.Tensor, weights, pre: str, m: dict, eps: float) -> torch.Tensor:
    T, W = h.shape
    H, D = m["heads"], m["dim"]
    prev = torch.cat([torch.zeros(1, W, dtype=F64), h[:-1]], 0)

    def mix(s):
        return h + (prev - h) * _w(weights, pre + "mu." + s)

    r = (mix("r") @ _w(weights, pre + "r").T).reshape(T, H, D)
    k = (mix("k") @ _w(weights, pre + "k").T).reshape(T, H, D)
    v = (mix("v") @ _w(weights, pre + "v").T).reshape(T, H, D)
    gz = mix("g") @ _w(weights, pre + "g").T
    gate = gz * torch.sigmoid(gz)
    dec = torch.tanh(mix("w") @ _w(weights, pre + "w1").T) @ _w(weights, pre + "w2").T + _w(weights, pre + "w0")
    w = torch.exp(-torch.exp(dec)).reshape(T, H, D)
    u = _w(weights, pre + "u")
    S = torch.zeros(H, D, D, dtype=F64)
    out = torch.zeros(T, H, D, dtype=F64)
    for t in range(T):
        kv = k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hdv,hd->hv", S + u[:, :, None] * kv, r[t])
        S = w[t][:, :, None] * S + kv
    o = rms_plain(out, eps).reshape(T, -1) * _w(weights, pre + "norm") * gate
    return o @ _w(weights, pre + "o").T


def mlstm(h: torch.Tensor, weights, pre: str, m: dict, eps: float) -> torch.Tensor:
    T = h.shape[0]
    H, D, Dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ _w(weights, pre + "q").T).reshape(T, H, D) * D ** -0.5
    k = (h @ _w(weights, pre + "k").T).reshape(T, H, D)
    v = (h @ _w(weights, pre + "v").T).reshape(T, H, Dv)
    ig = cap * torch.tanh((h @ _w(weights, pre + "i").T + _w(weights, pre + "i.b")) / cap)
    fg = torch.nn.functional.logsigmoid(
        cap * torch.tanh((h @ _w(weights, pre + "f").T + _w(weights, pre + "f.b")) / cap))
    S = torch.zeros(H, D, Dv, dtype=F64)
    n = torch.zeros(H, D, dtype=F64)
    mx = torch.zeros(H, dtype=F64)
    out = torch.zeros(T, H, Dv, dtype=F64)
    for t in range(T):
        m_new = torch.maximum(fg[t] + mx, ig[t])
        a = torch.exp(fg[t] + mx - m_new)
        b = torch.exp(ig[t] - m_new)
        S = a[:, None, None] * S + b[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = a[:, None] * n + b[:, None] * k[t]
        mx = m_new
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-mx)) + 1e-6
        out[t] = torch.einsum("hdv,hd->hv", S, q[t]) / den[:, None]
    gate = torch.sigmoid(h @ _w(weights, pre + "g").T)
    o = rms_plain(out, eps).reshape(T, -1) * _w(weights, pre + "norm") * gate
    return o @ _w(weights, pre + "o").T


def dense_ff(h: torch.Tensor, weights, pre: str, mlp: dict) -> torch.Tensor:
    lim = mlp["limit"]
    g = torch.clamp(h @ _w(weights, pre + "gate").T, max=lim)
    u = torch.clamp(h @ _w(weights, pre + "up").T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ _w(weights, pre + "down").T


def route(z: torch.Tensor, correction: torch.Tensor, top: int, group_count: int, group_keep: int):
    """One token's expert choice: softmax scores, choice = score + correction,
    only the best groups (by their largest choice score) stay eligible, the
    top choices win; weights are the plain scores renormalised."""
    s = torch.softmax(z, -1)
    c = s + correction
    n = c.numel()
    per = n // group_count
    gs = c.reshape(group_count, per).max(-1).values
    best = torch.topk(gs, group_keep).indices.tolist()
    allowed = [e for e in range(n) if e // per in best]
    allowed.sort(key=lambda e: (-float(c[e]), e))
    chosen = allowed[:top]
    wsum = sum(float(s[e]) for e in chosen) + 1e-20
    return chosen, [float(s[e]) / wsum for e in chosen]


def moe_ff(h: torch.Tensor, weights, pre: str, mlp: dict) -> torch.Tensor:
    r = mlp["router"]
    E, ident = r["experts"], r.get("identity", 0)
    z = h @ _w(weights, pre + "router").T
    corr = _w(weights, pre + "correction")
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        chosen, ws = route(z[t], corr, r["top"], r["groups"]["count"], r["groups"]["keep"])
        for e, wt in zip(chosen, ws):
            if e >= E:
                out[t] += wt * h[t]
                continue
            a = h[t] @ _w(weights, f"{pre}e{e}.gate").T
            b = h[t] @ _w(weights, f"{pre}e{e}.up").T
            out[t] += wt * ((a * torch.sigmoid(a) * b) @ _w(weights, f"{pre}e{e}.down").T)
    return out


def layer_schedule(cfg):
    """(layer index, starts a pass of the loop) of every layer run, in
    execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, False) for i in range(n)]
    a, b, times = lp["start"], lp["stop"], lp["times"]
    looped = [(i, i == a) for i in range(a, b)] * times
    return [(i, False) for i in range(a)] + looped + [(i, False) for i in range(b, n)]


def forward(tokens: List[int], weights: Dict[str, torch.Tensor], cfg: dict, return_layers: bool = False):
    """Logits [T, vocab] of a whole sequence (float64)."""
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x0 = embed_tokens(tokens, weights, cfg)
    x = x0.clone()
    layers_out = []
    for li, pass_start in layer_schedule(cfg):
        if pass_start:
            x = torch.cat([x, x0], -1) @ _w(weights, "loop.in").T
        spec = cfg["layers"][li]
        pre = f"l{li}."
        h1 = group_rms(x, _w(weights, pre + "norm1"), groups, eps)
        kind = spec["type"]
        if kind == "attention":
            y = attention(h1, weights, pre + "mix.", spec["mixer"], eps)
        elif kind == "wkv":
            y = wkv(h1, weights, pre + "mix.", spec["mixer"], eps)
        elif kind == "mlstm":
            y = mlstm(h1, weights, pre + "mix.", spec["mixer"], eps)
        else:
            raise ValueError(kind)
        mlp = spec.get("mlp")
        if mlp:
            h2 = group_rms(x, _w(weights, pre + "norm2"), groups, eps)
            if mlp["kind"] == "dense":
                y = y + dense_ff(h2, weights, pre + "mlp.", mlp)
            else:
                y = y + moe_ff(h2, weights, pre + "mlp.", mlp)
        x = x + y
        layers_out.append(x.clone())
    hf = group_rms(x, _w(weights, "final.norm"), groups, eps)
    logits = hf @ _w(weights, "head").T
    return (logits, layers_out) if return_layers else logits


def random_weights(cfg: dict, seed: int, decay_rank: int = 5) -> Dict[str, torch.Tensor]:
    """Random checkpoint for a config (values rounded to bfloat16, as a
    checkpoint stores them). Norm weights vary around 1, decays reach far
    back, gate biases are away from 0 so that every term matters."""
    g = torch.Generator().manual_seed(seed)
    W, V = cfg["width"], cfg["vocab"]

    def rn(*shape, std=1.0, mean=0.0):
        return (torch.randn(*shape, generator=g) * std + mean).bfloat16().float()

    def mat(o, i, gain=1.0):
        return rn(o, i, std=gain * i ** -0.5)

    w = {"embed": rn(V, W), "final.norm": rn(W, std=0.1, mean=1.0), "head": mat(V, W)}
    bg = (cfg.get("embedding") or {}).get("bigram")
    if bg:
        w["bigram"] = rn(bg["buckets"] + 1, W, std=0.5)
    if cfg.get("loop"):
        w["loop.in"] = mat(W, 2 * W, gain=1.4)
    for i, sp in enumerate(cfg["layers"]):
        p, m = f"l{i}.", sp["mixer"]
        w[p + "norm1"] = rn(W, std=0.1, mean=1.0)
        q = p + "mix."
        if sp["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            w.update({q + "q": mat(H * D, W), q + "k": mat(G * D, W), q + "v": mat(G * Dv, W),
                      q + "g": mat(H * Dv, W), q + "o": mat(W, H * Dv),
                      q + "q.norm": rn(D, std=0.2, mean=1.0), q + "k.norm": rn(D, std=0.2, mean=1.0)})
        elif sp["type"] == "wkv":
            H, D = m["heads"], m["dim"]
            for s in "rkvgw":
                w[q + "mu." + s] = torch.rand(W, generator=g).bfloat16().float()
            for s in "rkvg":
                w[q + s] = mat(H * D, W)
            w.update({q + "w1": mat(decay_rank, W), q + "w2": mat(H * D, decay_rank),
                      q + "w0": rn(H * D, std=0.8, mean=-2.5), q + "u": rn(H, D, std=0.5),
                      q + "norm": rn(H * D, std=0.1, mean=1.0), q + "o": mat(W, H * D)})
        else:
            H, D, Dv = m["heads"], m["dim"], m["vdim"]
            w.update({q + "q": mat(H * D, W), q + "k": mat(H * D, W), q + "v": mat(H * Dv, W),
                      q + "g": mat(H * Dv, W), q + "o": mat(W, H * Dv), q + "norm": rn(H * Dv, std=0.1, mean=1.0),
                      q + "i": mat(H, W, gain=2.0), q + "i.b": rn(H, std=0.5),
                      q + "f": mat(H, W, gain=2.0), q + "f.b": rn(H, std=0.5, mean=2.0)})
        mlp = sp.get("mlp")
        if not mlp:
            continue
        w[p + "norm2"] = rn(W, std=0.1, mean=1.0)
        q = p + "mlp."
        if mlp["kind"] == "dense":
            w.update({q + "gate": mat(mlp["ff"], W, gain=2.0), q + "up": mat(mlp["ff"], W, gain=2.0),
                      q + "down": mat(W, mlp["ff"])})
        else:
            r = mlp["router"]
            n = r["experts"] + r.get("identity", 0)
            w[q + "router"] = mat(n, W, gain=2.0)
            w[q + "correction"] = rn(n, std=0.1, mean=-0.05)
            ff = mlp["expert"]["ff"]
            for e in range(r["experts"]):
                w.update({f"{q}e{e}.gate": mat(ff, W, gain=1.5), f"{q}e{e}.up": mat(ff, W, gain=1.5),
                          f"{q}e{e}.down": mat(W, ff)})
    return w
