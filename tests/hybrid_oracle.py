"""Plain, slow oracle for the Zutalix design: one function per mechanism,
token-by-token loops, float64 throughout. It shares no code with the product
path (kllms_amd.models / kllms_amd.ops); tests build small random models and
compare the engine against these functions.

Notation: x is the residual stream [L, W] of ONE sequence (positions 0..L-1),
``w`` a dict name -> float64 tensor, ``cfg`` the parsed config dict.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_w(x, weight, eps):
    return rms(x, eps) * weight


def silu(x):
    return x * torch.sigmoid(x)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


# --- rotary ---------------------------------------------------------------

def rotary_freqs(rot):
    dims = int(rot["dims"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        if sc:
            wavelen = 2 * math.pi / f
            orig, lo, hi, fac = float(sc["original"]), float(sc["low"]), float(sc["high"]), float(sc["factor"])
            if wavelen < orig / hi:
                pass
            elif wavelen > orig / lo:
                f = f / fac
            else:
                s = (orig / wavelen - lo) / (hi - lo)
                f = (1 - s) * f / fac + s * f
        out.append(f)
    return out


def rotate_pairs(x, pos, freqs):
    """x [heads, dim] at position pos; interleaved pairs (2i, 2i+1) of the
    first 2*len(freqs) dims rotate, the rest pass through."""
    y = x.clone()
    for i, f in enumerate(freqs):
        a = pos * f
        c, s = math.cos(a), math.sin(a)
        u, v = x[:, 2 * i], x[:, 2 * i + 1]
        y[:, 2 * i] = u * c - v * s
        y[:, 2 * i + 1] = v * c + u * s
    return y


# --- mixers -----------------------------------------------------------------

def chunk_softmax_attention(h, w, pre, m, eps):
    """Left branch: GQA softmax attention whose values are the un-rotated
    keys, visibility limited to the query's own aligned block of mask.size
    positions, per-head sigmoid output gate."""
    L = h.shape[0]
    H, G, D = m["heads"], m["kv_heads"], m["dim"]
    q = (h @ w[pre + "q"].T + w[pre + "q.b"]).view(L, H, D)
    k = (h @ w[pre + "k"].T + w[pre + "k.b"]).view(L, G, D)
    gate = torch.sigmoid(h @ w[pre + "g"].T)  # [L, H]
    freqs = rotary_freqs(m["rot"])
    qr = torch.stack([rotate_pairs(q[t], t, freqs) for t in range(L)])
    kr = torch.stack([rotate_pairs(k[t], t, freqs) for t in range(L)])
    size = int(m["mask"]["size"])
    out = torch.zeros(L, H, D, dtype=F64)
    for t in range(L):
        lo = (t // size) * size
        for hh in range(H):
            g = hh // (H // G)
            s = (kr[lo:t + 1, g] @ qr[t, hh]) * float(m["scale"])
            p = torch.softmax(s, 0)
            out[t, hh] = (p[:, None] * k[lo:t + 1, g]).sum(0) * gate[t, hh]
    return out.reshape(L, H * D) @ w[pre + "o"].T


def decayed_linear_attention(h, w, pre, m, eps):
    """Right branch: S_t = decay_h S_{t-1} + k_t v_t^T; o_t = S_t^T q_t."""
    L = h.shape[0]
    H, D, V = m["heads"], m["dim"], m["vdim"]
    q = silu(h @ w[pre + "q"].T).view(L, H, D)
    k = silu(h @ w[pre + "k"].T).view(L, H, D)
    v = silu(h @ w[pre + "v"].T).view(L, H, V)
    S = torch.zeros(H, D, V, dtype=F64)
    o = torch.zeros(L, H, V, dtype=F64)
    for t in range(L):
        for hh in range(H):
            S[hh] = float(m["decay"][hh]) * S[hh] + torch.outer(k[t, hh], v[t, hh])
            o[t, hh] = S[hh].T @ q[t, hh]
    y = rms_w(o.reshape(L, H * V), w[pre + "norm"], eps) * torch.sigmoid(h @ w[pre + "g"].T)
    return y @ w[pre + "o"].T


def parallel_mixer(h, w, pre, m, eps):
    left = chunk_softmax_attention(h, w, pre + "left.", m["left"], eps)
    right = decayed_linear_attention(h, w, pre + "right.", m["right"], eps)
    return 0.5 * (rms_w(left, w[pre + "left.out"], eps) + rms_w(right, w[pre + "right.out"], eps))


def short_conv_silu(x, taps_w):
    """x [L, C], taps_w [C, K]; last column multiplies the current token."""
    L, C = x.shape
    K = taps_w.shape[1]
    y = torch.zeros_like(x)
    for t in range(L):
        for j in range(K):
            src = t - (K - 1 - j)
            if src >= 0:
                y[t] += taps_w[:, j] * x[src]
    return silu(y)


def channel_delta_mixer(h, w, pre, m, eps):
    L = h.shape[0]
    H, G, D, V = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = short_conv_silu(h @ w[pre + "q"].T, w[pre + "q.conv"]).view(L, G, D)
    k = short_conv_silu(h @ w[pre + "k"].T, w[pre + "k.conv"]).view(L, G, D)
    v = short_conv_silu(h @ w[pre + "v"].T, w[pre + "v.conv"]).view(L, H, V)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * D ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w[pre + "b"].T)  # [L, H]
    a = (h @ w[pre + "a1"].T) @ w[pre + "a2"].T + w[pre + "dt_bias"]
    decay = torch.exp(-torch.exp(w[pre + "A_log"])[None, :, None] * softplus(a).view(L, H, D))
    S = torch.zeros(H, D, V, dtype=F64)
    o = torch.zeros(L, H, V, dtype=F64)
    for t in range(L):
        for hh in range(H):
            g = hh // (H // G)
            S[hh] = decay[t, hh][:, None] * S[hh]
            u = beta[t, hh] * (v[t, hh] - S[hh].T @ k[t, g])
            S[hh] = S[hh] + torch.outer(k[t, g], u)
            o[t, hh] = S[hh].T @ q[t, g]
    gate = torch.sigmoid((h @ w[pre + "g1"].T) @ w[pre + "g2"].T).view(L, H, V)
    y = rms(o, eps) * w[pre + "norm"] * gate
    return y.reshape(L, H * V) @ w[pre + "o"].T


def clamped_glu(h, w, pre, mlp):
    lim = float(mlp["limit"])
    g = torch.clamp(h @ w[pre + "gate"].T, max=lim)
    u = torch.clamp(h @ w[pre + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1)) @ w[pre + "down"].T


# --- whole model ------------------------------------------------------------

MIXERS = {"parallel": parallel_mixer, "channel_delta": channel_delta_mixer}


def forward(cfg, w, tokens, return_layers=False):
    """Logits [L, vocab] of one sequence (float64)."""
    eps = float(cfg["norm"]["eps"])
    w = {k: v.to(F64) if v.is_floating_point() else v for k, v in w.items()}
    x = rms_w(w["embed"][torch.tensor(tokens)], w["embed.norm"], eps)
    layers = []
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[spec["type"]](rms_w(x, w[p + "norm1"], eps), w, p + "mix.", spec["mixer"], eps)
        x = x + rms_w(y, w[p + "norm1b"], eps)
        if spec.get("mlp"):
            y = clamped_glu(rms_w(x, w[p + "norm2"], eps), w, p + "mlp.", spec["mlp"])
            x = x + rms_w(y, w[p + "norm2b"], eps)
        layers.append(x)
    logits = rms_w(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(layers)) if return_layers else logits


def random_weights(cfg, seed=0, scale=1.0):
    """Random bf16-representable weights for a config dict (names as the
    checkpoint format uses them)."""
    g = torch.Generator().manual_seed(seed)
    W = cfg["width"]
    w = {}

    def lin(name, out, inp, s=None):
        s = s if s is not None else scale / math.sqrt(inp)
        w[name] = (torch.randn(out, inp, generator=g) * s).bfloat16().float()

    def vec(name, n, mean=1.0, std=0.1):
        w[name] = (mean + std * torch.randn(n, generator=g)).bfloat16().float()

    lin("embed", cfg["vocab"], W, 1.0)
    vec("embed.norm", W)
    for i, spec in enumerate(cfg["layers"]):
        p = f"l{i}."
        m = spec["mixer"]
        vec(p + "norm1", W)
        vec(p + "norm1b", W)
        if spec["type"] == "parallel":
            le, ri = m["left"], m["right"]
            lin(p + "mix.left.q", le["heads"] * le["dim"], W)
            vec(p + "mix.left.q.b", le["heads"] * le["dim"], 0.0, 0.2)
            lin(p + "mix.left.k", le["kv_heads"] * le["dim"], W)
            vec(p + "mix.left.k.b", le["kv_heads"] * le["dim"], 0.0, 0.2)
            lin(p + "mix.left.g", le["heads"], W)
            lin(p + "mix.left.o", W, le["heads"] * le["vdim"])
            lin(p + "mix.right.q", ri["heads"] * ri["dim"], W)
            lin(p + "mix.right.k", ri["heads"] * ri["dim"], W)
            lin(p + "mix.right.v", ri["heads"] * ri["vdim"], W)
            lin(p + "mix.right.g", ri["heads"] * ri["vdim"], W)
            lin(p + "mix.right.o", W, ri["heads"] * ri["vdim"])
            vec(p + "mix.right.norm", ri["heads"] * ri["vdim"])
            vec(p + "mix.left.out", W)
            vec(p + "mix.right.out", W)
        else:
            H, G, D, V, K = m["heads"], m["kv_heads"], m["dim"], m["vdim"], m["conv"]
            r = max(4, W // 16)
            for n, c in (("q", G * D), ("k", G * D), ("v", H * V)):
                lin(p + "mix." + n, c, W)
                w[p + f"mix.{n}.conv"] = (torch.randn(c, K, generator=g) * 0.5).bfloat16().float()
            lin(p + "mix.b", H, W)
            vec(p + "mix.A_log", H, 0.0, 0.5)
            vec(p + "mix.norm", V)
            lin(p + "mix.a1", r, W)
            lin(p + "mix.a2", H * D, r)
            vec(p + "mix.dt_bias", H * D, 0.0, 0.5)
            lin(p + "mix.g1", r, W)
            lin(p + "mix.g2", H * V, r)
            lin(p + "mix.o", W, H * V)
        if spec.get("mlp"):
            ff = spec["mlp"]["ff"]
            vec(p + "norm2", W)
            vec(p + "norm2b", W)
            lin(p + "mlp.gate", ff, W)
            lin(p + "mlp.up", ff, W)
            lin(p + "mlp.down", W, ff)
    vec("final.norm", W)
    lin("head", cfg["vocab"], W)
    return w
