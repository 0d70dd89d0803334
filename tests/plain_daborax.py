"""A plain, slow implementation of the Daborax decoder, written from its equations for the tests.

One function per mechanism, whole sequences at once, loops over tokens for the recurrences, dense score
matrices, no cache, no kernels and no code of the package.  Everything runs in one dtype (float64 by default).

Notation: T tokens, d the residual width, W a dict name -> tensor, linear weights [out, in], p a tensor prefix.
"""
import math

import torch


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


# ---- embedding ------------------------------------------------------------------------------------------
def position_vectors(T, width, dtype, base=10000.0, first=0):
    """Entry 2i = sin(p base^(-2i/width)), entry 2i+1 = cos of the same angle."""
    out = torch.zeros(T, width, dtype=dtype)
    for t in range(T):
        for j in range(width):
            i = j // 2
            a = (first + t) * base ** (-2.0 * i / width)
            out[t, j] = math.sin(a) if j % 2 == 0 else math.cos(a)
    return out


def embed(tokens, table, scale):
    x = table[torch.as_tensor(list(tokens), dtype=torch.long)] * scale
    return x + position_vectors(len(tokens), table.shape[1], table.dtype)


# ---- short causal convolution ---------------------------------------------------------------------------
def short_conv(x, w, b):
    """x [T, C], w [C, taps]; the last column multiplies the current token, zeros stand before the start."""
    T, C = x.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], dim=0)
    out = torch.zeros_like(x)
    for t in range(T):
        out[t] = b + (padded[t:t + taps] * w.T).sum(0)
    return out


# ---- state-space mixer ----------------------------------------------------------------------------------
def mamba2_mixer(h, W, p, heads, vdim, state, groups, norm_groups, eps):
    T = h.shape[0]
    inner, gn = heads * vdim, groups * state
    proj = h @ W[p + "in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * gn], proj[:, 2 * inner + 2 * gn:]
    xbc = silu(short_conv(xbc, W[p + "conv"], W[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, heads, vdim)
    B = xbc[:, inner:inner + gn].reshape(T, groups, state)
    C = xbc[:, inner + gn:].reshape(T, groups, state)
    dt = softplus(dt + W[p + "dt_bias"])
    rate = torch.exp(W[p + "A_log"])
    y = torch.zeros(T, heads, vdim, dtype=h.dtype)
    per_group = heads // groups
    for hd in range(heads):
        g = hd // per_group
        S = torch.zeros(state, vdim, dtype=h.dtype)
        for t in range(T):
            S = torch.exp(-rate[hd] * dt[t, hd]) * S + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    part = inner // norm_groups
    y = unit_rms(y.reshape(T, norm_groups, part), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


# ---- linear attention with a decay per head ---------------------------------------------------------------
def lightning_mixer(h, W, p, heads, dim, vdim, decay, eps):
    T = h.shape[0]
    q = silu(h @ W[p + "q"].T).reshape(T, heads, dim)
    k = silu(h @ W[p + "k"].T).reshape(T, heads, dim)
    v = silu(h @ W[p + "v"].T).reshape(T, heads, vdim)
    o = torch.zeros(T, heads, vdim, dtype=h.dtype)
    for hd in range(heads):
        S = torch.zeros(dim, vdim, dtype=h.dtype)
        for t in range(T):
            S = decay[hd] * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o.reshape(T, heads * vdim), eps) * W[p + "norm"]
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


# ---- softmax attention over a window, with a capped score and a learned sink ---------------------------------
def seen(n_queries, n_keys, window, first=0):
    """[queries, keys] True where query at position first + i sees key j: 0 <= (first + i) - j < window (no window: all earlier keys)."""
    i = torch.arange(first, first + n_queries)[:, None]
    j = torch.arange(n_keys)[None, :]
    ok = j <= i
    return ok if window is None else ok & (i - j < window)


def sink_softmax(scores, mask, sink, softcap=None):
    """Weights of the seen keys: the score is capped (cap * tanh(score / cap)), then exp(score) / (exp(sink) + sum exp(score));
    the sink has no key and is neither capped nor scaled.  ``sink`` None: a plain softmax."""
    if softcap:
        scores = softcap * torch.tanh(scores / softcap)
    scores = scores.masked_fill(~mask, float("-inf"))
    m = scores.max(-1, keepdim=True).values
    if sink is not None:
        m = torch.maximum(m, torch.as_tensor(sink, dtype=scores.dtype))
    e = torch.exp(scores - m)
    den = e.sum(-1, keepdim=True)
    if sink is not None:
        den = den + torch.exp(torch.as_tensor(sink, dtype=scores.dtype) - m)
    return e / den


def window_attention(h, W, p, heads, kv_heads, dim, vdim, scale, softcap, window, eps):
    T = h.shape[0]
    q = (h @ W[p + "q"].T + W[p + "q.b"]).reshape(T, heads, dim)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).reshape(T, kv_heads, dim)
    v = (h @ W[p + "v"].T + W[p + "v.b"]).reshape(T, kv_heads, vdim)
    q, k = unit_rms(q, eps), unit_rms(k, eps)
    mask = seen(T, T, window)
    per = heads // kv_heads
    out = []
    for hd in range(heads):
        g = hd // per
        w = sink_softmax((q[:, hd] @ k[:, g].T) * scale, mask, W[p + "sink"][hd], softcap)
        out.append(w @ v[:, g])
    return torch.cat(out, -1) @ W[p + "o"].T + W[p + "o.b"]


# ---- feed-forward -----------------------------------------------------------------------------------------
def clamped_glu(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


# ---- the model ----------------------------------------------------------------------------------------------
def run_mixer(h, W, p, kind, m, eps):
    if kind == "mamba2":
        return mamba2_mixer(h, W, p, m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"], eps)
    if kind == "lightning":
        return lightning_mixer(h, W, p, m["heads"], m["dim"], m["vdim"], m["decay"], eps)
    if kind == "attention":
        mask = m.get("mask") or {}
        return window_attention(h, W, p, m["heads"], m.get("kv_heads") or m["heads"], m["dim"], m.get("vdim") or m["dim"],
                                m["scale"], m.get("softcap"), mask.get("size"), eps)
    raise ValueError(kind)


def forward(cfg, W, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of one whole sequence.  ``layers_out``: a list that receives the residual stream after every layer."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps, mult = cfg["norm"]["eps"], cfg.get("residual_mult", 1.0)
    x = embed(tokens, W["embed"], (cfg.get("embedding") or {}).get("scale", 1.0))
    for i, l in enumerate(cfg["layers"]):
        src = l.get("weights_of", i)
        src = i if src is None else src
        p = "l%d." % src
        y = run_mixer(x, W, p + "mix.", l["type"], l["mixer"], eps)
        x = x + mult * (unit_rms(y, eps) * W[p + "norm1"] * W[p + "ls1"])
        if l.get("mlp"):
            y = clamped_glu(x, W, p + "mlp.", l["mlp"]["limit"])
            x = x + mult * (unit_rms(y, eps) * W[p + "norm2"] * W[p + "ls2"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T


# ---- random weights for the tests ---------------------------------------------------------------------------------
def random_weights(cfg, seed, std=1.0):
    """Every tensor of a configuration, float32: matrices with entries of size std / sqrt(inputs), norm weights and layer
    scales around one, biases, sinks and the recurrences' vectors of order one."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]
    lin = lambda o, i: torch.randn(o, i, generator=g) * (std / math.sqrt(i))
    around_one = lambda n: 1.0 + 0.2 * torch.randn(n, generator=g)
    W = {"embed": 0.5 * torch.randn(cfg["vocab"], d, generator=g), "head": lin(cfg["vocab"], d), "final.norm": around_one(d)}
    for i, l in enumerate(cfg["layers"]):
        if l.get("weights_of") is not None:
            continue
        p, m = "l%d." % i, l["mixer"]
        W[p + "norm1"], W[p + "ls1"] = around_one(d), 0.5 + torch.rand(d, generator=g)
        if l["type"] == "attention":
            H, G = m["heads"], m.get("kv_heads") or m["heads"]
            dk, dv = m["dim"], m.get("vdim") or m["dim"]
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = lin(H * dk, d), lin(G * dk, d), lin(G * dv, d)
            W[p + "mix.q.b"], W[p + "mix.k.b"], W[p + "mix.v.b"] = (0.3 * torch.randn(n, generator=g) for n in (H * dk, G * dk, G * dv))
            W[p + "mix.sink"] = torch.randn(H, generator=g)
            W[p + "mix.o"], W[p + "mix.o.b"] = lin(d, H * dv), 0.3 * torch.randn(d, generator=g)
        elif l["type"] == "lightning":
            H, dk, dv = m["heads"], m["dim"], m.get("vdim") or m["dim"]
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"], W[p + "mix.g"] = lin(H * dk, d), lin(H * dk, d), lin(H * dv, d), lin(H * dv, d)
            W[p + "mix.norm"], W[p + "mix.o"] = around_one(H * dv), lin(d, H * dv)
        else:
            H, P_, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * P_, H * P_ + 2 * G * N
            W[p + "mix.in"] = lin(2 * inner + 2 * G * N + H, d)
            W[p + "mix.conv"] = torch.randn(ch, m["conv"], generator=g) / math.sqrt(m["conv"])
            W[p + "mix.conv.b"] = 0.2 * torch.randn(ch, generator=g)
            W[p + "mix.dt_bias"], W[p + "mix.A_log"] = torch.randn(H, generator=g) - 1.0, 0.5 * torch.randn(H, generator=g)
            W[p + "mix.D"], W[p + "mix.norm"], W[p + "mix.o"] = torch.randn(H, generator=g), around_one(inner), lin(d, inner)
        if l.get("mlp"):
            ff = l["mlp"]["ff"]
            W[p + "norm2"], W[p + "ls2"] = around_one(d), 0.5 + torch.rand(d, generator=g)
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = 2.0 * lin(ff, d), 2.0 * lin(ff, d), lin(d, ff)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in W.items()}      # what a bfloat16 file holds
