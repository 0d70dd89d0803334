"""A plain, slow implementation of the Fizelix decoder, written from its equations for the tests.

One function per mechanism, whole sequences at once, loops over tokens and keys, no cache, no kernels and no
code of the package.  Everything runs in one dtype (float64 by default).

Notation: T tokens, d the residual width, W a dict name -> tensor, linear weights [out, in], p a tensor prefix,
r(z) = z / sqrt(mean(z^2) + eps) over the last axis.
"""
import math

import torch


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


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


# ---- rotation of adjacent pairs ---------------------------------------------------------------------------
def rotate_pairs(x, positions, dims, base):
    """x [T, heads, size]: entries (2i, 2i+1), 2i < dims, turn by the angle position * base^(-2i/dims); the rest stay."""
    out = x.clone()
    for i in range(dims // 2):
        a = torch.as_tensor([pos * base ** (-2.0 * i / dims) for pos in positions], dtype=x.dtype)[:, None]
        c, s = torch.cos(a), torch.sin(a)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


# ---- attention over a window of tokens and the means of the blocks before it --------------------------------
def visible(i, window, block):
    """What query position i sees: (token positions, block numbers).  Tokens j with 0 <= i - j < window; block b
    (positions b*block .. b*block + block - 1) once its last position is <= i - window."""
    tokens = [j for j in range(max(0, i - window + 1), i + 1)]
    blocks = []
    if block:
        b = 0
        while b * block + block - 1 <= i - window:
            blocks.append(b)
            b += 1
    return tokens, blocks


def seen_masks(T, window, block, first=0):
    """([T, first + T] tokens seen, [T, blocks] blocks seen) for queries at positions first .. first + T - 1, from ``visible``."""
    n_keys = first + T
    n_blocks = n_keys // block if (block and window) else 0
    tok = torch.zeros(T, n_keys, dtype=torch.bool)
    blk = torch.zeros(T, n_blocks, dtype=torch.bool)
    for t in range(T):
        tokens, blocks = visible(first + t, window if window else n_keys + 1, block if window else 0)
        tok[t, tokens] = True
        blk[t, blocks] = True
    return tok, blk


def pooled_sigmoid_attention(h, W, p, heads, kv_heads, dim, vdim, scale, window, block, rot_dims, rot_base):
    """Weights are sigmoid(score + bias of the head), for tokens and block means alike, and are not normalised over the
    keys.  ``window`` None: all earlier tokens and no blocks.  Dense score matrices under the masks of ``seen_masks``."""
    T = h.shape[0]
    positions = list(range(T))
    q = (h @ W[p + "q"].T).reshape(T, heads, dim)
    k = (h @ W[p + "k"].T).reshape(T, kv_heads, dim)
    v = (h @ W[p + "v"].T).reshape(T, kv_heads, vdim)
    if rot_dims:
        q, k = rotate_pairs(q, positions, rot_dims, rot_base), rotate_pairs(k, positions, rot_dims, rot_base)
    tok, blk = seen_masks(T, window, block)
    nb = blk.shape[1]
    per = heads // kv_heads
    out = []
    for hd in range(heads):
        g = hd // per
        bias = W[p + "pb"][hd] if (p + "pb") in W else 0.0
        w = torch.sigmoid((q[:, hd] @ k[:, g].T) * scale + bias) * tok
        o = w @ v[:, g]
        if nb:
            k_mean = k[:nb * block, g].reshape(nb, block, dim).mean(1)
            v_mean = v[:nb * block, g].reshape(nb, block, vdim).mean(1)
            o = o + (torch.sigmoid((q[:, hd] @ k_mean.T) * scale + bias) * blk) @ v_mean
        out.append(o)
    return torch.cat(out, -1) @ W[p + "o"].T


# ---- feed-forward -----------------------------------------------------------------------------------------
def gated_unit(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def routed_experts(h, W, p, experts, top, shared):
    """Every token goes to the ``top`` experts with the largest sigmoid(router logit); an expert sees the token times that
    sigmoid (the weight is on the INPUT and is not renormalised).  A shared expert sees every token as it is."""
    T = h.shape[0]
    s = torch.sigmoid(h @ W[p + "router"].T)
    out = torch.zeros(T, W[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(T):
        order = sorted(range(experts), key=lambda e: (-float(s[t, e]), e))[:top]
        for e in order:
            out[t] = out[t] + gated_unit((s[t, e] * h[t])[None], W, "%se%d." % (p, e))[0]
    if shared:
        out = out + gated_unit(h, W, p + "shared.")
    return out


def feed_forward(h, W, p, mlp):
    if mlp.get("kind", "dense") == "dense":
        return gated_unit(h, W, p)
    return routed_experts(h, W, p, mlp["router"]["experts"], mlp["router"]["top"], bool(mlp.get("shared")))


# ---- the model ----------------------------------------------------------------------------------------------
def run_mixer(h, W, p, kind, m, eps):
    if kind == "mamba2":
        return mamba2_mixer(h, W, p, m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"], eps)
    if kind == "attention":
        mask, rot = m.get("mask") or {}, m.get("rot") or {}
        return pooled_sigmoid_attention(h, W, p, m["heads"], m.get("kv_heads") or m["heads"], m["dim"], m.get("vdim") or m["dim"],
                                        m["scale"], mask.get("size"), mask.get("pool") or 0, rot.get("dims") or 0,
                                        rot.get("base") or 10000.0)
    raise ValueError(kind)


def run_order(cfg):
    """(layer, is the first layer of a pass after the first) in the order the layers run."""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = loop["start"], loop["stop"], loop["times"]
    out = [(i, False) for i in range(a)]
    for rep in range(times):
        out += [(i, rep > 0 and i == a) for i in range(a, b)]
    return out + [(i, False) for i in range(b, n)]


def sublayer(x, f, W, p, q, eps):
    """x + ls * r(f(h) * sigmoid(R h + b)) * w_out with h = r(x) * w_in: norms on both sides of the sublayer, a gate made
    from the sublayer's input on its result, a scale per column on the way back."""
    h = unit_rms(x, eps) * W["%snorm%d" % (p, q)]
    y = f(h)
    if "%srg%d" % (p, q) in W:
        y = y * torch.sigmoid(h @ W["%srg%d" % (p, q)].T + W["%srg%d.b" % (p, q)])
    y = unit_rms(y, eps) * W["%snorm%db" % (p, q)]
    if "%sls%d" % (p, q) in W:
        y = y * W["%sls%d" % (p, q)]
    return x + y


def token_side_input(x, tokens, W, p, index, dim, eps):
    """x + r(P (gelu_tanh(G x) * e)) * w, e the layer's slice of the token's row of a second embedding table."""
    e = W["side.embed"][torch.as_tensor(list(tokens), dtype=torch.long)][:, index * dim:(index + 1) * dim]
    g = gelu_tanh(x @ W[p + "side.gate"].T) * e
    return x + unit_rms(g @ W[p + "side.proj"].T, eps) * W[p + "side.norm"]


def forward(cfg, W, tokens, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of one whole sequence.  ``layers_out``: a list that receives the residual stream after every layer run."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    side = (cfg.get("token_side") or {}).get("dim")
    x0 = W["embed"][torch.as_tensor(list(tokens), dtype=torch.long)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    x = x0.clone()
    for i, again in run_order(cfg):
        l = cfg["layers"][i]
        p = "l%d." % i
        if again:
            x = x + x0
        x = sublayer(x, lambda h: run_mixer(h, W, p + "mix.", l["type"], l["mixer"], eps), W, p, 1, eps)
        if l.get("mlp"):
            x = sublayer(x, lambda h: feed_forward(h, W, p + "mlp.", l["mlp"]), W, p, 2, eps)
        if side:
            x = token_side_input(x, tokens, W, p, i, side, eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return (unit_rms(x, eps) * W["final.norm"]) @ W["head"].T * cfg.get("logit_scale", 1.0)


# ---- random weights for the tests ---------------------------------------------------------------------------------
def random_weights(cfg, seed, std=1.0):
    """Every tensor of a configuration, float32 values that bfloat16 holds exactly: matrices with entries of size
    std / sqrt(inputs), norm weights and layer scales around one, biases and the recurrence's vectors of order one."""
    g = torch.Generator().manual_seed(seed)
    d = cfg["width"]
    lin = lambda o, i, s=std: torch.randn(o, i, generator=g) * (s / math.sqrt(i))
    around_one = lambda n: 1.0 + 0.2 * torch.randn(n, generator=g)
    W = {"embed": torch.randn(cfg["vocab"], d, generator=g), "head": lin(cfg["vocab"], d), "final.norm": around_one(d)}
    side = (cfg.get("token_side") or {}).get("dim")
    if side:
        W["side.embed"] = torch.randn(cfg["vocab"], side * len(cfg["layers"]), generator=g)
    for i, l in enumerate(cfg["layers"]):
        p, m = "l%d." % i, l["mixer"]
        subs = (1, 2) if l.get("mlp") else (1,)
        for q in subs:
            W["%snorm%d" % (p, q)], W["%snorm%db" % (p, q)] = around_one(d), around_one(d)
            W["%sls%d" % (p, q)] = 0.5 + torch.rand(d, generator=g)
            W["%srg%d" % (p, q)], W["%srg%d.b" % (p, q)] = lin(d, d, 2.0), 0.5 * torch.randn(d, generator=g)
        if side:
            W[p + "side.gate"], W[p + "side.proj"], W[p + "side.norm"] = lin(side, d, 2.0), lin(d, side), 0.5 * around_one(d)
        if l["type"] == "attention":
            H, G = m["heads"], m.get("kv_heads") or m["heads"]
            dk, dv = m["dim"], m.get("vdim") or m["dim"]
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = lin(H * dk, d, 2.0), lin(G * dk, d, 2.0), lin(G * dv, d)
            W[p + "mix.pb"] = torch.randn(H, generator=g) - 2.0
            W[p + "mix.o"] = lin(d, H * dv)
        else:
            H, P_, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
            inner, ch = H * P_, H * P_ + 2 * G * N
            W[p + "mix.in"] = lin(2 * inner + 2 * G * N + H, d)
            W[p + "mix.conv"] = torch.randn(ch, m["conv"], generator=g) / math.sqrt(m["conv"])
            W[p + "mix.conv.b"] = 0.2 * torch.randn(ch, generator=g)
            W[p + "mix.dt_bias"], W[p + "mix.A_log"] = torch.randn(H, generator=g) - 1.0, 0.5 * torch.randn(H, generator=g)
            W[p + "mix.D"], W[p + "mix.norm"], W[p + "mix.o"] = torch.randn(H, generator=g), around_one(inner), lin(d, inner)
        mlp = l.get("mlp")
        if mlp and mlp.get("kind", "dense") == "dense":
            ff = mlp["ff"]
            W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"] = lin(ff, d, 2.0), lin(ff, d, 2.0), lin(d, ff)
        elif mlp:
            ff = mlp["expert"]["ff"]
            for e in range(mlp["router"]["experts"]):
                q = "%smlp.e%d." % (p, e)
                W[q + "gate"], W[q + "up"], W[q + "down"] = lin(ff, d, 2.0), lin(ff, d, 2.0), lin(d, ff)
            W[p + "mlp.router"] = lin(mlp["router"]["experts"], d, 2.0)
            if mlp.get("shared"):
                ff = mlp["shared"]["ff"]
                q = p + "mlp.shared."
                W[q + "gate"], W[q + "up"], W[q + "down"] = lin(ff, d, 2.0), lin(ff, d, 2.0), lin(d, ff)
    return {k: v.to(torch.bfloat16).to(torch.float32) for k, v in W.items()}
