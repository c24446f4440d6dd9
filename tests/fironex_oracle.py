"""Slow float64 oracle for the Fironex design, one function per mechanism.

Written from the design's equations only; shares no code with the engine.
Every function takes whole sequences (no cache, no state, no batches), so
anything the engine gets wrong through pages, slots, portions or batching
shows as a difference.

Layer i of a model reads tensors `l<i>.*`; `W` is a dict name -> tensor.
"""
import math

import torch

F64 = torch.float64


def d(t):
    return t.to(F64)


# -- small pieces --------------------------------------------------------------
def layer_norm(x, w, eps):
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * d(w)


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1 + torch.tanh(math.sqrt(2 / math.pi)
                                     * (z + 0.044715 * z ** 3)))


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + z.clamp(min=0)


def xielu(z, p, q):
    ap, aq = softplus(p), softplus(q)
    pos = ap * z * z + z / 2
    neg = (0.5 + aq) * (torch.exp(z.clamp(max=0)) - 1 - z) + z / 2
    return torch.where(z > 0, pos, neg)


def rope_freqs(rot):
    """Per-pair angular frequencies, with the optional long-context
    rescaling: long wavelengths are slowed by `factor`, short ones kept,
    and the band between them blends the two."""
    n = rot["dims"]
    f = torch.tensor([rot["base"] ** (-2.0 * i / n) for i in range(n // 2)],
                     dtype=F64)
    sc = rot.get("scaling")
    if sc:
        out = []
        for fi in f.tolist():
            wl = 2 * math.pi / fi
            if wl < sc["original"] / sc["high"]:
                out.append(fi)
            elif wl > sc["original"] / sc["low"]:
                out.append(fi / sc["factor"])
            else:
                s = (sc["original"] / wl - sc["low"]) / (sc["high"] - sc["low"])
                out.append((1 - s) * fi / sc["factor"] + s * fi)
        f = torch.tensor(out, dtype=F64)
    return f


def rotate(x, rot, interleaved):
    """x [T, n_vec, size]: rotate the first rot.dims entries of each vector
    by angle position * f_i; pairs are (2i, 2i+1) when interleaved, else
    (i, i + dims/2)."""
    T = x.shape[0]
    n = rot["dims"]
    f = rope_freqs(rot)
    ang = torch.arange(T, dtype=F64)[:, None] * f[None, :]      # [T, n/2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    y = x.clone()
    if interleaved:
        a, b = x[..., 0:n:2], x[..., 1:n:2]
        y[..., 0:n:2] = a * c - b * s
        y[..., 1:n:2] = b * c + a * s
    else:
        a, b = x[..., :n // 2], x[..., n // 2:n]
        y[..., :n // 2] = a * c - b * s
        y[..., n // 2:n] = b * c + a * s
    return y


def masked_softmax_attention(q, k, v, scale, window):
    """q [T, dk], k [T, dk], v [T, dv]; token i sees j with
    0 <= i - j < window (window None: all j <= i)."""
    T = q.shape[0]
    s = (q @ k.t()) * scale
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    ok = j <= i
    if window is not None:
        ok = ok & (i - j < window)
    s = s.masked_fill(~ok, -math.inf)
    return torch.softmax(s, -1) @ v


# -- mixers --------------------------------------------------------------------
def rglru_mixer(h, W, p, m):
    """Gated linear recurrent unit with a short causal convolution."""
    width, nb, taps = m["width"], m["blocks"], m["conv"]
    T = h.shape[0]
    y = gelu_tanh(h @ d(W[p + "y"]).t() + d(W[p + "y.b"]))
    xin = h @ d(W[p + "x"]).t() + d(W[p + "x.b"])
    cw, cb = d(W[p + "conv"]), d(W[p + "conv.b"])
    pad = torch.cat([torch.zeros(taps - 1, width, dtype=F64), xin], 0)
    u = torch.zeros(T, width, dtype=F64)
    for t in range(T):
        for j in range(taps):       # column taps-1 multiplies the current token
            u[t] += cw[:, j] * pad[t + j]
        u[t] += cb
    bw = width // nb
    r = torch.zeros_like(u)
    g = torch.zeros_like(u)
    for b in range(nb):
        ub = u[:, b * bw:(b + 1) * bw]
        r[:, b * bw:(b + 1) * bw] = torch.sigmoid(
            ub @ d(W[p + "ra"][b]).t() + d(W[p + "ra.b"][b]))
        g[:, b * bw:(b + 1) * bw] = torch.sigmoid(
            ub @ d(W[p + "ri"][b]).t() + d(W[p + "ri.b"][b]))
    log_a = -8.0 * r * softplus(d(W[p + "lam"]))
    a = torch.exp(log_a)
    S = torch.zeros(width, dtype=F64)
    out = torch.zeros(T, width, dtype=F64)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1 - a[t] ** 2) * g[t] * u[t]
        out[t] = S * y[t]
    return out @ d(W[p + "o"]).t()


def differential_attention_mixer(h, W, p, m, eps):
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ d(W[p + "q"]).t()).view(T, H * 2, dk)
    k = (h @ d(W[p + "k"]).t()).view(T, G * 2, dk)
    v = (h @ d(W[p + "v"]).t()).view(T, G, dv)
    q = rotate(q, m["rot"], True).view(T, H, 2, dk)
    k = rotate(k, m["rot"], True).view(T, G, 2, dk)
    window = (m.get("mask") or {}).get("size")
    lam = (math.exp(float((d(W[p + "lq1"]) * d(W[p + "lk1"])).sum()))
           - math.exp(float((d(W[p + "lq2"]) * d(W[p + "lk2"])).sum()))
           + m["diff"])
    gate = torch.sigmoid(h @ d(W[p + "g"]).t()).view(T, H, dv)
    heads = []
    for hh in range(H):
        g = hh // (H // G)
        a1 = masked_softmax_attention(q[:, hh, 0], k[:, g, 0], v[:, g],
                                      m["scale"], window)
        a2 = masked_softmax_attention(q[:, hh, 1], k[:, g, 1], v[:, g],
                                      m["scale"], window)
        o = rms_unit(a1 - lam * a2, eps) * (1 - m["diff"])
        heads.append(o * gate[:, hh])
    return torch.cat(heads, -1) @ d(W[p + "o"]).t()


def latent_kv(h, W, p, m, eps):
    """Compressed keys/values of a latent-attention layer: the normed latent
    [T, rank] and the rotated shared key part [T, rot_dim]."""
    rank, rd = m["kv_rank"], m["rot_dim"]
    z = h @ d(W[p + "dkv"]).t()
    c = rms_unit(z[:, :rank], eps) * d(W[p + "dkv.norm"])
    kr = rotate(z[:, None, rank:rank + rd], m["rot"], False)[:, 0]
    return c, kr


def latent_attention_mixer(h, W, p, m, c, kr):
    H, dk, rd, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ d(W[p + "q"]).t()).view(T, H, dk + rd)
    qn = q[..., :dk]
    qr = rotate(q[..., dk:], m["rot"], False)
    kn = (c @ d(W[p + "uk"]).t()).view(T, H, dk)
    v = (c @ d(W[p + "uv"]).t()).view(T, H, dv)
    gate = torch.sigmoid(h @ d(W[p + "g"]).t())          # [T, H]
    heads = []
    for hh in range(H):
        qq = torch.cat([qn[:, hh], qr[:, hh]], -1)
        kk = torch.cat([kn[:, hh], kr], -1)
        o = masked_softmax_attention(qq, kk, v[:, hh], m["scale"], None)
        heads.append(o * gate[:, hh:hh + 1])
    return torch.cat(heads, -1) @ d(W[p + "o"]).t()


def feed_forward(h, W, p):
    act = d(W[p + "act"])
    return xielu(h @ d(W[p + "up"]).t(), act[0], act[1]) @ d(W[p + "down"]).t()


# -- the model -----------------------------------------------------------------
def forward(cfg, W, tokens, taps=None):
    """Logits [T, vocab] (float64) of one whole sequence. `taps`, a list,
    receives the residual stream after every layer."""
    eps = cfg["norm"]["eps"]
    mult = cfg["residual_mult"]
    x = d(W["embed"])[torch.tensor(tokens)]
    latents = {}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        h = layer_norm(x, W[p + "norm1"], eps)
        if L["type"] == "rglru":
            y = rglru_mixer(h, W, p + "mix.", m)
        elif L["type"] == "attention":
            y = differential_attention_mixer(h, W, p + "mix.", m, eps)
        elif L["type"] == "latent_attention":
            src = m.get("kv_from")
            if src is None:
                latents[i] = latent_kv(h, W, p + "mix.", m, eps)
                src = i
            y = latent_attention_mixer(h, W, p + "mix.", m, *latents[src])
        else:
            raise ValueError(L["type"])
        x = x + mult * layer_norm(y, W[p + "norm1b"], eps)
        if L.get("mlp"):
            h = layer_norm(x, W[p + "norm2"], eps)
            x = x + mult * layer_norm(feed_forward(h, W, p + "mlp."),
                                      W[p + "norm2b"], eps)
        if taps is not None:
            taps.append(x.clone())
    x = layer_norm(x, W["final.norm"], eps)
    return x @ d(W["embed"]).t()
