"""Plain, slow model of the Bolatar design, one function per mechanism.

Written directly from the design's equations with explicit loops over
tokens and heads, in float64, for one sequence at a time. It shares no code
with dynamo_amd: the tests compare the engine against this file.

Weights are a dict name -> tensor under the checkpoint's tensor names
(`embed`, `pos`, `l<i>.norm1`, `l<i>.mix.*`, `l<i>.mlp.*`, `final.norm`,
`head`); `cfg` is the parsed config.json dictionary.
"""
import math

import torch

F64 = torch.float64


def _sig(x):
    return 1.0 / (1.0 + torch.exp(-x))


def _silu(x):
    return x * _sig(x)


def _softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def _logsig(x):
    return -_softplus(-x)


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def causal_conv_silu(x, w):
    """x [T, C]; w [C, taps], last column weighs the current token."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros_like(x)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * x[s]
    return _silu(y)


def delta_mixer(h, W, p, m, eps):
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = causal_conv_silu(h @ W[p + "q"].T, W[p + "q.conv"]).view(T, G, dk)
    k = causal_conv_silu(h @ W[p + "k"].T, W[p + "k.conv"]).view(T, G, dk)
    v = causal_conv_silu(h @ W[p + "v"].T, W[p + "v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = _sig(h @ W[p + "b"].T)
    g = torch.exp(-torch.exp(W[p + "A_log"]) *
                  _softplus(h @ W[p + "a"].T + W[p + "dt_bias"]))
    gate = _silu(h @ W[p + "g"].T).view(T, H, dv)
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        kv = hh // (H // G)
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = g[t, hh] * S
            u = beta[t, hh] * (v[t, hh] - S.T @ k[t, kv])
            S = S + torch.outer(k[t, kv], u)
            out[t, hh] = S.T @ q[t, kv]
    out = rms(out, eps) * W[p + "norm"] * gate
    return out.reshape(T, H * dv) @ W[p + "o"].T


def biased_attention(h, W, p, m, eps):
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, dk)
    k = (h @ W[p + "k"].T).view(T, G, dk)
    v = rms((h @ W[p + "v"].T).view(T, G, dv), eps)
    coef, every = m["q_temp"]["coef"], m["q_temp"]["every"]
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        temp = 1.0 + coef * math.log(math.floor((i + 1) / every) + 1)
        for hh in range(H):
            kv = hh // (H // G)
            r1, r2 = W[p + "r1"][hh], W[p + "r2"][hh]
            dist = (i - torch.arange(i + 1)).to(F64)
            s = (k[:i + 1, kv] @ (q[i, hh] * temp)) * m["scale"] \
                - r1 * torch.log(1 + r2 * dist)
            a = torch.softmax(s, 0)
            out[i, hh] = a @ v[:i + 1, kv]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def rwkv_mixer(h, W, p, m, eps):
    H, d = m["heads"], m["dim"]
    T = h.shape[0]
    prev = torch.cat([torch.zeros_like(h[:1]), h[:-1]], 0)

    def mix(s):
        return h + (prev - h) * W[p + "mu." + s]
    r = (mix("r") @ W[p + "r"].T).view(T, H, d)
    k = (mix("k") @ W[p + "k"].T).view(T, H, d)
    v = (mix("v") @ W[p + "v"].T).view(T, H, d)
    gate = _silu(mix("g") @ W[p + "g"].T)
    w = torch.exp(-torch.exp(
        torch.tanh(mix("w") @ W[p + "w1"].T) @ W[p + "w2"].T + W[p + "w0"]
    )).view(T, H, d)
    u = W[p + "u"]
    out = torch.zeros(T, H, d, dtype=F64)
    for hh in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(T):
            kv = torch.outer(k[t, hh], v[t, hh])
            out[t, hh] = (S + u[hh][:, None] * kv).T @ r[t, hh]
            S = w[t, hh][:, None] * S + kv
    out = rms(out, eps).reshape(T, H * d) * W[p + "norm"] * gate
    return out @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    a = biased_attention(h, W, p + "left.", m["left"], eps)
    b = rwkv_mixer(h, W, p + "right.", m["right"], eps)
    return 0.5 * (rms(a, eps) * W[p + "left.out"] +
                  rms(b, eps) * W[p + "right.out"])


def mlstm_mixer(h, W, p, m, eps):
    H, dk, dv, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    T = h.shape[0]
    q = (h @ W[p + "q"].T).view(T, H, dk) * dk ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, dk)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    ig = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    fg = _logsig(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    out = torch.zeros(T, H, dv, dtype=F64)
    for hh in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        n = torch.zeros(dk, dtype=F64)
        mx = torch.zeros((), dtype=F64)
        for t in range(T):
            new = torch.maximum(fg[t, hh] + mx, ig[t, hh])
            a, b = torch.exp(fg[t, hh] + mx - new), torch.exp(ig[t, hh] - new)
            S = a * S + b * torch.outer(k[t, hh], v[t, hh])
            n = a * n + b * k[t, hh]
            mx = new
            den = torch.maximum((n @ q[t, hh]).abs(), torch.exp(-mx)) + 1e-6
            out[t, hh] = S.T @ q[t, hh] / den
    out = rms(out, eps).reshape(T, H * dv) * W[p + "norm"] * _sig(h @ W[p + "g"].T)
    return out @ W[p + "o"].T


def feed_forward(h, W, p, m):
    lim = m["limit"]
    g = torch.clamp(h @ W[p + "gate"].T, max=lim)
    u = torch.clamp(h @ W[p + "up"].T, -lim, lim)
    return (g * _sig(1.702 * g) * (u + 1)) @ W[p + "down"].T


MIXERS = {"delta": delta_mixer, "parallel": parallel_mixer, "mlstm": mlstm_mixer}


def forward(cfg, weights, tokens, return_layers=False):
    """Logits [T, vocab] (float64) of one sequence given from its start."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    tok = torch.as_tensor(tokens, dtype=torch.long)
    x = W["embed"][tok] * cfg["embedding"]["scale"] + W["pos"][:len(tok)]
    layers = []
    for i, L in enumerate(cfg["layers"]):
        p = "l%d." % i
        x = x + MIXERS[L["type"]](rms(x, eps) * W[p + "norm1"], W,
                                  p + "mix.", L["mixer"], eps)
        if L.get("mlp"):
            x = x + feed_forward(rms(x, eps) * W[p + "norm2"], W, p + "mlp.",
                                 L["mlp"])
        layers.append(x)
    x = rms(x, eps) * W["final.norm"]
    logits = x @ W["head"].T
    cap = cfg["logit_softcap"]
    logits = cap * torch.tanh(logits / cap)
    return (logits, torch.stack(layers)) if return_layers else logits
