"""Plain, slow float64 implementations of the Pemidra decoder's mechanisms, written from their
equations, one function per mechanism, over whole sequences (no cache, no chunks, no batching,
token-by-token recurrences).  The tests compare the framework against these; nothing here imports
the package.

Notation: T tokens, W model width; linear weights are [out, in] and applied as W x; ``sd`` maps the
checkpoint's tensor names to float64 tensors; ``p`` is a name prefix such as ``l3.mix.``.
"""
import math

import torch

F64 = torch.float64


def rms_unit(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x, w, b, eps):
    mu = x.mean(-1, keepdim=True)
    d = x - mu
    return d / torch.sqrt((d * d).mean(-1, keepdim=True) + eps) * w + b


def silu(x):
    return x * torch.sigmoid(x)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def softplus(x):
    return torch.where(x > 30.0, x, torch.log1p(torch.exp(torch.clamp(x, max=30.0))))


def l2_unit(x):
    return x / torch.sqrt((x * x).sum(-1, keepdim=True) + 1e-6)


def causal_conv(x, w):
    """x [T, C], w [C, taps]; the last column multiplies the current token; zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for k in range(taps):
            src = t - (taps - 1) + k
            if src >= 0:
                y[t] += w[:, k] * x[src]
    return y


# ------------------------------------------------------------------ mixers
def retention(h, sd, p, m, eps):
    """Decayed linear attention: S <- d_h S + k v^T, o = S^T q; no softmax, no denominator."""
    T = h.shape[0]
    H, dk, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ sd[p + "q"].T).view(T, H, dk)
    k = (h @ sd[p + "k"].T).view(T, H, dk) * dk ** -0.5
    v = (h @ sd[p + "v"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = float(m["decay"][hd]) * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = rms_unit(o, eps).reshape(T, H * dv) * silu(h @ sd[p + "g"].T)
    return o @ sd[p + "o"].T


def chunk_softmax_attention(h, sd, p, m, eps):
    """Grouped-query attention inside fixed chunks of positions, q/k RMS-normed with a shared weight,
    partial rotation (rotate-half pairing), unit-RMS values, per-head temperature, a softmax whose
    denominator carries an extra 1, and one sigmoid gate per head."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    size, rd, base = m["mask"]["size"], m["rot"]["dims"], m["rot"]["base"]
    q = rms_unit((h @ sd[p + "q"].T).view(T, H, dk), eps) * sd[p + "q.norm"]
    k = rms_unit((h @ sd[p + "k"].T).view(T, G, dk), eps) * sd[p + "k.norm"]
    v = rms_unit((h @ sd[p + "v"].T).view(T, G, dv), eps)

    def rotate(x):
        y = x.clone()
        half = rd // 2
        for t in range(T):
            for i in range(half):
                a = t * base ** (-2.0 * i / rd)
                c, s = math.cos(a), math.sin(a)
                u, w = x[t, :, i], x[t, :, i + half]
                y[t, :, i] = u * c - w * s
                y[t, :, i + half] = w * c + u * s
        return y

    q, k = rotate(q), rotate(k)
    gate = torch.sigmoid(h @ sd[p + "g"].T)                     # [T, H]
    out = torch.zeros(T, H, dv, dtype=F64)
    for i in range(T):
        lo = (i // size) * size
        for hd in range(H):
            g = hd // (H // G)
            s = (k[lo:i + 1, g] @ q[i, hd]) * m["scale"] * float(sd[p + "temp"][hd])
            e = torch.exp(s)
            w = e / (1.0 + e.sum())
            out[i, hd] = (w[:, None] * v[lo:i + 1, g]).sum(0) * gate[i, hd]
    return out.reshape(T, H * dv) @ sd[p + "o"].T


def gated_delta(h, sd, p, m, eps):
    """Gated delta rule with a decay per head and key channel, short convolutions on q, k, v."""
    T = h.shape[0]
    H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = silu(causal_conv(h @ sd[p + "q"].T, sd[p + "q.conv"])).view(T, G, dk)
    k = silu(causal_conv(h @ sd[p + "k"].T, sd[p + "k.conv"])).view(T, G, dk)
    v = silu(causal_conv(h @ sd[p + "v"].T, sd[p + "v.conv"])).view(T, H, dv)
    q = l2_unit(q) * dk ** -0.5
    k = l2_unit(k)
    beta = torch.sigmoid(h @ sd[p + "b"].T)                     # [T, H]
    dt = softplus((h @ sd[p + "a1"].T) @ sd[p + "a2"].T + sd[p + "dt_bias"]).view(T, H, dk)
    g = torch.exp(-torch.exp(sd[p + "A_log"]).view(1, H, 1) * dt)
    o = torch.zeros(T, H, dv, dtype=F64)
    for hd in range(H):
        kh = hd // (H // G)
        S = torch.zeros(dk, dv, dtype=F64)
        for t in range(T):
            S = g[t, hd][:, None] * S
            u = beta[t, hd] * (v[t, hd] - S.T @ k[t, kh])
            S = S + torch.outer(k[t, kh], u)
            o[t, hd] = S.T @ q[t, kh]
    gate = torch.sigmoid((h @ sd[p + "g1"].T) @ sd[p + "g2"].T).view(T, H, dv)
    o = rms_unit(o, eps) * sd[p + "norm"] * gate
    return o.reshape(T, H * dv) @ sd[p + "o"].T


def parallel_mixer(h, sd, p, m, eps):
    """Attention and gated delta rule side by side on the same input; each result RMS-normed over the
    model width with its own weight; half their sum."""
    left = chunk_softmax_attention(h, sd, p + "left.", m["left"], eps)
    right = gated_delta(h, sd, p + "right.", m["right"], eps)
    return 0.5 * (rms_unit(left, eps) * sd[p + "left.out"] + rms_unit(right, eps) * sd[p + "right.out"])


def general_delta(h, sd, p, m, eps):
    """Generalized delta rule: decay and removal rate per head and key channel, both reading the old
    state: S <- diag(w) S - (a u)(u^T S) + k v^T with u the unit key; o = S^T r."""
    T = h.shape[0]
    H, d = m["heads"], m["dim"]
    r = (h @ sd[p + "r"].T).view(T, H, d)
    k = (h @ sd[p + "k"].T).view(T, H, d)
    v = (h @ sd[p + "v"].T).view(T, H, d)
    w = torch.exp(-math.exp(-0.5) * torch.sigmoid(torch.tanh(h @ sd[p + "w1"].T) @ sd[p + "w2"].T + sd[p + "w0"])).view(T, H, d)
    a = torch.sigmoid(h @ sd[p + "a"].T + sd[p + "a.b"]).view(T, H, d)
    u = l2_unit(k)
    o = torch.zeros(T, H, d, dtype=F64)
    for hd in range(H):
        S = torch.zeros(d, d, dtype=F64)
        for t in range(T):
            S = w[t, hd][:, None] * S - torch.outer(a[t, hd] * u[t, hd], S.T @ u[t, hd]) + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ r[t, hd]
    o = rms_unit(o, eps).reshape(T, H * d) * sd[p + "norm"] * torch.sigmoid(h @ sd[p + "g"].T)
    return o @ sd[p + "o"].T


MIXERS = {"retention": retention, "parallel": parallel_mixer, "general_delta": general_delta}


def feed_forward(h, sd, p):
    return (gelu_tanh(h @ sd[p + "gate"].T) * (h @ sd[p + "up"].T)) @ sd[p + "down"].T


# ------------------------------------------------------------------ the decoder
def forward(cfg: dict, sd: dict, tokens, taps: list = None):
    """cfg: the checkpoint's config as a dict -> logits [T, vocab] (float64) of one whole sequence.
    Post-norm layers: x <- LN1(alpha x + ls1 * mixer(x)); x <- LN2(alpha x + ls2 * ff(x))."""
    sd = {k: v.to(F64) for k, v in sd.items()}
    eps, alpha = cfg["norm"]["eps"], cfg["postln_alpha"]
    x = sd["embed"][torch.as_tensor(tokens, dtype=torch.long)]
    for i, L in enumerate(cfg["layers"]):
        b = f"l{i}."
        y = MIXERS[L["type"]](x, sd, b + "mix.", L["mixer"], eps) * sd[b + "ls1"]
        x = layer_norm(alpha * x + y, sd[b + "norm1"], sd[b + "norm1.b"], eps)
        if L.get("mlp"):
            y = feed_forward(x, sd, b + "mlp.") * sd[b + "ls2"]
            x = layer_norm(alpha * x + y, sd[b + "norm2"], sd[b + "norm2.b"], eps)
        if taps is not None:
            taps.append(x.clone())
    x = layer_norm(x, sd["final.norm"], sd["final.norm.b"], eps)
    return x @ sd["head"].T
