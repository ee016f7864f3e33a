"""Plain, slow float64 implementations of the hybrid decoder's mechanisms, written from their
equations, one function per mechanism, over whole sequences (no cache, no chunks, no batching).
The tests compare the framework against these; nothing here imports the package.

Notation: T tokens, W model width; linear weights are [out, in] and applied as W x.
"""
import math

import torch

F64 = torch.float64


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_rmsnorm(x, w, eps):
    """RMS norm whose weight is stored around zero."""
    return unit_rms(x, eps) * (1.0 + w)


def sigmoid_attention(h, wq, bq, wk, bk, wv, bv, wo, bo, r1, r2, pb, heads, kv_heads, dim, vdim, scale, eps):
    """Causal, unnormalised: weight(i, j) = sigmoid(scale q_i.k_j - r1 ln(1 + r2 (i - j)) + pb), j <= i,
    with q and k scaled to unit RMS per head."""
    T = h.shape[0]
    q = unit_rms((h @ wq.T + bq).view(T, heads, dim), eps)
    k = unit_rms((h @ wk.T + bk).view(T, kv_heads, dim), eps)
    v = (h @ wv.T + bv).view(T, kv_heads, vdim)
    rep = heads // kv_heads
    out = torch.zeros(T, heads, vdim, dtype=F64)
    for i in range(T):
        for hd in range(heads):
            g = hd // rep
            for j in range(i + 1):
                s = float(q[i, hd] @ k[j, g]) * scale - float(r1[hd]) * math.log(1.0 + float(r2[hd]) * (i - j))
                out[i, hd] += 1.0 / (1.0 + math.exp(-(s + float(pb[hd])))) * v[j, g]
    return out.reshape(T, heads * vdim) @ wo.T + bo


def sigmoid_attention_fast(h, wq, bq, wk, bk, wv, bv, wo, bo, r1, r2, pb, heads, kv_heads, dim, vdim, scale, eps):
    """The same as :func:`sigmoid_attention` with the three loops written as tensor products (for the
    longer sequences; test_oracle_forms_agree checks the two against each other)."""
    T = h.shape[0]
    q = unit_rms((h @ wq.T + bq).view(T, heads, dim), eps)
    k = unit_rms((h @ wk.T + bk).view(T, kv_heads, dim), eps).repeat_interleave(heads // kv_heads, 1)
    v = (h @ wv.T + bv).view(T, kv_heads, vdim).repeat_interleave(heads // kv_heads, 1)
    i = torch.arange(T).view(T, 1)
    j = torch.arange(T).view(1, T)
    dist = (i - j).clamp(min=0).to(F64)
    s = torch.einsum("ihd,jhd->hij", q, k) * scale - r1.view(-1, 1, 1) * torch.log(1.0 + r2.view(-1, 1, 1) * dist)
    w = torch.sigmoid(s + pb.view(-1, 1, 1)) * (j <= i)
    return torch.einsum("hij,jhd->ihd", w, v).reshape(T, heads * vdim) @ wo.T + bo


def causal_conv_silu(x, w, b):
    """x [T, C], w [C, taps] (last column multiplies the current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    y = torch.zeros(T, C, dtype=F64)
    for t in range(T):
        for k in range(taps):
            src = t - (taps - 1) + k
            if src >= 0:
                y[t] += w[:, k] * x[src]
    y = y + b
    return y * torch.sigmoid(y)


def mamba2(h, w_in, conv_w, conv_b, dt_bias, a_log, d_skip, norm_w, w_out, heads, vdim, state, groups, norm_groups, eps):
    """[z | x B C | dt] = W_in h; conv + silu over x B C; dt = softplus(dt + bias); per head
    S <- exp(-exp(a_log) dt) S + dt B x^T, y = S^T C + D x; out = W_out (grouprms(y silu(z)) * norm_w)."""
    T = h.shape[0]
    inner, gn = heads * vdim, groups * state
    u = h @ w_in.T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * gn], u[:, 2 * inner + 2 * gn:]
    xbc = causal_conv_silu(xbc, conv_w, conv_b)
    x = xbc[:, :inner].view(T, heads, vdim)
    B = xbc[:, inner:inner + gn].view(T, groups, state)
    C = xbc[:, inner + gn:].view(T, groups, state)
    dt = torch.log1p(torch.exp(dt + dt_bias))
    y = torch.zeros(T, heads, vdim, dtype=F64)
    per = heads // groups
    for hd in range(heads):
        S = torch.zeros(state, vdim, dtype=F64)
        g = hd // per
        for t in range(T):
            S = math.exp(-math.exp(float(a_log[hd])) * float(dt[t, hd])) * S + float(dt[t, hd]) * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S.T @ C[t, g] + d_skip[hd] * x[t, hd]
    y = y.reshape(T, inner) * (z * torch.sigmoid(z))
    y = unit_rms(y.view(T, norm_groups, inner // norm_groups), eps).reshape(T, inner) * norm_w
    return y @ w_out.T


def dense_ff(h, w_gate, w_up, w_down):
    g = h @ w_gate.T
    return (g * torch.sigmoid(g) * (h @ w_up.T)) @ w_down.T


def layer_runs(n_layers, loop):
    """[(layer, add the embedding output first)]: layers loop.start .. loop.stop - 1 run loop.times
    times in a row."""
    a, b, t = (loop["start"], loop["stop"], loop["times"]) if loop else (0, 0, 1)
    runs = [(i, False) for i in range(a)]
    for k in range(t):
        runs += [(i, k > 0 and i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n_layers)]


def forward(cfg, sd, tokens, streams=None):
    """cfg: the checkpoint's config dict; sd: name -> tensor (any float dtype).  Returns f64 logits
    [T, vocab]; ``streams`` (a list) receives the residual stream after every layer run."""
    W = {k: v.to(F64) for k, v in sd.items()}
    eps, m = cfg["norm"]["eps"], cfg["residual_mult"]
    T = len(tokens)
    x = W["embed"][torch.as_tensor(tokens)] + W["pos"][:T]
    emb = x.clone()
    for li, add in layer_runs(len(cfg["layers"]), cfg.get("loop")):
        if add:
            x = x + emb
        spec, p = cfg["layers"][li], f"l{li}."
        mx, a = spec["mixer"], p + "mix."
        h = offset_rmsnorm(x, W[p + "norm1"], eps)
        if spec["type"] == "attention":
            y = sigmoid_attention_fast(h, W[a + "q"], W[a + "q.b"], W[a + "k"], W[a + "k.b"], W[a + "v"], W[a + "v.b"],
                                       W[a + "o"], W[a + "o.b"], W[a + "r1"], W[a + "r2"], W[a + "pb"], mx["heads"],
                                       mx["kv_heads"], mx["dim"], mx["vdim"], mx["scale"], eps)
        else:
            y = mamba2(h, W[a + "in"], W[a + "conv"], W[a + "conv.b"], W[a + "dt_bias"], W[a + "A_log"], W[a + "D"],
                       W[a + "norm"], W[a + "o"], mx["heads"], mx["vdim"], mx["state"], mx["groups"], mx["norm_groups"], eps)
        if spec.get("mlp"):
            y = y + dense_ff(h, W[p + "mlp.gate"], W[p + "mlp.up"], W[p + "mlp.down"])
        x = x + m * y
        if streams is not None:
            streams.append(x.clone())
    z = offset_rmsnorm(x, W["final.norm"], eps) @ W["head"].T
    cap = cfg.get("logit_softcap") or 0.0
    return cap * torch.tanh(z / cap) if cap else z
