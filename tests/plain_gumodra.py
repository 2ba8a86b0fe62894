"""Plain implementation of the Gumodra design: whole sequences, no cache, float64, one function per mechanism.

It reads the raw config.json dictionary and the checkpoint's tensors by name and shares no code with the
package: every formula is restated here.  Positions count from 0; "rms" always has eps inside the root.

    norm            y = x / sqrt(mean(x^2) + eps) * g, g one number for the whole row
    layer           h = norm1(x);  x += sigmoid(R1 h + r1) * mixer(h) + sigmoid(R2 h + r2) * ff(h)
                    (one norm, both sub-layers read h; the second term is absent without a feed-forward)
    rotation        first `dims` features of a head, feature i with i + dims/2:
                    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = p * f_i, f_i = base^(-2i/dims)
    attention       q = Wq h + bq, k = Wk h + bk, values = k as projected; q and k divided by their rms per head
                    and multiplied by a weight shared by the heads, then rotated; score = q.k * scale;
                    query p sees key j <= p with p - j < size or j < keep_first; the softmax's denominator
                    holds exp(sink_head) as one more term without a value; Wo (.) + bo
    mlstm           q = Wq h / sqrt(dim), k = Wk h, v = Wv h; a = cap tanh((Wi h + bi)/cap),
                    b = logsigmoid(cap tanh((Wf h + bf)/cap)); m' = max(b + m, a);
                    S' = exp(b + m - m') S + exp(a - m') k v^T, n' likewise with k; m, S, n start at 0;
                    o = S'^T q / (max(|n'.q|, exp(-m')) + 1e-6); o / rms(o) per head, * w, * sigmoid(Wg h); Wo
    feed-forward    Wd (silu(Wg h) * (Wu h)); mixture: s = softmax(Wr h); choice c = s + correction; experts in
                    `count` equal groups of neighbours, a group's score its largest c, only the `keep` best groups
                    may be chosen from; the `top` largest c; weights s / (sum of the chosen s + 1e-20); plus a
                    shared expert times sigmoid(w_sg . h)
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def scalar_norm(x, g, eps):
    return rms(x, eps) * g


def silu(z):
    return z * torch.sigmoid(z)


def rotate(x, positions, rot):
    """x [T, heads, d]: the first rot.dims features rotated by position, the others unchanged."""
    dims = rot["dims"]
    if dims == 0:
        return x
    i = torch.arange(dims // 2, dtype=F64)
    f = rot["base"] ** (-2.0 * i / dims)
    a = positions.to(F64)[:, None] * f[None, :]
    cos, sin = torch.cos(a)[:, None, :], torch.sin(a)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


def visible(T, size=None, keep_first=0):
    """[query, key]: causal, and with a window the last `size` positions plus the first `keep_first`."""
    p = torch.arange(T)
    m = p[:, None] >= p[None, :]
    if size is not None:
        m = m & (((p[:, None] - p[None, :]) < size) | (p[None, :] < keep_first))
    return m


def sink_softmax(scores, mask, sink):
    """scores [H, T, T], sink [H] or None: weights whose rows sum to less than one by the sink's share."""
    s = scores.masked_fill(~mask, -math.inf)
    if sink is None:
        return torch.softmax(s, -1)
    T = s.shape[1]
    ext = torch.cat([s, sink.to(s.dtype)[:, None, None].expand(-1, T, 1)], -1)
    return torch.softmax(ext, -1)[..., :-1]


def attention(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d = m["heads"], m["kv_heads"], m["dim"]
    pos = torch.arange(T)
    q = (h @ W[p + "q"].T + W[p + "q.b"]).view(T, H, d)
    k = (h @ W[p + "k"].T + W[p + "k.b"]).view(T, G, d)
    v = k
    q = rotate(rms(q, eps) * W[p + "q.norm"], pos, m["rot"])
    k = rotate(rms(k, eps) * W[p + "k.norm"], pos, m["rot"])
    rep = H // G
    kk, vv = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
    scores = torch.einsum("ihd,jhd->hij", q, kk) * m["scale"]
    mask = m.get("mask") or {}
    w = sink_softmax(scores, visible(T, mask.get("size"), mask.get("keep_first", 0)), W.get(p + "sink"))
    o = torch.einsum("hij,jhd->ihd", w, vv).reshape(T, H * d)
    return o @ W[p + "o"].T + W[p + "o.b"]


def mlstm_gates(h, W, p, cap):
    """(log input gate, log forget gate) [T, heads]."""
    a = cap * torch.tanh((h @ W[p + "i"].T + W[p + "i.b"]) / cap)
    b = torch.nn.functional.logsigmoid(cap * torch.tanh((h @ W[p + "f"].T + W[p + "f.b"]) / cap))
    return a, b


def mlstm_recurrence(q, k, v, a, b):
    """q, k [T, H, d], v [T, H, dv], a, b [T, H] -> o [T, H, dv]; the stabiliser starts at 0."""
    T, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=q.dtype)
    n = torch.zeros(H, d, dtype=q.dtype)
    m = torch.zeros(H, dtype=q.dtype)
    out = []
    for t in range(T):
        m_new = torch.maximum(b[t] + m, a[t])
        keep, take = torch.exp(b[t] + m - m_new), torch.exp(a[t] - m_new)
        S = keep[:, None, None] * S + take[:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        n = keep[:, None] * n + take[:, None] * k[t]
        m = m_new
        num = torch.einsum("hdv,hd->hv", S, q[t])
        den = torch.maximum((n * q[t]).sum(-1).abs(), torch.exp(-m)) + 1e-6
        out.append(num / den[:, None])
    return torch.stack(out)


def mlstm(h, W, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    q = (h @ W[p + "q"].T).view(T, H, d) * d ** -0.5
    k = (h @ W[p + "k"].T).view(T, H, d)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    a, b = mlstm_gates(h, W, p, m["gate_cap"])
    o = rms(mlstm_recurrence(q, k, v, a, b), eps).reshape(T, H * dv)
    return (o * W[p + "norm"] * torch.sigmoid(h @ W[p + "g"].T)) @ W[p + "o"].T


def gated_ff(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def route(h, W, p, r):
    """(chosen experts [T, top], their weights [T, top])."""
    E, top = r["experts"], r["top"]
    s = torch.softmax(h @ W[p + "router"].T, -1)
    c = s + W[p + "correction"]
    g = r.get("groups")
    if g:
        per = E // g["count"]
        best = c.view(-1, g["count"], per).max(-1).values.topk(g["keep"], -1).indices
        allowed = torch.zeros(c.shape[0], g["count"], dtype=torch.bool).scatter_(1, best, True)
        c = c.masked_fill(~allowed.repeat_interleave(per, 1), -math.inf)
    idx = c.topk(top, -1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20)


def mixture_ff(h, W, p, mlp):
    idx, w = route(h, W, p, mlp["router"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, we in zip(idx[t].tolist(), w[t]):
            out[t] += we * gated_ff(h[t:t + 1], W, f"{p}e{e}.")[0]
    if mlp.get("shared"):
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * gated_ff(h, W, p + "shared.")
    return out


def feed_forward(h, W, p, mlp):
    return gated_ff(h, W, p) if mlp["kind"] == "dense" else mixture_ff(h, W, p, mlp)


def layer(x, W, i, L, eps):
    p = f"l{i}."
    h = scalar_norm(x, W[p + "norm1"], eps)
    mix = attention if L["type"] == "attention" else mlstm
    y = torch.sigmoid(h @ W[p + "rg1"].T + W[p + "rg1.b"]) * mix(h, W, p + "mix.", L["mixer"], eps)
    if L.get("mlp"):
        y = y + torch.sigmoid(h @ W[p + "rg2"].T + W[p + "rg2.b"]) * feed_forward(h, W, p + "mlp.", L["mlp"])
    return x + y


def forward(raw, W, tokens, return_layers=False):
    """Logits [T, vocab] of one whole sequence (float64); with return_layers also the residual after each layer."""
    W = {k: v.to(F64) for k, v in W.items()}
    eps = raw["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * raw.get("embedding", {}).get("scale", 1.0)
    after = []
    for i, L in enumerate(raw["layers"]):
        x = layer(x, W, i, L, eps)
        after.append(x)
    logits = scalar_norm(x, W["final.norm"], eps) @ W["head"].T
    return (logits, torch.stack(after)) if return_layers else logits
