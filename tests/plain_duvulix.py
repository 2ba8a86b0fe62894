"""Plain implementation of the Duvulix design: whole sequences, no cache, float64, one function per mechanism.

It reads the raw config.json dictionary and the checkpoint's tensors by name and shares no code with the
package: every formula is restated here.  Positions count from 0; "rms" always has eps inside the root.

    norm            y = x / sqrt(mean(x^2) + eps) * (1 + w)                      (weights stored around zero)
    layer           x += norm1b(mixer(norm1 x));  x += norm2b(ff(norm2 x))        (ff may be absent)
    rotation        first `dims` features of a head, feature i with i + dims/2:
                    (u, v) -> (u cos a - v sin a, v cos a + u sin a), a = p * f_i, f_i = base^(-2i/dims)
    YaRN            f_i <- f_i / factor * ramp_i + f_i (1 - ramp_i), cos and sin times 0.1 ln(factor) + 1
    attention       grouped heads, score = q.k * scale, causal, optionally only inside the query's chunk of
                    `size` positions counted from 0; softmax
    latent attn.    c = rms(W_dkv x [:rank]) * w, shared rotated key part = rot(W_dkv x [rank:]);
                    k_h = [W_uk,h c | shared], v_h = W_uv,h c, q_h = [plain | rot]; gate sigmoid(W_g x)_h
    mamba2          [z | x | B | C | dt] = W_in h; causal conv + silu on x, B, C; dt = softplus(dt + bias);
                    S = exp(-exp(A_log) dt) S + dt B x^T;  y = S^T C + D x;  y * silu(z); grouped rms * w; W_o
    feed-forward    W_down (a N(z) + b N(z^2) + c N(z^3) + e), z = W_up h, N(v) = v / sqrt(mean(v^2) + eps)
"""
import math

import torch

F64 = torch.float64


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    return rms(x, eps) * (1.0 + w)


def frequencies(rot):
    """(angular frequency per pair [dims/2], magnitude of cos and sin)."""
    dims, base = rot["dims"], rot["base"]
    i = torch.arange(dims // 2, dtype=F64)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0

    def feature_turning(t):
        return dims * math.log(sc["original"] / (2 * math.pi * t)) / (2 * math.log(base))
    lo = max(math.floor(feature_turning(sc["fast"])), 0)
    hi = min(math.ceil(feature_turning(sc["slow"])), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0, 1)
    return f / sc["factor"] * ramp + f * (1 - ramp), 0.1 * math.log(sc["factor"]) + 1.0


def rotate(x, positions, rot):
    """x [T, heads, d]: the first rot.dims features rotated by position, the others unchanged."""
    dims = rot["dims"]
    if dims == 0:
        return x
    f, mag = frequencies(rot)
    a = positions.to(F64)[:, None] * f[None, :]
    cos, sin = (torch.cos(a) * mag)[:, None, :], (torch.sin(a) * mag)[:, None, :]
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], -1)


def visible(T, chunk=None):
    p = torch.arange(T)
    m = p[:, None] >= p[None, :]
    if chunk:
        m = m & ((p[:, None] // chunk) == (p[None, :] // chunk))
    return m


def softmax_attend(scores, mask, v):
    """scores [H, T, T], v [T, H, dv] -> [T, H, dv]."""
    w = torch.softmax(scores.masked_fill(~mask, -math.inf), -1)
    return torch.einsum("hij,jhd->ihd", w, v)


def attention(h, W, p, m):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate((h @ W[p + "q"].T).view(T, H, d), pos, m["rot"])
    k = rotate((h @ W[p + "k"].T).view(T, G, d), pos, m["rot"]).repeat_interleave(H // G, 1)
    v = (h @ W[p + "v"].T).view(T, G, dv).repeat_interleave(H // G, 1)
    s = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    o = softmax_attend(s, visible(T, (m.get("mask") or {}).get("size")), v)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def latent_cache(h, W, p, m, eps):
    """(latent c [T, rank], shared rotated key part [T, rot_dim]) of a layer that has a down projection."""
    T, R = h.shape[0], m["kv_rank"]
    d = h @ W[p + "dkv"].T
    c = rms(d[:, :R], eps) * W[p + "dkv.norm"]
    kr = rotate(d[:, None, R:], torch.arange(T), m["rot"])[:, 0]
    return c, kr


def latent_attention(h, W, p, m, cache):
    T = h.shape[0]
    H, d, r, dv = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = cache
    q = (h @ W[p + "q"].T).view(T, H, d + r)
    q_plain, q_rot = q[..., :d], rotate(q[..., d:], torch.arange(T), m["rot"])
    k_plain = (c @ W[p + "uk"].T).view(T, H, d)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    s = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, kr)) * m["scale"]
    o = softmax_attend(s, visible(T), v) * torch.sigmoid(h @ W[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ W[p + "o"].T


def causal_conv_silu(x, w, b):
    """x [T, C], w [C, taps] (last column = current token), zeros before the start."""
    T, taps = x.shape[0], w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, x.shape[1], dtype=x.dtype), x], 0)
    y = sum(pad[k:k + T] * w[:, k] for k in range(taps)) + b
    return y * torch.sigmoid(y)


def softplus(x):
    return torch.where(x > 30, x, torch.log1p(torch.exp(torch.clamp(x, max=30))))


def ssm_recurrence(x, B, C, dt, A_log, D):
    """x [T, H, P], B and C [T, H, N] (already spread over heads), dt [T, H] after softplus -> y [T, H, P]."""
    T, H, P = x.shape
    S = torch.zeros(H, B.shape[-1], P, dtype=F64)
    A = torch.exp(A_log)
    ys = []
    for t in range(T):
        S = torch.exp(-A * dt[t])[:, None, None] * S + dt[t][:, None, None] * B[t][:, :, None] * x[t][:, None, :]
        ys.append(torch.einsum("hnp,hn->hp", S, C[t]) + D[:, None] * x[t])
    return torch.stack(ys)


def mamba2(h, W, p, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    u = h @ W[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = causal_conv_silu(xbc, W[p + "conv"], W[p + "conv.b"])
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, 1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, 1)
    y = ssm_recurrence(x, B, C, softplus(dt + W[p + "dt_bias"]), W[p + "A_log"], W[p + "D"]).reshape(T, inner)
    y = y * (z * torch.sigmoid(z))
    ng = m["norm_groups"]
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def poly_norm(z, coef, eps):
    a, b, c, e = [float(v) for v in coef]
    return a * rms(z, eps) + b * rms(z ** 2, eps) + c * rms(z ** 3, eps) + e


def feed_forward(h, W, p, eps):
    return poly_norm(h @ W[p + "up"].T, W[p + "act"], eps) @ W[p + "down"].T


def forward(cfg, weights, tokens, residuals=None):
    """float64 logits [T, vocab] of the whole sequence; ``residuals`` (a list) receives x after every layer."""
    W = {k: v.to(F64) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(list(tokens))]
    caches = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = offset_norm(x, W[p + "norm1"], eps)
        if layer["type"] == "latent_attention":
            if "kv_from" in m and m["kv_from"] is not None:
                cache = caches[m["kv_from"]]
            else:
                cache = caches[i] = latent_cache(h, W, p + "mix.", m, eps)
            b = latent_attention(h, W, p + "mix.", m, cache)
        elif layer["type"] == "attention":
            b = attention(h, W, p + "mix.", m)
        elif layer["type"] == "mamba2":
            b = mamba2(h, W, p + "mix.", m, eps)
        else:
            raise ValueError(layer["type"])
        x = x + offset_norm(b, W[p + "norm1b"], eps)
        if layer.get("mlp"):
            f = feed_forward(offset_norm(x, W[p + "norm2"], eps), W, p + "mlp.", eps)
            x = x + offset_norm(f, W[p + "norm2b"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    return offset_norm(x, W["final.norm"], eps) @ W["head"].T


def greedy(cfg, weights, prompt, n_new):
    toks = list(prompt)
    out = []
    for _ in range(n_new):
        nxt = int(forward(cfg, weights, toks)[-1].argmax())
        out.append(nxt)
        toks.append(nxt)
    return out
