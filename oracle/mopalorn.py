"""Plain PyTorch-CPU oracle of the Mopalorn decoder (test infrastructure only, one function per mechanism).

Mopalorn is a decoder with SANDWICH norms: x <- x + n1b(mixer(n1(x))), then x <- x + n2b(ff(n2(x))); every norm is a plain RMS norm with a weight.
Mixers: *latent_attention* (keys and values rebuilt from a cached low-rank latent, one rotated key part shared by all heads, rotate-half rotary, a
sliding window, a sigmoid output gate), *attention* (grouped queries, no rotation, a query temperature that grows with the logarithm of the position,
tanh-capped scores, all earlier keys visible) and *attention_2* (grouped queries, a sliding window plus one mean key / value for every block of tokens
that lies wholly before the window, a learned sink in the softmax denominator).  Layers marked ``v_mix`` blend their values with those of the first
such layer.  Feed-forward: one up and one down projection around the xIELU activation.  The head is the embedding table times a constant.

Everything here works on ONE whole sequence in the dtype handed in (fp64 by default), query by query, and shares no code with ``llm_quest_amd``.
``weights`` maps the checkpoint's tensor names to tensors; ``cfg`` is the parsed ``config.json``.
"""

import math

import torch


def rms_norm(x, w, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps) * w


def rotary_half(x, dims, base, first_position=0):
    """x [T, H, D]: the first ``dims`` entries of every head turn, entry i paired with entry i + dims/2, by the angle position * base^(-2i/dims)."""
    T, half = x.shape[0], dims // 2
    out = x.clone()
    pos = torch.arange(first_position, first_position + T, dtype=x.dtype)
    for i in range(half):
        ang = pos * base ** (-2.0 * i / dims)
        c, s = torch.cos(ang)[:, None], torch.sin(ang)[:, None]
        u, v = x[:, :, i], x[:, :, i + half]
        out[:, :, i] = u * c - v * s
        out[:, :, i + half] = v * c + u * s
    return out


def query_temperature(T, coef, every, dtype):
    """[T]: 1 + coef * ln(floor((p + 1) / every) + 1) for p = 0 .. T-1."""
    p = torch.arange(T)
    return 1.0 + coef * torch.log((torch.div(p + 1, every, rounding_mode="floor") + 1).to(dtype))


def soft_cap(s, cap):
    return cap * torch.tanh(s / cap)


def softmax_attention(q, k, v, scale, visible, cap=None, sink=None, extra=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads key / value head h // (H/G).  ``visible(i)`` lists the keys of query i; ``extra(i)``
    (optional) returns further (keys [n, G, d], values [n, G, dv]) that share the softmax; ``sink`` [H] adds exp(sink_h) to the denominator only."""
    T, H, d = q.shape
    G, dv = k.shape[1], v.shape[-1]
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for i in range(T):
        js = visible(i)
        ks, vs = k[js], v[js]
        if extra is not None:
            ek, ev = extra(i)
            ks, vs = torch.cat([ek, ks]), torch.cat([ev, vs])
        for h in range(H):
            g = h // (H // G)
            s = (ks[:, g] @ q[i, h]) * scale
            if cap:
                s = soft_cap(s, cap)
            m = s.max() if sink is None else torch.maximum(s.max(), sink[h])
            e = torch.exp(s - m)
            den = e.sum() + (torch.exp(sink[h] - m) if sink is not None else 0.0)
            out[i, h] = (e[:, None] * vs[:, g]).sum(dim=0) / den
    return out


def window_keys(i, size):
    """Keys j with 0 <= i - j < size (size 0 or None: every j <= i)."""
    return list(range(max(0, i - size + 1) if size else 0, i + 1))


def pooled_blocks(k, v, i, size, pool):
    """Means of the keys / values of every block of ``pool`` tokens that ends at or before position i - size."""
    n = max(0, (i - size + 1) // pool)
    G = k.shape[1]
    if n == 0:
        return k.new_zeros(0, G, k.shape[-1]), v.new_zeros(0, G, v.shape[-1])
    return k[: n * pool].reshape(n, pool, G, -1).mean(dim=1), v[: n * pool].reshape(n, pool, G, -1).mean(dim=1)


def mix_values(v, v_first, lam):
    return (1.0 - lam) * v + lam * v_first


def latent_attention_mixer(h, w, pre, m, eps, shared):
    T = h.shape[0]
    H, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    rot = m.get("rot") or {"dims": dr, "base": 10000.0}
    q = (h @ w[pre + "q"].T).reshape(T, H, dn + dr)
    down = h @ w[pre + "dkv"].T
    c = rms_norm(down[:, :R], w[pre + "dkv.norm"], eps)
    kr = rotary_half(down[:, R:].reshape(T, 1, dr), rot["dims"], rot["base"])
    qr = rotary_half(q[:, :, dn:], rot["dims"], rot["base"])
    k = torch.cat([(c @ w[pre + "uk"].T).reshape(T, H, dn), kr.expand(T, H, dr)], dim=-1)
    v = (c @ w[pre + "uv"].T).reshape(T, H, dv)
    size = (m.get("mask") or {}).get("size", 0)
    o = softmax_attention(torch.cat([q[:, :, :dn], qr], dim=-1), k, v, m["scale"], lambda i: window_keys(i, size))
    o = o.reshape(T, H * dv) * torch.sigmoid(h @ w[pre + "g"].T)
    return o @ w[pre + "o"].T


def _qkv(h, w, pre, m, shared):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = (h @ w[pre + "q"].T).reshape(T, H, d)
    k = (h @ w[pre + "k"].T).reshape(T, G, d)
    v = (h @ w[pre + "v"].T).reshape(T, G, dv)
    if m.get("v_mix"):
        if "v_first" in shared:
            v = mix_values(v, shared["v_first"], w[pre + "vmix"])
        else:
            shared["v_first"] = v
    return q, k, v


def attention_mixer(h, w, pre, m, eps, shared):
    T = h.shape[0]
    q, k, v = _qkv(h, w, pre, m, shared)
    qt = m.get("q_temp")
    if qt:
        q = q * query_temperature(T, qt["coef"], qt["every"], h.dtype)[:, None, None]
    o = softmax_attention(q, k, v, m["scale"], lambda i: window_keys(i, 0), cap=m.get("softcap"))
    return o.reshape(T, -1) @ w[pre + "o"].T


def attention_2_mixer(h, w, pre, m, eps, shared):
    T = h.shape[0]
    q, k, v = _qkv(h, w, pre, m, shared)
    size, pool = m["mask"]["size"], m["mask"].get("pool", 0)
    extra = (lambda i: pooled_blocks(k, v, i, size, pool)) if pool else None
    o = softmax_attention(q, k, v, m["scale"], lambda i: window_keys(i, size), sink=w.get(pre + "sink"), extra=extra)
    return o.reshape(T, -1) @ w[pre + "o"].T


def xielu(z, p, q):
    """z > 0: softplus(p) z^2 + z/2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z/2."""
    sp = torch.nn.functional.softplus
    pos = sp(p) * z * z + 0.5 * z
    neg = (0.5 + sp(q)) * (torch.expm1(z) - z) + 0.5 * z
    return torch.where(z > 0, pos, neg)


def dense_ff(h, w, pre):
    a = w[pre + "act"]
    return xielu(h @ w[pre + "up"].T, a[0], a[1]) @ w[pre + "down"].T


MIXERS = {"latent_attention": latent_attention_mixer, "attention": attention_mixer, "attention_2": attention_2_mixer}


def forward(tokens, weights, cfg, dtype=torch.float64, return_layers=False):
    """tokens: the ids of one whole sequence -> logits [T, vocab] (and the residual stream after every layer)."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(list(tokens))]
    layers, shared = [], {}
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        y = MIXERS[layer["type"]](rms_norm(x, w[p + "norm1"], eps), w, p + "mix.", layer["mixer"], eps, shared)
        x = x + rms_norm(y, w[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            y = dense_ff(rms_norm(x, w[p + "norm2"], eps), w, p + "mlp.")
            x = x + rms_norm(y, w[p + "norm2b"], eps)
        layers.append(x)
    logits = rms_norm(x, w["final.norm"], eps) @ w["embed"].T * cfg.get("logit_scale", 1.0)
    return (logits, layers) if return_layers else logits
