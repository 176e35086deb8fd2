"""Plain, slow restatement of the Fagunex layer stack: one function per mechanism, whole sequences,
token loops where the definition is a recurrence or a window.  Shares nothing with the product
path; the tests compare the engine against it.  Everything runs in `dtype` (float64 by default) on
the CPU.

Weights come as a dict name -> tensor with the checkpoint's names ('l<i>.mix.q', ...), the
configuration as the parsed config.json dict.

Notation: a sublayer reads n1(x) and adds n1b(sublayer output) to x, where every n is a Dynamic
Tanh, tanh(alpha x) w + b.  The mixer's input is blended with the previous token's (token shift).
After the feed-forward a per-layer token embedding enters through a gated low-rank path.
"""
import math

import torch


def rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dynamic_tanh(x, w, b, alpha):
    return torch.tanh(alpha * x) * w + b


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def token_shift(h, mix, previous=None):
    """h [T, W]: row t becomes h_t + (h_(t-1) - h_t) * mix, h_(-1) = `previous` (zeros when None)."""
    first = torch.zeros_like(h[:1]) if previous is None else previous[None]
    before = torch.cat([first, h[:-1]], dim=0)
    return h + (before - h) * mix


def rotate_interleaved(x, positions, dims, base):
    """x [T, ..., d]: dimension 2i pairs with 2i+1 for i < dims/2; the rest pass."""
    out = x.clone()
    for i in range(dims // 2):
        ang = positions.to(x.dtype) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(ang), torch.sin(ang)
        while c.dim() < x.dim() - 1:
            c, s = c[..., None], s[..., None]
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * c - v * s
        out[..., 2 * i + 1] = v * c + u * s
    return out


def rotate_halves(x, positions, dims, base):
    """x [T, ..., d]: dimension i pairs with i + dims/2 for i < dims/2; the rest pass."""
    out = x.clone()
    half = dims // 2
    for i in range(half):
        ang = positions.to(x.dtype) * (base ** (-2.0 * i / dims))
        c, s = torch.cos(ang), torch.sin(ang)
        while c.dim() < x.dim() - 1:
            c, s = c[..., None], s[..., None]
        u, v = x[..., i], x[..., i + half]
        out[..., i] = u * c - v * s
        out[..., i + half] = v * c + u * s
    return out


def gated_write_recurrence(q, f, v, state=None):
    """S_t = diag(f_t) S_(t-1) + (1 - f_t) v_t^T, o_t = S_t^T q_t.
    q, f [T, H, n], v [T, H, p] -> o [T, H, p], S [H, n, p]."""
    T, H, n = q.shape
    p = v.shape[-1]
    S = torch.zeros(H, n, p, dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(T, H, p, dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            S[h] = f[t, h][:, None] * S[h] + (1.0 - f[t, h])[:, None] * v[t, h][None, :]
            out[t, h] = S[h].T @ q[t, h]
    return out, S


def hgrn2_mixer(h, W, p, m, eps):
    H, n, pv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    T = h.shape[0]
    q = torch.nn.functional.silu(h @ W[p + "q"].T).view(T, H, n)
    v = (h @ W[p + "v"].T).view(T, H, pv)
    low = W[p + "lower"]
    f = (low + (1.0 - low) * torch.sigmoid(h @ W[p + "f"].T + W[p + "f.b"])).view(T, H, n)
    o, _ = gated_write_recurrence(q, f, v)
    o = rms(o, eps) * W[p + "norm"]
    return o.reshape(T, H * pv) @ W[p + "o"].T


def masked_softmax_attention(q, k, v, scale, window=None, sink=None):
    """q, k [T, H, d], v [T, H, dv].  Position i sees j <= i, and with a window only i - j < window.
    sink [H]: exp(sink_h) joins the denominator, with no value."""
    T, H, _ = q.shape
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for hd in range(H):
        for i in range(T):
            lo = 0 if window is None else max(0, i - window + 1)
            s = (k[lo:i + 1, hd] @ q[i, hd]) * scale
            if sink is None:
                w = torch.softmax(s, dim=0)
            else:
                z = torch.cat([s, sink[hd:hd + 1]])
                w = torch.softmax(z, dim=0)[:-1]
            out[i, hd] = w @ v[lo:i + 1, hd]
    return out


def latent_attention_mixer(h, W, p, m, eps, kind):
    """kind 1: queries through a normed latent, interleaved rotation, sliding window, sink, output gate.
    kind 2: direct queries, rotation of halves, causal, ordinary softmax."""
    H, d, r, dv, c_dim = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    T = h.shape[0]
    pos = torch.arange(T)
    if kind == 1:
        cq = rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
        q = (cq @ W[p + "uq"].T).view(T, H, d + r)
    else:
        q = (h @ W[p + "q"].T).view(T, H, d + r)
    dkv = h @ W[p + "dkv"].T
    c = rms(dkv[:, :c_dim], eps) * W[p + "dkv.norm"]
    k_rot = dkv[:, c_dim:]
    rotate = rotate_interleaved if kind == 1 else rotate_halves
    dims, base = int(m["rot"]["dims"]), float(m["rot"]["base"])
    q_rot = rotate(q[..., d:], pos, dims, base)
    k_rot = rotate(k_rot, pos, dims, base)
    k_plain = (c @ W[p + "uk"].T).view(T, H, d)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    qq = torch.cat([q[..., :d], q_rot], dim=-1)
    kk = torch.cat([k_plain, k_rot[:, None, :].expand(T, H, r)], dim=-1)
    if kind == 1:
        a = masked_softmax_attention(qq, kk, v, float(m["scale"]), int(m["mask"]["size"]), W[p + "sink"])
        a = a.reshape(T, H * dv) * torch.sigmoid(h @ W[p + "g"].T)
    else:
        a = masked_softmax_attention(qq, kk, v, float(m["scale"])).reshape(T, H * dv)
    return a @ W[p + "o"].T


def swiglu(h, gate, up, down):
    return (torch.nn.functional.silu(h @ gate.T) * (h @ up.T)) @ down.T


def routed_experts(h, W, p, mlp):
    """Top-k experts by router logit, weights = softmax over the chosen logits; plus a shared
    expert times sigmoid of one number per token."""
    E, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = h @ W[p + "router"].T
    out = torch.zeros(h.shape[0], W[p + "e0.down"].shape[0], dtype=h.dtype)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(z[t, e]), e))[:top]
        w = torch.softmax(z[t, order], dim=0)
        for j, e in enumerate(order):
            out[t] += w[j] * swiglu(h[t:t + 1], W[p + f"e{e}.gate"], W[p + f"e{e}.up"], W[p + f"e{e}.down"])[0]
    if mlp.get("shared"):
        s = swiglu(h, W[p + "shared.gate"], W[p + "shared.up"], W[p + "shared.down"])
        out = out + torch.sigmoid(h @ W[p + "shared.sg"].T) * s
    return out


def token_side_input(x, tokens, W, p, index, dim, eps):
    e = W["side.embed"][tokens][:, index * dim:(index + 1) * dim]
    g = gelu_tanh(x @ W[p + "side.gate"].T) * e
    y = g @ W[p + "side.proj"].T
    return x + rms(y, eps) * W[p + "side.norm"]


def layer_runs(config):
    """Indices of the layers in the order they run (a loop repeats a span in place)."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def forward(config, weights, tokens, dtype=torch.float64, residuals=None):
    """tokens: list of ids of ONE sequence from position 0 -> logits [T, vocab]."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    ids = torch.tensor(tokens, dtype=torch.long)
    x = W["embed"][ids]
    side = config.get("token_side")

    def norm(name, v):
        return dynamic_tanh(v, W[name], W[name + ".b"], W[name + ".alpha"])

    for i in layer_runs(config):
        layer, p = config["layers"][i], f"l{i}."
        h = token_shift(norm(p + "norm1", x), W[p + "shift"])
        if layer["type"] == "hgrn2":
            y = hgrn2_mixer(h, W, p + "mix.", layer["mixer"], eps)
        elif layer["type"] == "latent_attention":
            y = latent_attention_mixer(h, W, p + "mix.", layer["mixer"], eps, 1)
        elif layer["type"] == "latent_attention_2":
            y = latent_attention_mixer(h, W, p + "mix.", layer["mixer"], eps, 2)
        else:
            raise ValueError(layer["type"])
        x = x + norm(p + "norm1b", y)
        if layer.get("mlp"):
            x = x + norm(p + "norm2b", routed_experts(norm(p + "norm2", x), W, p + "mlp.", layer["mlp"]))
        if side:
            x = token_side_input(x, ids, W, p, i, int(side["dim"]), eps)
        if residuals is not None:
            residuals.append(x.clone())
    return norm("final.norm", x) @ W["head"].T
