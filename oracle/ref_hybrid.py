"""Plain, slow restatement of the Pagazen layer stack: one function per mechanism, whole sequences,
token loops where the definition is a recurrence.  Shares nothing with the product path; the
tests compare the engine against it.  Everything runs in `dtype` (float64 by default) on the CPU.

Weights come as a dict name -> tensor with the checkpoint's names ('l<i>.mix.in', ...), the
configuration as the parsed config.json dict.
"""
import torch


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm whose stored weight is an offset from one."""
    return unit_rms(x, eps) * (1.0 + w)


def relu_squared_mlp(h, up, down):
    a = torch.relu(h @ up.T)
    return (a * a) @ down.T


def rotate_half_pairs(x, positions, dims, base):
    """x [T, heads, dim]: dimension i pairs with i + dims/2 for i < dims/2; the rest pass."""
    half = dims // 2
    i = torch.arange(half, dtype=x.dtype)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(x.dtype)[:, None] * freq[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def windowed_softmax_attention(q, k, v, scale, window, slopes):
    """q [T,H,d], k [T,G,d], v [T,G,dv] -> [T,H,dv].  Position i sees j with 0 <= i-j < window;
    the score loses slopes[h] * (i - j)."""
    T, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    for h in range(H):
        g = h // (H // G)
        for i in range(T):
            lo = max(0, i - window + 1)
            s = (k[lo:i + 1, g] @ q[i, h]) * scale
            dist = torch.arange(i - lo, -1, -1, dtype=q.dtype)
            p = torch.softmax(s - slopes[h] * dist, dim=0)
            out[i, h] = p @ v[lo:i + 1, g]
    return out


def decayed_outer_product_scan(q, k, v, decay, gain, state=None):
    """S_t = decay[t,h] S_(t-1) + gain[t,h] k_t v_t^T ; o_t = S_t^T q_t.
    q, k [T,H,n], v [T,H,p], decay / gain [T,H] -> o [T,H,p], final S [H,n,p]."""
    T, H, n = k.shape
    p = v.shape[-1]
    S = torch.zeros(H, n, p, dtype=q.dtype) if state is None else state.clone()
    out = torch.zeros(T, H, p, dtype=q.dtype)
    for t in range(T):
        S = decay[t][:, None, None] * S + gain[t][:, None, None] * k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hnp,hn->hp", S, q[t])
    return out, S


def causal_conv_silu(x, w, b):
    """x [T,C], w [C,taps] (last column = current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    pad = torch.cat([torch.zeros(taps - 1, C, dtype=x.dtype), x], 0)
    y = b[None, :].clone().repeat(T, 1)
    for j in range(taps):
        y = y + pad[j:j + T] * w[:, j][None, :]
    return y * torch.sigmoid(y)


def left_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = unit_rms((h @ W[p + "q"].T).view(T, H, d), eps)
    k = unit_rms((h @ W[p + "k"].T).view(T, G, d), eps)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    slopes = [2.0 ** (-8.0 * (i + 1) / H) for i in range(H)]
    o = windowed_softmax_attention(q, k, v, m["scale"], m["mask"]["size"], slopes)
    return o.reshape(T, H * dv) @ W[p + "o"].T


def right_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    pos = torch.arange(T)
    q = rotate_half_pairs((h @ W[p + "q"].T).view(T, H, d), pos, m["rot"]["dims"], m["rot"]["base"])
    k = rotate_half_pairs((h @ W[p + "k"].T).view(T, H, d), pos, m["rot"]["dims"], m["rot"]["base"])
    k = k * d ** -0.5
    v = (h @ W[p + "v"].T).view(T, H, dv)
    decay = torch.tensor(m["decay"], dtype=h.dtype)[None, :].repeat(T, 1)
    o, _ = decayed_outer_product_scan(q, k, v, decay, torch.ones(T, H, dtype=h.dtype))
    o = unit_rms(o, eps).reshape(T, H * dv)
    gate = h @ W[p + "g"].T
    return (o * gate * torch.sigmoid(gate)) @ W[p + "o"].T


def parallel_mixer(h, W, p, m, eps):
    return m["left_scale"] * left_mixer(h, W, p + "left.", m["left"], eps) + \
        m["right_scale"] * right_mixer(h, W, p + "right.", m["right"], eps)


def mamba2_mixer(h, W, p, m, eps):
    T = h.shape[0]
    H, P, N, G = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = H * P
    zxbcdt = h @ W[p + "in"].T
    z = zxbcdt[:, :inner]
    xbc = causal_conv_silu(zxbcdt[:, inner:2 * inner + 2 * G * N], W[p + "conv"], W[p + "conv.b"])
    dt = torch.nn.functional.softplus(zxbcdt[:, 2 * inner + 2 * G * N:] + W[p + "dt_bias"], threshold=1e9)
    x = xbc[:, :inner].view(T, H, P)
    B = xbc[:, inner:inner + G * N].view(T, G, N).repeat_interleave(H // G, dim=1)
    C = xbc[:, inner + G * N:].view(T, G, N).repeat_interleave(H // G, dim=1)
    decay = torch.exp(-torch.exp(W[p + "A_log"])[None, :] * dt)
    y, _ = decayed_outer_product_scan(C, B, x, decay, dt)
    y = (y + W[p + "D"][None, :, None] * x).reshape(T, inner)
    y = y * z * torch.sigmoid(z)
    parts = m["norm_groups"]
    y = unit_rms(y.view(T, parts, inner // parts), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


def forward(config, weights, tokens, dtype=torch.float64, residuals=None):
    """Logits [T, vocab] of one whole sequence.  `residuals`, a list, receives the stream after every
    layer run."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps = config["norm"]["eps"]
    x = W["embed"][torch.as_tensor(tokens, dtype=torch.long)] * config["embedding"]["scale"]
    for i, layer in enumerate(config["layers"]):
        p = "l%d." % layer.get("weights_of", i)
        mix = {"parallel": parallel_mixer, "mamba2": mamba2_mixer}[layer["type"]]
        x = x + offset_norm(mix(x, W, p + "mix.", layer["mixer"], eps), W[p + "norm1"], eps)
        if layer.get("mlp"):
            assert layer["mlp"]["kind"] == "dense"
            x = x + offset_norm(relu_squared_mlp(x, W[p + "mlp.up"], W[p + "mlp.down"]), W[p + "norm2"], eps)
        if residuals is not None:
            residuals.append(x.clone())
    logits = offset_norm(x, W["final.norm"], eps) @ W["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(logits / cap) if cap else logits
