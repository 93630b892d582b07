"""The Pavodra design as plain, slow functions: one per mechanism, written from its equations in float64 on
the CPU, sharing no code with the package.  ``forward`` runs a whole token list and returns the logits of every
place and the residual stream after every layer; the tests compare the framework's steps with it.

Notation: ``T`` tokens, ``w`` a dict of float64 tensors by checkpoint name, ``p`` a layer's prefix (``l3``).
"""
import torch

F = torch.float64


def rms(x, eps):
    """x over the root of (its mean square plus eps), along the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_around_zero(x, weight, eps):
    """The layer norm of the design: the stored weight is the gain minus one."""
    return rms(x, eps) * (1.0 + weight)


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.where(z > 30, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def dense_ff(h, w, p):
    """down(relu(up h)^2)."""
    a = torch.relu(h @ w[p + ".mlp.up"].T)
    return (a * a) @ w[p + ".mlp.down"].T


def mingru(h, w, p, state=None):
    """A gated recurrence whose gate and candidate read the current token only; returns (out, last state)."""
    T = h.shape[0]
    z = torch.sigmoid(h @ w[p + ".mix.z"].T + w[p + ".mix.z.b"])
    u = h @ w[p + ".mix.x"].T + w[p + ".mix.x.b"]
    cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
    gate = silu(h @ w[p + ".mix.g"].T)
    s = torch.zeros(z.shape[1], dtype=F) if state is None else state.clone()
    rows = []
    for t in range(T):
        s = (1.0 - z[t]) * s + z[t] * cand[t]
        rows.append(s * gate[t])
    return torch.stack(rows) @ w[p + ".mix.o"].T, s


def mamba2(h, w, p, m, eps, state=None, tail=None):
    """A state-space layer with a scalar decay per head.  ``m``: the mixer's sizes.  Returns (out, state
    [heads, N, vdim], the last taps - 1 inputs of the convolution)."""
    T = h.shape[0]
    Hn, P, N, G, K = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner = Hn * P
    proj = h @ w[p + ".mix.in"].T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * G * N], proj[:, 2 * inner + 2 * G * N:]
    C = xbc.shape[1]
    past = torch.zeros(K - 1, C, dtype=F) if tail is None else tail.clone()
    padded = torch.cat([past, xbc], 0)  # row t + K - 1 is token t
    cw, cb = w[p + ".mix.conv"], w[p + ".mix.conv.b"]
    conv = torch.stack([(padded[t:t + K] * cw.T).sum(0) + cb for t in range(T)])  # the last tap is the token's own
    conv = silu(conv)
    x, B, Cm = conv[:, :inner].view(T, Hn, P), conv[:, inner:inner + G * N].view(T, G, N), conv[:, inner + G * N:].view(T, G, N)
    dt = softplus(dt + w[p + ".mix.dt_bias"])
    A = -torch.exp(w[p + ".mix.A_log"])
    S = torch.zeros(Hn, N, P, dtype=F) if state is None else state.clone()
    y = torch.zeros(T, Hn, P, dtype=F)
    per = Hn // G
    for t in range(T):
        for hd in range(Hn):
            g = hd // per
            S[hd] = torch.exp(A[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ Cm[t, g] + w[p + ".mix.D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = rms(y.view(T, ng, inner // ng), eps).reshape(T, inner) * w[p + ".mix.norm"]
    return y @ w[p + ".mix.o"].T, S, padded[T:T + K - 1] if K > 1 else past


def rotate_pairs(v, pos, dims, base):
    """Neighbouring elements (2i, 2i + 1) of the first ``dims`` of the last axis, turned by pos * base^(-2i/dims)."""
    out = v.clone()
    i = torch.arange(dims // 2, dtype=F)
    ang = pos.to(F)[:, None] * base ** (-2.0 * i / dims)
    c, s = torch.cos(ang), torch.sin(ang)
    while c.dim() < v.dim():
        c, s = c.unsqueeze(1), s.unsqueeze(1)
    a, b = v[..., 0:dims:2], v[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def latent_attention(h, w, p, m, eps, pos=None):
    """Attention whose keys and values are made from one small latent per token plus one rotated key part that all
    heads share.  Keys and values are expanded here for every token: the slow, direct way."""
    T = h.shape[0]
    Hn, dn, dr, dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    pos = torch.arange(T) if pos is None else pos
    q = (h @ w[p + ".mix.q"].T).view(T, Hn, dn + dr)
    down = h @ w[p + ".mix.dkv"].T
    c = rms(down[:, :R], eps) * w[p + ".mix.dkv.norm"]
    k_rot = rotate_pairs(down[:, R:], pos, m["rot"]["dims"], m["rot"]["base"])  # [T, dr], one for all heads
    q_rot = rotate_pairs(q[..., dn:], pos, m["rot"]["dims"], m["rot"]["base"])
    k = (c @ w[p + ".mix.uk"].T).view(T, Hn, dn)
    v = (c @ w[p + ".mix.uv"].T).view(T, Hn, dv)
    out = torch.zeros(T, Hn, dv, dtype=F)
    for hd in range(Hn):
        s = (q[:, hd, :dn] @ k[:, hd].T + q_rot[:, hd] @ k_rot.T) * m["scale"]
        s = s.masked_fill(torch.arange(T)[None, :] > torch.arange(T)[:, None], float("-inf"))
        out[:, hd] = torch.softmax(s, -1) @ v[:, hd]
    return out.reshape(T, Hn * dv) @ w[p + ".mix.o"].T


def forward(cfg, w, ids):
    """``(logits [T, vocab], residual stream after every layer [layers, T, width])`` of a whole sequence."""
    eps, mult = cfg["norm"]["eps"], cfg["residual_mult"]
    x = w["embed"][torch.as_tensor(ids)]
    outs, streams = [x], []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}"
        kind, m = layer["type"], layer["mixer"]
        if kind == "mingru":
            mixed = mingru(x, w, p)[0]
        elif kind == "mamba2":
            mixed = mamba2(x, w, p, m, eps)[0]
        elif kind == "latent_attention":
            mixed = latent_attention(x, w, p, m, eps)
        else:
            raise ValueError(kind)
        x = x + mult * norm_around_zero(mixed, w[p + ".norm1"], eps)
        if layer.get("mlp") is not None:
            x = x + mult * norm_around_zero(dense_ff(x, w, p), w[p + ".norm2"], eps)
        outs.append(x)
        a = w[p + ".dwa"]
        x = sum(a[j] * outs[j] for j in range(i + 2))
        streams.append(x)
    logits = norm_around_zero(x, w["final.norm"], eps) @ w["embed"].T * cfg["logit_scale"]
    return logits, torch.stack(streams)
