"""A plain, slow implementation of the Mezinex decoder, written from its equations for the tests.

One function per mechanism, whole sequences at once, loops over tokens for the recurrences, dense score
matrices, no cache, no kernels and no code of the package.  Everything runs in one dtype (float64 by default).

Notation: T tokens, d the residual width, weights a dict name -> tensor, linear weights [out, in].
"""
import math

import torch


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


# ---- embedding ------------------------------------------------------------------------------------------
def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every token: a hash of (previous, current); the first token takes the last row."""
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + int(t) * mul_cur) % buckets)
    return rows


def embed(tokens, table, pair_table=None, buckets=0, mul_prev=0, mul_cur=0):
    x = table[torch.as_tensor(list(tokens), dtype=torch.long)]
    if pair_table is not None:
        x = x + pair_table[torch.as_tensor(bigram_rows(tokens, buckets, mul_prev, mul_cur), dtype=torch.long)]
    return x


# ---- short causal convolution ---------------------------------------------------------------------------
def causal_conv(x, w, b):
    """x [T, C], w [C, taps] (the last column multiplies the current token), zeros before the start."""
    T, C = x.shape
    taps = w.shape[1]
    out = torch.zeros_like(x)
    for t in range(T):
        acc = b.clone()
        for k in range(taps):
            src = t - (taps - 1 - k)
            if src >= 0:
                acc = acc + w[:, k] * x[src]
        out[t] = acc
    return out


# ---- the gated linear recurrent unit ----------------------------------------------------------------------
def rglru_mixer(h, W, p, blocks):
    """Two branches: y = gelu(W_y h + b), u = conv(W_x h + b); gates per block of channels from u; a diagonal
    recurrence S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t with a_t = exp(-8 r_t softplus(lam)); out = W_o (S y)."""
    T = h.shape[0]
    y = gelu_tanh(h @ W[p + "y"].T + W[p + "y.b"])
    u = causal_conv(h @ W[p + "x"].T + W[p + "x.b"], W[p + "conv"], W[p + "conv.b"])
    width = u.shape[1]
    bw = width // blocks
    ub = u.view(T, blocks, bw)
    r = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, W[p + "ra"]) + W[p + "ra.b"]).reshape(T, width)
    i = torch.sigmoid(torch.einsum("tbi,boi->tbo", ub, W[p + "ri"]) + W[p + "ri.b"]).reshape(T, width)
    log_a = -8.0 * r * softplus(W[p + "lam"])
    a = torch.exp(log_a)
    S = torch.zeros(width, dtype=h.dtype)
    out = torch.zeros(T, width, dtype=h.dtype)
    for t in range(T):
        S = a[t] * S + torch.sqrt(1.0 - a[t] * a[t]) * i[t] * u[t]
        out[t] = S
    return (out * y) @ W[p + "o"].T


# ---- the state-space mixer ---------------------------------------------------------------------------------
def mamba2_mixer(h, W, p, heads, vdim, state, groups, norm_groups, eps):
    T = h.shape[0]
    inner, N, G = heads * vdim, state, groups
    proj = h @ W[p + "in"].T
    z = proj[:, :inner]
    xbc = silu(causal_conv(proj[:, inner:2 * inner + 2 * G * N], W[p + "conv"], W[p + "conv.b"]))
    dt = softplus(proj[:, 2 * inner + 2 * G * N:] + W[p + "dt_bias"])          # [T, heads]
    x = xbc[:, :inner].reshape(T, heads, vdim)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    decay_rate = torch.exp(W[p + "A_log"])
    S = torch.zeros(heads, N, vdim, dtype=h.dtype)
    y = torch.zeros(T, heads, vdim, dtype=h.dtype)
    per = heads // G
    for t in range(T):
        for hd in range(heads):
            g = hd // per
            S[hd] = torch.exp(-decay_rate[hd] * dt[t, hd]) * S[hd] + dt[t, hd] * torch.outer(B[t, g], x[t, hd])
            y[t, hd] = S[hd].T @ C[t, g] + W[p + "D"][hd] * x[t, hd]
    y = y.reshape(T, inner) * silu(z)
    y = rms(y.view(T, norm_groups, inner // norm_groups), eps).reshape(T, inner) * W[p + "norm"]
    return y @ W[p + "o"].T


# ---- latent attention -----------------------------------------------------------------------------------------
def rotate_pairs(x, positions, base, dims):
    """x [T, ..., n]: entries (2i, 2i+1) of the first ``dims`` entries turn by the angle p * base^(-2i/dims)."""
    out = x.clone()
    i = torch.arange(dims // 2, dtype=x.dtype)
    f = torch.pow(torch.tensor(base, dtype=x.dtype), -2.0 * i / dims)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [dims // 2]
    c, s = torch.cos(ang).view(shape), torch.sin(ang).view(shape)
    a, b = x[..., 0:dims:2], x[..., 1:dims:2]
    out[..., 0:dims:2] = a * c - b * s
    out[..., 1:dims:2] = b * c + a * s
    return out


def latent_attention(h, W, p, heads, dim, rot_dim, vdim, kv_rank, scale, rot_base, rot_dims, eps, first_position=0):
    T = h.shape[0]
    pos = torch.arange(first_position, first_position + T)
    cq = rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).view(T, heads, dim + rot_dim)
    q_plain, q_rot = q[..., :dim], rotate_pairs(q[..., dim:], pos, rot_base, rot_dims)
    kv = h @ W[p + "dkv"].T
    c = rms(kv[:, :kv_rank], eps) * W[p + "dkv.norm"]
    k_rot = rotate_pairs(kv[:, kv_rank:], pos, rot_base, rot_dims)              # one for all heads
    k_plain = (c @ W[p + "uk"].T).view(T, heads, dim)
    v = (c @ W[p + "uv"].T).view(T, heads, vdim)
    s = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihd,jd->hij", q_rot, k_rot)) * scale
    causal = torch.arange(T)[None, :] <= torch.arange(T)[:, None]
    s = s.masked_fill(~causal, float("-inf"))
    w = torch.softmax(s, dim=-1)
    o = torch.einsum("hij,jhd->ihd", w, v).reshape(T, heads * vdim)
    o = o * torch.sigmoid(h @ W[p + "g"].T)
    return o @ W[p + "o"].T


# ---- feed-forward ---------------------------------------------------------------------------------------------
def gated_ffn(h, W, p):
    return (silu(h @ W[p + "gate"].T) * (h @ W[p + "up"].T)) @ W[p + "down"].T


# ---- several residual streams -----------------------------------------------------------------------------------
def hyper_read(xs, w_in):
    """xs [S, T, d] -> the sublayer's input, sum_s in[s] x_s."""
    return torch.einsum("s,std->td", w_in, xs)


def hyper_write(xs, y, w_mix, w_out):
    """All streams at once from the old ones: x_t <- sum_s mix[s, t] x_s + out[t] y."""
    return torch.einsum("st,sid->tid", w_mix, xs) + w_out[:, None, None] * y[None]


# ---- the model --------------------------------------------------------------------------------------------------
def run_order(cfg):
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return list(range(n))
    a, b, times = loop["start"], loop["stop"], loop["times"]
    return list(range(a)) + list(range(a, b)) * times + list(range(b, n))


def mixer(kind, h, W, p, m, eps):
    if kind == "rglru":
        return rglru_mixer(h, W, p, m["blocks"])
    if kind == "mamba2":
        return mamba2_mixer(h, W, p, m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"], eps)
    if kind == "latent_attention":
        return latent_attention(h, W, p, m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"], m["scale"],
                                m["rot"]["base"], m["rot"]["dims"], eps)
    raise ValueError(kind)


def forward(cfg, W, tokens, dtype=torch.float64, layer_outputs=None):
    """Logits [T, vocab] of a whole sequence from empty state.  ``layer_outputs``: a list that receives the residual
    stream (the sum of the streams) after every layer run."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    eps = cfg["norm"]["eps"]
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        x = embed(tokens, W["embed"], W["bigram"], big["buckets"], big["mul_prev"], big["mul_cur"])
    else:
        x = embed(tokens, W["embed"])
    streams = cfg.get("streams")
    xs = torch.stack([x] * streams) if streams else None
    for li in run_order(cfg):
        layer = cfg["layers"][li]
        p = "l%d." % li
        subs = [(1, lambda h: mixer(layer["type"], h, W, p + "mix.", layer["mixer"], eps))]
        if layer.get("mlp"):
            subs.append((2, lambda h: gated_ffn(h, W, p + "mlp.")))
        for q, f in subs:
            nw = W[p + "norm%d" % q]
            if streams:
                u = hyper_read(xs, W[p + "hc%d.in" % q])
                y = f(rms(u, eps) * nw)
                xs = hyper_write(xs, y, W[p + "hc%d.mix" % q], W[p + "hc%d.out" % q])
            else:
                x = x + f(rms(x, eps) * nw)
        if layer_outputs is not None:
            layer_outputs.append(xs.sum(0) if streams else x.clone())
    if streams:
        x = xs.sum(0)
    return (rms(x, eps) * W["final.norm"]) @ W["head"].T * cfg.get("logit_scale", 1.0)


# ---- weights for the tests ----------------------------------------------------------------------------------------
def tensor_shapes(cfg):
    """Name -> shape of every tensor of a configuration."""
    d, V = cfg["width"], cfg["vocab"]
    S = cfg.get("streams")
    out = {"embed": (V, d), "final.norm": (d,), "head": (V, d)}
    big = (cfg.get("embedding") or {}).get("bigram")
    if big:
        out["bigram"] = (big["buckets"] + 1, d)
    for i, l in enumerate(cfg["layers"]):
        p, m = "l%d." % i, l["mixer"]
        out[p + "norm1"] = (d,)
        if l["type"] == "rglru":
            w, b = m["width"], m["blocks"]
            out.update({p + "mix.y": (w, d), p + "mix.y.b": (w,), p + "mix.x": (w, d), p + "mix.x.b": (w,),
                        p + "mix.conv": (w, m["conv"]), p + "mix.conv.b": (w,), p + "mix.ra": (b, w // b, w // b),
                        p + "mix.ra.b": (b, w // b), p + "mix.ri": (b, w // b, w // b), p + "mix.ri.b": (b, w // b),
                        p + "mix.lam": (w,), p + "mix.o": (d, w)})
        elif l["type"] == "mamba2":
            inner, gn = m["heads"] * m["vdim"], m["groups"] * m["state"]
            out.update({p + "mix.in": (2 * inner + 2 * gn + m["heads"], d), p + "mix.conv": (inner + 2 * gn, m["conv"]),
                        p + "mix.conv.b": (inner + 2 * gn,), p + "mix.dt_bias": (m["heads"],), p + "mix.A_log": (m["heads"],),
                        p + "mix.D": (m["heads"],), p + "mix.norm": (inner,), p + "mix.o": (d, inner)})
        else:
            H = m["heads"]
            out.update({p + "mix.dq": (m["q_rank"], d), p + "mix.dq.norm": (m["q_rank"],),
                        p + "mix.uq": (H * (m["dim"] + m["rot_dim"]), m["q_rank"]),
                        p + "mix.dkv": (m["kv_rank"] + m["rot_dim"], d), p + "mix.dkv.norm": (m["kv_rank"],),
                        p + "mix.uk": (H * m["dim"], m["kv_rank"]), p + "mix.uv": (H * m["vdim"], m["kv_rank"]),
                        p + "mix.g": (H * m["vdim"], d), p + "mix.o": (d, H * m["vdim"])})
        subs = [1]
        if l.get("mlp"):
            ff = l["mlp"]["ff"]
            out.update({p + "norm2": (d,), p + "mlp.gate": (ff, d), p + "mlp.up": (ff, d), p + "mlp.down": (d, ff)})
            subs.append(2)
        if S:
            for q in subs:
                out.update({p + "hc%d.in" % q: (S,), p + "hc%d.out" % q: (S,), p + "hc%d.mix" % q: (S, S)})
    return out


def random_weights(cfg, seed):
    """Weights at scales that keep every mechanism alive: products near unit gain, decays spread over (0, 1), streams
    that mix but do not blow up.  Values are rounded to bfloat16 (what a folder stores)."""
    g = torch.Generator().manual_seed(seed)
    S = cfg.get("streams") or 1
    W = {}
    for name, shape in tensor_shapes(cfg).items():
        r = torch.randn(*shape, generator=g, dtype=torch.float64)
        leaf = name.split(".", 1)[1] if name.startswith("l") and "." in name else name
        if leaf in ("norm1", "norm2", "mix.norm", "mix.dq.norm", "mix.dkv.norm", "mix.D") or name == "final.norm":
            t = 1.0 + 0.2 * r
        elif leaf.endswith(".b") or leaf in ("mix.dt_bias", "mix.A_log"):
            t = 0.5 * r
        elif leaf == "mix.lam":
            t = 1.5 * r - 1.0
        elif leaf == "mix.conv":
            t = 0.6 * r
        elif leaf.endswith(".in"):
            t = 1.0 / S + 0.3 * r
        elif leaf.endswith(".out"):
            t = 1.0 + 0.3 * r
        elif leaf.endswith(".mix"):
            t = torch.eye(S, dtype=torch.float64) + 0.15 * r
        elif name in ("embed", "bigram"):
            t = r
        else:
            t = r / math.sqrt(shape[-1])
        W[name] = t.to(torch.bfloat16).to(torch.float64)
    return W
