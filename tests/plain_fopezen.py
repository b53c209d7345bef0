"""A plain, slow implementation of the Fopezen decoder, written from its equations for the tests.

One function per mechanism, whole sequences at once, dense score matrices, no cache, no kernels and
no code of the package.  Everything runs in one dtype (float32 by default, float64 to see rounding).

Notation: T tokens, d the residual width, H query heads, G key/value heads, dk the query/key size
per head, dv the value size per head.  Weights are a dict name -> tensor, linear weights [out, in].
"""
import math

import torch


def rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def norm_one_plus(x, w, eps):
    """The layer norm of this design: unit root mean square, then times (1 + w)."""
    return rms(x, eps) * (1.0 + w)


def sinusoid(positions, width, dtype):
    """Entry 2i is sin(p * 10000^(-2i/width)), entry 2i+1 the cosine of the same angle."""
    i = torch.arange((width + 1) // 2, dtype=dtype)          # the arithmetic of the exponent is done in ``dtype``
    freq = torch.pow(torch.tensor(10000.0, dtype=dtype), -2.0 * i / width)
    ang = positions.to(dtype)[:, None] * freq[None, :]
    out = torch.zeros(len(positions), width, dtype=dtype)
    out[:, 0::2] = torch.sin(ang)
    out[:, 1::2] = torch.cos(ang)[:, :width // 2]            # an odd width ends on a sine
    return out


def embed(tokens, table, first_position=0):
    T = len(tokens)
    pos = torch.arange(first_position, first_position + T)
    return table[torch.as_tensor(tokens, dtype=torch.long)] + sinusoid(pos, table.shape[1], table.dtype)


def visible(T, size, keep_first):
    """vis[i, j]: query i sees key j when j <= i and (i - j < size or j < keep_first).  size None: every earlier key."""
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    near = (i - j < size) if size else torch.ones(T, T, dtype=torch.bool)
    return (j <= i) & (near | (j < keep_first))


def weights_of_scores(s, vis, sink):
    """Softmax over the visible keys; with ``sink`` one more term exp(0) in the denominator that has no value."""
    s = s.masked_fill(~vis, float("-inf"))
    m = s.max(-1, keepdim=True).values
    if sink:
        m = torch.clamp(m, min=0.0)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True)
    if sink:
        den = den + torch.exp(-m)
    return e / den


def qk_norm_per_head(x, w, H, eps):
    """x [T, H*dk]: each head's dk entries to unit root mean square, times w [dk] (the same for all heads)."""
    T = x.shape[0]
    return (rms(x.view(T, H, -1), eps) * w).reshape(T, -1)


def qk_norm_whole(x, w, eps):
    """x [T, H*dk]: the whole row to unit root mean square, times w [H*dk]."""
    return rms(x, eps) * w


def mix_values(v, v_first, lam):
    return (1.0 - lam) * v + lam * v_first


def attend(q, k, v, H, G, scale, vis, sink):
    """q [T, H*dk], k [T, G*dk], v [T, G*dv] -> [T, H*dv]; query head h reads key/value head h // (H/G)."""
    T = q.shape[0]
    q = q.view(T, H, -1)
    k = k.view(T, G, -1)
    v = v.view(T, G, -1)
    out = []
    for h in range(H):
        g = h // (H // G)
        s = (q[:, h] @ k[:, g].T) * scale
        out.append(weights_of_scores(s, vis, sink) @ v[:, g])
    return torch.cat(out, dim=-1)


def mixer(kind, h, W, p, cfg, eps, carry):
    """One attention mixer.  kind 'attention': norms per head, sink softmax, output gate, bias on the output
    projection.  kind 'attention_2': norms over the whole projection, plain softmax, no gate.  ``carry`` holds the
    values of the first value-mixing layer."""
    H, G = cfg["heads"], cfg["kv_heads"]
    q = h @ W[p + "q"].T + W[p + "q.b"]
    k = h @ W[p + "k"].T + W[p + "k.b"]
    v = h @ W[p + "v"].T + W[p + "v.b"]
    if kind == "attention":
        q = qk_norm_per_head(q, W[p + "q.norm"], H, eps)
        k = qk_norm_per_head(k, W[p + "k.norm"], G, eps)
    else:
        q = qk_norm_whole(q, W[p + "q.norm"], eps)
        k = qk_norm_whole(k, W[p + "k.norm"], eps)
    if cfg.get("v_mix"):
        if "v_first" in carry:
            v = mix_values(v, carry["v_first"], W[p + "vmix"])
        else:
            carry["v_first"] = v
    mask = cfg.get("mask") or {}
    vis = visible(h.shape[0], mask.get("size"), mask.get("keep_first", 0))
    a = attend(q, k, v, H, G, cfg["scale"], vis, sink=(kind == "attention"))
    if kind == "attention":
        a = a * torch.sigmoid(h @ W[p + "g"].T)
        return a @ W[p + "o"].T + W[p + "o.b"]
    return a @ W[p + "o"].T


def feed_forward(h, W, p):
    """down(relu(up h)^2)."""
    return torch.relu(h @ W[p + "up"].T).square() @ W[p + "down"].T


def forward(config, W, tokens, dtype=torch.float32, layers_out=None):
    """Logits [T, vocab] of a whole sequence; ``layers_out`` (a list) receives the residual stream after every layer."""
    W = {n: t.to(dtype) for n, t in W.items()}
    eps = config["norm"]["eps"]
    x = embed(tokens, W["embed"])
    carry = {}
    for i, layer in enumerate(config["layers"]):
        p = "l%d." % i
        y = mixer(layer["type"], x, W, p + "mix.", layer["mixer"], eps, carry)
        x = x + norm_one_plus(y, W[p + "norm1"], eps)
        if layer.get("mlp"):
            y = feed_forward(x, W, p + "mlp.")
            x = x + norm_one_plus(y, W[p + "norm2"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_one_plus(x, W["final.norm"], eps) @ W["embed"].T


def random_weights(config, seed, std=None):
    """Random weights of a configuration, rounded to bfloat16 values (held in float32)."""
    g = torch.Generator().manual_seed(seed)
    d, V = config["width"], config["vocab"]

    def mat(o, i, s=None):
        return (torch.randn(o, i, generator=g) * (s if s is not None else 1.0 / math.sqrt(i))).to(torch.bfloat16).float()

    def vec(n, s=0.1, mean=0.0):
        return (torch.randn(n, generator=g) * s + mean).to(torch.bfloat16).float()

    W = {"embed": mat(V, d, 1.0), "final.norm": vec(d)}
    for i, layer in enumerate(config["layers"]):
        p, m = "l%d." % i, layer["mixer"]
        H, G, dk, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"] = vec(d)
        W[p + "mix.q"], W[p + "mix.q.b"] = mat(H * dk, d), vec(H * dk)
        W[p + "mix.k"], W[p + "mix.k.b"] = mat(G * dk, d), vec(G * dk)
        W[p + "mix.v"], W[p + "mix.v.b"] = mat(G * dv, d), vec(G * dv)
        per_head = layer["type"] == "attention"
        W[p + "mix.q.norm"] = vec(dk if per_head else H * dk, 0.2, 1.0)
        W[p + "mix.k.norm"] = vec(dk if per_head else G * dk, 0.2, 1.0)
        if m.get("v_mix"):
            W[p + "mix.vmix"] = vec(1, 0.15, 0.4).reshape(())
        W[p + "mix.o"] = mat(d, H * dv)
        if per_head:
            W[p + "mix.g"] = mat(H * dv, d)
            W[p + "mix.o.b"] = vec(d)
        if layer.get("mlp"):
            W[p + "norm2"] = vec(d)
            W[p + "mlp.up"] = mat(layer["mlp"]["ff"], d)
            W[p + "mlp.down"] = mat(d, layer["mlp"]["ff"])
    return W
