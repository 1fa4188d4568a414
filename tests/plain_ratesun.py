"""A plain, slow rendition of the Ratesun design on one whole sequence: no cache, no batch, one function per
mechanism, written from the design's equations with torch tensor arithmetic only. It shares no code with the
package and is what the package's parts, kernels and engine are tested against.

A model is `(cfg, w)`: `cfg` the dictionary of its config.json, `w` a dictionary of tensors by checkpoint name.
Everything is computed in the dtype of `w`'s tensors after `widen` (float64 by default), whole sequence at once.

Notation: T tokens, D the model's width, H heads; for a head, n unrotated and r rotated query/key elements,
v value elements; R the size of the key/value latent, Q that of the query latent.
"""
import math

import torch


def widen(w, dtype=torch.float64):
    return {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}


# ---------------------------------------------------------------- norms and activations

def layer_norm(x, weight, bias, eps):
    """(x - mean) / sqrt(var + eps) * weight + bias over the last axis; var is the mean squared deviation."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight + bias


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def rms_norm(x, weight, eps):
    return unit_rms(x, eps) * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def poly_norm(z, coeffs, eps):
    """a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, N = `unit_rms` over a token's values."""
    a, b, c, e = (coeffs[i] for i in range(4))
    return a * unit_rms(z, eps) + b * unit_rms(z * z, eps) + c * unit_rms(z * z * z, eps) + e


# ---------------------------------------------------------------- the input end

def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    """Row of the pair table for every token: (previous * mul_prev + token * mul_cur) mod buckets, and row
    `buckets` for the first token of the sequence."""
    rows = []
    for i, t in enumerate(tokens):
        rows.append(buckets if i == 0 else (int(tokens[i - 1]) * mul_prev + int(t) * mul_cur) % buckets)
    return rows


def embed(cfg, w, tokens):
    x = w["embed"][torch.tensor(tokens)]
    pair = (cfg.get("embedding") or {}).get("bigram")
    if pair:
        x = x + w["bigram"][torch.tensor(bigram_rows(tokens, pair["buckets"], pair["mul_prev"], pair["mul_cur"]))]
    return x


# ---------------------------------------------------------------- the short convolution before a sublayer

def input_conv(h, weight):
    """h + conv(h): conv(h)_t = sum_j weight[:, j] * h_(t - taps + 1 + j), zeros before the start.
    h `[T, D]`, weight `[D, taps]`."""
    taps = weight.shape[1]
    out = h.clone()
    for t in range(h.shape[0]):
        for j in range(taps):
            s = t - taps + 1 + j
            if s >= 0:
                out[t] = out[t] + weight[:, j] * h[s]
    return out


# ---------------------------------------------------------------- rotary positions

def rotate_pairs(x, positions, base, dims):
    """Turns the first `dims` elements of the last axis, element 2i with 2i + 1, by the angle
    position * base^(-2i / dims); the rest pass. x `[T, ..., n]`, positions `[T]`."""
    out = x.clone()
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        a = positions.to(x.dtype) * f
        shape = [-1] + [1] * (x.dim() - 2)
        cos, sin = torch.cos(a).reshape(shape), torch.sin(a).reshape(shape)
        u, v = x[..., 2 * i], x[..., 2 * i + 1]
        out[..., 2 * i] = u * cos - v * sin
        out[..., 2 * i + 1] = v * cos + u * sin
    return out


# ---------------------------------------------------------------- the mixer

def kv_latent(h, w, p, m, eps, positions):
    """The latent c `[T, R]` (normed) and the shared rotated key part `[T, r]` (turned by its position)."""
    R, r = m["kv_rank"], m["rot_dim"]
    d = h @ w[p + "dkv"].T
    c = rms_norm(d[:, :R], w[p + "dkv.norm"], eps)
    k_rot = rotate_pairs(d[:, R:R + r], positions, m["rot"]["base"], m["rot"]["dims"])
    return c, k_rot


def latent_attention(h, w, p, m, eps, positions, c, k_rot):
    """One latent-attention mixer on `h` `[T, D]` with the latent `c` and rotated key part `k_rot` of its own
    layer or of the layer it borrows them from. Scores (q_n . k_n + q_r . k_r) * scale, a window of
    `mask.size` keys ending at the query, softmax, values, output projection."""
    T = h.shape[0]
    H, n, r, v = m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    cq = rms_norm(h @ w[p + "dq"].T, w[p + "dq.norm"], eps)
    q = (cq @ w[p + "uq"].T).reshape(T, H, n + r)
    q_n = q[..., :n]
    q_r = rotate_pairs(q[..., n:], positions, m["rot"]["base"], m["rot"]["dims"])
    k_n = (c @ w[p + "uk"].T).reshape(T, H, n)
    val = (c @ w[p + "uv"].T).reshape(T, H, v)
    scores = torch.einsum("ihd,jhd->hij", q_n, k_n) + torch.einsum("ihd,jd->hij", q_r, k_rot)
    scores = scores * m["scale"]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    seen = (j <= i)
    size = (m.get("mask") or {}).get("size")
    if size is not None:
        seen = seen & (i - j < size)
    scores = scores.masked_fill(~seen[None], float("-inf"))
    prob = torch.softmax(scores, dim=-1)
    out = torch.einsum("hij,jhd->ihd", prob, val).reshape(T, H * v)
    return out @ w[p + "o"].T


# ---------------------------------------------------------------- the feed-forward and the token input of a layer

def feed_forward(h, w, p, eps):
    return poly_norm(h @ w[p + "up"].T, w[p + "act"], eps) @ w[p + "down"].T


def token_side(x, w, layer, tokens, dim, eps):
    """y = proj (gelu_tanh(gate x) * e), e the layer's part of the token's side row; returns y scaled to unit
    root mean square, times the weight."""
    e = w["side.embed"][torch.tensor(tokens)][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ w[f"l{layer}.side.gate"].T) * e
    y = g @ w[f"l{layer}.side.proj"].T
    return unit_rms(y, eps) * w[f"l{layer}.side.norm"]


# ---------------------------------------------------------------- the whole model

def forward(cfg, w, tokens, taps=None):
    """Logits `[T, vocab]`. `taps`, a dictionary, gets the stream after every layer under "layers" (what goes
    on to the next layer) and "own" (the layer's own result before the average over depth)."""
    eps = cfg["norm"]["eps"]
    mult = cfg["residual_mult"]
    T = len(tokens)
    positions = torch.arange(T)
    x = embed(cfg, w, tokens)
    results = [x]
    latents = {}
    side = cfg.get("token_side")
    for i, layer in enumerate(cfg["layers"]):
        L = f"l{i}."
        m = layer["mixer"]

        def norm(t, name):
            return layer_norm(t, w[L + name], w[L + name + ".b"], eps)

        h = norm(x, "norm1")
        if L + "canon1" in w:
            h = input_conv(h, w[L + "canon1"])
        src = m.get("kv_from")
        if src is None:
            latents[i] = kv_latent(h, w, L + "mix.", m, eps, positions)
            src = i
        c, k_rot = latents[src]
        x = x + mult * norm(latent_attention(h, w, L + "mix.", m, eps, positions, c, k_rot), "norm1b")
        if layer.get("mlp") is not None:
            h = norm(x, "norm2")
            if L + "canon2" in w:
                h = input_conv(h, w[L + "canon2"])
            x = x + mult * norm(feed_forward(h, w, L + "mlp.", eps), "norm2b")
        if side:
            x = x + mult * token_side(x, w, i, tokens, side["dim"], eps)
        results.append(x)
        if L + "dwa" in w:
            x = sum(w[L + "dwa"][j] * results[j] for j in range(i + 2))
        if taps is not None:
            taps.setdefault("own", []).append(results[-1])
            taps.setdefault("layers", []).append(x)
    x = layer_norm(x, w["final.norm"], w["final.norm.b"], eps)
    return (x @ w["embed"].T) * cfg["logit_scale"]
