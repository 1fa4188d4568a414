"""A plain, slow rendition of the Sunatar design on one whole sequence: no cache, no batch, one function per
mechanism, written from the design's equations with torch tensor arithmetic only. It shares no code with the
package and is what the package's parts, kernels and engine are tested against.

A model is `(cfg, w)`: `cfg` the dictionary of its config.json, `w` a dictionary of tensors by checkpoint name.
Everything is computed in the dtype of `w`'s tensors after `widen` (float64 by default), token after token where
the design is a recurrence.

Notation: T tokens, D the model's width, H query heads, G key/value heads, n the query/key size of a head,
v its value size.
"""
import math

import torch


def widen(w, dtype=torch.float64):
    return {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in w.items()}


# ---------------------------------------------------------------- norms and activations

def layer_norm(x, weight, eps):
    """(x - mean) / sqrt(var + eps) * weight over the last axis; var is the mean squared deviation."""
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * weight


def unit_rms(x, eps):
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def log_sigmoid(z):
    """log(1 / (1 + exp(-z))), written so that neither side overflows."""
    return torch.minimum(z, torch.zeros_like(z)) - torch.log1p(torch.exp(-z.abs()))


def soft_cap(z, cap):
    return cap * torch.tanh(z / cap)


# ---------------------------------------------------------------- rotary positions

def rotary_frequencies(base, dims, scaling=None):
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` = {factor, low, high, original} a frequency whose
    wavelength 2 pi / f is longer than original / low is divided by factor, one shorter than original / high is
    kept, and between the two the divided and the kept one are blended linearly in original / wavelength."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if scaling:
        factor, low, high, orig = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
        out = []
        for fi in f:
            wavelength = 2.0 * math.pi / fi
            if wavelength < orig / high:
                out.append(fi)
            elif wavelength > orig / low:
                out.append(fi / factor)
            else:
                s = (orig / wavelength - low) / (high - low)
                out.append((1.0 - s) * fi / factor + s * fi)
        f = out
    return torch.tensor(f, dtype=torch.float64)


def rotate_halves(x, positions, freqs):
    """x `[T, heads, n]`: of the first dims = 2 len(freqs) elements of a head, element i is paired with element
    i + dims / 2; the pair (u, v) at position p becomes (u cos a - v sin a, v cos a + u sin a), a = p f_i."""
    half = freqs.numel()
    angle = positions.to(torch.float64)[:, None, None] * freqs[None, None, :]
    cos, sin = torch.cos(angle).to(x.dtype), torch.sin(angle).to(x.dtype)
    u, v = x[..., :half], x[..., half:2 * half]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., 2 * half:]], dim=-1)


# ---------------------------------------------------------------- attention

def window_softmax(scores, window):
    """scores `[heads, T, T]`: softmax over the keys j with 0 <= i - j < window (all j <= i without one)."""
    t = scores.shape[-1]
    i = torch.arange(t)[:, None]
    j = torch.arange(t)[None, :]
    seen = (j <= i) & ((i - j < window) if window else torch.ones_like(j <= i))
    return torch.softmax(scores.masked_fill(~seen, float("-inf")), dim=-1)


def attention_values(m, w, p, h, eps):
    """The values a layer makes on its own, before any mixing: `[T, G, v]`."""
    return (h @ w[p + "v"].T + w[p + "v.b"]).view(h.shape[0], m["kv_heads"], m["vdim"])


def attention(m, w, p, h, eps, v_first=None):
    """The attention mixer of one layer on `h` `[T, D]`; `p` is the tensors' prefix ('l3.mix.'). `v_first`: the
    values of the first value-mixing layer, or None where this layer is that one or mixes nothing.
    Returns (output `[T, D]`, this layer's own values)."""
    t = h.shape[0]
    heads, groups, n, v = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = h @ w[p + "q"].T + w[p + "q.b"]
    k = h @ w[p + "k"].T + w[p + "k.b"]
    # one norm over the whole projection, all heads at once
    q = unit_rms(q, eps) * w[p + "q.norm"]
    k = unit_rms(k, eps) * w[p + "k.norm"]
    rot = m["rot"]
    freqs = rotary_frequencies(rot["base"], rot["dims"], rot.get("scaling"))
    positions = torch.arange(t)
    q = rotate_halves(q.view(t, heads, n), positions, freqs)
    k = rotate_halves(k.view(t, groups, n), positions, freqs)
    own = attention_values(m, w, p, h, eps)
    val = own
    if v_first is not None:
        lam = w[p + "vmix"]
        val = (1.0 - lam) * own + lam * v_first
    per = heads // groups
    k = k.repeat_interleave(per, dim=1)
    val = val.repeat_interleave(per, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"]
    weights = window_softmax(scores, (m.get("mask") or {}).get("size"))
    o = torch.einsum("hij,jhd->ihd", weights, val).reshape(t, heads * v)
    return o @ w[p + "o"].T, own


# ---------------------------------------------------------------- the matrix memory

def mlstm(m, w, p, h, eps):
    """The matrix-memory mixer on `h` `[T, D]`, token after token from an empty memory."""
    t = h.shape[0]
    heads, n, v, cap = m["heads"], m["dim"], m["vdim"], m["gate_cap"]
    q = (h @ w[p + "q"].T).view(t, heads, n) * n ** -0.5
    k = (h @ w[p + "k"].T).view(t, heads, n)
    val = (h @ w[p + "v"].T).view(t, heads, v)
    gi = soft_cap(h @ w[p + "i"].T + w[p + "i.b"], cap)                       # log of the input gate
    gf = log_sigmoid(soft_cap(h @ w[p + "f"].T + w[p + "f.b"], cap))          # log of the forget gate
    mem = torch.zeros(heads, n, v, dtype=h.dtype)
    norm = torch.zeros(heads, n, dtype=h.dtype)
    peak = torch.zeros(heads, dtype=h.dtype)                                  # the running maximum starts at 0
    out = []
    for s in range(t):
        new_peak = torch.maximum(gf[s] + peak, gi[s])
        keep = torch.exp(gf[s] + peak - new_peak)
        take = torch.exp(gi[s] - new_peak)
        mem = keep[:, None, None] * mem + take[:, None, None] * k[s][:, :, None] * val[s][:, None, :]
        norm = keep[:, None] * norm + take[:, None] * k[s]
        peak = new_peak
        top = torch.einsum("hnv,hn->hv", mem, q[s])
        below = torch.maximum((norm * q[s]).sum(-1).abs(), torch.exp(-peak)) + 1e-6
        out.append(top / below[:, None])
    o = unit_rms(torch.stack(out), eps).reshape(t, heads * v) * w[p + "norm"]
    o = o * torch.sigmoid(h @ w[p + "g"].T)
    return o @ w[p + "o"].T


# ---------------------------------------------------------------- the feed-forward

def gated_expert(w, p, h):
    """W_down (silu(W_gate h) * (W_up h))."""
    return (silu(h @ w[p + "gate"].T) * (h @ w[p + "up"].T)) @ w[p + "down"].T


def route(z, top):
    """Scores sigmoid(z) `[T, E]`; the `top` largest of a token (the lower index where two are equal) and their
    scores as they are."""
    s = torch.sigmoid(z)
    order = torch.sort(s, dim=-1, descending=True, stable=True).indices[:, :top]
    return order, torch.gather(s, 1, order)


def mixture(mlp, w, p, h):
    """The chosen experts on score * h, summed, plus the shared expert on h."""
    chosen, score = route(h @ w[p + "router"].T, mlp["router"]["top"])
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, s in zip(chosen[t].tolist(), score[t]):
            out[t] = out[t] + gated_expert(w, f"{p}e{e}.", s * h[t])
    if mlp.get("shared"):
        out = out + gated_expert(w, p + "shared.", h)
    return out


# ---------------------------------------------------------------- the model

def forward(cfg, w, tokens, return_layers=False):
    """Logits `[T, vocab]` of a whole sequence; with `return_layers` also the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = w["embed"][torch.tensor(tokens)] * (cfg.get("embedding") or {}).get("scale", 1.0)
    v_first = None
    streams = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = layer_norm(x, w[p + "norm1"], eps)
        m = layer["mixer"]
        if layer["type"] == "attention":
            mixes = bool(m.get("v_mix"))
            y, own = attention(m, w, p + "mix.", h, eps, v_first if mixes else None)
            if mixes and v_first is None:
                v_first = own
        elif layer["type"] == "mlstm":
            y = mlstm(m, w, p + "mix.", h, eps)
        else:
            raise ValueError(layer["type"])
        if layer.get("mlp") is not None:
            y = y + mixture(layer["mlp"], w, p + "mlp.", h)
        x = x + y
        streams.append(x)
    logits = layer_norm(x, w["final.norm"], eps) @ w["head"].T
    return (logits, torch.stack(streams)) if return_layers else logits
