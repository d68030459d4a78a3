"""A plain, slow implementation of the Biberax decoder in float64 on the CPU: one function per
mechanism, written from the equations, sharing no code with the engine.  It reads the same
``config.json`` dictionary and the same tensor names as the engine and runs whole sequences
only (no cache, no portions): what the engine must reproduce however it cuts the work.

Notation: ``h`` a layer's normalised input ``[T, width]``; positions count from 0; ``i`` is the
position of a query and ``j`` of a key."""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def root_mean_square_norm(x, eps, weight=None):
    """x / sqrt(mean(x^2) + eps) over the last dimension, times ``weight`` if given."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def scaled_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i/dims) for the dims/2 pairs; with ``scaling`` (factor, low, high, original) a
    frequency whose wavelength 2 pi / f is longer than original/low is divided by factor, one
    shorter than original/high stays, and between the two the divided and the plain frequency are
    blended linearly in original/wavelength."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling:
            factor, low, high, original = (float(scaling[key]) for key in ("factor", "low", "high", "original"))
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return torch.tensor(out, dtype=F64)


def rotate_neighbours(x, positions, frequencies):
    """Rotary encoding of the first 2 * len(frequencies) dimensions of every head of ``x [T, heads, d]``:
    dimension 2i is paired with 2i + 1, and the pair (u, v) at position p becomes
    (u cos a - v sin a, v cos a + u sin a) with a = p f_i.  Later dimensions pass."""
    dims = 2 * len(frequencies)
    angle = positions.to(F64)[:, None] * frequencies[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * cos - v * sin
    out[..., 1:dims:2] = v * cos + u * sin
    return out


def causal(n):
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    return j <= i


def same_chunk(n, size):
    """visible[i, j]: j <= i and both lie in the same run of ``size`` positions counted from 0."""
    i, j = torch.arange(n)[:, None], torch.arange(n)[None, :]
    return (j <= i) & (i // size == j // size)


def distance_bucket(n, rows, farthest):
    """The row of a bias table of ``rows`` rows for the distance n >= 0: the first half of the rows
    are the distances themselves, the second half are spaced evenly in the logarithm up to
    ``farthest``; everything beyond shares the last row."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(farthest / half) * (rows - half))))


def distance_bias(n, table, farthest):
    """bias[h, i, j] = table[bucket(i - j), h] for j <= i (zero elsewhere: masked anyway)."""
    rows, heads = table.shape
    out = torch.zeros((heads, n, n), dtype=F64)
    for i in range(n):
        for j in range(i + 1):
            out[:, i, j] = table[distance_bucket(i - j, rows, farthest)]
    return out


def attention_with_sink(q, k, v, scale, visible, sink, bias=None):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads kv head h // (H/G).
    s = scale q.k (+ bias[h]); p_j = exp(s_j) / (exp(sink_h) + sum_visible exp(s_j)): the sink is a
    score without key or value.  ``sink`` is [H] (zeros: a one in the denominator) or None (no sink)."""
    n, heads, _ = q.shape
    group = heads // k.shape[1]
    out = torch.zeros((n, heads, v.shape[2]), dtype=F64)
    for h in range(heads):
        s = (q[:, h] @ k[:, h // group].T) * scale
        if bias is not None:
            s = s + bias[h]
        s = s.masked_fill(~visible, float("-inf"))
        top = s.max(dim=-1, keepdim=True).values
        if sink is not None:
            top = torch.maximum(top, sink[h].reshape(1, 1))
        e = torch.exp(s - top)
        total = e.sum(dim=-1, keepdim=True)
        if sink is not None:
            total = total + torch.exp(sink[h] - top)
        out[:, h] = (e / total) @ v[:, h // group]
    return out


def tensor(weights, name):
    return weights[name].to(F64)


def rotary_chunked_mixer(h, positions, m, weights, prefix):
    """The mixer called ``attention``: grouped heads, rotation of the leading dimensions in neighbouring
    pairs, keys of the query's own chunk only, a one in the softmax's denominator, a sigmoid gate on
    the heads' outputs."""
    n = h.shape[0]
    heads, groups, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ tensor(weights, prefix + ".q").T).view(n, heads, d)
    k = (h @ tensor(weights, prefix + ".k").T).view(n, groups, d)
    v = (h @ tensor(weights, prefix + ".v").T).view(n, groups, dv)
    rot = m.get("rot")
    if rot and rot.get("dims"):
        f = scaled_frequencies(int(rot["dims"]), rot["base"], rot.get("scaling"))
        q, k = rotate_neighbours(q, positions, f), rotate_neighbours(k, positions, f)
    mask = m.get("mask")
    visible = same_chunk(n, int(mask["size"])) if mask and mask.get("size") else causal(n)
    o = attention_with_sink(q, k, v, float(m["scale"]), visible, torch.zeros(heads, dtype=F64))
    gate = torch.sigmoid(h @ tensor(weights, prefix + ".g").T)
    return (o.reshape(n, heads * dv) * gate) @ tensor(weights, prefix + ".o").T


def biased_shared_kv_mixer(h, m, weights, prefix, eps):
    """The mixer called ``attention_2``: biased projections, values that are the keys as projected,
    one norm over all of q and over all of k, a learned bias by distance, all earlier keys, a learned
    sink a head, a sigmoid gate, a biased output projection."""
    n = h.shape[0]
    heads, groups, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = h @ tensor(weights, prefix + ".q").T + tensor(weights, prefix + ".q.b")
    k = h @ tensor(weights, prefix + ".k").T + tensor(weights, prefix + ".k.b")
    v = k.view(n, groups, d)
    q = root_mean_square_norm(q, eps, tensor(weights, prefix + ".q.norm")).view(n, heads, d)
    k = root_mean_square_norm(k, eps, tensor(weights, prefix + ".k.norm")).view(n, groups, d)
    bias = distance_bias(n, tensor(weights, prefix + ".rel"), float(m["bias_max"]))
    o = attention_with_sink(q, k, v, float(m["scale"]), causal(n), tensor(weights, prefix + ".sink"), bias)
    gate = torch.sigmoid(h @ tensor(weights, prefix + ".g").T)
    return (o.reshape(n, heads * d) * gate) @ tensor(weights, prefix + ".o").T + tensor(weights, prefix + ".o.b")


def dense_feed_forward(h, weights, prefix):
    return (gelu_tanh(h @ tensor(weights, prefix + ".gate").T) * (h @ tensor(weights, prefix + ".up").T)) \
        @ tensor(weights, prefix + ".down").T


def bounded_gated_unit(h, weights, prefix, limit, slope=1.702):
    """down(g sigmoid(slope g) (u + 1)), g = min(gate h, limit), u = clamp(up h, -limit, limit)."""
    g = torch.clamp(h @ tensor(weights, prefix + ".gate").T, max=limit)
    u = torch.clamp(h @ tensor(weights, prefix + ".up").T, min=-limit, max=limit)
    return (g * torch.sigmoid(slope * g) * (u + 1.0)) @ tensor(weights, prefix + ".down").T


def routed_feed_forward(h, mlp, weights, prefix, router_input=None):
    """Every token goes to the ``top`` experts with the largest router logits, weighted by the softmax
    over those logits alone; a shared expert, if the layer has one, is added for every token.
    ``router_input``: what the router reads in place of ``h`` (its rounding, say)."""
    experts, top = int(mlp["router"]["experts"]), int(mlp["router"]["top"])
    z = (h if router_input is None else router_input) @ tensor(weights, prefix + ".router").T + tensor(weights, prefix + ".router.b")
    out = torch.zeros((h.shape[0], tensor(weights, prefix + ".e0.down").shape[0]), dtype=F64)
    for t in range(h.shape[0]):
        order = sorted(range(experts), key=lambda e: (-float(z[t, e]), e))[:top]
        chosen = torch.stack([z[t, e] for e in order])
        share = torch.softmax(chosen, dim=0)
        for w, e in zip(share, order):
            out[t] += w * bounded_gated_unit(h[t:t + 1], weights, f"{prefix}.e{e}", float(mlp["expert"]["limit"]))[0]
    if mlp.get("shared"):
        out = out + bounded_gated_unit(h, weights, prefix + ".shared", float(mlp["shared"]["limit"]))
    return out


def forward(config, weights, tokens, keep_layers=False, round_router_input=None):
    """Logits [T, vocab] of one whole sequence; with ``keep_layers`` also the residual stream after
    every layer.  ``round_router_input``: a dtype the routers' input is rounded to first."""
    eps = float(config["norm"]["eps"])
    n = len(tokens)
    positions = torch.arange(n)
    x = tensor(weights, "embed")[torch.tensor(list(tokens), dtype=torch.long)]
    streams = []
    for i, layer in enumerate(config["layers"]):
        p = f"l{i}"
        h = root_mean_square_norm(x, eps, tensor(weights, p + ".norm1"))
        if layer["type"] == "attention":
            x = x + rotary_chunked_mixer(h, positions, layer["mixer"], weights, p + ".mix")
        elif layer["type"] == "attention_2":
            x = x + biased_shared_kv_mixer(h, layer["mixer"], weights, p + ".mix", eps)
        else:
            raise ValueError(f"unknown layer type {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            h = root_mean_square_norm(x, eps, tensor(weights, p + ".norm2"))
            if mlp["kind"] == "dense":
                x = x + dense_feed_forward(h, weights, p + ".mlp")
            else:
                rounded = None if round_router_input is None else h.to(round_router_input).to(F64)
                x = x + routed_feed_forward(h, mlp, weights, p + ".mlp", rounded)
        streams.append(x)
    logits = root_mean_square_norm(x, eps, tensor(weights, "final.norm")) @ tensor(weights, "head").T
    return (logits, torch.stack(streams)) if keep_layers else logits


class PlainBiberax:
    """The functions above bound to one configuration and one set of weights."""

    def __init__(self, config, weights):
        self.config, self.weights = config, weights

    def forward(self, tokens, **kwargs):
        return forward(self.config, self.weights, tokens, **kwargs)

    def generate_greedy(self, prompt, n):
        """``n`` tokens after ``prompt``, each the lowest id among the largest logits."""
        tokens = list(prompt)
        for _ in range(n):
            tokens.append(int(torch.argmax(self.forward(tokens)[-1])))
        return tokens[len(prompt):]
