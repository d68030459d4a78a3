"""A plain, slow implementation of the Bikovik decoder in float64 on the CPU: one function per
mechanism, written from the equations, sharing no code with the engine.  It reads the same
``config.json`` dictionary and the same tensor names as the engine and runs whole sequences
only (no cache, no portions): what the engine must reproduce however it cuts the work.

Notation: ``h`` a layer's normalised input ``[T, width]``; positions count from 0."""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def dynamic_tanh(x, weight, bias, alpha):
    """y = tanh(alpha x) * w + b, elementwise; no statistics of the row enter."""
    return torch.tanh(alpha * x) * weight + bias


def root_mean_square_norm(x, eps, weight=None):
    """x / sqrt(mean(x^2) + eps) over the last dimension, times ``weight`` if given."""
    y = x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)
    return y if weight is None else y * weight


def rotate_pairs(x, positions, dims, base):
    """Rotary encoding of the first ``dims`` dimensions of every head of ``x [T, heads, d]``:
    dimension i < dims/2 is paired with i + dims/2; the pair turns by position * base^(-2i/dims)."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    angle = positions.to(F64)[:, None] * freq[None, :]
    cos, sin = angle.cos()[:, None, :], angle.sin()[:, None, :]
    lo, hi = x[..., :half], x[..., half:dims]
    out = x.clone()
    out[..., :half] = lo * cos - hi * sin
    out[..., half:dims] = hi * cos + lo * sin
    return out


def window_with_kept_first(n, size, keep_first):
    """visible[i, j]: j <= i and (i - j < size or j < keep_first)."""
    i = torch.arange(n)[:, None]
    j = torch.arange(n)[None, :]
    return (j <= i) & ((i - j < size) | (j < keep_first))


def talking_heads_attention(q, k, v, scale, talk, visible):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; query head h reads kv head h // (H/G).  The
    scores of all heads at one (query, key) pair are mixed by ``talk [H, H]`` before the mask
    and the softmax."""
    n, heads, _ = q.shape
    group = heads // k.shape[1]
    out = torch.zeros((n, heads, v.shape[2]), dtype=F64)
    raw = torch.stack([q[:, h] @ k[:, h // group].T for h in range(heads)]) * scale       # [H, T, T]
    mixed = torch.einsum("hg,gij->hij", talk, raw)
    mixed = mixed.masked_fill(~visible[None], float("-inf"))
    weights = torch.softmax(mixed, dim=-1)
    for h in range(heads):
        out[:, h] = weights[h] @ v[:, h // group]
    return out


def gated_outer_product_recurrence(q, decay_rows, write_rows, v, state=None):
    """S_t = diag(decay_rows_t) S_(t-1) + write_rows_t v_t^T;  o_t = S_t^T q_t, one head.
    q, decay_rows, write_rows [T, d]; v [T, dv]; returns o [T, dv] and the last state."""
    n, d = q.shape
    s = torch.zeros((d, v.shape[1]), dtype=F64) if state is None else state.clone()
    out = torch.zeros((n, v.shape[1]), dtype=F64)
    for t in range(n):
        s = decay_rows[t][:, None] * s + write_rows[t][:, None] * v[t][None, :]
        out[t] = s.T @ q[t]
    return out, s


def clamped_gated_unit(gate, up, limit):
    g = torch.clamp(gate, max=limit)
    u = torch.clamp(up, min=-limit, max=limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def soft_cap(x, cap):
    return cap * torch.tanh(x / cap)


class PlainBikovik:
    def __init__(self, config: dict, tensors: dict):
        self.c = config
        self.w = {name: t.to(F64) for name, t in tensors.items()}
        self.first_mixed = next((i for i, layer in enumerate(config["layers"])
                                 if layer["type"] == "attention" and layer["mixer"].get("v_mix")), None)

    def norm(self, x, name):
        return dynamic_tanh(x, self.w[name], self.w[name + ".b"], self.w[name + ".alpha"])

    # -- mixers ----------------------------------------------------------------
    def attention(self, i, m, h, positions, shared):
        w, p = self.w, f"l{i}.mix."
        n = h.shape[0]
        heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        q = (h @ w[p + "q"].T + w[p + "q.b"]).view(n, heads, d)
        k = (h @ w[p + "k"].T + w[p + "k.b"]).view(n, groups, d)
        v = (h @ w[p + "v"].T + w[p + "v.b"]).view(n, groups, dv)
        q = rotate_pairs(q, positions, m["rot"]["dims"], m["rot"]["base"])
        k = rotate_pairs(k, positions, m["rot"]["dims"], m["rot"]["base"])
        if m.get("v_mix"):
            if i == self.first_mixed:
                shared["v_first"] = v
            else:
                lam = w[p + "vmix"]
                v = (1.0 - lam) * v + lam * shared["v_first"]
        visible = window_with_kept_first(n, m["mask"]["size"], m["mask"]["keep_first"])
        o = talking_heads_attention(q, k, v, m["scale"], w[p + "talk"], visible)
        return o.reshape(n, heads * dv) @ w[p + "o"].T

    def hgrn2(self, i, m, h):
        w, p = self.w, f"l{i}.mix."
        n = h.shape[0]
        heads, d, dv = m["heads"], m["dim"], m["vdim"]
        q = torch.nn.functional.silu(h @ w[p + "q"].T).view(n, heads, d)
        lower = w[p + "lower"]
        f = (lower + (1.0 - lower) * torch.sigmoid(h @ w[p + "f"].T + w[p + "f.b"])).view(n, heads, d)
        v = (h @ w[p + "v"].T).view(n, heads, dv)
        out = []
        for head in range(heads):
            o, _ = gated_outer_product_recurrence(q[:, head], f[:, head], 1.0 - f[:, head], v[:, head])
            out.append(root_mean_square_norm(o, self.c["norm"]["eps"], w[p + "norm"]))
        return torch.cat(out, dim=1) @ w[p + "o"].T

    def retention(self, i, m, h, positions):
        w, p = self.w, f"l{i}.mix."
        n = h.shape[0]
        heads, d, dv = m["heads"], m["dim"], m["vdim"]
        q = rotate_pairs((h @ w[p + "q"].T).view(n, heads, d), positions, m["rot"]["dims"], m["rot"]["base"])
        k = rotate_pairs((h @ w[p + "k"].T).view(n, heads, d), positions, m["rot"]["dims"], m["rot"]["base"])
        k = k * d ** -0.5
        v = (h @ w[p + "v"].T).view(n, heads, dv)
        out = []
        for head in range(heads):
            decay = torch.full((n, d), float(m["decay"][head]), dtype=F64)
            o, _ = gated_outer_product_recurrence(q[:, head], decay, k[:, head], v[:, head])
            out.append(root_mean_square_norm(o, self.c["norm"]["eps"]))
        gate = torch.nn.functional.silu(h @ w[p + "g"].T)
        return (torch.cat(out, dim=1) * gate) @ w[p + "o"].T

    def feed_forward(self, i, m, h):
        w, p = self.w, f"l{i}.mlp."
        return clamped_gated_unit(h @ w[p + "gate"].T, h @ w[p + "up"].T, m["limit"]) @ w[p + "down"].T

    # -- the whole model ---------------------------------------------------------
    def forward(self, tokens, return_layers: bool = False):
        """Logits ``[T, vocab]`` (float64) of a whole sequence; with ``return_layers`` also the
        residual stream after every layer ``[layers, T, width]``."""
        c, w = self.c, self.w
        tokens = torch.as_tensor(tokens, dtype=torch.long)
        positions = torch.arange(tokens.shape[0])
        x = w["embed"][tokens] * c["embedding"]["scale"]
        shared, after = {}, []
        for i, layer in enumerate(c["layers"]):
            h = self.norm(x, f"l{i}.norm1")
            kind, m = layer["type"], layer["mixer"]
            if kind == "attention":
                x = x + self.attention(i, m, h, positions, shared)
            elif kind == "hgrn2":
                x = x + self.hgrn2(i, m, h)
            elif kind == "retention":
                x = x + self.retention(i, m, h, positions)
            else:
                raise ValueError(f"unknown layer type {kind!r}")
            if layer.get("mlp") is not None:
                x = x + self.feed_forward(i, layer["mlp"], self.norm(x, f"l{i}.norm2"))
            after.append(x)
        logits = soft_cap(self.norm(x, "final.norm") @ w["head"].T, c["logit_softcap"])
        return (logits, torch.stack(after)) if return_layers else logits

    def generate_greedy(self, prompt, n_new: int):
        tokens = list(prompt)
        for _ in range(n_new):
            tokens.append(int(self.forward(tokens)[-1].argmax()))
        return tokens[len(prompt):]
