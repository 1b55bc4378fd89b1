"""The Depunex decoder in plain, slow arithmetic: float64, whole sequences, no cache, no batch, one function per mechanism.

It shares no code with the package. `tensors` maps checkpoint names to torch tensors, `config` is config.json as a dict.
x is the residual stream [tokens, width], h what a sublayer reads, t a token's index in its sequence (its position).
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

F = torch.float64


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def silu(z):
    return z * torch.sigmoid(z)


def softplus(z):
    return torch.clamp(z, min=0) + torch.log1p(torch.exp(-z.abs()))


def rms_divided(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x, w, eps):
    """RMS norm with the gain 1 + w."""
    return rms_divided(x, eps) * (1.0 + w.to(F))


# ---- embedding -----------------------------------------------------------------------------------------------------

def bigram_rows(tokens, buckets, mul_prev, mul_cur):
    rows = []
    for t, token in enumerate(tokens):
        rows.append(buckets if t == 0 else (tokens[t - 1] * mul_prev + token * mul_cur) % buckets)
    return rows


def embedding(tokens, table, scale, bigram=None, buckets=0, mul_prev=0, mul_cur=0):
    ids = torch.tensor(list(tokens), dtype=torch.long)
    x = table.to(F)[ids] * scale
    if bigram is not None:
        x = x + bigram.to(F)[torch.tensor(bigram_rows(list(tokens), buckets, mul_prev, mul_cur), dtype=torch.long)]
    return x


# ---- short causal convolution with bias, then silu ----------------------------------------------------------------------

def causal_conv_silu(u, w, b):
    """u [tokens, channels], w [channels, taps] (last column: the current token), b [channels]."""
    tokens, channels = u.shape
    taps = w.shape[1]
    padded = torch.cat([torch.zeros(taps - 1, channels, dtype=F), u])
    y = torch.zeros_like(u)
    for j in range(taps):
        y = y + padded[j:j + tokens] * w.to(F)[:, j]
    return silu(y + b.to(F))


# ---- Mamba-2: a matrix state per head with one decay per head and token ------------------------------------------------------

def mamba2(h, p, m, eps):
    """p: the mixer's tensors by their short names; m: the mixer's sizes."""
    heads, vdim, n, groups, norm_groups = m["heads"], m["vdim"], m["state"], m["groups"], m["norm_groups"]
    inner = heads * vdim
    tokens = h.shape[0]
    proj = h @ p["in"].to(F).T
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * groups * n], proj[:, 2 * inner + 2 * groups * n:]
    xbc = causal_conv_silu(xbc, p["conv"], p["conv.b"])
    x = xbc[:, :inner].reshape(tokens, heads, vdim)
    b = xbc[:, inner:inner + groups * n].reshape(tokens, groups, n)
    c = xbc[:, inner + groups * n:].reshape(tokens, groups, n)
    dt = softplus(dt + p["dt_bias"].to(F))                                   # [tokens, heads]
    rate = torch.exp(p["A_log"].to(F))
    y = torch.zeros(tokens, heads, vdim, dtype=F)
    for head in range(heads):
        group = head // (heads // groups)
        state = torch.zeros(n, vdim, dtype=F)
        for t in range(tokens):
            state = torch.exp(-rate[head] * dt[t, head]) * state + dt[t, head] * torch.outer(b[t, group], x[t, head])
            y[t, head] = state.T @ c[t, group] + p["D"].to(F)[head] * x[t, head]
    y = y.reshape(tokens, inner) * silu(z)
    y = rms_divided(y.reshape(tokens, norm_groups, inner // norm_groups), eps).reshape(tokens, inner) * p["norm"].to(F)
    return y @ p["o"].to(F).T


# ---- Mamba: a vector state per channel, decays per channel, state and token ----------------------------------------------------

def mamba(h, p, m):
    inner, n, rank = m["inner"], m["state"], m["dt_rank"]
    tokens = h.shape[0]
    proj = h @ p["in"].to(F).T
    x, z = proj[:, :inner], proj[:, inner:]
    x = causal_conv_silu(x, p["conv"], p["conv.b"])
    low = x @ p["x"].to(F).T
    dt = softplus(low[:, :rank] @ p["dt"].to(F).T + p["dt.b"].to(F))          # [tokens, inner]
    b, c = low[:, rank:rank + n], low[:, rank + n:]
    a = -torch.exp(p["A_log"].to(F))                                          # [inner, n]
    state = torch.zeros(inner, n, dtype=F)
    y = torch.zeros(tokens, inner, dtype=F)
    for t in range(tokens):
        state = torch.exp(dt[t][:, None] * a) * state + (dt[t] * x[t])[:, None] * b[t][None, :]
        y[t] = state @ c[t] + p["D"].to(F) * x[t]
    return (y * silu(z)) @ p["o"].to(F).T


# ---- attention inside chunks, rotary positions with stretched frequencies ------------------------------------------------------

def rotary_frequencies(dims, base, scaling):
    out = []
    for i in range(dims // 2):
        f = base ** (-2.0 * i / dims)
        if scaling is not None:
            factor, low, high, original = scaling["factor"], scaling["low"], scaling["high"], scaling["original"]
            wavelength = 2.0 * math.pi / f
            if wavelength < original / high:
                pass
            elif wavelength > original / low:
                f = f / factor
            else:
                s = (original / wavelength - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate(x, dims, frequencies):
    """x [tokens, heads, dim]: the pairs (i, i + dims / 2) of the first dims dims turn by position * f_i."""
    tokens = x.shape[0]
    half = dims // 2
    angle = torch.arange(tokens, dtype=F)[:, None] * torch.tensor(frequencies, dtype=F)[None, :]
    cos, sin = torch.cos(angle)[:, None, :], torch.sin(angle)[:, None, :]
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * cos - v * sin, v * cos + u * sin, x[..., dims:]], dim=-1)


def chunked_attention(h, p, m):
    heads, kv_heads, dim, vdim = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    tokens = h.shape[0]
    q = (h @ p["q"].to(F).T).reshape(tokens, heads, dim)
    k = (h @ p["k"].to(F).T).reshape(tokens, kv_heads, dim)
    v = (h @ p["v"].to(F).T).reshape(tokens, kv_heads, vdim)
    rot = m.get("rot")
    if rot is not None:
        frequencies = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        q, k = rotate(q, rot["dims"], frequencies), rotate(k, rot["dims"], frequencies)
    i = torch.arange(tokens)
    visible = i[None, :] <= i[:, None]
    if m.get("mask") is not None:
        size = m["mask"]["size"]
        visible = visible & ((i[None, :] // size) == (i[:, None] // size))
    out = torch.zeros(tokens, heads, vdim, dtype=F)
    for head in range(heads):
        shared = head // (heads // kv_heads)
        scores = (q[:, head] @ k[:, shared].T) * m["scale"]
        scores = scores.masked_fill(~visible, float("-inf"))
        out[:, head] = torch.softmax(scores, dim=-1) @ v[:, shared]
    return out.reshape(tokens, heads * vdim) @ p["o"].to(F).T


def parallel_mixer(h, p, m):
    left = chunked_attention(h, {name[5:]: t for name, t in p.items() if name.startswith("left.")}, m["left"])
    right = mamba(h, {name[6:]: t for name, t in p.items() if name.startswith("right.")}, m["right"])
    return m["left_scale"] * left + m["right_scale"] * right


# ---- feed-forwards ---------------------------------------------------------------------------------------------------

def dense_ff(h, p, mlp):
    limit = mlp["limit"]
    g = torch.clamp(h @ p["gate"].to(F).T, max=limit)
    u = torch.clamp(h @ p["up"].to(F).T, min=-limit, max=limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ p["down"].to(F).T


def route(h, router, experts, top, group_count=1, group_keep=1):
    """(chosen experts [tokens, top], their weights [tokens, top]). One group: every expert can be chosen."""
    scores = torch.sigmoid(h @ router.to(F).T)                                # [tokens, experts]
    tokens = h.shape[0]
    per_group = experts // group_count
    grouped = scores.reshape(tokens, group_count, per_group)
    group_score = grouped.topk(min(2, per_group), dim=-1).values.sum(dim=-1)
    kept = group_score.topk(group_keep, dim=-1).indices                       # [tokens, keep]
    allowed = torch.zeros(tokens, group_count, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed[:, :, None].expand(-1, -1, per_group).reshape(tokens, experts), scores,
                         torch.full_like(scores, -1.0))
    chosen = masked.topk(top, dim=-1).indices
    weights = scores.gather(1, chosen)
    return chosen, weights / (weights.sum(dim=-1, keepdim=True) + 1e-20)


def moe_ff(h, p, mlp):
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    chosen, weights = route(h, p["router"], r["experts"], r["top"], groups["count"], groups["keep"])
    out = torch.zeros(h.shape[0], p["e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for e, w in zip(chosen[t].tolist(), weights[t]):
            gate, up, down = p[f"e{e}.gate"].to(F), p[f"e{e}.up"].to(F), p[f"e{e}.down"].to(F)
            out[t] += w * (down @ (silu(gate @ h[t]) * (up @ h[t])))
    return out


# ---- the per-layer token input -------------------------------------------------------------------------------------------

def side_input(x, tokens, layer, dim, side_table, p, eps):
    e = side_table.to(F)[torch.tensor(list(tokens), dtype=torch.long)][:, layer * dim:(layer + 1) * dim]
    g = gelu_tanh(x @ p["side.gate"].to(F).T) * e
    y = g @ p["side.proj"].to(F).T
    return rms_divided(y, eps) * p["side.norm"].to(F)


# ---- the model -------------------------------------------------------------------------------------------------------------

def under(tensors, prefix):
    return {name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)}


def layer_forward(x, tokens, index, layer, tensors, config):
    eps = config["norm"]["eps"]
    p = under(tensors, f"l{index}.")
    h = offset_norm(x, p["norm1"], eps)
    mix = under(p, "mix.")
    mixed = mamba2(h, mix, layer["mixer"], eps) if layer["type"] == "mamba2" else parallel_mixer(h, mix, layer["mixer"])
    total = mixed * p["ls1"].to(F)
    mlp = layer["mlp"]
    if mlp is not None:
        ff = dense_ff(h, under(p, "mlp."), mlp) if mlp["kind"] == "dense" else moe_ff(h, under(p, "mlp."), mlp)
        total = total + ff * p["ls2"].to(F)
    x = x + total
    side = config.get("token_side")
    if side is not None:
        x = x + side_input(x, tokens, index, side["dim"], tensors["side.embed"], p, eps)
    return x


def forward(tokens, tensors, config, streams=None):
    """Logits [tokens, vocab] of one whole sequence; `streams`, a list, receives the residual stream after every layer."""
    e = config.get("embedding") or {}
    b = e.get("bigram")
    if b is None:
        x = embedding(tokens, tensors["embed"], e.get("scale", 1.0))
    else:
        x = embedding(tokens, tensors["embed"], e.get("scale", 1.0), tensors["bigram"], b["buckets"], b["mul_prev"], b["mul_cur"])
    for index, layer in enumerate(config["layers"]):
        x = layer_forward(x, tokens, index, layer, tensors, config)
        if streams is not None:
            streams.append(x.clone())
    y = offset_norm(x, tensors["final.norm"], config["norm"]["eps"])
    logits = y @ tensors["embed"].to(F).T
    cap = config.get("logit_softcap")
    return logits if cap is None else cap * torch.tanh(logits / cap)



def read_folder(folder):
    """(config.json as a dict, {name: tensor as stored}) of a model folder; the file's layout is read here, by hand."""
    with open(os.path.join(folder, "config.json")) as handle:
        raw = json.load(handle)
    with open(os.path.join(folder, "model.safetensors"), "rb") as handle:
        size = struct.unpack("<Q", handle.read(8))[0]
        header = json.loads(handle.read(size))
        data = handle.read()
    kinds = {"BF16": torch.bfloat16, "F32": torch.float32, "F16": torch.float16, "I32": torch.int32}
    tensors = {}
    for name, entry in header.items():
        if name != "__metadata__":
            lo, hi = entry["data_offsets"]
            tensors[name] = torch.frombuffer(bytearray(data[lo:hi]), dtype=kinds[entry["dtype"]]).reshape(entry["shape"])
    return raw, tensors


class PlainModel:
    def __init__(self, folder):
        self.raw, self.tensors = read_folder(folder)

    def logits(self, tokens):
        with torch.no_grad():
            return forward(list(tokens), self.tensors, self.raw).to(torch.float32)


def generate_greedy(model, prompt, count):
    ids, out = list(prompt), []
    for _ in range(count):
        token = int(model.logits(ids)[-1].argmax())
        out.append(token)
        ids.append(token)
    return out
