"""The Renapel decoder in plain, slow arithmetic: float64, whole sequences, no cache, no batch, one function per mechanism.

It shares no code with the package. `tensors` maps checkpoint names to torch tensors, `config` is config.json as a dict.
X is the residual stream in its copies [copies, tokens, width], h what a sublayer reads, t a token's index in its sequence
(its position), H heads, d the key size and e the value size of a head.
"""
from __future__ import annotations

import json
import math
import os
import struct

import torch

F = torch.float64
SWISH_ALPHA = 1.702
WEIGHT_FLOOR = 1e-20


def silu(z):
    return z * torch.sigmoid(z)


def rms_divided(x, eps):
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def rms_norm(x, w, eps):
    return rms_divided(x, eps) * w.to(F)


# ---- the residual stream in several copies ------------------------------------------------------------------------------

def copies_read(X, weights):
    """What a sublayer's norm reads: the copies weighted and summed. X [copies, tokens, width], weights [copies]."""
    return torch.einsum("s,stw->tw", weights.to(F), X)


def copies_write(X, y, mix, out):
    """All copies at once from the old ones: new copy b = sum over a of mix[a, b] * old copy a, plus out[b] * y."""
    return torch.einsum("ab,atw->btw", mix.to(F), X) + out.to(F)[:, None, None] * y[None]


# ---- a matrix state per head with a fixed decay ---------------------------------------------------------------------------

def lightning(h, p, m, eps):
    heads, d, e = m["heads"], m["dim"], m["vdim"]
    tokens = h.shape[0]
    q = silu(h @ p["q"].to(F).T).reshape(tokens, heads, d)
    k = silu(h @ p["k"].to(F).T).reshape(tokens, heads, d)
    v = silu(h @ p["v"].to(F).T).reshape(tokens, heads, e)
    decay = torch.tensor(m["decay"], dtype=F)
    state = torch.zeros(heads, d, e, dtype=F)
    out = torch.zeros(tokens, heads, e, dtype=F)
    for t in range(tokens):
        state = decay[:, None, None] * state + k[t][:, :, None] * v[t][:, None, :]
        out[t] = torch.einsum("hde,hd->he", state, q[t])
    o = rms_norm(out.reshape(tokens, heads * e), p["norm"], eps)
    o = o * torch.sigmoid(h @ p["g"].to(F).T)
    return o @ p["o"].to(F).T


# ---- softmax attention whose denominator holds one more term ----------------------------------------------------------------

def softmax_with_sink(scores, sink):
    """scores [heads, queries, keys] with -inf where a key is not seen; sink [heads]: exp(sink) joins the denominator."""
    top = torch.maximum(scores.max(dim=-1).values, sink[:, None])
    weights = torch.exp(scores - top[..., None])
    return weights / (weights.sum(dim=-1) + torch.exp(sink[:, None] - top))[..., None]


def causal_mask(tokens):
    return torch.tril(torch.ones(tokens, tokens, dtype=torch.bool))


def distance_bucket(n, rows, far):
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(far / half) * (rows - half))))


def distance_bias(table, tokens, far):
    """[heads, queries, keys] from the table [rows, heads]; keys ahead of the query get row 0 (they are masked anyway)."""
    rows = table.shape[0]
    index = torch.tensor([[distance_bucket(i - j, rows, far) if j <= i else 0 for j in range(tokens)] for i in range(tokens)])
    return table.to(F)[index].permute(2, 0, 1)


def query_temperature(tokens, coef, every):
    return torch.tensor([1.0 + coef * math.log((t + 1) // every + 1) for t in range(tokens)], dtype=F)


def attention_keys_values(h, p, m, eps):
    """What a softmax attention layer keeps of its tokens: keys (each head divided by its root mean square) and values."""
    kv_heads, d, e = m["kv_heads"], m["dim"], m["vdim"]
    tokens = h.shape[0]
    k = (h @ p["k"].to(F).T + p["k.b"].to(F)).reshape(tokens, kv_heads, d)
    v = (h @ p["v"].to(F).T + p["v.b"].to(F)).reshape(tokens, kv_heads, e)
    return rms_divided(k, eps), v


def attention(h, p, m, eps, keys_values=None):
    """keys_values: those of another layer, for a layer that has none of its own."""
    heads, kv_heads, d, e = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    tokens = h.shape[0]
    k, v = attention_keys_values(h, p, m, eps) if keys_values is None else keys_values
    q = rms_divided((h @ p["q"].to(F).T + p["q.b"].to(F)).reshape(tokens, heads, d), eps)
    temp = m.get("q_temp")
    if temp is not None:
        q = q * query_temperature(tokens, temp["coef"], temp["every"])[:, None, None]
    share = heads // kv_heads
    k, v = k.repeat_interleave(share, dim=1), v.repeat_interleave(share, dim=1)
    scores = torch.einsum("ihd,jhd->hij", q, k) * m["scale"] + distance_bias(p["rel"], tokens, m["bias_max"])
    scores = scores.masked_fill(~causal_mask(tokens), -math.inf)
    weights = softmax_with_sink(scores, p["sink"].to(F))
    return torch.einsum("hij,jhe->ihe", weights, v).reshape(tokens, heads * e) @ p["o"].to(F).T


# ---- attention through a latent ---------------------------------------------------------------------------------------------

def rotate_neighbours(x, dims, base):
    """x [tokens, ..., n]: the first `dims` of the last axis turn in pairs (2i, 2i + 1) by t * base^(-2i / dims)."""
    tokens = x.shape[0]
    frequencies = torch.tensor([base ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=F)
    angles = torch.arange(tokens, dtype=F)[:, None] * frequencies
    shape = [tokens] + [1] * (x.dim() - 2) + [dims // 2]
    cos, sin = torch.cos(angles).reshape(shape), torch.sin(angles).reshape(shape)
    first, second = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = first * cos - second * sin
    out[..., 1:dims:2] = second * cos + first * sin
    return out


def latent_attention(h, p, m, eps):
    heads, d, r, e, rank = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    tokens = h.shape[0]
    rot = m["rot"]
    q = rms_norm(h @ p["dq"].to(F).T, p["dq.norm"], eps) @ p["uq"].to(F).T
    q = q.reshape(tokens, heads, d + r)
    q_plain, q_turned = q[..., :d], rotate_neighbours(q[..., d:], rot["dims"], rot["base"])
    down = h @ p["dkv"].to(F).T
    latent = rms_norm(down[:, :rank], p["dkv.norm"], eps)
    k_turned = rotate_neighbours(down[:, rank:], rot["dims"], rot["base"])          # one for all heads
    k_plain = (latent @ p["uk"].to(F).T).reshape(tokens, heads, d)
    v = (latent @ p["uv"].to(F).T).reshape(tokens, heads, e)
    scores = (torch.einsum("ihd,jhd->hij", q_plain, k_plain) + torch.einsum("ihr,jr->hij", q_turned, k_turned)) * m["scale"]
    scores = scores.masked_fill(~causal_mask(tokens), -math.inf)
    weights = softmax_with_sink(scores, p["sink"].to(F))
    return torch.einsum("hij,jhe->ihe", weights, v).reshape(tokens, heads * e) @ p["o"].to(F).T


# ---- experts ------------------------------------------------------------------------------------------------------------------

def route(h, router_matrix, router):
    """Weights [tokens, experts], zero for experts not chosen."""
    experts, top = router["experts"], router["top"]
    scores = torch.softmax(h @ router_matrix.to(F).T, dim=-1)
    allowed = torch.ones_like(scores, dtype=torch.bool)
    groups = router.get("groups")
    if groups is not None:
        size = experts // groups["count"]
        best = scores.reshape(-1, groups["count"], size).max(dim=-1).values
        kept = torch.zeros_like(best, dtype=torch.bool)
        kept.scatter_(1, best.topk(groups["keep"], dim=-1).indices, True)
        allowed = kept.repeat_interleave(size, dim=1)
    chosen = scores.masked_fill(~allowed, -1.0).topk(top, dim=-1).indices
    picked = torch.gather(scores, 1, chosen)
    weights = torch.zeros_like(scores)
    weights.scatter_(1, chosen, picked / (picked.sum(dim=-1, keepdim=True) + WEIGHT_FLOOR) * router.get("scale", 1.0))
    return weights


def expert(h, gate, up, down, limit):
    g = torch.clamp(h @ gate.to(F).T, max=limit)
    u = torch.clamp(h @ up.to(F).T, min=-limit, max=limit)
    return (g * torch.sigmoid(SWISH_ALPHA * g) * (u + 1.0)) @ down.to(F).T


def experts_ff(h, p, mlp):
    weights = route(h, p["router"], mlp["router"])
    y = torch.zeros(h.shape[0], p["e0.down"].shape[0], dtype=F)
    for n in range(mlp["router"]["experts"]):
        y = y + weights[:, n:n + 1] * expert(h, p[f"e{n}.gate"], p[f"e{n}.up"], p[f"e{n}.down"], mlp["expert"]["limit"])
    return y


# ---- the model ------------------------------------------------------------------------------------------------------------------

def under(tensors, prefix):
    return {name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)}


def sublayer(X, connection, norm_weight, eps, run):
    """One sublayer on the copies: read, norm, run, write. A model without copies has one stream and adds to it."""
    if connection is None:
        return X + run(rms_norm(X[0], norm_weight, eps))[None]
    y = run(rms_norm(copies_read(X, connection["in"]), norm_weight, eps))
    return copies_write(X, y, connection["mix"], connection["out"])


def forward(tokens, tensors, config, streams=None):
    """Logits [tokens, vocab] of one whole sequence; `streams`, a list, receives the sum of the copies after every layer."""
    eps = config["norm"]["eps"]
    x = tensors["embed"].to(F)[torch.tensor(list(tokens), dtype=torch.long)]
    copies = config.get("streams")
    X = x[None].repeat(1 if copies is None else copies, 1, 1)
    kept = {}                   # layer -> its keys and values, for the layers that read them
    for index, layer in enumerate(config["layers"]):
        p = under(tensors, f"l{index}.")
        mix, m, kind = under(p, "mix."), layer["mixer"], layer["type"]

        def mixer(h):
            if kind == "lightning":
                return lightning(h, mix, m, eps)
            if kind == "latent_attention":
                return latent_attention(h, mix, m, eps)
            if "kv_from" in m:
                return attention(h, mix, m, eps, kept[m["kv_from"]])
            kept[index] = attention_keys_values(h, mix, m, eps)
            return attention(h, mix, m, eps, kept[index])

        X = sublayer(X, None if copies is None else under(p, "hc1."), p["norm1"], eps, mixer)
        if layer.get("mlp") is not None:
            X = sublayer(X, None if copies is None else under(p, "hc2."), p["norm2"], eps,
                         lambda h: experts_ff(h, under(p, "mlp."), layer["mlp"]))
        if streams is not None:
            streams.append(X.sum(dim=0))
    return rms_norm(X.sum(dim=0), tensors["final.norm"], eps) @ tensors["head"].to(F).T


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
