"""Plain Golepel: whole sequences, no cache, one function per mechanism, float64 by default.

Written from the design's equations; it shares no code with the engine.  Every function takes its sizes and
constants as arguments.  A model is a config dict (the config.json object) and {tensor name: tensor}.

  layer          x <- x + norm1(mixer(x + conv1(x)));  x <- x + norm2(ff(x + conv2(x)))   (no norm in front)
  norm           the vector in `groups` equal consecutive parts, each divided by its own sqrt(mean(part^2) + eps),
                 the whole times w
  conv           conv(h)_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros before the sequence
  mixer          attention through a latent: keys and values of every head are products of one vector c per token
                 (a normed down-projection) and one rotated key part shared by the heads
  feed-forward   dense silu-gated, or a mixture of experts with a clamped gate
"""
import json
import math
import os
import struct

import torch

_DT = {"F32": torch.float32, "F16": torch.float16, "BF16": torch.bfloat16, "F64": torch.float64,
       "I32": torch.int32, "I64": torch.int64}


def read_folder(folder, dtype=torch.float64):
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    out = {}
    with open(os.path.join(folder, "model.safetensors"), "rb") as f:
        raw = f.read()
    n = struct.unpack("<Q", raw[:8])[0]
    hdr = json.loads(raw[8:8 + n])
    for name, meta in hdr.items():
        if name == "__metadata__":
            continue
        s, e = meta["data_offsets"]
        t = torch.frombuffer(bytearray(raw[8 + n + s:8 + n + e]), dtype=_DT[meta["dtype"]]).reshape(meta["shape"])
        out[name] = t.to(dtype) if t.dtype.is_floating_point else t
    return cfg, out


# ---- mechanisms ---------------------------------------------------------------------------------------------------
def group_rms_norm(x, w, eps, groups):
    """x [..., D]: each of `groups` consecutive parts over its own root mean square (eps inside the root), times w."""
    parts = x.reshape(*x.shape[:-1], groups, x.shape[-1] // groups)
    parts = parts / torch.sqrt((parts * parts).mean(-1, keepdim=True) + eps)
    return parts.reshape(x.shape) * w


def causal_conv(h, w):
    """h [T, D], w [D, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j), rows before the first count as zero."""
    T, taps = h.shape[0], w.shape[1]
    out = torch.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += w[:, j] * h[:T - back]
    return out


def rotate_halves(x, positions, base, dims):
    """x [T, ..., n]: the first `dims` elements turn in pairs (i, i + dims/2) by the angle p * base^(-2i/dims)."""
    half = dims // 2
    f = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=x.dtype)
    ang = positions.to(x.dtype)[:, None] * f[None, :]
    shape = [x.shape[0]] + [1] * (x.dim() - 2) + [half]
    c, s = torch.cos(ang).reshape(shape), torch.sin(ang).reshape(shape)
    u, v = x[..., :half], x[..., half:dims]
    return torch.cat([u * c - v * s, v * c + u * s, x[..., dims:]], dim=-1)


def latent_keys(h, w_dkv, w_norm, eps, kv_rank, positions, rot):
    """What a layer caches of each token: the latent c [T, kv_rank] and the rotated key part [T, rot_dim]."""
    d = h @ w_dkv.T
    c = d[:, :kv_rank]
    c = c / torch.sqrt((c * c).mean(-1, keepdim=True) + eps) * w_norm
    return c, rotate_halves(d[:, kv_rank:], positions, rot["base"], rot["dims"])


def latent_attention(h, W, p, m, positions, latent):
    """h [T, width] -> [T, width].  W: tensors, p: the mixer's name prefix, m: its sizes, latent: (c, rotated key part)."""
    T, H, dim, rd, vd = h.shape[0], m["heads"], m["dim"], m["rot_dim"], m["vdim"]
    c, kr = latent
    q = (h @ W[p + "q"].T).reshape(T, H, dim + rd)
    qn, qr = q[..., :dim], rotate_halves(q[..., dim:], positions, m["rot"]["base"], m["rot"]["dims"])
    kn = (c @ W[p + "uk"].T).reshape(T, H, dim)
    v = (c @ W[p + "uv"].T).reshape(T, H, vd)
    s = (torch.einsum("thd,shd->hts", qn, kn) + torch.einsum("thd,sd->hts", qr, kr)) * m["scale"]
    s = s.masked_fill(~torch.tril(torch.ones(T, T, dtype=torch.bool)), float("-inf"))
    o = torch.einsum("hts,shd->thd", torch.softmax(s, -1), v).reshape(T, H * vd)
    return o @ W[p + "o"].T


def dense_ff(h, W, p):
    g = h @ W[p + "gate"].T
    return ((g * torch.sigmoid(g)) * (h @ W[p + "up"].T)) @ W[p + "down"].T


def expert_ff(h, W, p, limit):
    g = torch.clamp(h @ W[p + "gate"].T, max=limit)
    u = torch.clamp(h @ W[p + "up"].T, -limit, limit)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def route(h, w_router, top):
    """Scores over all experts; the `top` largest are chosen and weigh in with their scores as they are."""
    s = torch.softmax(h @ w_router.T, -1)
    val, idx = torch.topk(s, top, dim=-1)
    return idx, val


def moe_ff(h, W, p, mlp):
    idx, val = route(h, W[p + "router"], mlp["router"]["top"])
    out = torch.zeros_like(h)
    for e in range(mlp["router"]["experts"]):
        rows, slot = torch.nonzero(idx == e, as_tuple=True)
        if rows.numel():
            out[rows] += val[rows, slot][:, None] * expert_ff(h[rows], W, f"{p}e{e}.", mlp["expert"]["limit"])
    return out


# ---- the model ----------------------------------------------------------------------------------------------------
def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one sequence; layers_out: a list that receives the stream after every layer."""
    dtype = W["embed"].dtype
    eps, groups = cfg["norm"]["eps"], cfg["norm"]["groups"]
    x = W["embed"][torch.tensor(tokens)]
    positions = torch.arange(len(tokens))
    latents = {}
    for i, layer in enumerate(cfg["layers"]):
        L = f"l{i}."
        m = layer["mixer"]
        assert layer["type"] == "latent_attention"
        h = x + causal_conv(x, W[L + "canon1"])
        if m.get("kv_from") is None:
            latents[i] = latent_keys(h, W[L + "mix.dkv"], W[L + "mix.dkv.norm"], eps, m["kv_rank"], positions, m["rot"])
            lat = latents[i]
        else:
            lat = latents[m["kv_from"]]
        x = x + group_rms_norm(latent_attention(h, W, L + "mix.", m, positions, lat), W[L + "norm1"], eps, groups)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = x + causal_conv(x, W[L + "canon2"])
            y = dense_ff(h, W, L + "mlp.") if mlp["kind"] == "dense" else moe_ff(h, W, L + "mlp.", mlp)
            x = x + group_rms_norm(y, W[L + "norm2"], eps, groups)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = group_rms_norm(x, W["final.norm"], eps, groups)
    return (x @ W["embed"].T) * cfg["logit_scale"]


def greedy_generate(cfg, W, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        z = forward(cfg, W, toks)[-1]
        t = int(torch.nonzero(z == z.max())[0])
        out.append(t)
        toks.append(t)
    return out
