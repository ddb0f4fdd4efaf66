"""Plain Lutovik: whole sequences, no cache, one function per mechanism, float64 by default.

Written from the design's equations; it shares no code with the engine.  Every function takes its sizes and
constants as arguments.  A model is a config dict (the config.json object) and {tensor name: tensor}.

  layer      x <- x + n1b(mixer(n1(x)));  x <- x + n2b(ff(n2(x)))   with n(v) = v / sqrt(mean(v^2) + eps) * (1 + w)
  mixers     "attention": grouped-query softmax attention, rotation of neighbouring pairs with optional scaling of
             the frequencies by wavelength, optionally on the keys and values another layer made;
             "parallel": an attention with split-half rotation and a sigmoid gate on its heads' outputs, next to a
             state-space layer (short convolution, a decaying matrix state per head, gate, grouped norm); the two
             outputs are normed and averaged
  ff         a relu-gated layer, or a mixture of silu-gated experts chosen by the largest sigmoid scores, the score
             scaling the expert's input, plus an expert every token uses
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


# ---- small functions ----------------------------------------------------------------------------------------------
def unit_rms(v, eps):
    """v [..., n] over its root mean square, eps inside the root."""
    return v / torch.sqrt((v * v).mean(-1, keepdim=True) + eps)


def norm_one_plus(v, w, eps):
    return unit_rms(v, eps) * (1.0 + w)


def silu(z):
    return z / (1.0 + torch.exp(-z))


def softplus(z):
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0.0)


# ---- rotation -------------------------------------------------------------------------------------------------------
def frequencies(base, dims, scaling=None):
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` {factor, low, high, original} a frequency whose wavelength
    2 pi / f exceeds original / low is divided by factor, one below original / high stays, and between the two the
    divided and the plain value are mixed linearly in original / wavelength."""
    out = []
    for i in range(dims // 2):
        f = float(base) ** (-2.0 * i / dims)
        if scaling is not None:
            wave = 2.0 * math.pi / f
            if wave > scaling["original"] / scaling["low"]:
                f = f / scaling["factor"]
            elif wave >= scaling["original"] / scaling["high"]:
                s = (scaling["original"] / wave - scaling["low"]) / (scaling["high"] - scaling["low"])
                f = (1.0 - s) * f / scaling["factor"] + s * f
        out.append(f)
    return torch.tensor(out, dtype=torch.float64)


def rotate(x, freqs, layout):
    """x [T, heads, d]; position t turns pair i of a head's first 2 len(freqs) elements by t * f_i.  layout
    "neighbours": pair i = elements (2i, 2i + 1); "halves": (i, i + len(freqs))."""
    T, n = x.shape[0], freqs.numel()
    if n == 0:
        return x
    ang = torch.arange(T, dtype=x.dtype)[:, None] * freqs.to(x.dtype)[None, :]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = x.clone()
    if layout == "neighbours":
        a, b = x[..., 0:2 * n:2], x[..., 1:2 * n:2]
        out[..., 0:2 * n:2] = a * c - b * s
        out[..., 1:2 * n:2] = b * c + a * s
    else:
        a, b = x[..., :n], x[..., n:2 * n]
        out[..., :n] = a * c - b * s
        out[..., n:2 * n] = b * c + a * s
    return out


# ---- attention ----------------------------------------------------------------------------------------------------
def keys_values(h, wk, wv, kv_heads, dim, vdim, freqs, layout):
    """What an attention layer keeps per token: rotated keys [T, G, dim] and values [T, G, vdim]."""
    T = h.shape[0]
    k = rotate((h @ wk.T).reshape(T, kv_heads, dim), freqs, layout)
    v = (h @ wv.T).reshape(T, kv_heads, vdim)
    return k, v


def softmax_attention(q, k, v, scale):
    """q [T, H, dim], k [T, G, dim], v [T, G, vdim] -> [T, H, vdim]; query t sees keys 0 .. t."""
    T, H = q.shape[0], q.shape[1]
    per = H // k.shape[1]
    out = torch.zeros(T, H, v.shape[-1], dtype=q.dtype)
    hidden = torch.triu(torch.ones(T, T, dtype=torch.bool), diagonal=1)
    for head in range(H):
        g = head // per
        s = (q[:, head] @ k[:, g].T) * scale
        s = s.masked_fill(hidden, float("-inf"))
        out[:, head] = torch.softmax(s, dim=-1) @ v[:, g]
    return out


def attention(h, t, p, m, layout, kv=None, gated=False):
    """t: tensors, p: their prefix, m: the mixer's config.  kv: (keys, values) of the layer named by kv_from, else this
    layer makes its own.  Returns (output [T, width], (keys, values))."""
    T, H, G, dim, vdim = h.shape[0], m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    rot = m["rot"]
    freqs = frequencies(rot["base"], rot["dims"], rot.get("scaling"))
    q = rotate((h @ t[p + "q"].T).reshape(T, H, dim), freqs, layout)
    if kv is None:
        kv = keys_values(h, t[p + "k"], t[p + "v"], G, dim, vdim, freqs, layout)
    heads = softmax_attention(q, kv[0], kv[1], m["scale"]).reshape(T, H * vdim)
    if gated:
        heads = heads * torch.sigmoid(h @ t[p + "g"].T)
    return heads @ t[p + "o"].T, kv


# ---- the state-space layer --------------------------------------------------------------------------------------------
def short_conv(u, w, b):
    """u [T, C], w [C, taps], b [C]: out_t = b + sum_j w[:, j] u_(t - taps + 1 + j), zeros before the first token."""
    T, taps = u.shape[0], w.shape[1]
    out = b.expand(T, -1).clone()
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += w[:, j] * u[:T - back]
    return out


def state_scan(x, B, C, dt, a_log, skip):
    """x [T, heads, P], B and C [T, groups, N], dt [T, heads] (positive), a_log and skip [heads].
    S_t = exp(-exp(a_log) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + skip x_t."""
    T, heads, P = x.shape
    per = heads // B.shape[1]
    y = torch.zeros_like(x)
    for head in range(heads):
        g = head // per
        S = torch.zeros(B.shape[-1], P, dtype=x.dtype)
        rate = torch.exp(a_log[head])
        for s in range(T):
            S = torch.exp(-rate * dt[s, head]) * S + dt[s, head] * torch.outer(B[s, g], x[s, head])
            y[s, head] = S.T @ C[s, g] + skip[head] * x[s, head]
    return y


def state_space(h, t, p, m, eps):
    T, heads, P, N, G = h.shape[0], m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * P
    u = h @ t[p + "in"].T
    z, xbc, dt = u[:, :inner], u[:, inner:2 * inner + 2 * G * N], u[:, 2 * inner + 2 * G * N:]
    xbc = silu(short_conv(xbc, t[p + "conv"], t[p + "conv.b"]))
    x = xbc[:, :inner].reshape(T, heads, P)
    B = xbc[:, inner:inner + G * N].reshape(T, G, N)
    C = xbc[:, inner + G * N:].reshape(T, G, N)
    dt = softplus(dt + t[p + "dt_bias"])
    y = state_scan(x, B, C, dt, t[p + "A_log"], t[p + "D"]).reshape(T, inner) * silu(z)
    ng = m["norm_groups"]
    y = unit_rms(y.reshape(T, ng, inner // ng), eps).reshape(T, inner) * t[p + "norm"]
    return y @ t[p + "o"].T


def parallel(h, t, p, m, eps):
    left, kv = attention(h, t, p + "left.", m["left"], "halves", gated=True)
    right = state_space(h, t, p + "right.", m["right"], eps)
    return 0.5 * (unit_rms(left, eps) * t[p + "left.out"] + unit_rms(right, eps) * t[p + "right.out"]), kv


# ---- feed-forward -----------------------------------------------------------------------------------------------------
def gated_ff(h, t, p, act):
    return (act(h @ t[p + "gate"].T) * (h @ t[p + "up"].T)) @ t[p + "down"].T


def mixture(h, t, p, mlp):
    E, top = mlp["router"]["experts"], mlp["router"]["top"]
    s = torch.sigmoid(h @ t[p + "router"].T)
    order = torch.argsort(-s, dim=-1, stable=True)[:, :top]
    out = torch.zeros_like(h)
    for r in range(h.shape[0]):
        for e in order[r].tolist():
            out[r] += gated_ff(s[r, e] * h[r:r + 1], t, f"{p}e{e}.", silu)[0]
    if mlp.get("shared") is not None:
        out = out + gated_ff(h, t, p + "shared.", silu)
    return out


def feed_forward(h, t, p, mlp):
    if mlp["kind"] == "dense":
        return gated_ff(h, t, p, torch.relu)
    return mixture(h, t, p, mlp)


# ---- the model ----------------------------------------------------------------------------------------------------
def forward(cfg, t, tokens, layers_out=None):
    """Logits [T, vocab] of a whole sequence.  layers_out: a list that receives the stream after every layer."""
    eps = cfg["norm"]["eps"]
    x = t["embed"][torch.as_tensor(tokens, dtype=torch.long)] * cfg["embedding"]["scale"]
    kept = {}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        h = norm_one_plus(x, t[p + "norm1"], eps)
        if layer["type"] == "attention":
            a, kept[i] = attention(h, t, p + "mix.", m, "neighbours", kv=kept[m["kv_from"]] if m.get("kv_from") is not None else None)
        elif layer["type"] == "parallel":
            a, kept[i] = parallel(h, t, p + "mix.", m, eps)
        else:
            raise ValueError(f"layer {i}: unknown type {layer['type']!r}")
        x = x + norm_one_plus(a, t[p + "norm1b"], eps)
        if layer.get("mlp") is not None:
            f = feed_forward(norm_one_plus(x, t[p + "norm2"], eps), t, p + "mlp.", layer["mlp"])
            x = x + norm_one_plus(f, t[p + "norm2b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    return norm_one_plus(x, t["final.norm"], eps) @ t["head"].T


def greedy_generate(cfg, t, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        z = forward(cfg, t, toks)[-1]
        tok = int(torch.nonzero(z == z.max())[0])
        out.append(tok)
        toks.append(tok)
    return out
