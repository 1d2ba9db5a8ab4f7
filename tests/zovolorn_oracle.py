"""Zovolorn in plain float64 NumPy: every mechanism as one function over a whole sequence, without caches, batches or kernels.  It shares nothing with the
product path (uzu_amd/, csrc/): the tests hold the engine to these equations.

Notation: T positions, d = model width, x [T, d] the residual stream.  Weights are dicts of float64 arrays keyed by the tensor names of a model directory
(linear weights [out, in]); `cfg` is the parsed config.json.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import numpy as np

UNIT_EPS = 1e-6  # inside the root of the unit vectors of the delta rule's queries and keys


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def grouped_rms_norm(y, w, groups: int, eps: float):
    """y [T, n] cut into `groups` equal consecutive parts, each divided by sqrt(mean(part^2) + eps); the whole times w"""
    T, n = y.shape
    parts = y.reshape(T, groups, n // groups)
    parts = parts / np.sqrt((parts ** 2).mean(axis=-1, keepdims=True) + eps)
    return parts.reshape(T, n) * w


def causal_conv(h, w):
    """h [T, C], w [C, taps]: out_t = sum_j w[:, j] * h_(t - taps + 1 + j), zeros in front of the sequence (the last tap weighs the current position)"""
    T, C = h.shape
    taps = w.shape[1]
    out = np.zeros_like(h)
    for j in range(taps):
        back = taps - 1 - j
        if back < T:
            out[back:] += w[:, j] * h[:T - back]
    return out


def embed_rows(tokens, table, scale: float, bigram=None, buckets: int = 0, mul_prev: int = 0, mul_cur: int = 0):
    """table[token] * scale (+ the row of `bigram` hashed from (previous token, token); the first token of a sequence takes the last row)"""
    tokens = np.asarray(tokens, dtype=np.int64)
    x = table[tokens] * scale
    if bigram is not None:
        rows = np.empty(len(tokens), dtype=np.int64)
        rows[0] = buckets
        rows[1:] = (tokens[:-1] * mul_prev + tokens[1:] * mul_cur) % buckets
        x = x + bigram[rows]
    return x


def rotate_pairs(a, dims: int, base: float, first_position: int = 0):
    """a [T, heads, width]: coordinates (2i, 2i + 1), i < dims / 2, of every head turn by the angle position * base^(-2i / dims); the rest stay"""
    T = a.shape[0]
    out = a.copy()
    i = np.arange(dims // 2)
    ang = (first_position + np.arange(T))[:, None] * (float(base) ** (-2.0 * i / dims))[None, :]
    c, s = np.cos(ang)[:, None, :], np.sin(ang)[:, None, :]
    u, v = a[..., 0:dims:2], a[..., 1:dims:2]
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def distance_bucket(n: int, rows: int, far: float) -> int:
    """row of a distance-bias table with `rows` rows: exact below rows // 2, then logarithmic steps up to `far`, the last row beyond"""
    exact = rows // 2
    if n < exact:
        return n
    if rows == 1:  # one row for every distance
        return 0
    return min(rows - 1, exact + int(math.floor(math.log(n / exact) / math.log(far / exact) * (rows - exact))))


def masked_softmax_attention(q, k, v, scale, visible, head_scale=None, bias=None, sink=None):
    """q [T, H, dk], k [T, G, dk], v [T, G, dv]; query head a reads key / value head a // (H / G).  scores = q.k * scale (* head_scale[a]) (+ bias[a, i, j]),
    softmax over the keys j with visible[i, j]; `sink` [H]: one more term exp(sink[a]) in the denominator, without a value.  -> [T, H, dv]"""
    T, H, _ = q.shape
    G = k.shape[1]
    out = np.zeros((T, H, v.shape[2]))
    for a in range(H):
        g = a // (H // G)
        s = (q[:, a, :] @ k[:, g, :].T) * scale
        if head_scale is not None:
            s = s * head_scale[a]
        if bias is not None:
            s = s + bias[a]
        s = np.where(visible, s, -np.inf)
        m = s.max(axis=1, keepdims=True)
        if sink is not None:
            m = np.maximum(m, sink[a])
        e = np.exp(s - m)
        den = e.sum(axis=1, keepdims=True)
        if sink is not None:
            den = den + np.exp(sink[a] - m)
        out[:, a, :] = (e / den) @ v[:, g, :]
    return out


def attention_mixer(h, w: Dict[str, np.ndarray], p: str, mx: dict, eps: float):
    """the `attention` mixer on its input rows h [T, d]; p = the tensor prefix '<layer>.mix.'"""
    T = h.shape[0]
    H, G, dk, dv = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    q, k, v = h @ w[p + "q"].T, h @ w[p + "k"].T, h @ w[p + "v"].T
    # one RMS norm over the whole projection (all heads at once)
    q = q / np.sqrt((q ** 2).mean(axis=1, keepdims=True) + eps) * w[p + "q.norm"]
    k = k / np.sqrt((k ** 2).mean(axis=1, keepdims=True) + eps) * w[p + "k.norm"]
    q, k, v = q.reshape(T, H, dk), k.reshape(T, G, dk), v.reshape(T, G, dv)
    rot = mx.get("rot")
    if rot and int(rot.get("dims") or 0):
        q, k = rotate_pairs(q, int(rot["dims"]), float(rot["base"])), rotate_pairs(k, int(rot["dims"]), float(rot["base"]))
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    o = masked_softmax_attention(q, k, v, float(mx["scale"]), j <= i, sink=w[p + "sink"])
    o = o * sigmoid(h @ w[p + "g"].T)[:, :, None]
    return o.reshape(T, H * dv) @ w[p + "o"].T


def chunk_attention(h, w, p: str, mx: dict, eps: float):
    """the left half of the `parallel` mixer: attention inside chunks of positions, values = the keys as projected, a temperature per head, a distance bias"""
    T = h.shape[0]
    H, G, dk = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"])
    q, k = (h @ w[p + "q"].T).reshape(T, H, dk), (h @ w[p + "k"].T).reshape(T, G, dk)
    v = k  # before the norm
    qn = q / np.sqrt((q ** 2).mean(axis=-1, keepdims=True) + eps) * w[p + "q.norm"]
    kn = k / np.sqrt((k ** 2).mean(axis=-1, keepdims=True) + eps) * w[p + "k.norm"]
    rel = w[p + "rel"]
    size = int(mx["mask"]["size"])
    i, j = np.arange(T)[:, None], np.arange(T)[None, :]
    visible = (j <= i) & (i // size == j // size)
    by_distance = np.array([distance_bucket(n, rel.shape[0], float(mx["bias_max"])) for n in range(T)], dtype=np.int64)
    bucket = by_distance[np.maximum(i - j, 0)]
    bias = np.stack([rel[bucket, a] for a in range(H)])
    o = masked_softmax_attention(qn, kn, v, float(mx["scale"]), visible, head_scale=w[p + "temp"], bias=bias)
    return o.reshape(T, H * dk) @ w[p + "o"].T


def delta_rule(q, k, v, beta, decay, state=None):
    """q, k [T, dk], v [T, dv], beta [T], decay [T, dk] of ONE head; S [dk, dv] from `state` (zeros):  S <- decay_t * S (rows), u = beta_t (v_t - S^T k_t),
    S <- S + k_t u^T, o_t = S^T q_t.  -> (o [T, dv], S)"""
    T, dk = q.shape
    S = np.zeros((dk, v.shape[1])) if state is None else state.copy()
    o = np.zeros((T, v.shape[1]))
    for t in range(T):
        S = decay[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + np.outer(k[t], u)
        o[t] = S.T @ q[t]
    return o, S


def delta_mixer(h, w, p: str, mx: dict, eps: float):
    """the right half of the `parallel` mixer: the gated delta rule with a decay per head and key channel"""
    T = h.shape[0]
    H, G, dk, dv = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    q = silu(causal_conv(h @ w[p + "q"].T, w[p + "q.conv"])).reshape(T, G, dk)
    k = silu(causal_conv(h @ w[p + "k"].T, w[p + "k.conv"])).reshape(T, G, dk)
    v = silu(causal_conv(h @ w[p + "v"].T, w[p + "v.conv"])).reshape(T, H, dv)
    q = q / np.sqrt((q ** 2).sum(axis=-1, keepdims=True) + UNIT_EPS) * dk ** -0.5
    k = k / np.sqrt((k ** 2).sum(axis=-1, keepdims=True) + UNIT_EPS)
    beta = sigmoid(h @ w[p + "b"].T)  # [T, H]
    step = softplus((h @ w[p + "a1"].T) @ w[p + "a2"].T + w[p + "dt_bias"]).reshape(T, H, dk)
    decay = np.exp(-np.exp(w[p + "A_log"])[None, :, None] * step)
    gate = sigmoid((h @ w[p + "g1"].T) @ w[p + "g2"].T).reshape(T, H, dv)
    o = np.zeros((T, H, dv))
    for a in range(H):
        g = a // (H // G)
        o[:, a, :], _ = delta_rule(q[:, g, :], k[:, g, :], v[:, a, :], beta[:, a], decay[:, a, :])
    o = o / np.sqrt((o ** 2).mean(axis=-1, keepdims=True) + eps) * w[p + "norm"] * gate
    return o.reshape(T, H * dv) @ w[p + "o"].T


def parallel_mixer(h, w, p: str, mx: dict, eps: float):
    return float(mx["left_scale"]) * chunk_attention(h, w, p + "left.", mx["left"], eps) + float(mx["right_scale"]) * delta_mixer(h, w, p + "right.", mx["right"], eps)


def dense_mlp(h, w, p: str):
    """down(gelu_tanh(gate h + b) * (up h + b)) + b; p = '<layer>.mlp.'"""
    g = h @ w[p + "gate"].T + w[p + "gate.b"]
    u = h @ w[p + "up"].T + w[p + "up.b"]
    return (gelu_tanh(g) * u) @ w[p + "down"].T + w[p + "down.b"]


def forward(cfg: dict, w: Dict[str, np.ndarray], tokens) -> Tuple[np.ndarray, List[np.ndarray]]:
    """-> (logits [T, vocab], the residual stream behind every layer)"""
    w = {n: np.asarray(a, dtype=np.float64) for n, a in w.items()}
    eps, groups = float(cfg["norm"]["eps"]), int(cfg["norm"].get("groups", 1))
    em = cfg["embedding"]
    bg = em.get("bigram")
    x = embed_rows(tokens, w["embed"], float(em.get("scale", 1.0)), w["bigram"] if bg else None, int(bg["buckets"]) if bg else 0, int(bg["mul_prev"]) if bg else 0,
                   int(bg["mul_cur"]) if bg else 0)
    streams = []
    for i, lc in enumerate(cfg["layers"]):
        p = f"l{i}."
        h = x + causal_conv(x, w[p + "canon1"])
        if lc["type"] == "attention":
            m = attention_mixer(h, w, p + "mix.", lc["mixer"], eps)
        elif lc["type"] == "parallel":
            m = parallel_mixer(h, w, p + "mix.", lc["mixer"], eps)
        else:
            raise ValueError(lc["type"])
        x = x + grouped_rms_norm(m, w[p + "norm1"], groups, eps)
        if lc.get("mlp") is not None:
            h = x + causal_conv(x, w[p + "canon2"])
            x = x + grouped_rms_norm(dense_mlp(h, w, p + "mlp."), w[p + "norm2"], groups, eps)
        streams.append(x.copy())
    y = grouped_rms_norm(x, w["final.norm"], groups, eps)
    logits = y @ w["embed"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    if cap:
        logits = cap * np.tanh(logits / cap)
    return logits, streams


# ------------------------------------------------------------------------------------------------ the tests' own configurations, weights and model directories
def dense(ff):
    return {"kind": "dense", "ff": int(ff)}


def attention_layer(heads, kv_heads, dim, vdim, rot_dims=0, rot_base=10000.0, scale=None, mlp=None):
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(scale if scale is not None else dim ** -0.5)}
    if rot_dims:
        mx["rot"] = {"dims": int(rot_dims), "base": float(rot_base)}
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def parallel_layer(heads, kv_heads, dim, chunk, rel_rows, bias_max, d_heads, d_kv_heads, d_dim, d_vdim, conv, rank=3, scale=None, left_scale=1.0, right_scale=1.0, mlp=None, gate_rank=None):
    """`rel_rows`, `rank` (of the decay's two factors) and `gate_rank` (of the gate's; default: the same) size tensors only (a reader takes them from the shapes):
    they are kept under '_sizes', which a reader ignores"""
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": int(chunk)}, "bias_max": float(bias_max),
            "scale": float(scale if scale is not None else dim ** -0.5)}
    right = {"heads": d_heads, "kv_heads": d_kv_heads, "dim": d_dim, "vdim": d_vdim, "conv": int(conv)}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": float(left_scale), "right_scale": float(right_scale)}, "mlp": mlp,
            "_sizes": {"rel_rows": int(rel_rows), "rank": int(rank), "gate_rank": int(gate_rank if gate_rank is not None else rank)}}


def config(vocab, width, layers, eps=1e-5, groups=1, taps=4, embed_scale=1.0, bigram=None, logit_softcap=0.0):
    """bigram = (buckets, mul_prev, mul_cur)"""
    em = {"scale": float(embed_scale)}
    if bigram:
        em["bigram"] = {"buckets": int(bigram[0]), "mul_prev": int(bigram[1]), "mul_cur": int(bigram[2])}
    return {"architecture": "Zovolorn", "vocab": int(vocab), "width": int(width), "norm": {"eps": float(eps), "groups": int(groups)}, "canon": {"taps": int(taps)},
            "embedding": em, "layers": layers, "logit_softcap": float(logit_softcap)}


def bf16_bits(a):
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def to_bf16(a):
    return (bf16_bits(a).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(a))


def weights(cfg, seed):
    """random tensors (bf16-representable f32) for a configuration: products ~ N(0, gain^2 / in), norm weights around 1, decays from fast to slow"""
    rng = np.random.default_rng(seed)
    vocab, width, taps = cfg["vocab"], cfg["width"], cfg["canon"]["taps"]
    W = {}

    def lin(name, n, k, gain=1.0, bias=False):
        W[name] = to_bf16(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            W[name + ".b"] = to_bf16(rng.standard_normal(n) * 0.2)

    def vec(name, n, centre, spread):
        W[name] = to_bf16(centre + spread * (rng.random(n) - 0.5))

    W["embed"] = to_bf16(rng.standard_normal((vocab, width)) / cfg["embedding"]["scale"])
    bg = cfg["embedding"].get("bigram")
    if bg:
        W["bigram"] = to_bf16(rng.standard_normal((bg["buckets"] + 1, width)) * 0.5)
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        vec(p + "norm1", width, 1.0, 0.6)
        W[p + "canon1"] = to_bf16(rng.standard_normal((width, taps)) * 0.3)
        if lc["type"] == "attention":
            H, G, dk, dv = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            q = p + "mix."
            lin(q + "q", H * dk, width, 2.0), lin(q + "k", G * dk, width, 2.0), lin(q + "v", G * dv, width), lin(q + "g", H, width, 2.0)
            vec(q + "q.norm", H * dk, 1.5, 0.6), vec(q + "k.norm", G * dk, 1.5, 0.6), vec(q + "sink", H, 0.5, 3.0)
            lin(q + "o", width, H * dv)
        else:
            lm, rm, sz = mx["left"], mx["right"], lc["_sizes"]
            H, G, dk = lm["heads"], lm["kv_heads"], lm["dim"]
            q = p + "mix.left."
            lin(q + "q", H * dk, width, 2.0), lin(q + "k", G * dk, width, 2.0)
            vec(q + "q.norm", dk, 1.5, 0.6), vec(q + "k.norm", dk, 1.5, 0.6), vec(q + "temp", H, 1.0, 1.0)
            W[q + "rel"] = to_bf16(rng.standard_normal((sz["rel_rows"], H)) * 1.5)
            lin(q + "o", width, H * dk)
            Hd, Gd, dk, dv, ct, rank = rm["heads"], rm["kv_heads"], rm["dim"], rm["vdim"], rm["conv"], sz["rank"]
            q = p + "mix.right."
            lin(q + "q", Gd * dk, width, 2.0), lin(q + "k", Gd * dk, width, 2.0), lin(q + "v", Hd * dv, width, 1.5), lin(q + "b", Hd, width, 2.0)
            for n, ch in (("q", Gd * dk), ("k", Gd * dk), ("v", Hd * dv)):
                W[q + n + ".conv"] = to_bf16(rng.standard_normal((ch, ct)) * 0.6)
            lin(q + "a1", rank, width), lin(q + "a2", Hd * dk, rank, 2.0), lin(q + "g1", sz["gate_rank"], width), lin(q + "g2", Hd * dv, sz["gate_rank"], 2.0)
            vec(q + "A_log", Hd, -1.0, 3.0), vec(q + "dt_bias", Hd * dk, -1.0, 3.0), vec(q + "norm", dv, 1.0, 0.6)
            lin(q + "o", width, Hd * dv)
        if lc.get("mlp") is not None:
            ff = lc["mlp"]["ff"]
            vec(p + "norm2", width, 1.0, 0.6)
            W[p + "canon2"] = to_bf16(rng.standard_normal((width, taps)) * 0.3)
            lin(p + "mlp.gate", ff, width, 1.5, True), lin(p + "mlp.up", ff, width, 1.5, True), lin(p + "mlp.down", width, ff, 1.0, True)
    vec("final.norm", width, 1.0, 0.6)
    return W


def write_model_dir(path, cfg, W):
    """config.json + model.safetensors (bf16) in the design's layout, written with nothing but the file format"""
    import json
    import os
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(cfg, f)
    header, blobs, off = {}, [], 0
    for name in sorted(W):
        b = bf16_bits(W[name]).tobytes()
        header[name] = {"dtype": "BF16", "shape": list(np.shape(W[name])), "data_offsets": [off, off + len(b)]}
        blobs.append(b)
        off += len(b)
    hj = json.dumps(header).encode()
    hj += b" " * (-len(hj) % 8)
    with open(os.path.join(path, "model.safetensors"), "wb") as f:
        f.write(len(hj).to_bytes(8, "little") + hj + b"".join(blobs))


def logit_error(got, want):
    """per row: RMS over the vocabulary of the difference with its mean taken off, relative to the RMS of the centred expected row"""
    d = np.asarray(got, dtype=np.float64) - np.asarray(want, dtype=np.float64)
    d = d - d.mean(-1, keepdims=True)
    w = np.asarray(want, dtype=np.float64)
    w = w - w.mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt((w * w).mean(-1) + 1e-30)


def greedy(cfg, W, prompt, n):
    """n tokens by arg-max, every step a forward pass over the whole sequence"""
    toks = list(prompt)
    for _ in range(n):
        logits, _ = forward(cfg, W, toks)
        toks.append(int(np.argmax(logits[-1])))
    return toks[len(prompt):]
