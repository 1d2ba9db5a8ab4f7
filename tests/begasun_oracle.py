"""Begasun in float64 NumPy: every mechanism of the design as one plain function over a whole sequence (no cache, no batching, no state objects).

This is test infrastructure: it shares no code with the product (uzu_amd.begasun, the engine).  `forward` returns the logits of every position and the residual
rows behind every layer run, which is what the tests hold the engine to.  Weights come in as a dict name -> float array (the names of the model directory).

Notation: T positions, d the stream's width, rms(u) = u / sqrt(mean(u^2) + eps) over the last axis.
"""
import math
from typing import Dict, List, Optional, Tuple

import numpy as np

GATE_SLOPE = 1.702   # the sigmoid's slope in the feed-forward's gate
UP_SHIFT = 1.0       # the feed-forward's linear branch enters as (u + 1)
DECAY_RATE = 8.0     # log a = -DECAY_RATE * r * softplus(lam) in the recurrent unit
YARN_MAG = 0.1       # cos / sin are multiplied by YARN_MAG * ln(factor) + 1 under scaled frequencies


def f64(a):
    return np.asarray(a, dtype=np.float64)


def gelu_tanh(z):
    return 0.5 * z * (1.0 + np.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def softplus(z):
    return np.logaddexp(0.0, z)


def rms(u, eps):
    return u / np.sqrt(np.mean(u * u, axis=-1, keepdims=True) + eps)


def norm_one_plus(u, w, eps):
    """the model's norm: the weight is stored around zero"""
    return rms(u, eps) * (1.0 + f64(w))


def norm_plain(u, w, eps):
    return rms(u, eps) * f64(w)


def rotation_table(dims: int, base: float, scaling: Optional[dict]) -> Tuple[np.ndarray, float]:
    """angular frequencies [dims / 2] and the factor on cos / sin"""
    i = np.arange(dims // 2, dtype=np.float64)
    f = base ** (-2.0 * i / dims)
    if not scaling:
        return f, 1.0
    factor, orig = float(scaling["factor"]), float(scaling["original"])
    turn = lambda t: dims * math.log(orig / (2.0 * math.pi * t)) / (2.0 * math.log(base))
    lo = max(math.floor(turn(float(scaling["fast"]))), 0)
    hi = min(math.ceil(turn(float(scaling["slow"]))), dims - 1)
    ramp = np.clip((i - lo) / max(hi - lo, 0.001), 0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), YARN_MAG * math.log(factor) + 1.0


def rotate(x, positions, dims: int, base: float, scaling: Optional[dict], interleaved: bool):
    """x [T, ..., width]: the first `dims` coordinates of the last axis turn by position * frequency; pairs (2i, 2i + 1) or (i, i + dims / 2)"""
    x = f64(x).copy()
    if not dims:
        return x
    f, mag = rotation_table(dims, base, scaling)
    ang = f64(positions)[:, None] * f[None, :]
    shape = (x.shape[0],) + (1,) * (x.ndim - 2) + (dims // 2,)
    c, s = (np.cos(ang) * mag).reshape(shape), (np.sin(ang) * mag).reshape(shape)
    if interleaved:
        u, v = x[..., 0:dims:2].copy(), x[..., 1:dims:2].copy()
        x[..., 0:dims:2], x[..., 1:dims:2] = u * c - v * s, v * c + u * s
    else:
        h = dims // 2
        u, v = x[..., :h].copy(), x[..., h:dims].copy()
        x[..., :h], x[..., h:dims] = u * c - v * s, v * c + u * s
    return x


def causal_attention(q, k, v, scale):
    """q, k [T, H, dk], v [T, H, dv]: position i reads j <= i through a softmax of scale * q.k"""
    T = q.shape[0]
    s = np.einsum("ihd,jhd->hij", q, k) * scale
    s = np.where(np.tril(np.ones((T, T), dtype=bool))[None], s, -np.inf)
    p = np.exp(s - s.max(axis=-1, keepdims=True))
    p /= p.sum(axis=-1, keepdims=True)
    return np.einsum("hij,jhd->ihd", p, v)


def latent_attention(h, W: Dict[str, np.ndarray], p: str, mx: dict, eps: float, positions):
    """keys and values are up-projections of one normed low-rank row per position; one rotated key part is shared by the heads; a sigmoid gate per head"""
    T = h.shape[0]
    H, dim, rd, vd, rank = int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]), int(mx["kv_rank"])
    rot = mx["rot"]
    q = (h @ f64(W[p + "q"]).T).reshape(T, H, dim + rd)
    down = h @ f64(W[p + "dkv"]).T
    c = norm_plain(down[:, :rank], W[p + "dkv.norm"], eps)
    turn = lambda a: rotate(a, positions, rd, float(rot["base"]), rot.get("scaling"), interleaved=True)
    k_rot = turn(down[:, rank:])                                   # [T, rd], the same for every head
    q_rot = turn(q[:, :, dim:])
    k_plain = (c @ f64(W[p + "uk"]).T).reshape(T, H, dim)
    val = (c @ f64(W[p + "uv"]).T).reshape(T, H, vd)
    qq = np.concatenate([q[:, :, :dim], q_rot], axis=-1)
    kk = np.concatenate([k_plain, np.broadcast_to(k_rot[:, None, :], (T, H, rd))], axis=-1)
    o = causal_attention(qq, kk, val, float(mx["scale"]))
    o = o * sigmoid(h @ f64(W[p + "g"]).T)[:, :, None]
    return o.reshape(T, H * vd) @ f64(W[p + "o"]).T


def grouped_attention(h, W, p: str, mx: dict, eps: float, positions):
    """H query heads on G key / value heads, per-head RMS norm of queries and keys in front of the rotation (half-split pairing)"""
    T = h.shape[0]
    H, G, dim, vd = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
    rot = mx.get("rot") or {}
    q = norm_plain((h @ f64(W[p + "q"]).T).reshape(T, H, dim), W[p + "q.norm"], eps)
    k = norm_plain((h @ f64(W[p + "k"]).T).reshape(T, G, dim), W[p + "k.norm"], eps)
    v = (h @ f64(W[p + "v"]).T).reshape(T, G, vd)
    dims = int(rot.get("dims") or 0)
    if dims:
        q = rotate(q, positions, dims, float(rot["base"]), rot.get("scaling"), interleaved=False)
        k = rotate(k, positions, dims, float(rot["base"]), rot.get("scaling"), interleaved=False)
    rep = H // G
    o = causal_attention(q, np.repeat(k, rep, axis=1), np.repeat(v, rep, axis=1), float(mx["scale"]))
    return o.reshape(T, H * vd) @ f64(W[p + "o"]).T


def causal_conv(x, taps, bias):
    """x [T, C], taps [C, K] (the last column weighs the current position), zeros in front of the sequence"""
    T, C = x.shape
    K = taps.shape[1]
    pad = np.concatenate([np.zeros((K - 1, C)), x], axis=0)
    out = np.tile(f64(bias)[None, :], (T, 1))
    for j in range(K):
        out += pad[j:j + T] * f64(taps)[None, :, j]
    return out


def gated_linear_recurrence(u, r, i, lam):
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) i_t u_t from S = 0, a_t = exp(-DECAY_RATE r_t softplus(lam)); returns S_t for every t"""
    a = np.exp(-DECAY_RATE * r * softplus(f64(lam))[None, :])
    b = np.sqrt(1.0 - a * a) * i * u
    S = np.zeros(u.shape[1])
    out = np.empty_like(u)
    for t in range(u.shape[0]):
        S = a[t] * S + b[t]
        out[t] = S
    return out


def rglru(h, W, p: str, mx: dict):
    """two branches of `width` channels: gelu(linear) times the gated linear recurrence over a short causal convolution of the other linear"""
    width, blocks = int(mx["width"]), int(mx["blocks"])
    y = gelu_tanh(h @ f64(W[p + "y"]).T + f64(W[p + "y.b"]))
    u = causal_conv(h @ f64(W[p + "x"]).T + f64(W[p + "x.b"]), f64(W[p + "conv"]), W[p + "conv.b"])
    bw = width // blocks
    ub = u.reshape(-1, blocks, bw)
    r = sigmoid(np.einsum("tbi,boi->tbo", ub, f64(W[p + "ra"])) + f64(W[p + "ra.b"])[None]).reshape(-1, width)
    i = sigmoid(np.einsum("tbi,boi->tbo", ub, f64(W[p + "ri"])) + f64(W[p + "ri.b"])[None]).reshape(-1, width)
    S = gated_linear_recurrence(u, r, i, W[p + "lam"])
    return (S * y) @ f64(W[p + "o"]).T


def feed_forward(h, W, p: str, ml: dict):
    lim = float(ml["limit"]) if ml.get("limit") is not None else math.inf
    g = np.minimum(h @ f64(W[p + "gate"]).T, lim)
    u = np.clip(h @ f64(W[p + "up"]).T, -lim, lim)
    return (g * sigmoid(GATE_SLOPE * g) * (u + UP_SHIFT)) @ f64(W[p + "down"]).T


def token_side(x, tokens, W, layer: int, dim: int, eps: float):
    """a per-layer slice of a second embedding table, gated by the stream, projected back and added behind a plain-weight RMS norm"""
    e = f64(W["side.embed"])[np.asarray(tokens), layer * dim:(layer + 1) * dim]
    p = f"l{layer}.side."
    g = gelu_tanh(x @ f64(W[p + "gate"]).T) * e
    return x + norm_plain(g @ f64(W[p + "proj"]).T, W[p + "norm"], eps)


def layer_order(cfg: dict) -> List[Tuple[int, bool]]:
    """(layer index, the run opens a pass of the loop) for every layer run"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def forward(cfg: dict, W: Dict[str, np.ndarray], tokens) -> Tuple[np.ndarray, np.ndarray]:
    """logits [T, vocab] and the residual rows behind every layer run [runs, T, d]"""
    tokens = np.asarray(tokens, dtype=np.int64)
    eps = float(cfg["norm"]["eps"])
    positions = np.arange(len(tokens))
    x0 = f64(W["embed"])[tokens] * float(cfg["embedding"]["scale"])
    x = x0
    side = cfg.get("token_side")
    taps = []
    for i, opens in layer_order(cfg):
        lc = cfg["layers"][i]
        p = f"l{i}."
        if opens:
            x = np.concatenate([x, x0], axis=-1) @ f64(W["loop.in"]).T
        h = norm_one_plus(x, W[p + "norm1"], eps)
        kind = lc["type"]
        if kind == "latent_attention":
            m = latent_attention(h, W, p + "mix.", lc["mixer"], eps, positions)
        elif kind == "attention":
            m = grouped_attention(h, W, p + "mix.", lc["mixer"], eps, positions)
        elif kind == "rglru":
            m = rglru(h, W, p + "mix.", lc["mixer"])
        else:
            raise ValueError(kind)
        x = x + norm_one_plus(m, W[p + "norm1b"], eps) * f64(W[p + "ls1"])
        if lc.get("mlp") is not None:
            h = norm_one_plus(x, W[p + "norm2"], eps)
            x = x + norm_one_plus(feed_forward(h, W, p + "mlp.", lc["mlp"]), W[p + "norm2b"], eps) * f64(W[p + "ls2"])
        if side:
            x = token_side(x, tokens, W, i, int(side["dim"]), eps)
        taps.append(x)
    out = norm_one_plus(x, W["final.norm"], eps)
    return out @ f64(W["head"]).T * float(cfg.get("logit_scale", 1.0)), np.stack(taps)


# ---------------------------------------------------------------------------------------------- configurations, random weights and files of the tests' own making
def rot(dims, base=10000.0, scaling=None):
    r = {"dims": int(dims), "base": float(base)}
    if scaling:
        r["scaling"] = dict(scaling)
    return r


def dense(ff, limit=7.0):
    return {"kind": "dense", "ff": int(ff), "limit": float(limit)}


def latent_layer(heads, dim, rot_dim, vdim, kv_rank, rotation, scale=None, mlp=None):
    return {"type": "latent_attention", "mlp": mlp, "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rotation,
                                                              "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5)}}


def attention_layer(heads, kv_heads, dim, vdim, rotation, scale=None, mlp=None):
    return {"type": "attention", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rotation,
                                                       "scale": float(scale if scale is not None else dim ** -0.5)}}


def rglru_layer(width, blocks, conv, mlp=None):
    return {"type": "rglru", "mlp": mlp, "mixer": {"width": int(width), "blocks": int(blocks), "conv": int(conv)}}


def config(vocab, width, layers, eps=1e-6, embed_scale=None, logit_scale=1.0, loop=None, side_dim=0):
    cfg = {"architecture": "Begasun", "vocab": int(vocab), "width": int(width), "norm": {"eps": float(eps)},
           "embedding": {"scale": float(embed_scale if embed_scale is not None else width ** 0.5)}, "layers": layers, "logit_scale": float(logit_scale)}
    if loop:
        cfg["loop"] = {"start": int(loop[0]), "stop": int(loop[1]), "times": int(loop[2])}
    if side_dim:
        cfg["token_side"] = {"dim": int(side_dim)}
    return cfg


def bf16_bits(a):
    u = np.ascontiguousarray(a, dtype=np.float32).view(np.uint32).astype(np.uint64)
    return ((u + 0x7FFF + ((u >> 16) & 1)) >> 16).astype(np.uint16)


def to_bf16(a):
    return (bf16_bits(a).astype(np.uint32) << 16).view(np.float32).reshape(np.shape(a))


def weights(cfg, seed, logit_gain=1.0):
    """bf16-representable float32 tensors of every name the configuration implies"""
    rng = np.random.default_rng(seed)
    d, V = cfg["width"], cfg["vocab"]
    W = {}

    def lin(name, n, k, gain=1.0, bias=False):
        W[name] = to_bf16(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            W[name + ".b"] = to_bf16(rng.standard_normal(n) * 0.2)

    def vec(name, n, centre, spread):
        W[name] = to_bf16(centre + spread * (rng.random(n) - 0.5))

    W["embed"] = to_bf16(rng.standard_normal((V, d)) / cfg["embedding"]["scale"])
    if cfg.get("loop"):
        lin("loop.in", d, 2 * d, gain=1.4)
    side = cfg.get("token_side")
    if side:
        W["side.embed"] = to_bf16(rng.standard_normal((V, len(cfg["layers"]) * side["dim"])))
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        vec(p + "norm1", d, 0.0, 0.4), vec(p + "norm1b", d, 0.0, 0.4), vec(p + "ls1", d, 0.8, 0.8)
        if lc["type"] == "latent_attention":
            H, dim, rd, vd, rank = mx["heads"], mx["dim"], mx["rot_dim"], mx["vdim"], mx["kv_rank"]
            lin(p + "mix.q", H * (dim + rd), d, 2.5), lin(p + "mix.dkv", rank + rd, d, 2.5), lin(p + "mix.g", H, d, 2.0)
            vec(p + "mix.dkv.norm", rank, 1.0, 0.6)
            lin(p + "mix.uk", H * dim, rank, 1.5), lin(p + "mix.uv", H * vd, rank), lin(p + "mix.o", d, H * vd)
        elif lc["type"] == "attention":
            H, G, dim, vd = mx["heads"], mx["kv_heads"], mx["dim"], mx["vdim"]
            lin(p + "mix.q", H * dim, d, 2.0), lin(p + "mix.k", G * dim, d, 2.0), lin(p + "mix.v", G * vd, d)
            vec(p + "mix.q.norm", dim, 1.6, 0.8), vec(p + "mix.k.norm", dim, 1.6, 0.8)
            lin(p + "mix.o", d, H * vd)
        else:
            w, blocks, taps = mx["width"], mx["blocks"], mx["conv"]
            bw = w // blocks
            lin(p + "mix.y", w, d, 1.5, bias=True), lin(p + "mix.x", w, d, 1.5, bias=True)
            W[p + "mix.conv"] = to_bf16(rng.standard_normal((w, taps)) * 0.6)
            W[p + "mix.conv.b"] = to_bf16(rng.standard_normal(w) * 0.1)
            for g in ("ra", "ri"):
                W[p + "mix." + g] = to_bf16(rng.standard_normal((blocks, bw, bw)) * 1.5 / np.sqrt(bw))
                W[p + "mix." + g + ".b"] = to_bf16(rng.standard_normal((blocks, bw)) * 0.3)
            vec(p + "mix.lam", w, -3.0, 4.0)   # decays from about 0.3 up to 0.99 per position
            lin(p + "mix.o", d, w)
        if lc.get("mlp") is not None:
            ff = lc["mlp"]["ff"]
            vec(p + "norm2", d, 0.0, 0.4), vec(p + "norm2b", d, 0.0, 0.4), vec(p + "ls2", d, 0.8, 0.8)
            lin(p + "mlp.gate", ff, d, 1.5), lin(p + "mlp.up", ff, d, 1.5), lin(p + "mlp.down", d, ff)
        if side:
            lin(p + "side.gate", side["dim"], d, 1.5), lin(p + "side.proj", d, side["dim"])
            vec(p + "side.norm", d, 0.5, 0.6)
    vec("final.norm", d, 0.0, 0.4)
    lin("head", V, d, logit_gain)
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
    d = f64(got) - f64(want)
    d = d - d.mean(-1, keepdims=True)
    w = f64(want) - f64(want).mean(-1, keepdims=True)
    return np.sqrt((d * d).mean(-1)) / np.sqrt((w * w).mean(-1) + 1e-30)


def greedy(cfg, W, prompt, n):
    toks, out = list(prompt), []
    for _ in range(n):
        out.append(int(np.argmax(forward(cfg, W, toks)[0][-1])))
        toks.append(out[-1])
    return out
