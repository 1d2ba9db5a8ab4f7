"""Begasun: a decoder-only design over an f32 residual stream (include/uzu_model_desc.h: ``f32_stream``) with a looped stack of mixed layers, read from its own
``config.json`` schema.

A model directory holds ``config.json`` (``"architecture": "Begasun"``) and ``model.safetensors`` (bf16 tensors, linear weights ``[out, in]``).  This module turns it
into the engine's :class:`uzu_amd.desc.ModelBundle` -- the object every other model becomes, so `HipModel`, states, batched steps, sampling and the generate loop are
the engine's own -- and writes such a directory from a configuration and random weights (tests, benchmarks).

The design, in this package's terms (every size comes from ``config.json`` or a tensor's shape, every constant that can differ between models from ``config.json``):

* ``x = embed[token] * embedding.scale``; the read-out is ``head`` behind ``final.norm``, times ``logit_scale``.
* the model's norm is an RMS norm whose weight is stored around zero: ``x / sqrt(mean(x^2) + norm.eps) * (1 + w)`` (desc.NORM_STATISTICS with scale_offset 1).
* ``layers[i]``: ``x <- x + ls1 * norm1b(mixer(norm1(x)))``, then (``mlp`` not null) ``x <- x + ls2 * norm2b(mlp(norm2(x)))``: a norm in front of and behind every
  sublayer, and a layer scale (a vector) on each result.
* ``token_side``: behind that, ``x <- x + rms(proj(gelu(gate x) * e)) * side.norm`` with ``e`` layer i's ``dim``-wide slice of the token's row of ``side.embed``.
* ``loop {start, stop, times}``: layers start .. stop - 1 run ``times`` times with the same tensors, each pass opened by ``x <- loop.in [x ; x0]`` (x0 = the embedding
  rows); every run has its own sequence state.  The bundle lists layer RUNS: a repeated run names the run whose tensors it uses (``weights_of_layer``).
* ``type: latent_attention`` (desc.MIXER_LATENT_ATTENTION): ``mix.q`` (heads x [dim | rot_dim]), ``mix.dkv`` (``kv_rank`` latent numbers, RMS-normed with
  ``mix.dkv.norm``, + ``rot_dim`` numbers of ONE rotated key part for all heads), ``mix.g`` (a sigmoid gate per head), packed into one projection; per-head keys
  ``mix.uk`` and values ``mix.uv`` of the latent; rotation in interleaved pairs, frequencies optionally YaRN-scaled; causal softmax; ``mix.o``.
* ``type: attention`` (desc.MIXER_ATTENTION): ``heads`` query heads on ``kv_heads`` key / value heads (``mix.q / k / v`` packed, no biases), per-head RMS norm of
  queries and keys (``mix.q.norm`` / ``mix.k.norm``) in front of the half-split rotation of the first ``rot.dims`` coordinates, causal softmax, ``mix.o``.
* ``type: rglru`` (desc.MIXER_GATED_LRU): ``mix.y`` / ``mix.x`` (+ biases, packed), a causal convolution per channel (``mix.conv`` [channels, taps], ``mix.conv.b``),
  block-diagonal gates ``mix.ra / ri`` (+ ``.b``), ``mix.lam``; ``S <- a S + sqrt(1 - a^2) i u`` with ``a = exp(-8 r softplus(lam))``; ``mix.o (S * gelu(y))``.
* ``mlp.kind = dense``: ``down(g * sigmoid(1.702 g) * (u + 1))`` with ``g = min(gate h, limit)``, ``u = clamp(up h, -limit, limit)``.
"""
from __future__ import annotations

import dataclasses
import json
import os
from typing import Dict, List, Optional

import numpy as np

from . import desc as D
from .design_tensors import Tensors as _Tensors, bits_to_f32 as _bits_to_f32, f32_to_bf16_bits as _f32_to_bf16_bits, full_linear as _full

ARCHITECTURE = "Begasun"
GATE_ALPHA = 1.702   # the sigmoid's slope in the dense block's gate
UP_OFFSET = 1.0      # the dense block's up branch enters the product as (u + 1)
LRU_DECAY_RATE = 8.0  # log a = -8 r softplus(lam)


def _rope(rot: dict, max_positions: int) -> D.RopeConfig:
    sc = rot.get("scaling")
    if not sc:
        return D.RopeConfig(kind=D.ROPE_UNSCALED, head_dim=int(rot["dims"]), max_sequence_length=max_positions, base=float(rot["base"]))
    return D.RopeConfig(kind=D.ROPE_YARN, head_dim=int(rot["dims"]), max_sequence_length=max_positions, base=float(rot["base"]), scaling_factor=float(sc["factor"]),
                        original_context_length=int(sc["original"]), beta_fast=float(sc["fast"]), beta_slow=float(sc["slow"]), truncate=True)


def layer_runs(cfg: dict) -> List[tuple]:
    """(layer index, the run opens a pass of the loop) for every layer run, in order"""
    n = len(cfg["layers"])
    loop = cfg.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    runs = [(i, False) for i in range(a)]
    for _ in range(times):
        runs += [(i, i == a) for i in range(a, b)]
    return runs + [(i, False) for i in range(b, n)]


def load(path: str, cfg: dict, st, max_context_length: Optional[int], name: Optional[str], errors) -> D.ModelBundle:
    """config.json (already parsed) + model.safetensors (uzu_amd.loader.SafeTensors) -> ModelBundle.  `errors` = (ModelFormatError, UnsupportedModelError)."""
    bad, unsupported = errors
    t = _Tensors(st, bad)
    vocab, width = t.shape("embed")
    for key, have in (("vocab", vocab), ("width", width)):
        if cfg.get(key) is not None and int(cfg[key]) != have:
            raise bad(f"config.json: {key} = {cfg[key]} but 'embed' is {[vocab, width]}")
    eps = float((cfg.get("norm") or {}).get("eps", 1e-6))
    max_ctx = int(max_context_length or cfg.get("max_context_length") or 4096)
    layer_cfgs = cfg.get("layers")
    if not isinstance(layer_cfgs, list) or not layer_cfgs:
        raise bad("config.json: 'layers' must be a non-empty array")
    n_layers = len(layer_cfgs)
    loop = cfg.get("loop")
    if loop:
        a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
        if not (0 <= a < b <= n_layers and times >= 1):
            raise bad(f"config.json: loop = {loop}: 0 <= start < stop <= {n_layers} layers, times >= 1")
    side = cfg.get("token_side")
    side_dim = int(side["dim"]) if side else 0
    ropes: List[D.RopeConfig] = []

    def rope_index(rot: Optional[dict], where: str, exactly: Optional[int] = None, at_most: Optional[int] = None) -> Optional[int]:
        if not rot or not int(rot.get("dims") or 0):
            return None
        dims = int(rot["dims"])
        if dims % 2 or (exactly is not None and dims != exactly) or (at_most is not None and dims > at_most):
            raise bad(f"config.json: {where}.rot.dims = {dims}: an even number of coordinates, " + (f"the rotated part's {exactly}" if exactly is not None else f"at most dim = {at_most}"))
        r = _rope(rot, max_ctx)
        for i, have in enumerate(ropes):
            if have == r:
                return i
        ropes.append(r)
        return len(ropes) - 1

    one_plus = lambda n, dim: D.NormWeights(present=True, epsilon=eps, scale_offset=1.0, scales=np.ascontiguousarray(t.f32(n, (dim,))))
    plain = lambda n, dim: D.NormWeights(present=True, epsilon=eps, scale_offset=0.0, scales=np.ascontiguousarray(t.f32(n, (dim,))))

    def layer(i: int) -> D.LayerWeights:
        lc = layer_cfgs[i]
        p, kind, mx = f"l{i}.", lc.get("type"), lc.get("mixer") or {}
        where = f"layers[{i}].mixer"
        lw = D.LayerWeights(mixer_kind=D.MIXER_ATTENTION, hidden_dim=0, activation=D.ACT_SILU, pre_mixer_norm=one_plus(p + "norm1", width), pre_mlp_norm=D.ABSENT_NORM,
                            up_projection=None, down_projection=None, post_mixer_norm=one_plus(p + "norm1b", width),
                            layer_scale_mixer=np.ascontiguousarray(t.f32(p + "ls1", (width,))))
        if kind == "latent_attention":
            H, dim, rd, vd, rank = int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]), int(mx["kv_rank"])
            ri = rope_index(mx.get("rot"), where, exactly=rd) if rd else None
            if rd and ri is None:
                raise bad(f"config.json: {where}: rot_dim = {rd} without a rotation")
            lw.mixer_kind, lw.num_heads, lw.num_groups, lw.head_dim, lw.value_head_dim, lw.latent_rank, lw.latent_rope_dim = D.MIXER_LATENT_ATTENTION, H, H, dim, vd, rank, rd
            lw.use_rope, lw.rope_index, lw.rope_interleaved, lw.latent_packed, lw.has_gate = ri is not None, ri or 0, True, True, True
            lw.attention_scale = float(mx["scale"]) if mx.get("scale") is not None else float(dim + rd) ** -0.5
            packed = np.concatenate([t.bits(p + "mix.q", (H * (dim + rd), width)), t.bits(p + "mix.dkv", (rank + rd, width)), t.bits(p + "mix.g", (H, width))], axis=0)
            lw.qkv_projection = _full(np.ascontiguousarray(packed))
            lw.latent_norm = plain(p + "mix.dkv.norm", rank)
            lw.latent_up_keys = _full(t.bits(p + "mix.uk", (H * dim, rank)))
            lw.latent_up_values = _full(t.bits(p + "mix.uv", (H * vd, rank)))
            lw.out_projection = _full(t.bits(p + "mix.o", (width, H * vd)))
        elif kind == "attention":
            H, dim, vd = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
            G = int(mx.get("kv_heads") or H)
            if H % G:
                raise bad(f"config.json: {where}: {H} heads on {G} kv_heads")
            ri = rope_index(mx.get("rot"), where, at_most=dim)
            lw.num_heads, lw.num_groups, lw.head_dim, lw.value_head_dim = H, G, dim, vd
            lw.use_rope, lw.rope_index = ri is not None, ri or 0
            lw.attention_scale = float(mx["scale"]) if mx.get("scale") is not None else float(dim) ** -0.5
            packed = np.concatenate([t.bits(p + "mix.q", (H * dim, width)), t.bits(p + "mix.k", (G * dim, width)), t.bits(p + "mix.v", (G * vd, width))], axis=0)
            lw.qkv_projection = _full(np.ascontiguousarray(packed))
            lw.query_norm, lw.key_norm = plain(p + "mix.q.norm", dim), plain(p + "mix.k.norm", dim)
            lw.out_projection = _full(t.bits(p + "mix.o", (width, H * vd)))
        elif kind == "rglru":
            w, blocks, taps = int(mx["width"]), int(mx["blocks"]), int(mx["conv"])
            if blocks < 1 or w % blocks or taps < 1:
                raise bad(f"config.json: {where}: width = {w} in {blocks} blocks, {taps} taps")
            bw = w // blocks
            lw.mixer_kind, lw.lru_width, lw.lru_blocks, lw.lru_decay_rate, lw.dn_kernel_size = D.MIXER_GATED_LRU, w, blocks, LRU_DECAY_RATE, taps
            packed = np.concatenate([t.bits(p + "mix.y", (w, width)), t.bits(p + "mix.x", (w, width))], axis=0)
            lw.qkv_projection = _full(np.ascontiguousarray(packed), np.ascontiguousarray(np.concatenate([t.bits(p + "mix.y.b", (w,)), t.bits(p + "mix.x.b", (w,))])))
            lw.dn_conv_weights = np.ascontiguousarray(t.f32(p + "mix.conv", (w, taps)))
            lw.dn_conv_biases = np.ascontiguousarray(t.f32(p + "mix.conv.b", (w,)))
            # per block: the recurrence gate's rows, then the input gate's
            lw.lru_gate_weights = np.ascontiguousarray(np.concatenate([t.bits(p + "mix.ra", (blocks, bw, bw)), t.bits(p + "mix.ri", (blocks, bw, bw))], axis=1))
            lw.lru_gate_biases = np.ascontiguousarray(np.concatenate([t.f32(p + "mix.ra.b", (blocks, bw)), t.f32(p + "mix.ri.b", (blocks, bw))], axis=1))
            lw.lru_lambda = np.ascontiguousarray(t.f32(p + "mix.lam", (w,)))
            lw.out_projection = _full(t.bits(p + "mix.o", (width, w)))
        else:
            raise unsupported(f"config.json: layers[{i}].type = {kind!r} (latent_attention | attention | rglru)")
        ml = lc.get("mlp")
        if ml is None:
            lw.no_mlp = True
        elif ml.get("kind") == "dense":
            ff = int(ml.get("ff") or t.shape(p + "mlp.gate")[0])
            limit = float(ml["limit"]) if ml.get("limit") is not None else float("inf")
            lw.hidden_dim = ff
            lw.pre_mlp_norm, lw.post_mlp_norm = one_plus(p + "norm2", width), one_plus(p + "norm2b", width)
            lw.layer_scale_mlp = np.ascontiguousarray(t.f32(p + "ls2", (width,)))
            lw.up_projection = _full(np.ascontiguousarray(np.concatenate([t.bits(p + "mlp.up", (ff, width)), t.bits(p + "mlp.gate", (ff, width))], axis=0)))  # [up ; gate]
            lw.down_projection = _full(t.bits(p + "mlp.down", (width, ff)))
            lw.gated_act = (GATE_ALPHA, (float("-inf"), limit), (-limit, limit), UP_OFFSET)
        else:
            raise unsupported(f"config.json: layers[{i}].mlp.kind = {ml.get('kind')!r} (dense, or mlp: null)")
        if side_dim:
            lw.ple = D.PleLayerWeights(ple_dim=side_dim, activation=D.ACT_GELU_APPROX, gate=_full(t.bits(p + "side.gate", (side_dim, width))),
                                       projection=_full(t.bits(p + "side.proj", (width, side_dim))), norm=plain(p + "side.norm", width))
            lw.ple_slice = i
        return lw

    own: Dict[int, int] = {}   # layer index -> its first run
    runs: List[D.LayerWeights] = []
    reentry = _full(t.bits("loop.in", (width, 2 * width))) if loop else None
    for i, opens in layer_runs(cfg):
        if i in own:
            runs.append(dataclasses.replace(runs[own[i]], weights_of_layer=own[i]))
            continue
        lw = layer(i)
        if opens:
            lw.stream_reentry = reentry
        own[i] = len(runs)
        runs.append(lw)
    bundle = D.ModelBundle(name=name or os.path.basename(os.path.normpath(path)), vocab_size=int(vocab), model_dim=int(width), max_context_length=max_ctx,
                           rope=D.RopeConfig(), embedding=_full(t.bits("embed", (vocab, width))), output_norm=one_plus("final.norm", width), layers=runs,
                           tied_embeddings=False, output_embedding=_full(t.bits("head", (vocab, width))), input_scale=float((cfg.get("embedding") or {}).get("scale", 1.0)),
                           logit_scale=float(cfg.get("logit_scale", 1.0)), ropes=ropes or None, f32_stream=True, architecture=ARCHITECTURE,
                           side_table=_full(t.bits("side.embed", (vocab, n_layers * side_dim))) if side_dim else None, side_dim=side_dim)
    st.assert_all_consumed()
    return bundle


# ------------------------------------------------------------------------------------------------ writer: a configuration + random weights -> a model directory
def random_tensors(cfg: dict, seed: int = 0) -> Dict[str, np.ndarray]:
    """f32 values (already bf16-representable) of every tensor a configuration names, from a seeded generator: linear weights ~ N(0, gain^2 / in), norm weights
    near 0, layer scales near 1, recurrent decays spread over (0.3, 0.99)"""
    rng = np.random.default_rng(seed)
    rb = lambda a: _bits_to_f32(_f32_to_bf16_bits(np.asarray(a, dtype=np.float32)))
    vocab, width = int(cfg["vocab"]), int(cfg["width"])
    out: Dict[str, np.ndarray] = {}

    def lin(name, n, k, bias=False, gain=1.0):
        out[name] = rb(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            out[name + ".b"] = rb(rng.standard_normal(n) * 0.2)

    vec = lambda name, n, centre, spread: out.__setitem__(name, rb(centre + spread * (rng.random(n) - 0.5)))
    out["embed"] = rb(rng.standard_normal((vocab, width)) / float(cfg["embedding"]["scale"]))
    if cfg.get("loop"):
        lin("loop.in", width, 2 * width, gain=1.4)
    side = cfg.get("token_side")
    if side:
        out["side.embed"] = rb(rng.standard_normal((vocab, len(cfg["layers"]) * int(side["dim"]))))
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        vec(p + "norm1", width, 0.0, 0.3), vec(p + "norm1b", width, 0.0, 0.3), vec(p + "ls1", width, 0.8, 0.6)
        if lc["type"] == "latent_attention":
            H, dim, rd, vd, rank = int(mx["heads"]), int(mx["dim"]), int(mx["rot_dim"]), int(mx["vdim"]), int(mx["kv_rank"])
            lin(p + "mix.q", H * (dim + rd), width, gain=2.0), lin(p + "mix.dkv", rank + rd, width, gain=2.0), lin(p + "mix.g", H, width, gain=2.0)
            vec(p + "mix.dkv.norm", rank, 1.0, 0.4)
            lin(p + "mix.uk", H * dim, rank, gain=1.5), lin(p + "mix.uv", H * vd, rank), lin(p + "mix.o", width, H * vd)
        elif lc["type"] == "attention":
            H, G, dim, vd = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
            lin(p + "mix.q", H * dim, width, gain=2.0), lin(p + "mix.k", G * dim, width, gain=2.0), lin(p + "mix.v", G * vd, width)
            vec(p + "mix.q.norm", dim, 1.5, 0.6), vec(p + "mix.k.norm", dim, 1.5, 0.6)
            lin(p + "mix.o", width, H * vd)
        else:
            w, blocks, taps = int(mx["width"]), int(mx["blocks"]), int(mx["conv"])
            bw = w // blocks
            lin(p + "mix.y", w, width, bias=True, gain=1.5), lin(p + "mix.x", w, width, bias=True, gain=1.5)
            out[p + "mix.conv"] = rb(rng.standard_normal((w, taps)) * 0.6)
            out[p + "mix.conv.b"] = rb(rng.standard_normal(w) * 0.1)
            for g in ("ra", "ri"):
                out[p + "mix." + g] = rb(rng.standard_normal((blocks, bw, bw)) * 1.5 / np.sqrt(bw))
                out[p + "mix." + g + ".b"] = rb(rng.standard_normal((blocks, bw)) * 0.3)
            vec(p + "mix.lam", w, -2.75, 3.5)
            lin(p + "mix.o", width, w)
        ml = lc.get("mlp")
        if ml is not None:
            ff = int(ml["ff"])
            vec(p + "norm2", width, 0.0, 0.3), vec(p + "norm2b", width, 0.0, 0.3), vec(p + "ls2", width, 0.8, 0.6)
            lin(p + "mlp.gate", ff, width, gain=1.5), lin(p + "mlp.up", ff, width, gain=1.5), lin(p + "mlp.down", width, ff)
        if side:
            sd = int(side["dim"])
            lin(p + "side.gate", sd, width, gain=1.5), lin(p + "side.proj", width, sd)
            vec(p + "side.norm", width, 0.5, 0.4)
    vec("final.norm", width, 0.0, 0.3)
    lin("head", vocab, width)
    return out


def save(path: str, cfg: dict, tensors: Dict[str, np.ndarray]):
    """Write config.json + model.safetensors (every tensor as bf16) in this design's layout."""
    from .loader import write_safetensors
    os.makedirs(path, exist_ok=True)
    full = dict(cfg)
    full["architecture"] = ARCHITECTURE
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(full, f, indent=1, sort_keys=True)
    write_safetensors(os.path.join(path, "model.safetensors"), {k: ("BF16", _f32_to_bf16_bits(v).reshape(np.shape(v))) for k, v in tensors.items()}, {})


def rotation(dims: int, base: float = 10000.0, scaling: Optional[dict] = None) -> dict:
    r = {"dims": int(dims), "base": float(base)}
    if scaling:
        r["scaling"] = {k: scaling[k] for k in ("factor", "original", "fast", "slow")}
    return r


def dense_mlp(ff: int, limit: float = 7.0) -> dict:
    return {"kind": "dense", "ff": int(ff), "limit": float(limit)}


def latent_attention_layer(heads: int, dim: int, rot_dim: int, vdim: int, kv_rank: int, rot: dict, scale: Optional[float] = None, mlp: Optional[dict] = None) -> dict:
    return {"type": "latent_attention", "mlp": mlp,
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "rot": rot, "scale": float(scale if scale is not None else (dim + rot_dim) ** -0.5)}}


def attention_layer(heads: int, kv_heads: int, dim: int, vdim: int, rot: dict, scale: Optional[float] = None, mlp: Optional[dict] = None) -> dict:
    return {"type": "attention", "mlp": mlp, "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "rot": rot, "scale": float(scale if scale is not None else dim ** -0.5)}}


def rglru_layer(width: int, blocks: int, conv: int, mlp: Optional[dict] = None) -> dict:
    return {"type": "rglru", "mlp": mlp, "mixer": {"width": int(width), "blocks": int(blocks), "conv": int(conv)}}


def config(vocab: int, width: int, layers: List[dict], eps: float = 1e-6, embed_scale: Optional[float] = None, logit_scale: float = 1.0, loop: Optional[tuple] = None,
           side_dim: int = 0) -> dict:
    cfg = {"vocab": int(vocab), "width": int(width), "norm": {"eps": float(eps)}, "embedding": {"scale": float(embed_scale if embed_scale is not None else width ** 0.5)},
           "layers": layers, "logit_scale": float(logit_scale)}
    if loop:
        cfg["loop"] = {"start": int(loop[0]), "stop": int(loop[1]), "times": int(loop[2])}
    if side_dim:
        cfg["token_side"] = {"dim": int(side_dim)}
    return cfg
