"""Zovolorn: a decoder-only design over an f32 residual stream (include/uzu_model_desc.h: ``f32_stream``) whose sublayers read the stream through a short causal
convolution and join it behind a grouped RMS norm, with attention layers and layers that run a chunked attention and a gated delta rule side by side; read from its own
``config.json`` schema.

A model directory holds ``config.json`` (``"architecture": "Zovolorn"``) and ``model.safetensors`` (bf16 tensors, linear weights ``[out, in]``).  This module turns it
into the engine's :class:`uzu_amd.desc.ModelBundle` -- the object every other model becomes, so `HipModel`, states, batched steps, sampling and the generate loop are
the engine's own -- and writes such a directory from a configuration and random weights (tests, benchmarks).

The design, in this package's terms (every size comes from ``config.json`` or a tensor's shape, every constant that can differ between models from ``config.json``):

* ``x = embed[token] * embedding.scale + bigram[(previous * mul_prev + token * mul_cur) mod buckets]`` (a sequence's first token reads the table's last row;
  ModelBundle.bigram); the read-out is the embedding table itself behind ``final.norm``, capped by ``logit_softcap * tanh(. / logit_softcap)``.
* the model's norm is an RMS norm in ``norm.groups`` equal parts of the row, each divided by its own root mean square, times a plain weight (NormWeights.groups).
* ``layers[i]``: ``x <- x + norm1(mixer(h))`` with ``h = x + conv(x)``, then (``mlp`` not null) ``x <- x + norm2(mlp(h'))`` with ``h' = x + conv'(x)``: no norm in
  front of a sublayer; ``canon1`` / ``canon2`` are causal convolutions over positions on every channel, ``canon.taps`` taps, the last on the current position
  (LayerWeights.input_conv_*).
* ``type: attention`` (desc.MIXER_ATTENTION): ``heads`` query heads on ``kv_heads`` key / value heads (``mix.q / k / v / g`` packed), ONE RMS norm over the whole
  query projection and one over the whole key projection (``qk_norm_whole``), rotation of the first ``rot.dims`` coordinates in interleaved pairs, causal softmax with
  a learned sink logit per head (``mix.sink``), each head's result times ``sigmoid(mix.g h)`` (``has_gate``), ``mix.o``.
* ``type: parallel``: ``left_scale * left + right_scale * right`` (``pair_mixer``), both reading ``h``.
  ``left`` = attention inside chunks of ``mask.size`` positions (``attention_chunk_size``) whose values are the keys as projected (``values_are_keys``), per-head RMS
  norm of queries and keys with one shared weight, no rotation, scores ``scale * temp[head] * q.k + rel[bucket(distance), head]`` (``head_temperature``, ``rel_bias``),
  plain softmax.  ``right`` = the gated delta rule with a decay per head and key channel (desc.MIXER_DELTA_NET + ``dn_channel_decay``): q, k, v through a causal
  convolution of ``conv`` taps and silu, q and k as unit vectors, ``beta = sigmoid(b h)``, decays ``exp(-exp(A_log) softplus(a2 (a1 h) + dt_bias))``, per-head RMS of
  the result times ``norm`` times ``sigmoid(g2 (g1 h))``.
* ``mlp.kind = dense``: ``down(gelu_tanh(gate h + b) * (up h + b)) + b``.
"""
from __future__ import annotations

import json
import os
from typing import Dict, List, Optional

import numpy as np

from . import desc as D
from .design_tensors import Tensors as _Tensors, bits_to_f32 as _bits_to_f32, f32_to_bf16_bits as _f32_to_bf16_bits, full_linear as _full

ARCHITECTURE = "Zovolorn"


def load(path: str, cfg: dict, st, max_context_length: Optional[int], name: Optional[str], errors) -> D.ModelBundle:
    """config.json (already parsed) + model.safetensors (uzu_amd.loader.SafeTensors) -> ModelBundle.  `errors` = (ModelFormatError, UnsupportedModelError)."""
    bad, unsupported = errors
    t = _Tensors(st, bad)
    vocab, width = t.shape("embed")
    for key, have in (("vocab", vocab), ("width", width)):
        if cfg.get(key) is not None and int(cfg[key]) != have:
            raise bad(f"config.json: {key} = {cfg[key]} but 'embed' is {[vocab, width]}")
    norm_cfg = cfg.get("norm") or {}
    eps, groups = float(norm_cfg.get("eps", 1e-6)), int(norm_cfg.get("groups") or 1)
    if groups < 1 or width % groups:
        raise bad(f"config.json: norm.groups = {groups} does not divide width = {width}")
    max_ctx = int(max_context_length or cfg.get("max_context_length") or 4096)
    layer_cfgs = cfg.get("layers")
    if not isinstance(layer_cfgs, list) or not layer_cfgs:
        raise bad("config.json: 'layers' must be a non-empty array")
    taps = int((cfg.get("canon") or {}).get("taps") or 0)
    ropes: List[D.RopeConfig] = []

    def rope_index(rot: Optional[dict], where: str, at_most: int) -> Optional[int]:
        if not rot or not int(rot.get("dims") or 0):
            return None
        dims = int(rot["dims"])
        if dims % 2 or dims > at_most:
            raise bad(f"config.json: {where}.rot.dims = {dims}: an even number of coordinates, at most dim = {at_most}")
        r = D.RopeConfig(kind=D.ROPE_UNSCALED, head_dim=dims, max_sequence_length=max_ctx, base=float(rot["base"]))
        for i, have in enumerate(ropes):
            if have == r:
                return i
        ropes.append(r)
        return len(ropes) - 1

    grouped = lambda n: D.NormWeights(present=True, epsilon=eps, scales=np.ascontiguousarray(t.f32(n, (width,))), groups=groups)
    plain = lambda n, dim: D.NormWeights(present=True, epsilon=eps, scales=np.ascontiguousarray(t.f32(n, (dim,))))
    conv = lambda n: np.ascontiguousarray(t.f32(n, (width, taps))) if taps else None

    def heads_of(mx: dict, where: str):
        H, dim, vd = int(mx["heads"]), int(mx["dim"]), int(mx["vdim"])
        G = int(mx.get("kv_heads") or H)
        if H < 1 or G < 1 or H % G:
            raise bad(f"config.json: {where}: {H} heads on {G} kv_heads")
        return H, G, dim, vd

    def layer(i: int) -> D.LayerWeights:
        lc = layer_cfgs[i]
        p, kind, mx = f"l{i}.", lc.get("type"), lc.get("mixer") or {}
        where = f"layers[{i}].mixer"
        lw = D.LayerWeights(mixer_kind=D.MIXER_ATTENTION, hidden_dim=0, activation=D.ACT_GELU_APPROX, pre_mixer_norm=D.ABSENT_NORM, pre_mlp_norm=D.ABSENT_NORM, up_projection=None,
                            down_projection=None, post_mixer_norm=grouped(p + "norm1"), input_conv_taps=taps, input_conv_mixer=conv(p + "canon1"))
        if kind == "attention":
            H, G, dim, vd = heads_of(mx, where)
            ri = rope_index(mx.get("rot"), where, dim)
            lw.num_heads, lw.num_groups, lw.head_dim, lw.value_head_dim = H, G, dim, vd
            lw.use_rope, lw.rope_index, lw.rope_interleaved = ri is not None, ri or 0, True
            lw.attention_scale = float(mx["scale"]) if mx.get("scale") is not None else float(dim) ** -0.5
            packed = np.concatenate([t.bits(p + "mix.q", (H * dim, width)), t.bits(p + "mix.k", (G * dim, width)), t.bits(p + "mix.v", (G * vd, width)), t.bits(p + "mix.g", (H, width))], axis=0)
            lw.qkv_projection, lw.has_gate = _full(np.ascontiguousarray(packed)), True
            lw.query_norm, lw.key_norm, lw.qk_norm_whole = plain(p + "mix.q.norm", H * dim), plain(p + "mix.k.norm", G * dim), True
            lw.sinks = np.ascontiguousarray(t.bits(p + "mix.sink", (H,)))
            lw.out_projection = _full(t.bits(p + "mix.o", (width, H * vd)))
        elif kind == "parallel":
            lm, rm = mx.get("left") or {}, mx.get("right") or {}
            H, G, dim, vd = heads_of(lm, where + ".left")
            if vd != dim:
                raise bad(f"config.json: {where}.left: vdim = {vd} but the values are the keys (dim = {dim})")
            q = p + "mix.left."
            lw.num_heads, lw.num_groups, lw.head_dim, lw.value_head_dim, lw.values_are_keys = H, G, dim, dim, True
            lw.attention_scale = float(lm["scale"]) if lm.get("scale") is not None else float(dim) ** -0.5
            lw.qkv_projection = _full(np.ascontiguousarray(np.concatenate([t.bits(q + "q", (H * dim, width)), t.bits(q + "k", (G * dim, width))], axis=0)))
            lw.query_norm, lw.key_norm = plain(q + "q.norm", dim), plain(q + "k.norm", dim)
            lw.attention_chunk_size = int((lm.get("mask") or {}).get("size") or 0)
            rows = t.shape(q + "rel")[0]
            lw.rel_bias, lw.rel_bias_max = np.ascontiguousarray(t.bits(q + "rel", (rows, H))), float(lm["bias_max"])
            if rows > 1 and lw.rel_bias_max <= rows // 2:
                raise bad(f"config.json: {where}.left.bias_max = {lw.rel_bias_max}: beyond half of the {rows} rows of '{q}rel'")
            lw.head_temperature = np.ascontiguousarray(t.f32(q + "temp", (H,)))
            lw.out_projection = _full(t.bits(q + "o", (width, H * dim)))
            # the delta rule beside it
            Hd, Gd, dk, dv = heads_of(rm, where + ".right")
            ct = int(rm.get("conv") or 1)
            q = p + "mix.right."
            ra, rg = t.shape(q + "a1")[0], t.shape(q + "g1")[0]
            lw.pair_mixer, lw.pair_scales, lw.dn_channel_decay = D.MIXER_DELTA_NET, (float(mx.get("left_scale", 1.0)), float(mx.get("right_scale", 1.0))), True
            lw.dn_num_heads, lw.dn_num_groups, lw.dn_head_dim, lw.dn_value_head_dim, lw.dn_kernel_size, lw.dn_norm_epsilon = Hd, Gd, dk, dv, ct, eps
            lw.dn_in_proj = _full(np.ascontiguousarray(np.concatenate([t.bits(q + "q", (Gd * dk, width)), t.bits(q + "k", (Gd * dk, width)), t.bits(q + "v", (Hd * dv, width)),
                                                                      t.bits(q + "b", (Hd, width)), t.bits(q + "a1", (ra, width)), t.bits(q + "g1", (rg, width))], axis=0)))
            lw.dn_conv_weights = np.ascontiguousarray(np.concatenate([t.f32(q + "q.conv", (Gd * dk, ct)), t.f32(q + "k.conv", (Gd * dk, ct)), t.f32(q + "v.conv", (Hd * dv, ct))], axis=0))
            lw.dn_a_log, lw.dn_dt_bias = np.ascontiguousarray(t.f32(q + "A_log", (Hd,))), np.ascontiguousarray(t.f32(q + "dt_bias", (Hd * dk,)))
            lw.dn_norm_scales = np.ascontiguousarray(t.f32(q + "norm", (dv,)))
            lw.dn_decay_up, lw.dn_gate_up = _full(t.bits(q + "a2", (Hd * dk, ra))), _full(t.bits(q + "g2", (Hd * dv, rg)))
            lw.dn_out_proj = _full(t.bits(q + "o", (width, Hd * dv)))
        else:
            raise unsupported(f"config.json: layers[{i}].type = {kind!r} (attention | parallel)")
        ml = lc.get("mlp")
        if ml is None:
            lw.no_mlp = True
            for spare in (p + "norm2", p + "canon2"):  # a layer without a dense block has no use for them; a file that carries them all the same is read
                if t.has(spare):
                    st.consumed.add(spare)
        elif ml.get("kind") == "dense":
            ff = int(ml.get("ff") or t.shape(p + "mlp.gate")[0])
            lw.hidden_dim = ff
            lw.post_mlp_norm, lw.input_conv_mlp = grouped(p + "norm2"), conv(p + "canon2")
            lw.up_projection = _full(np.ascontiguousarray(np.concatenate([t.bits(p + "mlp.up", (ff, width)), t.bits(p + "mlp.gate", (ff, width))], axis=0)),  # [up ; gate]
                                     np.ascontiguousarray(np.concatenate([t.bits(p + "mlp.up.b", (ff,)), t.bits(p + "mlp.gate.b", (ff,))])))
            lw.down_projection = _full(t.bits(p + "mlp.down", (width, ff)), np.ascontiguousarray(t.bits(p + "mlp.down.b", (width,))))
        else:
            raise unsupported(f"config.json: layers[{i}].mlp.kind = {ml.get('kind')!r} (dense, or mlp: null)")
        return lw

    layers = [layer(i) for i in range(len(layer_cfgs))]
    em = cfg.get("embedding") or {}
    bg = em.get("bigram")
    bigram, mul = None, (0, 0)
    if bg:
        buckets = int(bg["buckets"])
        if buckets < 1:
            raise bad(f"config.json: embedding.bigram.buckets = {buckets}")
        bigram, mul = _full(t.bits("bigram", (buckets + 1, width))), (int(bg["mul_prev"]), int(bg["mul_cur"]))
    bundle = D.ModelBundle(name=name or os.path.basename(os.path.normpath(path)), vocab_size=int(vocab), model_dim=int(width), max_context_length=max_ctx, rope=D.RopeConfig(),
                           embedding=_full(t.bits("embed", (vocab, width))), output_norm=grouped("final.norm"), layers=layers, tied_embeddings=True,
                           input_scale=float(em.get("scale", 1.0)), logit_soft_cap=float(cfg.get("logit_softcap") or 0.0), ropes=ropes or None, f32_stream=True,
                           architecture=ARCHITECTURE, bigram=bigram, bigram_mul=mul)
    st.assert_all_consumed()
    return bundle


# ------------------------------------------------------------------------------------------------ writer: a configuration + random weights -> a model directory
def random_tensors(cfg: dict, seed: int = 0) -> Dict[str, np.ndarray]:
    """f32 values (already bf16-representable) of every tensor a configuration names, from a seeded generator: linear weights ~ N(0, gain^2 / in), norm weights
    around 1, convolution taps and biases small, decays spread between fast and slow"""
    rng = np.random.default_rng(seed)
    rb = lambda a: _bits_to_f32(_f32_to_bf16_bits(np.asarray(a, dtype=np.float32)))
    vocab, width = int(cfg["vocab"]), int(cfg["width"])
    taps = int((cfg.get("canon") or {}).get("taps") or 0)
    out: Dict[str, np.ndarray] = {}

    def lin(name, n, k, bias=False, gain=1.0):
        out[name] = rb(rng.standard_normal((n, k)) * gain / np.sqrt(k))
        if bias:
            out[name + ".b"] = rb(rng.standard_normal(n) * 0.2)

    vec = lambda name, n, centre, spread: out.__setitem__(name, rb(centre + spread * (rng.random(n) - 0.5)))
    em = cfg["embedding"]
    out["embed"] = rb(rng.standard_normal((vocab, width)) / float(em.get("scale", 1.0)))
    if em.get("bigram"):
        out["bigram"] = rb(rng.standard_normal((int(em["bigram"]["buckets"]) + 1, width)) * 0.5)
    for i, lc in enumerate(cfg["layers"]):
        p, mx = f"l{i}.", lc["mixer"]
        vec(p + "norm1", width, 1.0, 0.6)
        if taps:
            out[p + "canon1"] = rb(rng.standard_normal((width, taps)) * 0.3)
        if lc["type"] == "attention":
            H, G, dim, vd = int(mx["heads"]), int(mx["kv_heads"]), int(mx["dim"]), int(mx["vdim"])
            q = p + "mix."
            lin(q + "q", H * dim, width, gain=2.0), lin(q + "k", G * dim, width, gain=2.0), lin(q + "v", G * vd, width), lin(q + "g", H, width, gain=2.0)
            vec(q + "q.norm", H * dim, 1.5, 0.6), vec(q + "k.norm", G * dim, 1.5, 0.6), vec(q + "sink", H, 0.5, 3.0)
            lin(q + "o", width, H * vd)
        else:
            lm, rm = mx["left"], mx["right"]
            H, G, dim = int(lm["heads"]), int(lm["kv_heads"]), int(lm["dim"])
            q = p + "mix.left."
            lin(q + "q", H * dim, width, gain=2.0), lin(q + "k", G * dim, width, gain=2.0)
            vec(q + "q.norm", dim, 1.5, 0.6), vec(q + "k.norm", dim, 1.5, 0.6), vec(q + "temp", H, 1.0, 1.0)
            out[q + "rel"] = rb(rng.standard_normal((int(lm["rel_rows"]), H)) * 1.5)
            lin(q + "o", width, H * dim)
            Hd, Gd, dk, dv, ct, rank = int(rm["heads"]), int(rm["kv_heads"]), int(rm["dim"]), int(rm["vdim"]), int(rm["conv"]), int(rm.get("rank", 4))
            q = p + "mix.right."
            lin(q + "q", Gd * dk, width, gain=2.0), lin(q + "k", Gd * dk, width, gain=2.0), lin(q + "v", Hd * dv, width, gain=1.5), lin(q + "b", Hd, width, gain=2.0)
            for n, ch in (("q", Gd * dk), ("k", Gd * dk), ("v", Hd * dv)):
                out[q + n + ".conv"] = rb(rng.standard_normal((ch, ct)) * 0.6)
            lin(q + "a1", rank, width), lin(q + "a2", Hd * dk, rank, gain=2.0), lin(q + "g1", rank, width), lin(q + "g2", Hd * dv, rank, gain=2.0)
            vec(q + "A_log", Hd, -1.0, 3.0), vec(q + "dt_bias", Hd * dk, -1.0, 3.0), vec(q + "norm", dv, 1.0, 0.6)
            lin(q + "o", width, Hd * dv)
        ml = lc.get("mlp")
        if ml is not None:
            ff = int(ml["ff"])
            vec(p + "norm2", width, 1.0, 0.6)
            if taps:
                out[p + "canon2"] = rb(rng.standard_normal((width, taps)) * 0.3)
            lin(p + "mlp.gate", ff, width, bias=True, gain=1.5), lin(p + "mlp.up", ff, width, bias=True, gain=1.5), lin(p + "mlp.down", width, ff, bias=True)
    vec("final.norm", width, 1.0, 0.6)
    return out


def save(path: str, cfg: dict, tensors: Dict[str, np.ndarray]):
    """Write config.json + model.safetensors (every tensor as bf16) in this design's layout (`rel_rows` / `rank` of a layer are sizes of the writer only: a reader
    takes them from the tensors' shapes)."""
    from .loader import write_safetensors
    os.makedirs(path, exist_ok=True)
    full = json.loads(json.dumps(cfg))
    full["architecture"] = ARCHITECTURE
    for lc in full["layers"]:
        if lc["type"] == "parallel":
            lc["mixer"]["left"].pop("rel_rows", None), lc["mixer"]["right"].pop("rank", None)
    with open(os.path.join(path, "config.json"), "w", encoding="utf-8") as f:
        json.dump(full, f, indent=1, sort_keys=True)
    write_safetensors(os.path.join(path, "model.safetensors"), {k: ("BF16", _f32_to_bf16_bits(v).reshape(np.shape(v))) for k, v in tensors.items()}, {})


def dense_mlp(ff: int) -> dict:
    return {"kind": "dense", "ff": int(ff)}


def attention_layer(heads: int, kv_heads: int, dim: int, vdim: int, rot_dims: int = 0, rot_base: float = 10000.0, scale: Optional[float] = None, mlp: Optional[dict] = None) -> dict:
    mx = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": float(scale if scale is not None else dim ** -0.5)}
    if rot_dims:
        mx["rot"] = {"dims": int(rot_dims), "base": float(rot_base)}
    return {"type": "attention", "mixer": mx, "mlp": mlp}


def parallel_layer(heads: int, kv_heads: int, dim: int, chunk: int, rel_rows: int, bias_max: float, d_heads: int, d_kv_heads: int, d_dim: int, d_vdim: int, conv: int, rank: int = 4,
                   scale: Optional[float] = None, left_scale: float = 1.0, right_scale: float = 1.0, mlp: Optional[dict] = None) -> dict:
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "mask": {"size": int(chunk)}, "bias_max": float(bias_max), "rel_rows": int(rel_rows),
            "scale": float(scale if scale is not None else dim ** -0.5)}
    right = {"heads": d_heads, "kv_heads": d_kv_heads, "dim": d_dim, "vdim": d_vdim, "conv": int(conv), "rank": int(rank)}
    return {"type": "parallel", "mixer": {"left": left, "right": right, "left_scale": float(left_scale), "right_scale": float(right_scale)}, "mlp": mlp}


def config(vocab: int, width: int, layers: List[dict], eps: float = 1e-5, groups: int = 1, taps: int = 4, embed_scale: float = 1.0, bigram: Optional[tuple] = None,
           logit_softcap: float = 0.0) -> dict:
    """bigram = (buckets, mul_prev, mul_cur)"""
    em = {"scale": float(embed_scale)}
    if bigram:
        em["bigram"] = {"buckets": int(bigram[0]), "mul_prev": int(bigram[1]), "mul_cur": int(bigram[2])}
    return {"vocab": int(vocab), "width": int(width), "norm": {"eps": float(eps), "groups": int(groups)}, "canon": {"taps": int(taps)}, "embedding": em, "layers": layers,
            "logit_softcap": float(logit_softcap)}
