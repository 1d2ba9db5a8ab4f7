"""Zovolorn on the host: identities of the float64 oracle (what the GPU tests lean on), and the config.json reader -- every branch of the schema, the engine
description it produces (packed projections, the second mixer's fields, absent pre norms), its refusals, and what the writer writes read back.  No GPU."""
import json
import os

import numpy as np
import pytest

import zovolorn_oracle as O
from uzu_amd import desc as D, loader, zovolorn


def test_oracle_rotation_norm_in_parts_and_convolution():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((9, 3, 12))
    r = O.rotate_pairs(x, 8, 1e4, first_position=5)
    assert np.allclose(r[..., 8:], x[..., 8:])  # the tail passes unchanged
    assert np.allclose((r[..., 2:4] ** 2).sum(-1), (x[..., 2:4] ** 2).sum(-1))  # a rotation keeps the length of every pair (2i, 2i + 1)
    assert np.allclose(O.rotate_pairs(x, 8, 1e4)[0], x[0])  # position 0 turns nothing
    q, k = rng.standard_normal((1, 1, 8)), rng.standard_normal((1, 1, 8))
    s = lambda a, b: float(O.rotate_pairs(q, 8, 1e4, a)[0, 0] @ O.rotate_pairs(k, 8, 1e4, b)[0, 0])
    assert np.isclose(s(10, 3), s(107, 100))  # scores of rotated queries and keys depend on the distance only
    # the norm in parts: every part has mean square 1 in front of the weight
    y, w = rng.standard_normal((4, 12)) * np.array([1.0] * 6 + [50.0] * 6), rng.random(12) + 0.5
    n = O.grouped_rms_norm(y, w, 2, 0.0) / w
    assert np.allclose((n[:, :6] ** 2).mean(-1), 1.0) and np.allclose((n[:, 6:] ** 2).mean(-1), 1.0)
    assert not np.allclose((O.grouped_rms_norm(y, w, 1, 0.0)[:, :6] / w[:6]) ** 2, n[:, :6] ** 2)
    assert np.allclose(O.grouped_rms_norm(y, w, 12, 0.0), np.sign(y) * w)  # every coordinate its own part
    # the convolution: zeros in front of the sequence, the last tap weighs the current position
    h, taps = rng.standard_normal((20, 5)), rng.standard_normal((5, 4))
    c = O.causal_conv(h, taps)
    assert np.allclose(c[0], taps[:, 3] * h[0]) and np.allclose(c[7], sum(taps[:, j] * h[7 - 3 + j] for j in range(4)))
    assert np.allclose(O.causal_conv(h, taps[:, 3:]), taps[:, 3] * h)  # one tap: a scale


def test_oracle_distance_buckets_and_the_token_pair_table():
    b = [O.distance_bucket(n, 32, 240.0) for n in range(400)]
    assert b[:16] == list(range(16)) and b[16] == 16 and b[239] == 31 and b[240] == 31 and b[399] == 31
    assert all(y - x in (0, 1) for x, y in zip(b, b[1:])) and sorted(set(b)) == list(range(32))  # monotone, no bucket skipped at these sizes
    assert [O.distance_bucket(n, 1, 5.0) for n in range(4)] == [0, 0, 0, 0]
    assert [O.distance_bucket(n, 2, 3.0) for n in range(4)] == [0, 1, 1, 1]
    assert [O.distance_bucket(n, 5, 9.0) for n in range(10)][:3] == [0, 1, 2]  # five rows: two exact, three logarithmic
    table, pair = np.arange(12.0).reshape(6, 2), np.arange(100.0, 116.0).reshape(8, 2)
    x = O.embed_rows([5, 1, 1, 3], table, 0.5, pair, 7, 3, 2)
    assert np.allclose(x[0], table[5] * 0.5 + pair[7])  # the first token: the last row
    assert np.allclose(x[1], table[1] * 0.5 + pair[(5 * 3 + 1 * 2) % 7]) and np.allclose(x[3], table[3] * 0.5 + pair[(1 * 3 + 3 * 2) % 7])


def test_oracle_delta_rule_and_sink():
    rng = np.random.default_rng(1)
    T, dk, dv = 12, 5, 3
    q, k, v = rng.standard_normal((T, dk)), rng.standard_normal((T, dk)), rng.standard_normal((T, dv))
    k = k / np.linalg.norm(k, axis=-1, keepdims=True)
    ones = np.ones((T, dk))
    # beta = 1 and no decay: after writing (k_t, v_t) the state returns v_t for the query k_t (the rule overwrites what k_t pointed at)
    o, S = O.delta_rule(k, k, v, np.ones(T), ones)
    assert np.allclose(o, v)
    # beta = 0: nothing is ever written
    assert np.allclose(O.delta_rule(q, k, v, np.zeros(T), ones)[0], 0.0)
    # the state carries: two halves equal the whole; the decay acts on the rows that belong to key channels
    dec = rng.random((T, dk)) * 0.5 + 0.5
    beta = rng.random(T)
    whole, S_all = O.delta_rule(q, k, v, beta, dec)
    first, S1 = O.delta_rule(q[:7], k[:7], v[:7], beta[:7], dec[:7])
    second, S2 = O.delta_rule(q[7:], k[7:], v[7:], beta[7:], dec[7:], state=S1)
    assert np.allclose(np.concatenate([first, second]), whole) and np.allclose(S2, S_all)
    one, S_one = O.delta_rule(q[:1], k[:1], v[:1], beta[:1], dec[:1], state=np.ones((dk, dv)))
    kept = dec[0][:, None] * np.ones((dk, dv))
    assert np.allclose(S_one, kept + np.outer(k[0], beta[0] * (v[0] - kept.T @ k[0])))
    # a sink takes weight and gives nothing: with one key the result is v * e^s / (e^s + e^sink)
    qq, kk, vv = rng.standard_normal((1, 1, 4)), rng.standard_normal((1, 1, 4)), rng.standard_normal((1, 1, 2))
    s = float(qq[0, 0] @ kk[0, 0]) * 0.5
    out = O.masked_softmax_attention(qq, kk, vv, 0.5, np.ones((1, 1), bool), sink=np.array([1.25]))
    assert np.allclose(out[0, 0], vv[0, 0] * np.exp(s) / (np.exp(s) + np.exp(1.25)))


def cfg_full():
    return O.config(vocab=37, width=24, eps=1e-4, groups=3, taps=3, embed_scale=0.5, bigram=(19, 5, 3), logit_softcap=8.0, layers=[
        O.parallel_layer(4, 2, 6, 10, 7, 25.0, 4, 2, 5, 3, 2, rank=3, gate_rank=4, scale=0.3, left_scale=0.6, right_scale=0.9, mlp=O.dense(20)),
        O.attention_layer(6, 3, 4, 8, rot_dims=2, rot_base=500.0, scale=0.7, mlp=None),
        O.attention_layer(2, 2, 8, 4, rot_dims=0, mlp=O.dense(12)),
    ])


def test_oracle_is_causal_and_chunks_hide_what_lies_in_front():
    cfg = cfg_full()
    W = {k: v.astype(np.float64) for k, v in O.weights(cfg, 2).items()}
    a, streams = O.forward(cfg, W, [3, 1, 4, 1, 5, 9, 2, 6])
    b, _ = O.forward(cfg, W, [3, 1, 4, 1, 5, 9, 7, 7])
    assert np.allclose(a[:6], b[:6]) and not np.allclose(a[6], b[6]) and len(streams) == 3
    assert np.abs(a).max() < 8.0  # the cap
    # the chunked attention alone: a position sees its own chunk and nothing in front of it
    h = np.random.default_rng(3).standard_normal((25, 24))
    mx = dict(cfg["layers"][0]["mixer"]["left"])
    full = O.chunk_attention(h, W, "l0.mix.left.", mx, 1e-4)
    assert np.allclose(O.chunk_attention(h[10:], W, "l0.mix.left.", mx, 1e-4), full[10:])  # the first chunk cut off: the rest does not notice
    assert not np.allclose(O.chunk_attention(h[9:], W, "l0.mix.left.", mx, 1e-4)[1:], full[10:])  # cut one position earlier: the chunks shift


def write(tmp_path, cfg, W, name="m"):
    O.write_model_dir(str(tmp_path / name), cfg, W)
    return str(tmp_path / name)


def test_reader_maps_every_branch_of_the_schema(tmp_path):
    cfg = cfg_full()
    W = O.weights(cfg, 3)
    b = loader.load_model_dir(write(tmp_path, cfg, W), max_context_length=64)
    assert b.architecture == "Zovolorn" and b.f32_stream and b.tied_embeddings and b.vocab_size == 37 and b.model_dim == 24
    assert b.input_scale == 0.5 and b.logit_soft_cap == 8.0 and b.output_norm.groups == 3 and b.bigram.n == 20 and b.bigram_mul == (5, 3)
    p, a, c = b.layers
    for lw in b.layers:  # no norm in front of a sublayer; a grouped norm behind it; the input convolutions
        assert not lw.pre_mixer_norm.present and not lw.pre_mlp_norm.present and lw.post_mixer_norm.groups == 3 and lw.input_conv_taps == 3
        assert lw.input_conv_mixer.shape == (24, 3)
    # the pair: chunked attention as the main mixer, the delta rule in the dn_* fields
    assert p.mixer_kind == D.MIXER_ATTENTION and p.pair_mixer == D.MIXER_DELTA_NET and p.pair_scales == (0.6, 0.9) and p.dn_channel_decay
    assert (p.num_heads, p.num_groups, p.head_dim, p.value_head_dim) == (4, 2, 6, 6) and p.values_are_keys and p.attention_chunk_size == 10 and not p.use_rope
    assert p.qkv_projection.n == 4 * 6 + 2 * 6 and p.rel_bias.shape == (7, 4) and p.rel_bias_max == 25.0 and p.head_temperature.shape == (4,) and not p.qk_norm_whole
    assert p.query_norm.scales.shape == (6,) and p.sinks is None and not p.has_gate
    assert (p.dn_num_heads, p.dn_num_groups, p.dn_head_dim, p.dn_value_head_dim, p.dn_kernel_size) == (4, 2, 5, 3, 2)
    assert p.dn_in_proj.n == 2 * 2 * 5 + 4 * 3 + 4 + 3 + 4 and p.dn_conv_weights.shape == (2 * 2 * 5 + 4 * 3, 2) and p.dn_dt_bias.shape == (20,)
    assert (p.dn_decay_up.n, p.dn_decay_up.k, p.dn_gate_up.n, p.dn_gate_up.k) == (20, 3, 12, 4) and p.dn_norm_epsilon == pytest.approx(1e-4)
    assert np.array_equal(p.dn_in_proj.weights[20:32], O.bf16_bits(W["l0.mix.right.v"]))  # rows q | k | v | beta | decay down | gate down
    assert np.array_equal(p.dn_in_proj.weights[36:39], O.bf16_bits(W["l0.mix.right.a1"]))
    assert p.hidden_dim == 20 and p.activation == D.ACT_GELU_APPROX and p.up_projection.n == 40 and p.up_projection.out_biases.shape == (40,) and p.post_mlp_norm.groups == 3
    assert np.array_equal(p.up_projection.weights[:20], O.bf16_bits(W["l0.mlp.up"])) and p.down_projection.out_biases is not None and p.input_conv_mlp is not None
    # attention: grouped heads, one norm over the whole projection, interleaved partial rotation, sinks, gate rows behind the values
    assert a.pair_mixer is None and (a.num_heads, a.num_groups, a.head_dim, a.value_head_dim) == (6, 3, 4, 8) and a.qk_norm_whole and a.has_gate and a.rope_interleaved and a.use_rope
    assert a.qkv_projection.n == 6 * 4 + 3 * 4 + 3 * 8 + 6 and a.query_norm.scales.shape == (24,) and a.key_norm.scales.shape == (12,) and a.sinks.shape == (6,)
    assert a.no_mlp and a.input_conv_mlp is None and a.attention_scale == pytest.approx(0.7) and not a.attention_chunk_size and not a.values_are_keys
    assert b.ropes[a.rope_index].head_dim == 2 and b.ropes[a.rope_index].base == 500.0 and not c.use_rope and len(b.ropes) == 1
    spare = dict(W)  # a layer without a dense block whose file still carries the second sublayer's norm and convolution: read, not used
    spare["l1.norm2"], spare["l1.canon2"] = W["l1.norm1"], W["l1.canon1"]
    assert loader.load_model_dir(write(tmp_path, cfg, spare, "spare"), max_context_length=64).layers[1].no_mlp
    d = b.desc()  # the ctypes description carries them
    assert d.bigram_buckets == 19 and d.layers[0].pair_mixer == 1 + D.MIXER_DELTA_NET and d.layers[0].rel_bias_rows == 7 and d.layers[1].qk_norm_whole == 1
    assert d.layers[0].dn_decay_rank == 3 and d.layers[0].dn_gate_rank == 4 and d.output_norm.groups == 3 and d.logit_soft_cap == 8.0
    # no convolution, no table, one group, no cap
    bare = O.config(vocab=37, width=24, layers=[O.attention_layer(2, 1, 4, 4)], taps=1)
    del bare["canon"], bare["norm"]["groups"]
    Wb = O.weights(dict(bare, canon={"taps": 1}), 1)
    del Wb["l0.canon1"]
    b2 = loader.load_model_dir(write(tmp_path, bare, Wb, "bare"), max_context_length=64)
    assert b2.bigram is None and b2.layers[0].input_conv_mixer is None and b2.layers[0].input_conv_taps == 0 and b2.output_norm.groups == 1 and b2.logit_soft_cap == 0.0


def test_reader_refusals(tmp_path):
    def broken(change, name):
        cfg = cfg_full()
        W = O.weights(cfg, 3)
        change(cfg, W)
        return write(tmp_path, cfg, W, name)

    def kind(c, W): c["layers"][1]["type"] = "convolution"
    def moe(c, W): c["layers"][0]["mlp"]["kind"] = "moe"
    def shape(c, W): W["l1.mix.k"] = W["l1.mix.k"][:-1]
    def extra(c, W): W["l1.mix.extra"] = W["l1.mix.q"]
    def missing(c, W): del W["l0.mix.right.A_log"]
    def odd(c, W): c["layers"][1]["mixer"]["rot"]["dims"] = 3
    def wide(c, W): c["layers"][1]["mixer"]["rot"]["dims"] = 6
    def heads(c, W): c["layers"][1]["mixer"]["kv_heads"] = 4
    def delta_heads(c, W): c["layers"][0]["mixer"]["right"]["kv_heads"] = 3
    def values(c, W): c["layers"][0]["mixer"]["left"]["vdim"] = 8
    def near(c, W): c["layers"][0]["mixer"]["left"]["bias_max"] = 3.0
    def groups(c, W): c["norm"]["groups"] = 5
    def width(c, W): c["width"] = 25
    def buckets(c, W): c["embedding"]["bigram"]["buckets"] = 18
    def taps(c, W): c["canon"]["taps"] = 4
    for i, (change, err) in enumerate([(kind, loader.UnsupportedModelError), (moe, loader.UnsupportedModelError), (shape, loader.ModelFormatError), (extra, loader.ModelFormatError),
                                       (missing, loader.ModelFormatError), (odd, loader.ModelFormatError), (wide, loader.ModelFormatError), (heads, loader.ModelFormatError),
                                       (delta_heads, loader.ModelFormatError), (values, loader.ModelFormatError), (near, loader.ModelFormatError), (groups, loader.ModelFormatError),
                                       (width, loader.ModelFormatError), (buckets, loader.ModelFormatError), (taps, loader.ModelFormatError)]):
        with pytest.raises(err):
            loader.load_model_dir(broken(change, f"bad{i}"), max_context_length=64)


def test_what_the_writer_writes_reads_back(tmp_path):
    cfg = zovolorn.config(37, 16, [
        zovolorn.parallel_layer(2, 1, 8, 12, 6, 30.0, 2, 1, 4, 8, 3, rank=2, left_scale=0.6, right_scale=0.9, mlp=zovolorn.dense_mlp(8)),
        zovolorn.attention_layer(2, 1, 8, 4, rot_dims=4, mlp=None)], groups=2, taps=2, embed_scale=0.25, bigram=(11, 3, 2), logit_softcap=5.0)
    T = zovolorn.random_tensors(cfg, seed=4)
    zovolorn.save(str(tmp_path / "w"), cfg, T)
    on_disk = json.load(open(os.path.join(str(tmp_path / "w"), "config.json")))
    assert on_disk["architecture"] == "Zovolorn" and "rel_rows" not in on_disk["layers"][0]["mixer"]["left"]
    b = loader.load_model_dir(str(tmp_path / "w"), max_context_length=32)
    assert len(b.layers) == 2 and b.layers[0].pair_mixer == D.MIXER_DELTA_NET and b.layers[0].rel_bias.shape == (6, 2) and b.logit_soft_cap == 5.0
    assert np.array_equal(b.embedding.weights, O.bf16_bits(T["embed"]))
    # the oracle reads what the writer wrote
    assert O.forward(on_disk, {k: v.astype(np.float64) for k, v in T.items()}, [1, 2, 3])[0].shape == (3, 37)
