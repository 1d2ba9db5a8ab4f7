"""Begasun on the host: identities of the float64 oracle (what the GPU tests lean on), and the config.json reader -- every branch of the schema, the engine
description it produces (layer runs of a loop, packed projections, shared tensors), its refusals, and the writer's round trip.  No GPU."""
import json
import os

import numpy as np
import pytest

import begasun_oracle as O
from uzu_amd import begasun, desc as D, loader

YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.5}


def test_oracle_rotation_pairings_and_scaled_frequencies():
    rng = np.random.default_rng(0)
    x = rng.standard_normal((9, 3, 12))
    pos = np.arange(9) + 5
    inter, half = O.rotate(x, pos, 8, 1e4, None, True), O.rotate(x, pos, 8, 1e4, None, False)
    assert np.allclose(inter[..., 8:], x[..., 8:]) and np.allclose(half[..., 8:], x[..., 8:])  # the tail passes unchanged
    # the two pairings are one rotation under a permutation of the coordinates: (2i, 2i + 1) <-> (i, i + 4)
    perm = [0, 2, 4, 6, 1, 3, 5, 7]
    assert np.allclose(O.rotate(x[..., perm + [8, 9, 10, 11]], pos, 8, 1e4, None, False)[..., :8], inter[..., perm])
    # a rotation keeps the length of every pair; scaled frequencies multiply it by 0.1 ln(factor) + 1
    assert np.allclose((inter[..., 0:2] ** 2).sum(-1), (x[..., 0:2] ** 2).sum(-1))
    f, mag = O.rotation_table(8, 1e4, YARN)
    plain, one = O.rotation_table(8, 1e4, None)
    assert one == 1.0 and np.isclose(mag, 0.1 * np.log(4.0) + 1.0)
    assert np.isclose(f[0], plain[0]) and np.isclose(f[-1], plain[-1] / 4.0) and np.all(f <= plain + 1e-15) and np.all(f >= plain / 4.0 - 1e-15)
    sc = O.rotate(x, pos, 8, 1e4, YARN, True)
    assert np.allclose((sc[..., 0:2] ** 2).sum(-1), (x[..., 0:2] ** 2).sum(-1) * mag ** 2)
    # scores of rotated queries and keys depend on the distance only
    q, k = rng.standard_normal((1, 8)), rng.standard_normal((1, 8))
    s = lambda a, b: float(O.rotate(q, [a], 8, 1e4, YARN, True)[0] @ O.rotate(k, [b], 8, 1e4, YARN, True)[0])
    assert np.isclose(s(10, 3), s(107, 100))


def test_oracle_convolution_and_recurrence():
    rng = np.random.default_rng(1)
    x, taps, bias = rng.standard_normal((20, 5)), rng.standard_normal((5, 4)), rng.standard_normal(5)
    y = O.causal_conv(x, taps, bias)
    assert np.allclose(y[0], bias + taps[:, 3] * x[0])  # zeros in front of the sequence, the last tap weighs the current position
    assert np.allclose(y[7], bias + sum(taps[:, j] * x[7 - 3 + j] for j in range(4)))
    assert np.allclose(O.causal_conv(x, taps[:, 3:], bias), bias + taps[:, 3] * x)  # one tap: a scale
    # constant gates: S_t = sum_j a^(t - j) b u_j
    u = rng.standard_normal((30, 3))
    r, i, lam = np.full((30, 3), 0.5), np.full((30, 3), 0.25), np.array([-2.0, 0.0, 1.0])
    S = O.gated_linear_recurrence(u, r, i, lam)
    a = np.exp(-8.0 * 0.5 * np.log1p(np.exp(lam)))
    direct = sum(a ** (29 - j) * np.sqrt(1 - a * a) * 0.25 * u[j] for j in range(30))
    assert np.allclose(S[29], direct)
    assert np.allclose(S[0], np.sqrt(1 - a * a) * 0.25 * u[0])  # the first token starts from S = 0 like every other


def test_oracle_is_causal_and_the_loop_order():
    cfg = O.config(29, 16, [O.rglru_layer(8, 2, 3, mlp=O.dense(8)), O.latent_layer(2, 4, 2, 4, 6, O.rot(2)), O.attention_layer(2, 1, 4, 4, O.rot(4))], loop=(1, 3, 2), side_dim=3)
    W = {k: v.astype(np.float64) for k, v in O.weights(cfg, 2).items()}
    a, taps = O.forward(cfg, W, [3, 1, 4, 1, 5, 9, 2, 6])
    b, _ = O.forward(cfg, W, [3, 1, 4, 1, 5, 9, 7, 7])
    assert np.allclose(a[:6], b[:6]) and not np.allclose(a[6], b[6])
    assert taps.shape == (5, 8, 16)
    assert O.layer_order(cfg) == [(0, False), (1, True), (2, False), (1, True), (2, False)] == begasun.layer_runs(cfg)
    assert O.layer_order(dict(cfg, loop=None)) == [(0, False), (1, False), (2, False)]
    assert O.layer_order(dict(cfg, loop={"start": 0, "stop": 1, "times": 3})) == [(0, True), (0, True), (0, True), (1, False), (2, False)]


def cfg_full():
    return O.config(vocab=43, width=24, eps=2e-5, embed_scale=3.0, logit_scale=0.5, loop=(1, 3, 2), side_dim=4, layers=[
        O.rglru_layer(12, 3, 4, mlp=None),
        O.latent_layer(3, 4, 6, 5, 10, O.rot(6, 5000.0, YARN), scale=0.4, mlp=O.dense(16, 0.75)),
        O.attention_layer(4, 2, 6, 10, O.rot(4, 100.0), scale=0.3, mlp=O.dense(8, 2.0)),
        O.latent_layer(1, 8, 2, 4, 6, O.rot(2, 100.0), mlp=None),
    ])


def write(tmp_path, cfg, W, name="m"):
    path = str(tmp_path / name)
    O.write_model_dir(path, cfg, W)
    return path


def test_reader_maps_every_branch_of_the_schema(tmp_path):
    cfg = cfg_full()
    W = O.weights(cfg, 3)
    b = loader.load_model_dir(write(tmp_path, cfg, W), max_context_length=64)
    assert b.f32_stream and b.architecture == "Begasun" and not b.tied_embeddings and b.input_scale == 3.0 and b.logit_scale == 0.5
    assert b.output_norm.kind == D.NORM_STATISTICS and b.output_norm.scale_offset == 1.0 and b.output_norm.epsilon == pytest.approx(2e-5)
    assert b.side_dim == 4 and b.side_table.n == 43 and b.side_table.k == 4 * 4
    runs = b.layers
    assert [l.mixer_kind for l in runs] == [D.MIXER_GATED_LRU, D.MIXER_LATENT_ATTENTION, D.MIXER_ATTENTION, D.MIXER_LATENT_ATTENTION, D.MIXER_ATTENTION, D.MIXER_LATENT_ATTENTION]
    assert [l.weights_of_layer for l in runs] == [None, None, None, 1, 2, None]
    assert [l.stream_reentry is not None for l in runs] == [False, True, False, True, False, False] and runs[1].stream_reentry.k == 48
    assert [l.ple_slice for l in runs] == [0, 1, 2, 1, 2, 3] and all(l.ple.ple_dim == 4 and l.ple.norm.scale_offset == 0.0 for l in runs)
    lru = runs[0]
    assert lru.no_mlp and lru.lru_width == 12 and lru.lru_blocks == 3 and lru.dn_kernel_size == 4 and lru.lru_decay_rate == 8.0
    assert lru.qkv_projection.n == 24 and lru.qkv_projection.out_biases.shape == (24,) and lru.out_projection.k == 12
    assert np.array_equal(lru.qkv_projection.weights[12:], O.bf16_bits(W["l0.mix.x"]))  # gate branch first, then the recurrent branch
    assert lru.lru_gate_weights.shape == (3, 8, 4) and np.array_equal(lru.lru_gate_weights[1, 4:], O.bf16_bits(W["l0.mix.ri"][1]))
    assert np.array_equal(lru.lru_gate_biases[2, :4], W["l0.mix.ra.b"][2])
    assert lru.post_mixer_norm.present and lru.post_mixer_norm.scale_offset == 1.0 and np.array_equal(lru.layer_scale_mixer, W["l0.ls1"])
    lat = runs[1]
    assert (lat.num_heads, lat.head_dim, lat.latent_rope_dim, lat.value_head_dim, lat.latent_rank) == (3, 4, 6, 5, 10) and lat.latent_packed and lat.has_gate and lat.rope_interleaved
    assert lat.qkv_projection.n == 3 * 10 + 16 + 3 and lat.attention_scale == pytest.approx(0.4) and lat.latent_norm.scale_offset == 0.0
    assert np.array_equal(lat.qkv_projection.weights[30:46], O.bf16_bits(W["l1.mix.dkv"])) and np.array_equal(lat.qkv_projection.weights[46:], O.bf16_bits(W["l1.mix.g"]))
    assert lat.hidden_dim == 16 and lat.gated_act == (1.702, (float("-inf"), 0.75), (-0.75, 0.75), 1.0) and lat.up_projection.n == 32
    assert np.array_equal(lat.up_projection.weights[:16], O.bf16_bits(W["l1.mlp.up"]))  # [up ; gate]
    assert lat.post_mlp_norm.present and np.array_equal(lat.layer_scale_mlp, W["l1.ls2"])
    att = runs[2]
    assert (att.num_heads, att.num_groups, att.head_dim, att.value_head_dim) == (4, 2, 6, 10) and att.query_norm.present and att.key_norm.scales.shape == (6,) and not att.rope_interleaved
    assert att.qkv_projection.n == 24 + 12 + 20 and att.qkv_projection.out_biases is None
    assert len(b.ropes) == 3 and b.ropes[lat.rope_index].kind == D.ROPE_YARN and b.ropes[att.rope_index].head_dim == 4 and b.ropes[runs[5].rope_index].head_dim == 2
    d = b.desc()  # the ctypes description builds
    assert d.num_layers == 6 and d.has_ple == 1 and d.layers[3].weights_of_layer == 2 and d.layers[1].latent_rope_dim == 6
    # no loop, no token input
    cfg2 = O.config(19, 8, [O.attention_layer(1, 1, 4, 4, O.rot(0))])
    b2 = loader.load_model_dir(write(tmp_path, cfg2, O.weights(cfg2, 1), "plain"), max_context_length=16)
    assert b2.side_table is None and b2.layers[0].ple is None and b2.layers[0].stream_reentry is None and not b2.layers[0].use_rope and b2.ropes is None


def test_reader_refusals(tmp_path):
    def broken(change, name):
        cfg = cfg_full()
        W = O.weights(cfg, 3)
        change(cfg, W)
        return write(tmp_path, cfg, W, name)

    def kind(c, W): c["layers"][3]["type"] = "convolution"
    def moe(c, W): c["layers"][1]["mlp"]["kind"] = "moe"
    def shape(c, W): W["l2.mix.k"] = W["l2.mix.k"][:-1]
    def extra(c, W): W["l3.mix.extra"] = W["l3.mix.q"]
    def missing(c, W): del W["l0.mix.lam"]
    def odd(c, W): c["layers"][2]["mixer"]["rot"]["dims"] = 3
    def rot_part(c, W): c["layers"][1]["mixer"]["rot"]["dims"] = 4
    def groups(c, W): c["layers"][2]["mixer"]["kv_heads"] = 3
    def blocks(c, W): c["layers"][0]["mixer"]["blocks"] = 5
    def loop(c, W): c["loop"]["stop"] = 9
    def width(c, W): c["width"] = 25
    def side(c, W): c["token_side"]["dim"] = 5
    for i, (change, err) in enumerate([(kind, loader.UnsupportedModelError), (moe, loader.UnsupportedModelError), (shape, loader.ModelFormatError), (extra, loader.ModelFormatError),
                                       (missing, loader.ModelFormatError), (odd, loader.ModelFormatError), (rot_part, loader.ModelFormatError), (groups, loader.ModelFormatError),
                                       (blocks, loader.ModelFormatError), (loop, loader.ModelFormatError), (width, loader.ModelFormatError), (side, loader.ModelFormatError)]):
        with pytest.raises(err):
            loader.load_model_dir(broken(change, f"bad{i}"), max_context_length=64)


def test_writer_round_trip(tmp_path):
    cfg = begasun.config(37, 16, [
        begasun.rglru_layer(8, 2, 3, mlp=begasun.dense_mlp(8, limit=2.0)),
        begasun.latent_attention_layer(2, 4, 4, 4, 8, begasun.rotation(4, 1e4, YARN), mlp=None),
        begasun.attention_layer(2, 1, 8, 4, begasun.rotation(4, 1e4), mlp=begasun.dense_mlp(12))], loop=(0, 2, 2), side_dim=3, logit_scale=0.25)
    T = begasun.random_tensors(cfg, seed=4)
    begasun.save(str(tmp_path / "w"), cfg, T)
    assert json.load(open(os.path.join(str(tmp_path / "w"), "config.json")))["architecture"] == "Begasun"
    b = loader.load_model_dir(str(tmp_path / "w"), max_context_length=32)
    assert len(b.layers) == 5 and b.layers[0].mixer_kind == D.MIXER_GATED_LRU and b.layers[0].gated_act[1][1] == 2.0 and b.logit_scale == 0.25
    assert np.array_equal(b.embedding.weights, O.bf16_bits(T["embed"]))
    # the oracle reads what the writer wrote, and its own weight maker names the same tensors with the same shapes
    full = dict(cfg, architecture="Begasun")
    assert O.forward(full, {k: v.astype(np.float64) for k, v in T.items()}, [1, 2, 3])[0].shape == (3, 37)
    mine = O.weights(full, 1)
    assert {k: np.shape(v) for k, v in mine.items()} == {k: np.shape(v) for k, v in T.items()}
