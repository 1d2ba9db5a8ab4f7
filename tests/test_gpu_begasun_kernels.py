"""The kernels Begasun added to the f32-stream designs, each alone through the one-sequence C entries of csrc/capi_stream32.hip, against the float64 oracle's statement
of the same mechanism: the gated linear recurrent unit (both forms, against each other and against the recurrence; rows around the 32-row pieces; state and
convolution window carried through portions of many sizes; a far input that only the state carries; decays next to 1; NaN state ignored at position 0), the
latent append with a rotated key part (both pairings, far positions, both cache precisions), the post norm that joins a sublayer to the stream (with and without the
layer scale and the next sublayer's norm), and the per-head norm in front of the rotation."""
import ctypes as C

import numpy as np
import pytest

import begasun_oracle as O
from uzu_amd import _ffi

pytestmark = pytest.mark.gpu

f32 = lambda a: np.ascontiguousarray(a, dtype=np.float32)
ptr = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
u32, f32c = C.c_uint32, C.c_float


def tables(positions, dims, base, scaling=None):
    """cos / sin [positions][dims], both halves filled, as the engine's rotation tables"""
    f, mag = O.rotation_table(dims, base, scaling)
    ang = np.arange(positions, dtype=np.float64)[:, None] * f[None, :]
    return f32(np.concatenate([np.cos(ang), np.cos(ang)], axis=1) * mag), f32(np.concatenate([np.sin(ang), np.sin(ang)], axis=1) * mag)


def lru_weights(w, blocks, taps, seed, lam=(-3.0, 4.0)):
    rng = np.random.default_rng(seed)
    bw = w // blocks
    return {"conv": O.to_bf16(rng.standard_normal((w, taps)) * 0.6), "conv.b": O.to_bf16(rng.standard_normal(w) * 0.1),
            "ra": O.to_bf16(rng.standard_normal((blocks, bw, bw)) * 1.5 / np.sqrt(bw)), "ri": O.to_bf16(rng.standard_normal((blocks, bw, bw)) * 1.5 / np.sqrt(bw)),
            "ra.b": O.to_bf16(rng.standard_normal((blocks, bw)) * 0.3), "ri.b": O.to_bf16(rng.standard_normal((blocks, bw)) * 0.3),
            "lam": O.to_bf16(lam[0] + lam[1] * (rng.random(w) - 0.5))}


def lru_oracle(W, branches):
    """branches [T, 2 w] (gate branch | recurrent branch) -> S * gelu(gate branch) for the whole sequence from position 0"""
    w = W["lam"].size
    blocks = W["ra"].shape[0]
    x = O.f64(branches)
    u = O.causal_conv(x[:, w:], O.f64(W["conv"]), W["conv.b"])
    ub = u.reshape(-1, blocks, w // blocks)
    r = O.sigmoid(np.einsum("tbi,boi->tbo", ub, O.f64(W["ra"])) + O.f64(W["ra.b"])[None]).reshape(-1, w)
    i = O.sigmoid(np.einsum("tbi,boi->tbo", ub, O.f64(W["ri"])) + O.f64(W["ri.b"])[None]).reshape(-1, w)
    return O.gated_linear_recurrence(u, r, i, W["lam"]) * O.gelu_tanh(x[:, :w])


def lru(ctx, W, branches, state, conv_state, start, form):
    w, taps = W["lam"].size, W["conv"].shape[1]
    blocks = W["ra"].shape[0]
    rows = branches.shape[0]
    gate_w = np.ascontiguousarray(np.concatenate([O.bf16_bits(W["ra"]), O.bf16_bits(W["ri"])], axis=1))
    gate_b = f32(np.concatenate([W["ra.b"], W["ri.b"]], axis=1))
    st, cs, out = f32(state).copy(), f32(conv_state).copy(), np.empty((rows, w), dtype=np.float32)
    _ffi.call("uzu_hip_s32_gated_lru", ctx._h, ptr(f32(branches)), ptr(f32(W["conv"])), ptr(f32(W["conv.b"])), ptr(gate_w), ptr(gate_b), ptr(f32(W["lam"])), f32c(8.0), ptr(st), ptr(cs),
              ptr(out), u32(rows), u32(start), u32(w), u32(blocks), u32(taps), u32(form))
    return out, st, cs


def fresh_state(w, taps, fill=np.nan):
    return np.full(w, fill, dtype=np.float32), np.full((max(taps - 1, 1), w), fill, dtype=np.float32)


@pytest.mark.parametrize("shape", [(24, 3, 4), (7, 7, 5), (40, 1, 1), (64, 2, 2), (300, 4, 3)])
def test_recurrent_unit_forms_against_the_recurrence(hip_ctx, shape):
    w, blocks, taps = shape
    W = lru_weights(w, blocks, taps, seed=w)
    rng = np.random.default_rng(1)
    for rows in (1, 2, 31, 32, 33, 64, 65, 200):  # on both sides of the pieces' borders
        x = f32(rng.standard_normal((rows, 2 * w)))
        want = lru_oracle(W, x)
        got = {form: lru(hip_ctx, W, x, *fresh_state(w, taps), 0, form) for form in (0, 1, 2)}  # (NaN state: position 0 must not read it)
        for form, (out, st, cs) in got.items():
            assert np.abs(out - want).max() < 2e-5 * max(np.abs(want).max(), 1.0), (rows, form)
            assert np.isfinite(st).all()
            if taps > 1:  # the window behind the rows: the last taps - 1 inputs of the recurrent branch, zeros in front of position 0
                tail = np.concatenate([np.zeros((taps - 1, w), dtype=np.float32), x[:, w:]])[-(taps - 1):]
                assert np.array_equal(cs, tail), (rows, form)
        assert np.abs(got[1][0] - got[2][0]).max() < 2e-5 * max(np.abs(want).max(), 1.0)
        assert np.abs(got[1][1] - got[2][1]).max() < 2e-5


@pytest.mark.parametrize("taps", [1, 2, 4])
def test_recurrent_unit_carries_state_and_window_through_portions(hip_ctx, taps):
    """1000 positions with slow decays in portions of 64 / 1 / 2 / 200 / ... rows: only the state carries position 3 to the end, only the window carries the
    convolution across a cut (also across several one-row portions in a row, where the window shifts by one)."""
    w, blocks = 48, 3
    W = lru_weights(w, blocks, taps, seed=9, lam=(-9.0, 1.0))
    rng = np.random.default_rng(2)
    x = f32(rng.standard_normal((1000, 2 * w)))
    want = lru_oracle(W, x)
    x2 = x.copy()
    x2[3, w:] += 6.0
    assert np.abs(lru_oracle(W, x2)[-1] - want[-1]).max() > 3e-3 * np.abs(want[-1]).max(), "the oracle itself does not carry the input: slow the decays"
    for force in (0, 2):
        st, cs = fresh_state(w, taps)
        outs, at = [], 0
        for n in (64, 1, 2, 200, 33, 31, 1, 1, 1, 1, 300, 365):
            form = force if n >= 2 or force == 0 else 1
            out, st, cs = lru(hip_ctx, W, x[at:at + n], st, cs, at, form)
            outs.append(out)
            at += n
        assert at == 1000
        assert np.abs(np.concatenate(outs) - want).max() < 3e-5 * np.abs(want).max(), force


def test_recurrent_unit_decays_next_to_one(hip_ctx):
    """lambda very negative: a = 1 - O(1e-5), where 1 - a^2 in f32 would lose most of its digits"""
    w, blocks, taps = 32, 2, 3
    W = lru_weights(w, blocks, taps, seed=4, lam=(-13.0, 2.0))
    x = f32(np.random.default_rng(3).standard_normal((300, 2 * w)))
    want = lru_oracle(W, x)
    for form in (1, 2):
        out, _, _ = lru(hip_ctx, W, x, *fresh_state(w, taps), 0, form)
        assert np.abs(out - want).max() < 3e-5 * np.abs(want).max(), form


@pytest.mark.parametrize("interleaved", [1, 0])
@pytest.mark.parametrize("bf16", [0, 1])
@pytest.mark.parametrize("start", [0, 900])
def test_latent_append_with_a_rotated_key_part(hip_ctx, interleaved, bf16, start):
    H, dim, rd, rank, rows, eps = 3, 6, 4, 12, 70, 1e-5
    scaling = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.5}
    rng = np.random.default_rng(5)
    x = f32(rng.standard_normal((rows, H * (dim + rd) + rank + rd)))
    scales = f32(1.0 + 0.3 * rng.standard_normal(rank))
    cs, sn = tables(start + rows, rd, 5000.0, scaling)
    old = f32(rng.standard_normal((start + rows, rank + rd)))
    cache = old.copy()
    qlat = np.empty((rows, H, rank + rd), dtype=np.float32)
    _ffi.call("uzu_hip_s32_latent_rope_append", hip_ctx._h, ptr(x), ptr(scales), f32c(eps), ptr(cs), ptr(sn), ptr(cache), ptr(qlat), u32(bf16), u32(interleaved), u32(start), u32(rows),
              u32(H), u32(dim + rd), u32(rank), u32(rd))
    pos = np.arange(start, start + rows)
    down = O.f64(x[:, H * (dim + rd):])
    want_c = O.norm_plain(down[:, :rank], scales, eps)
    want_k = O.rotate(down[:, rank:], pos, rd, 5000.0, scaling, bool(interleaved))
    q = O.f64(x[:, :H * (dim + rd)]).reshape(rows, H, dim + rd)
    want_q = O.rotate(q[:, :, dim:], pos, rd, 5000.0, scaling, bool(interleaved))
    # a bf16 cache rounds every number once (2^-9 of it); f32 tables at position 900: the angle itself carries 1e-5
    close = lambda got, want: bool((np.abs(got - want) <= (2.0 ** -8 * np.abs(want) + 1e-6 if bf16 else 1e-4)).all())
    assert close(cache[start:, :rank], want_c) and close(cache[start:, rank:], want_k)
    keep = O.to_bf16(old[:start]) if bf16 else old[:start]
    assert np.array_equal(cache[:start], keep)  # rows of earlier positions are not touched
    assert np.abs(qlat[:, :, rank:] - want_q).max() < 1e-4 and np.isnan(qlat[:, :, :rank]).all()  # the folded key projection fills the other columns


@pytest.mark.parametrize("d", [37, 2048 + 5])
@pytest.mark.parametrize("with_scale", [False, True])
@pytest.mark.parametrize("with_next", [False, True])
def test_post_norm_joins_the_stream_and_leaves_the_next_norm(hip_ctx, d, with_scale, with_next):
    rng = np.random.default_rng(d)
    rows, eps, eps2 = 5, 1e-5, 1e-3
    y, res = f32(rng.standard_normal((rows, d)) * 3.0), f32(rng.standard_normal((rows, d)))
    w, ls, w2 = f32(0.2 * rng.standard_normal(d)), f32(0.5 + rng.random(d)) if with_scale else None, f32(0.2 * rng.standard_normal(d))
    out, nxt = np.empty((rows, d), dtype=np.float32), np.empty((rows, d), dtype=np.float32) if with_next else None
    _ffi.call("uzu_hip_s32_rms_norm_add", hip_ctx._h, ptr(y), ptr(res), ptr(out), ptr(w), f32c(1.0), ptr(ls), f32c(eps), u32(rows), u32(d), ptr(nxt), ptr(w2) if with_next else None,
              f32c(1.0), f32c(eps2))
    want = O.f64(res) + O.norm_one_plus(O.f64(y), w, eps) * (O.f64(ls) if with_scale else 1.0)
    assert np.abs(out - want).max() < 2e-6 * np.abs(want).max()
    if with_next:
        assert np.abs(nxt - O.norm_one_plus(want, w2, eps2)).max() < 5e-6 * 4.0


@pytest.mark.parametrize("rope", [0, 6, 12])
def test_head_norms_in_front_of_the_rotation(hip_ctx, rope):
    H, G, dim, rows, start, eps = 4, 2, 12, 40, 17, 1e-4
    rng = np.random.default_rng(rope)
    x = f32(rng.standard_normal((rows, (H + G) * dim)) * 2.0)
    qn, kn = f32(1.0 + 0.5 * rng.standard_normal(dim)), f32(1.0 + 0.5 * rng.standard_normal(dim))
    cs, sn = tables(start + rows, rope, 1e4) if rope else (None, None)
    got = x.copy()
    _ffi.call("uzu_hip_s32_rotate_normed", hip_ctx._h, ptr(got), ptr(cs), ptr(sn), ptr(qn), ptr(kn), f32c(eps), u32(rows), u32(start), u32(H), u32(G), u32(dim), u32(rope))
    pos = np.arange(start, start + rows)
    q = O.norm_plain(O.f64(x[:, :H * dim]).reshape(rows, H, dim), qn, eps)
    k = O.norm_plain(O.f64(x[:, H * dim:]).reshape(rows, G, dim), kn, eps)
    if rope:
        q, k = O.rotate(q, pos, rope, 1e4, None, False), O.rotate(k, pos, rope, 1e4, None, False)
    want = np.concatenate([q.reshape(rows, -1), k.reshape(rows, -1)], axis=1)
    assert np.abs(got - want).max() < 2e-5
    only_q = x.copy()  # one of the two norms alone
    _ffi.call("uzu_hip_s32_rotate_normed", hip_ctx._h, ptr(only_q), ptr(cs), ptr(sn), ptr(qn), None, f32c(eps), u32(rows), u32(start), u32(H), u32(G), u32(dim), u32(rope))
    k_raw = O.f64(x[:, H * dim:]).reshape(rows, G, dim)
    if rope:
        k_raw = O.rotate(k_raw, pos, rope, 1e4, None, False)
    assert np.abs(only_q[:, H * dim:] - k_raw.reshape(rows, -1)).max() < 2e-5 and np.abs(only_q[:, :H * dim] - q.reshape(rows, -1)).max() < 2e-5
