"""Pins the CPU oracle before anything is compared with it.

Checks, chosen so that a dropped term, a wrong sign or index, or a transposed
operand fails at least one of them:
  * the reference's own naive layers (committed vectors in tests/golden/ and,
    where oracle/_ref is built, live calls) -- bit exact;
  * closed forms: all-ones, delta and shift kernels, linearity, zero input;
  * Winograd: per-tile brute force (valid 8x8 (*) 3x3 correlation in float64),
    stage layouts against numpy einsum, edge shapes against the naive conv;
  * im2col: hand-counted index map, agreement with the naive conv.
"""
import os

import numpy as np
import pytest

from oracle import oracle as O

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "naive_ref_vectors.npz")


def _cases():
    z = np.load(GOLD)
    names = sorted({k.split("/")[0] for k in z.files})
    return z, names


def test_golden_vectors_match_reference_naive_layers():
    z, names = _cases()
    assert len(names) == 10
    for name in names:
        s = O.Shape(*[int(v) for v in z[name + "/shape"]])
        x, w, y_ref = z[name + "/x"], z[name + "/w"], z[name + "/y"]
        if name + "/bias_elems" in z.files:
            y = O.naive_conv_f32(s, x, w, np.ascontiguousarray(z[name + "/bias_elems"]), bias_mode=2)
        else:
            y = O.naive_conv_f32(s, x, w)
        assert y.shape == y_ref.shape, name
        assert np.array_equal(y, y_ref), name          # same summation order: bit exact
        y64 = O.naive_conv_f64(s, x, w)
        if name + "/bias_elems" not in z.files:
            assert O.max_rel_err(y_ref, y64) < 2e-6, name


@pytest.mark.skipif(O.ref_lib() is None, reason="oracle/_ref not built (no reference checkout)")
@pytest.mark.parametrize("shape", [
    (1, 64, 56, 56, 64, 3, 3, 1, 1, 1, 1, 1, 1),      # the single-layer case the reference itself runs on a CPU: 64 -> 64 channels at 56x56
    (1, 16, 28, 28, 24, 3, 3, 1, 1, 1, 1, 1, 1),
])
def test_live_reference_naive_3x3(shape):
    s = O.Shape(*shape)
    x, w = O.make_inputs(s, seed=3)
    y = O.naive_conv_f32(s, x, w)
    assert np.array_equal(y, O.ref_naive_3x3s1(s, x, w))
    assert np.array_equal(y, O.ref_naive_general(s, x, w))


@pytest.mark.skipif(O.ref_lib() is None, reason="oracle/_ref not built (no reference checkout)")
@pytest.mark.parametrize("shape", [
    (1, 32, 28, 28, 16, 3, 3, 2, 2, 1, 1, 1, 1),
    (1, 64, 14, 14, 32, 1, 1, 1, 1, 0, 0, 0, 0),
    (1, 3, 32, 32, 8, 7, 7, 2, 2, 3, 3, 3, 3),
])
def test_live_reference_naive_general(shape):
    s = O.Shape(*shape)
    x, w = O.make_inputs(s, seed=4)
    assert np.array_equal(O.naive_conv_f32(s, x, w), O.ref_naive_general(s, x, w))


def test_output_size_formula():
    # conv_layer.h:68-69, hand-evaluated
    assert O.out_hw(O.shape(1, 1, 224, 224, 1, 7, 7, 2, 2, 3)) == (112, 112)
    assert O.out_hw(O.shape(1, 1, 56, 56, 1, 3, 3, 2, 2, 1)) == (28, 28)
    assert O.out_hw(O.shape(1, 1, 56, 56, 1, 1, 1, 2, 2, 0)) == (28, 28)
    assert O.out_hw(O.shape(1, 1, 7, 9, 1, 3, 3, 1, 1, 0)) == (5, 7)
    assert O.out_hw(O.Shape(1, 1, 11, 12, 1, 5, 3, 1, 2, 0, 1, 2, 1)) == (8, 7)


def _taps_in_bounds(s):
    oh, ow = O.out_hw(s)
    cnt = np.zeros((oh, ow))
    for i in range(oh):
        for j in range(ow):
            for u in range(s.kh):
                for v in range(s.kw):
                    h, w_ = i * s.sh - s.pt + u, j * s.sw - s.pl + v
                    cnt[i, j] += (0 <= h < s.H) and (0 <= w_ < s.W)
    return cnt


@pytest.mark.parametrize("shape", [
    (2, 8, 9, 9, 3, 3, 3, 2, 2, 1, 1, 1, 1),
    (1, 5, 12, 10, 2, 3, 3, 1, 1, 1, 1, 1, 1),
    (1, 4, 11, 12, 3, 5, 3, 1, 2, 0, 1, 2, 1),
])
def test_all_ones_closed_form(shape):
    s = O.Shape(*shape)
    x = np.ones((s.N, s.C, s.H, s.W), np.float32)
    w = np.ones((s.K, s.C, s.kh, s.kw), np.float32)
    expect = s.C * _taps_in_bounds(s)
    for y in (O.naive_conv_f32(s, x, w), O.naive_conv_f64(s, x, w), O.im2col_conv_f32(s, x, w)):
        assert np.array_equal(y, np.broadcast_to(expect, y.shape))
    if s.kh == 3 and s.kw == 3 and s.sh == 1:
        assert np.allclose(O.wino_conv_f32(s, x, w), expect, rtol=0, atol=1e-4)
    # by hand for 8 channels, 9x9, stride 2, padding 1: a corner output sees 2x2 taps (32), a centre one 3x3 (72)
    if shape[1] == 8:
        assert expect[0, 0] == 32 and expect[2, 2] == 72


def test_delta_and_shift_kernels():
    s = O.shape(2, 3, 10, 13, 3)
    x, _ = O.make_inputs(s, seed=9)
    for (u, v) in [(1, 1), (0, 0), (2, 1), (1, 2), (0, 2)]:
        w = np.zeros((3, 3, 3, 3), np.float32)
        for k in range(3):
            w[k, k, u, v] = 1.0                    # output k = input k shifted by (u-1, v-1)
        xp = np.pad(x, ((0, 0), (0, 0), (1, 1), (1, 1)))
        expect = xp[:, :, u:u + 10, v:v + 13]
        assert np.array_equal(O.naive_conv_f32(s, x, w), expect)
        assert np.array_equal(O.im2col_conv_f32(s, x, w), expect)
        assert O.max_rel_err(O.wino_conv_f32(s, x, w), expect) < 1e-4   # F(6,3) fp32 rounding


def test_linearity_and_zero():
    s = O.shape(1, 6, 9, 9, 4, 3, 3, 2, 2, 1)
    x1, w = O.make_inputs(s, seed=1)
    x2, _ = O.make_inputs(s, seed=2)
    a = O.naive_conv_f64(s, x1, w) + 2.0 * O.naive_conv_f64(s, x2, w)
    b = O.naive_conv_f64(s, (x1.astype(np.float64) + 2.0 * x2).astype(np.float32), w)
    assert np.allclose(a, b, rtol=0, atol=1e-5)
    assert not O.naive_conv_f32(s, np.zeros_like(x1), w).any()


def test_naive_against_independent_numpy_correlation():
    # an einsum over explicitly gathered windows: no shared code with the oracle
    s = O.Shape(2, 5, 9, 8, 4, 3, 2, 2, 1, 1, 0, 0, 1)
    x, w = O.make_inputs(s, seed=5)
    oh, ow = O.out_hw(s)
    xp = np.pad(x.astype(np.float64), ((0, 0), (0, 0), (s.pt, s.pb), (s.pl, s.pr)))
    win = np.empty((s.N, s.C, oh, ow, s.kh, s.kw))
    for i in range(oh):
        for j in range(ow):
            win[:, :, i, j] = xp[:, :, i * s.sh:i * s.sh + s.kh, j * s.sw:j * s.sw + s.kw]
    expect = np.einsum("ncijuv,kcuv->nkij", win, w.astype(np.float64))
    assert np.allclose(O.naive_conv_f64(s, x, w), expect, rtol=0, atol=1e-12)
    assert O.max_rel_err(O.naive_conv_f32(s, x, w), expect) < 1e-6


# ------------------------------------------------------------------ Winograd

def test_winograd_tile_identity_brute_force():
    BT, G, AT = [m.astype(np.float64) for m in O.wino_matrices()]
    # exact rationals the float tables round from
    G[1] = [-2 / 9, -2 / 9, -2 / 9]; G[2] = [-2 / 9, 2 / 9, -2 / 9]
    G[3] = [1 / 90, 1 / 45, 2 / 45]; G[4] = [1 / 90, -1 / 45, 2 / 45]
    G[5] = [1 / 45, 1 / 90, 1 / 180]; G[6] = [1 / 45, -1 / 90, 1 / 180]
    rng = np.random.default_rng(0)
    for _ in range(5):
        d = rng.standard_normal((8, 8))
        g = rng.standard_normal((3, 3))
        y = AT @ ((G @ g @ G.T) * (BT @ d @ BT.T)) @ AT.T
        brute = np.array([[np.sum(d[i:i + 3, j:j + 3] * g) for j in range(6)] for i in range(6)])
        assert np.allclose(y, brute, rtol=0, atol=1e-10)
    # the float G table is the rounding of those rationals
    assert np.array_equal(O.wino_matrices()[1], G.astype(np.float32))


def test_winograd_stage_layouts():
    s = O.shape(2, 3, 8, 11, 5)                   # OH=8, OW=11 -> 2x2 tiles, clipped edges
    x, w = O.make_inputs(s, seed=11)
    BT, G, AT = [m.astype(np.float64) for m in O.wino_matrices()]
    th, tw = O.tiles_hw(s)
    assert (th, tw) == (2, 2)
    U = O.wino_filter_transform(w)
    Ue = np.einsum("ia,kcab,jb->ijkc", G, w.astype(np.float64), G).reshape(64, s.K, s.C)
    assert np.allclose(U, Ue, rtol=0, atol=1e-6)
    # tiles gathered by hand: origin 6*index - pad, zeros outside the image
    xp = np.zeros((s.N, s.C, th * 6 + 2, tw * 6 + 2))
    xp[:, :, 1:1 + s.H, 1:1 + s.W] = x
    d = np.empty((s.C, s.N, th, tw, 8, 8))
    for a in range(th):
        for b in range(tw):
            d[:, :, a, b] = xp[:, :, a * 6:a * 6 + 8, b * 6:b * 6 + 8].transpose(1, 0, 2, 3)
    Ve = np.einsum("ia,cnxyab,jb->ijcnxy", BT, d, BT).reshape(64, s.C, -1)
    V = O.wino_input_transform(s, x)
    assert np.allclose(V, Ve, rtol=0, atol=1e-4)
    M = O.wino_gemm(U, V)
    Me = np.einsum("fkc,fct->fkt", U.astype(np.float64), V.astype(np.float64))
    assert np.allclose(M, Me, rtol=0, atol=1e-4)
    bias = np.arange(s.K, dtype=np.float32)
    y = O.wino_output_transform(s, M, bias)
    Ye = np.einsum("ia,abknxy,jb->knxiyj", AT, Me.reshape(8, 8, s.K, s.N, th, tw), AT)
    Ye = Ye.reshape(s.K, s.N, th * 6, tw * 6)[:, :, :8, :11].transpose(1, 0, 2, 3)
    Ye = Ye + bias[None, :, None, None]
    assert np.allclose(y, Ye, rtol=0, atol=1e-3)
    assert O.max_rel_err(y, O.naive_conv_f64(s, x, w, bias)) < 1e-5


@pytest.mark.parametrize("hw", [(6, 6), (7, 7), (8, 5), (13, 14), (14, 14), (28, 28), (56, 56)])
@pytest.mark.parametrize("ck", [(1, 1), (3, 7), (64, 6)])
def test_winograd_edge_shapes_against_naive(hw, ck):
    s = O.shape(1, ck[0], hw[0], hw[1], ck[1])
    x, w = O.make_inputs(s, seed=hw[0] * 100 + ck[0])
    truth = O.naive_conv_f64(s, x, w)
    assert O.max_rel_err(O.wino_conv_f32(s, x, w), truth) < 1e-4
    assert O.max_rel_err(O.im2col_conv_f32(s, x, w), truth) < 1e-5


def test_winograd_pad0_and_pad2():
    for pad in (0, 2):
        s = O.shape(2, 4, 12, 9, 3, pt=pad)
        x, w = O.make_inputs(s, seed=pad)
        assert O.max_rel_err(O.wino_conv_f32(s, x, w), O.naive_conv_f64(s, x, w)) < 1e-4


def test_winograd_rejects_other_kernels():
    s = O.shape(1, 2, 8, 8, 2, 3, 3, 2, 2, 1)
    x, w = O.make_inputs(s)
    with pytest.raises(ValueError):
        O.wino_conv_f32(s, x, w)


# -------------------------------------------------------------------- im2col

def test_im2col_index_map_hand_counted():
    # 1 channel, 3x3 image 1..9, 2x2 kernel, stride 1, pad 0 -> rows (u,v), cols (i,j)
    s = O.Shape(1, 1, 3, 3, 1, 2, 2, 1, 1, 0, 0, 0, 0)
    x = np.arange(1, 10, dtype=np.float32).reshape(1, 1, 3, 3)
    assert np.array_equal(O.im2col(s, x), np.array(
        [[1, 2, 4, 5], [2, 3, 5, 6], [4, 5, 7, 8], [5, 6, 8, 9]], np.float32))
    # pad 1, stride 2, 3x3 kernel: output 2x2; row (u=0,v=0) reads x[-1+2i][-1+2j]
    s = O.Shape(1, 1, 3, 3, 1, 3, 3, 2, 2, 1, 1, 1, 1)
    col = O.im2col(s, x)
    assert col.shape == (9, 4)
    assert np.array_equal(col[0], [0, 0, 0, 5])
    assert np.array_equal(col[4], [1, 3, 7, 9])
    assert np.array_equal(col[8], [5, 0, 0, 0])


@pytest.mark.parametrize("shape", [
    (2, 6, 15, 15, 7, 3, 3, 2, 2, 1, 1, 1, 1),
    (1, 16, 7, 7, 9, 1, 1, 1, 1, 0, 0, 0, 0),
    (1, 3, 17, 17, 4, 7, 7, 2, 2, 3, 3, 3, 3),
    (2, 4, 11, 12, 3, 5, 3, 1, 2, 0, 1, 2, 1),
])
def test_im2col_conv_against_naive(shape):
    s = O.Shape(*shape)
    x, w = O.make_inputs(s, seed=21)
    bias = O.rng_uniform(5, (s.K,))
    truth = O.naive_conv_f64(s, x, w, bias)
    assert O.max_rel_err(O.im2col_conv_f32(s, x, w, bias), truth) < 1e-6


# ------------------------------------------------------------------- metrics

def test_diff_legacy_hand_vectors():
    a = np.array([1.0, 2.0, 3.0, 4.0], np.float32)
    b = np.array([1.0, 2.5, 3.0, 3.0], np.float32)
    assert O.diff_legacy(a, b) == pytest.approx(0.75)       # (0.5 + 1.0) / 2
    assert O.diff_legacy(a, a) == 0.0
    c = a + np.float32(5e-6)                                 # below the 1e-5 threshold
    assert O.diff_legacy(a, c) == 0.0


def test_max_rel_err():
    ref = np.array([1.0, -4.0, 2.0])
    y = np.array([1.0, -4.0, 2.5], np.float32)
    assert O.max_rel_err(y, ref) == pytest.approx(0.125)
    assert np.isnan(O.max_rel_err(np.array([np.nan, 1, 1], np.float32), ref)) or \
        O.max_rel_err(np.array([np.nan, 1, 1], np.float32), ref) > 1.0


# ----------------------------------------------------------------------- rng

def _py_xoshiro(seed, n):
    mask = (1 << 64) - 1

    def rotl(v, k):
        return ((v << k) | (v >> (64 - k))) & mask
    st, sm = [], seed
    for _ in range(4):
        sm = (sm + 0x9e3779b97f4a7c15) & mask
        z = sm
        z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & mask
        z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & mask
        st.append(z ^ (z >> 31))
    out = []
    for _ in range(n):
        out.append((rotl((st[1] * 5) & mask, 7) * 9) & mask)
        t = (st[1] << 17) & mask
        st[2] ^= st[0]; st[3] ^= st[1]; st[1] ^= st[2]; st[0] ^= st[3]
        st[2] ^= t
        st[3] = rotl(st[3], 45)
    return out


def test_rng_stream_and_distributions():
    assert [int(v) for v in O.rng_raw(1234567, 6)] == _py_xoshiro(1234567, 6)
    # first splitmix64 output for seed 1234567, as published with the generator
    mask = (1 << 64) - 1
    z = (1234567 + 0x9e3779b97f4a7c15) & mask
    z = ((z ^ (z >> 30)) * 0xbf58476d1ce4e5b9) & mask
    z = ((z ^ (z >> 27)) * 0x94d049bb133111eb) & mask
    assert (z ^ (z >> 31)) == 6457827717110365317
    u = O.rng_uniform(0, (200000,))
    assert u.min() >= -1.0 and u.max() < 1.0
    assert abs(u.mean()) < 0.01 and abs(u.var() - 1.0 / 3.0) < 0.01
    g = O.rng_normal(0, (200001,), 0.5)
    assert abs(g.mean()) < 0.01 and abs(g.std() - 0.5) < 0.01
    assert np.array_equal(O.rng_uniform(7, (100,)), O.rng_uniform(7, (100,)))
    assert not np.array_equal(O.rng_uniform(7, (100,)), O.rng_uniform(8, (100,)))
