"""Pins the rotary-embedding oracle (oracle/rope_oracle.c) without the GPU.

The reference holds no stored vectors for this step: its test compares the CUDA kernels with the
torch expressions of refs.py live, unseeded, at atol 5e-3 (reference: test/kernels.py:76-96).  The
pins here are (i) the reference's own torch call sequence (polar / view_as_complex, refs.py:19-27 and
37-47) evaluated in float64, a code path that shares nothing with the oracle's C loops, (ii) known
answers and invariants the mathematics fixes, each chosen so that a wrong sign, a wrong pairing, a
wrong exponent or an off-by-one position fails it, and (iii) committed golden vectors."""
import math
import os

import numpy as np
import pytest
import torch

import oracle

IL, NEOX = oracle.ROPE_INTERLEAVED, oracle.ROPE_NEOX


def torch_complex_rope(style, x, rotary_dim, start_pos, base):
    """The reference's formulation (complex multiplication by exp(i*theta)) in float64."""
    x = torch.as_tensor(x, dtype=torch.float64)
    L = x.shape[1]
    f = torch.arange(rotary_dim // 2, dtype=torch.float64)
    f = base ** (-2.0 * f / rotary_dim)
    ang = (torch.arange(L, dtype=torch.float64) + start_pos)[:, None] * f[None, :]
    rot = torch.polar(torch.ones_like(ang), ang)[None, :, None, :]
    y = x.clone()
    if style == IL:
        xc = torch.view_as_complex(x[..., :rotary_dim].reshape(*x.shape[:-1], rotary_dim // 2, 2).contiguous())
        y[..., :rotary_dim] = torch.view_as_real(xc * rot).flatten(-2)
    else:
        h = rotary_dim // 2
        xc = torch.view_as_complex(torch.stack([x[..., :h], x[..., h:rotary_dim]], dim=-1).contiguous())
        yr = torch.view_as_real(xc * rot)
        y[..., :h] = yr[..., 0]
        y[..., h:rotary_dim] = yr[..., 1]
    return y.numpy()


@pytest.mark.parametrize("style", [IL, NEOX])
@pytest.mark.parametrize("shape,rd,start,base", [
    ((2, 7, 3, 16), 16, 0, 1e4), ((1, 5, 2, 32), 8, 2048, 1e6), ((3, 4, 1, 128), 64, 100000, 5e5), ((1, 1, 4, 64), 2, 7, 10.0),
])
def test_matches_complex_formulation(style, shape, rd, start, base):
    x = np.random.default_rng(1).standard_normal(shape).astype(np.float32)
    got = oracle.rope(style, x, rd, start, base)
    want = torch_complex_rope(style, x, rd, start, base)
    assert np.abs(got - want).max() < 1e-6     # float32 storage of a float64 result
    assert np.array_equal(got[..., rd:], x[..., rd:])   # the tail is untouched bit for bit


def test_known_answers():
    # pair 0 has frequency 1: x = (1, 0) at position p becomes (cos p, sin p); x = (0, 1) becomes (-sin p, cos p)
    for style in (IL, NEOX):
        x = np.zeros((1, 4, 1, 8), np.float32)
        i1 = 1 if style == IL else 4      # partner of element 0 (rotary_dim 8)
        x[..., 0] = 1.0
        y = oracle.rope(style, x, 8, 3, 1e4)
        for l in range(4):
            assert y[0, l, 0, 0] == pytest.approx(math.cos(3 + l), abs=1e-7)
            assert y[0, l, 0, i1] == pytest.approx(math.sin(3 + l), abs=1e-7)
        x[:] = 0.0
        x[..., i1] = 1.0
        y = oracle.rope(style, x, 8, 3, 1e4)
        assert y[0, 2, 0, 0] == pytest.approx(-math.sin(5), abs=1e-7) and y[0, 2, 0, i1] == pytest.approx(math.cos(5), abs=1e-7)
    # the last pair of rotary_dim 8 at base 1e4 has frequency 1e4^(-6/8); a unit vector there turns by pos * that
    x = np.zeros((1, 1, 1, 8), np.float32)
    x[..., 6] = 1.0                        # interleaved pair 3 = elements (6, 7)
    y = oracle.rope(IL, x, 8, 1000, 1e4)
    th = 1000 * 1e4 ** (-0.75)
    assert y[0, 0, 0, 6] == pytest.approx(math.cos(th), abs=1e-7) and y[0, 0, 0, 7] == pytest.approx(math.sin(th), abs=1e-7)
    x[:] = 0.0
    x[..., 3] = 1.0                        # NeoX pair 3 = elements (3, 7)
    y = oracle.rope(NEOX, x, 8, 1000, 1e4)
    assert y[0, 0, 0, 3] == pytest.approx(math.cos(th), abs=1e-7) and y[0, 0, 0, 7] == pytest.approx(math.sin(th), abs=1e-7)


def test_invariants():
    rng = np.random.default_rng(2)
    x = rng.standard_normal((2, 6, 3, 32)).astype(np.float32)
    for style in (IL, NEOX):
        # position 0 is the identity; pair norms are preserved; base 1 turns every pair by the position
        y0 = oracle.rope(style, x[:, :1], 32, 0, 1e4)
        assert np.array_equal(y0, x[:, :1])
        y = oracle.rope(style, x, 32, 11, 1e4)
        pairs = (lambda a: a.reshape(2, 6, 3, 16, 2)) if style == IL else (lambda a: np.stack([a[..., :16], a[..., 16:]], -1))
        assert np.allclose((pairs(y) ** 2).sum(-1), (pairs(x) ** 2).sum(-1), atol=1e-5)
        yb = oracle.rope(style, x, 32, 5, 1.0)
        for l in range(6):
            c, s = math.cos(5 + l), math.sin(5 + l)
            px, py = pairs(x)[:, l], pairs(yb)[:, l]
            assert np.allclose(py[..., 0], c * px[..., 0] - s * px[..., 1], atol=1e-5)
            assert np.allclose(py[..., 1], s * px[..., 0] + c * px[..., 1], atol=1e-5)
        # rotations compose: rope at start a, then again at start b on a length-1 sequence, is rope at a + b
        x1 = x[:, :1]
        assert np.allclose(oracle.rope(style, oracle.rope(style, x1, 32, 300, 1e4), 32, 45, 1e4),
                           oracle.rope(style, x1, 32, 345, 1e4), atol=1e-5)
        # token l at start s equals token 0 at start s + l
        assert np.allclose(y[:, 4:5], oracle.rope(style, x[:, 4:5], 32, 15, 1e4), atol=1e-6)
    # the two styles are the same rotation under the permutation (2i, 2i+1) <-> (i, i + rd/2)
    perm = np.concatenate([np.arange(0, 32, 2), np.arange(1, 32, 2)])
    assert np.allclose(oracle.rope(IL, x, 32, 9, 1e4)[..., perm], oracle.rope(NEOX, x[..., perm], 32, 9, 1e4), atol=1e-6)


def test_kv_append_is_rope_plus_scatter():
    rng = np.random.default_rng(3)
    B, L, Hq, Hkv, D, Lmax, rd = 3, 5, 4, 2, 16, 12, 8
    q = rng.standard_normal((B, L, Hq, D)).astype(np.float32)
    k = rng.standard_normal((B, L, Hkv, D)).astype(np.float32)
    v = rng.standard_normal((B, L, Hkv, D)).astype(np.float32)
    kc = rng.standard_normal((B, Hkv, Lmax, D)).astype(np.float32)
    vc = rng.standard_normal((B, Hkv, Lmax, D)).astype(np.float32)
    pos = np.array([0, 7, 9], np.int32)      # sequence 2 runs past the end of the cache (rows 12, 13 dropped)
    for style in (IL, NEOX):
        q2, kc2, vc2 = oracle.rope_kv_append(style, q, k, v, pos, kc, vc, rd, 1e4)
        for b in range(B):
            assert np.array_equal(q2[b:b + 1], oracle.rope(style, q[b:b + 1], rd, int(pos[b]), 1e4))
            kr = oracle.rope(style, k[b:b + 1], rd, int(pos[b]), 1e4)[0]        # [L, Hkv, D]
            n = min(L, Lmax - int(pos[b]))
            assert np.array_equal(kc2[b, :, pos[b]:pos[b] + n], kr[:n].transpose(1, 0, 2))
            assert np.array_equal(vc2[b, :, pos[b]:pos[b] + n], v[b, :n].transpose(1, 0, 2))
            untouched = np.ones(Lmax, bool)
            untouched[pos[b]:pos[b] + n] = False
            assert np.array_equal(kc2[b][:, untouched], kc[b][:, untouched])
            assert np.array_equal(vc2[b][:, untouched], vc[b][:, untouched])


def test_bad_arguments():
    x = np.zeros((1, 1, 1, 8), np.float32)
    for args in ((IL, x, 7, 0, 1e4), (IL, x, 10, 0, 1e4), (5, x, 8, 0, 1e4), (IL, x, 8, 0, 0.0)):
        with pytest.raises(ValueError):
            oracle.rope(*args)


def test_golden_vectors():
    path = os.path.join(os.path.dirname(__file__), "golden", "rope_small.npz")
    z = np.load(path)
    for style, name in ((IL, "il"), (NEOX, "neox")):
        got = oracle.rope(style, z["x"], int(z["rotary_dim"]), int(z["start_pos"]), float(z["freq_base"]))
        assert np.abs(got - z[f"y_{name}"]).max() < 1e-6
