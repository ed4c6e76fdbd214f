"""Pins of the oracle's rotary embedding (a restatement of the Hugging Face function the reference's model
forward calls): it is a plane rotation of the pairs (x[d], x[d + D/2]) by the angle whose cosine and sine
the tables hold."""
import numpy as np

from oracle import blockrank_oracle as orc


def _tables(B, S, D, rng):
    ang = rng.uniform(-np.pi, np.pi, size=(B, S, D // 2))
    ang = np.concatenate([ang, ang], axis=-1)             # the model's tables repeat the D/2 frequencies
    return ang, np.cos(ang), np.sin(ang)


def test_rotation_properties():
    rng = np.random.default_rng(0)
    B, N, S, D = 2, 3, 7, 16
    x = rng.standard_normal((B, N, S, D))
    ang, c, s = _tables(B, S, D, rng)
    y = orc.rotary_embedding(x, c, s)
    h = D // 2
    # the same thing as a complex multiplication of (x1 + i x2) by exp(i angle)
    z = (x[..., :h] + 1j * x[..., h:]) * np.exp(1j * ang[:, None, :, :h])
    np.testing.assert_allclose(y[..., :h], z.real, atol=1e-12)
    np.testing.assert_allclose(y[..., h:], z.imag, atol=1e-12)
    # pair norms are preserved; angle 0 is the identity; rotating back restores x
    np.testing.assert_allclose(y[..., :h] ** 2 + y[..., h:] ** 2, x[..., :h] ** 2 + x[..., h:] ** 2, atol=1e-12)
    np.testing.assert_allclose(orc.rotary_embedding(x, np.ones_like(c), np.zeros_like(s)), x, atol=0)
    np.testing.assert_allclose(orc.rotary_embedding(y, c, -s), x, atol=1e-12)


def test_unit_vector_and_broadcast_table():
    B, N, S, D = 2, 1, 3, 4
    x = np.zeros((B, N, S, D))
    x[..., 0] = 1.0                                         # the pair (x[0], x[2]) = (1, 0)
    ang = np.array([[[0.3, 1.1, 0.3, 1.1], [0.0, 0.5, 0.0, 0.5], [2.0, -1.0, 2.0, -1.0]]])   # one table for the batch
    y = orc.rotary_embedding(x, np.cos(ang), np.sin(ang))
    for b in range(B):
        np.testing.assert_allclose(y[b, 0, :, 0], np.cos(ang[0, :, 0]), atol=1e-15)
        np.testing.assert_allclose(y[b, 0, :, 2], np.sin(ang[0, :, 0]), atol=1e-15)
        assert (y[b, 0, :, 1] == 0).all() and (y[b, 0, :, 3] == 0).all()
