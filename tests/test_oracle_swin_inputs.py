"""Pins the closed-form Swin side inputs against the constructive definitions."""
import numpy as np
import pytest
import torch

from oracle import swin_inputs as si


def _painted_mask(R, ws, shift):
    """Label image painted region by region, cut into windows, compared pairwise."""
    img = np.zeros((R, R))
    spans = ((0, R - ws), (R - ws, R - shift), (R - shift, R))
    label = 0
    for r0, r1 in spans:
        for c0, c1 in spans:
            img[r0:r1, c0:c1] = label
            label += 1
    g = R // ws
    out = np.zeros((g * g, ws * ws, ws * ws))
    for wr in range(g):
        for wc in range(g):
            tile = img[wr * ws:(wr + 1) * ws, wc * ws:(wc + 1) * ws].reshape(-1)
            out[wr * g + wc] = np.where(tile[None, :] - tile[:, None] != 0, -100.0, 0.0)
    return out


@pytest.mark.parametrize("R,ws,shift", [(32, 8, 4), (64, 8, 4), (128, 16, 8), (14, 7, 3), (24, 12, 6)])
def test_mask_closed_form(R, ws, shift):
    m = si.shifted_window_mask(R, ws, shift).numpy()
    np.testing.assert_array_equal(m, _painted_mask(R, ws, shift))
    g = R // ws
    assert m.shape == (g * g, ws * ws, ws * ws)
    assert set(np.unique(m)) <= {0.0, -100.0}
    np.testing.assert_array_equal(m, m.transpose(0, 2, 1))
    assert np.all(np.diagonal(m, axis1=1, axis2=2) == 0)
    nonzero = [w for w in range(g * g) if m[w].any()]
    assert len(nonzero) == 2 * g - 1
    assert all((w // g == g - 1) or (w % g == g - 1) for w in nonzero)


def test_relative_position_index():
    wh, ww = 4, 3
    idx = si.relative_position_index(wh, ww).numpy()
    for i in range(wh * ww):
        for j in range(wh * ww):
            dr, dc = i // ww - j // ww, i % ww - j % ww
            assert idx[i, j] == (dr + wh - 1) * (2 * ww - 1) + dc + ww - 1
    assert idx.min() == 0 and idx.max() == (2 * wh - 1) * (2 * ww - 1) - 1
    # i == j hits the table centre
    assert np.all(np.diag(idx) == ((2 * wh - 1) * (2 * ww - 1)) // 2)


def test_relative_coords_table():
    t = si.relative_coords_table(8, 8).numpy()
    assert t.shape == (1, 15, 15, 2)
    edge = np.log2(9.0) / 3.0        # |x| = 8 at the table edge
    assert abs(t[0, 14, 7, 0] - edge) < 1e-6 and abs(t[0, 0, 7, 0] + edge) < 1e-6
    assert abs(t[0, 8, 7, 0] - np.log2(8.0 / 7.0 + 1.0) / 3.0) < 1e-6
    assert t[0, 7, 7].tolist() == [0.0, 0.0]
    np.testing.assert_allclose(t[0, :, :, 0], -t[0, ::-1, :, 0], atol=1e-7)


def test_make_inputs_is_seeded_and_shaped():
    a = si.make_inputs(**si.CONFIGS["C1"], dtype=torch.bfloat16, seed=3)
    b = si.make_inputs(**si.CONFIGS["C1"], dtype=torch.bfloat16, seed=3)
    assert a["q"].shape == (32, 4, 64, 32) and a["mask"].shape == (16, 64, 64) and a["bias"].shape == (4, 64, 64)
    for key in a:
        assert torch.equal(a[key], b[key])
    assert float(a["bias"].min()) > 0 and float(a["bias"].max()) < 16.01
    assert abs(float(a["logit_scale"][0]) - 2.296875) < 1e-6  # ln 10 rounded to bf16
