"""The torch-CPU restatement used as bench.py's cpu_baseline against the C oracle."""
import numpy as np
import pytest
import torch

import oracle
from oracle import torch_cpu_path as tcp


@pytest.mark.parametrize("mode", ["factorized", "generic"])
@pytest.mark.parametrize("cfg", [dict(kh=1, kw=1, padding="VALID"), dict(kh=3, kw=3, padding="SAME"),
                                 dict(kh=3, kw=3, padding="SAME", stride=2, h=9, w=9)])
def test_torch_cpu_path_matches_oracle(cfg, mode):
    r = np.random.default_rng(3)
    kw = dict(n=2, ci=5, co=6, h=8, w=8, stride=1, dilation=1)
    kw.update(cfg)
    g = oracle.make_geom(**kw)
    if g.pt != g.pb or g.pl != g.pr:
        pytest.skip("asymmetric padding not on the timed path")
    x = r.standard_normal((4 * g.n, g.ci, g.h, g.w)).astype(np.float32)
    w = r.standard_normal((4, g.co, g.ci, g.kh, g.kw)).astype(np.float32)
    b = r.standard_normal((4, g.co)).astype(np.float32)
    gr = r.standard_normal((4 * g.n, g.co, g.ho, g.wo)).astype(np.float32)
    y = tcp.conv2d_fwd(g, torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b), mode).numpy()
    dw, dx = tcp.conv2d_bwd(g, torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(gr), mode)
    want_y = oracle.conv2d_fwd(g, x, w, b, "hamilton")
    want_dw, want_dx = oracle.conv2d_bwd(g, x, w, gr, "hamilton")
    for got, want in ((y, want_y), (dw.numpy(), want_dw), (dx.numpy(), want_dx)):
        assert np.abs(got - want).max() / np.abs(want).max() < 1e-5


@pytest.mark.parametrize("mode", ["factorized", "generic"])
@pytest.mark.parametrize("shape", [(3, 5, 7), (32, 128, 128)])
@pytest.mark.parametrize("use_bias", [False, True])
def test_torch_cpu_dense_path_matches_oracle(shape, mode, use_bias):
    """The Dense port (8 / 16 scalar matmuls by torch's CPU backend + lane maps) against the C oracle in fp64,
    ragged sizes and the benchmark's 32 x 128 -> 128 layer."""
    n, ni, no = shape
    r = np.random.default_rng(11)
    x = r.standard_normal((4 * n, ni)).astype(np.float32)
    w = r.standard_normal((4, ni, no)).astype(np.float32)
    b = r.standard_normal((4, no)).astype(np.float32) if use_bias else None
    gr = r.standard_normal((4 * n, no)).astype(np.float32)
    tb = torch.from_numpy(b) if use_bias else None
    y = tcp.dense_fwd(torch.from_numpy(x), torch.from_numpy(w), tb, mode).numpy()
    dw, dx = tcp.dense_bwd(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(gr), mode)
    want_y = oracle.dense_fwd(x, w, b, "generic")
    want_dw, want_dx = oracle.dense_bwd(x, w, gr, "generic")
    for got, want in ((y, want_y), (dw.numpy(), want_dw), (dx.numpy(), want_dx)):
        assert got.shape == want.shape
        assert np.abs(got - want).max() / np.abs(want).max() < 2e-5
    dw2, dx2 = tcp.dense_bwd(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(gr), mode, need_dx=False)
    assert dx2 is None and torch.equal(dw2, dw)
