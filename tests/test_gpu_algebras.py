"""GPU parity of the other algebras (REAL, COMPLEX, GA_300), which run as compositions on the quaternion kernels
(phoenix_core_amd/algebras.py): the reference's known-answer vectors (tests/golden/reference_kats.json, from
tests/tests.cpp:224-290, 371-423, 562-648) exactly, and forward / backward passes of random problems against the
oracle's generic path, which walks the reference's sign tables.  Tolerances as in test_gpu_parity.py."""
import json
import os

import numpy as np
import pytest
import torch

import oracle
import phoenix_core_amd as phx
from phoenix_core_amd import algebras

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-4, torch.float16: 2e-2}
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


class Ctx(phx.Context):
    def __init__(self, mode, policy="fp32"):
        env = {"UPSTRIDE_CONV_FP16_POLICY": policy}
        if mode == 16:
            env["UPSTRIDE_MEMORY_OPTIMIZED"] = "1"
        super().__init__(env)


def close(got, want, dtype, what):
    got = got.astype(np.float64)
    assert got.shape == want.shape, what
    d = np.abs(got - want)
    e_max = d.max() / max(np.abs(want).max(), 1e-30)
    e_l2 = np.sqrt((d ** 2).sum()) / max(np.sqrt((want ** 2).sum()), 1e-30)
    assert np.isfinite(got).all(), what
    assert e_max <= TOL[dtype] and e_l2 <= TOL[dtype], "%s: rel max %.3e, rel l2 %.3e" % (what, e_max, e_l2)


@pytest.mark.parametrize("mode", [8, 16])
@pytest.mark.parametrize("kat", [k for k in KATS["conv2d"] if k["algebra"] != phx.QUATERNION], ids=lambda k: k["name"])
def test_reference_conv_vectors(kat, mode):
    d = algebras.DIMS[kat["algebra"]]
    x = torch.tensor(kat["input"], dtype=torch.float32, device="cuda").reshape(d * kat["n"], kat["ci"], kat["h"], kat["w"])
    w = torch.tensor(kat["filter"], dtype=torch.float32, device="cuda").reshape(d, kat["co"], kat["ci"], kat["kh"], kat["kw"])
    desc = phx.Conv2DDescriptor(x.shape, w.shape, 1, 1, kat["padding"], algebra=kat["algebra"], context=Ctx(mode))
    y = phx.conv2d_fwd(x, w, None, desc)
    assert y.flatten().tolist() == [float(v) for v in kat["output"]]


@pytest.mark.parametrize("mode", [8, 16])
@pytest.mark.parametrize("kat", KATS["dense"], ids=lambda k: k["name"])
def test_reference_dense_vectors(kat, mode):
    d = algebras.DIMS[kat["algebra"]]
    x = torch.tensor(kat["input"], dtype=torch.float32, device="cuda").reshape(d * kat["n"], kat["ni"])
    w = torch.tensor(kat["filter"], dtype=torch.float32, device="cuda").reshape(d, kat["ni"], kat["no"])
    desc = phx.DenseDescriptor(x.shape, w.shape, algebra=kat["algebra"], context=Ctx(mode))
    y = phx.dense_fwd(x, w, None, desc)
    assert y.flatten().tolist() == [float(v) for v in kat["output"]]


# n, ci, co, h, w, kh, kw, stride, dilation, padding
SHAPES = [
    (2, 5, 7, 9, 11, 1, 1, 1, 1, "VALID"),
    (2, 6, 4, 10, 13, 3, 3, 1, 1, "SAME"),
    (1, 3, 8, 15, 14, 3, 3, 2, 1, "SAME"),
    (3, 4, 4, 8, 9, 3, 2, (1, 2), (2, 1), (2, 0, 1, 3)),
    # batches of 2 (above) and 4, 8: COMPLEX and REAL run in place on paired / quadrupled images (csrc/phx_algebra.hip);
    # odd batches take the embedding with zero components
    (4, 6, 4, 10, 13, 3, 3, 1, 1, "SAME"),
    (8, 16, 24, 12, 12, 1, 1, 1, 1, "VALID"),
    (4, 5, 9, 11, 9, 3, 3, 2, 1, "SAME"),
]


@pytest.mark.parametrize("dtype,policy", [(torch.float32, "fp32"), (torch.float16, "full16")], ids=["f32", "f16"])
@pytest.mark.parametrize("mode", [8, 16])
@pytest.mark.parametrize("shape", SHAPES, ids=lambda s: "n%d_k%dx%d_%dx%d" % (s[0], s[5], s[6], s[3], s[4]))
@pytest.mark.parametrize("algebra", [phx.REAL, phx.COMPLEX, phx.GA_300], ids=["real", "complex", "ga300"])
def test_conv_against_the_sign_tables(algebra, shape, mode, dtype, policy):
    n, ci, co, h, w, kh, kw, stride, dilation, padding = shape
    d = algebras.DIMS[algebra]
    r = np.random.default_rng(100 * algebra + kh * kw + h)
    npdt = np.float32 if dtype == torch.float32 else np.float16
    scale = 1.0 if dtype == torch.float32 else 0.5
    g = oracle.make_geom(n, ci, co, h, w, kh, kw, stride, dilation, padding)
    x = (scale * r.standard_normal((d * n, ci, h, w))).astype(npdt)
    wt = (scale * r.standard_normal((d, co, ci, kh, kw)) * np.sqrt(2.0 / (ci * kh * kw))).astype(npdt)
    b = (scale * r.standard_normal((d, co))).astype(npdt)
    gr = (scale * r.standard_normal((d * n, co, g.ho, g.wo))).astype(npdt)
    real = algebra == phx.REAL  # a real filter / bias has no blade axis
    w_dev, b_dev = (wt[0], b[0]) if real else (wt, b)
    desc = phx.Conv2DDescriptor(x.shape, w_dev.shape, stride, dilation, padding, algebra=algebra, use_bias=True,
                                dtype=dtype, context=Ctx(mode, policy))
    assert desc.output_shape == gr.shape
    xd, wd, bd, gd = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (x, w_dev, b_dev, gr))
    y = phx.conv2d_fwd(xd, wd, bd, desc)
    dw, dx = phx.conv2d_bwd(xd, wd, gd, desc)
    x64, w64, b64, g64 = (a.astype(np.float64) for a in (x, wt, b, gr))
    want_y = oracle.conv2d_fwd(g, x64, w64, b64, "generic", algebra=algebra)
    want_dw, want_dx = oracle.conv2d_bwd(g, x64, w64, g64, "generic", algebra=algebra)
    close(y.cpu().numpy(), want_y, dtype, "fwd")
    close(dx.cpu().numpy(), want_dx, dtype, "dgrad")
    got_dw = dw.cpu().numpy()
    close(got_dw[None] if real else got_dw, want_dw, dtype, "wgrad")


@pytest.mark.parametrize("dtype,policy", [(torch.float32, "fp32"), (torch.float16, "full16")], ids=["f32", "f16"])
@pytest.mark.parametrize("n", [7, 8])
@pytest.mark.parametrize("algebra", [phx.REAL, phx.COMPLEX, phx.GA_300], ids=["real", "complex", "ga300"])
def test_dense_against_the_sign_tables(algebra, n, dtype, policy):
    d = algebras.DIMS[algebra]
    r = np.random.default_rng(200 + algebra)
    ni, no = 33, 20
    npdt = np.float32 if dtype == torch.float32 else np.float16
    scale = 1.0 if dtype == torch.float32 else 0.5
    x = (scale * r.standard_normal((d * n, ni))).astype(npdt)
    wt = (r.uniform(-1, 1, (d, ni, no)) * np.sqrt(6.0 / (ni + no))).astype(npdt)
    b = (scale * r.standard_normal((d, no))).astype(npdt)
    gr = (scale * r.standard_normal((d * n, no))).astype(npdt)
    real = algebra == phx.REAL
    w_dev, b_dev = (wt[0], b[0]) if real else (wt, b)
    desc = phx.DenseDescriptor(x.shape, w_dev.shape, algebra=algebra, use_bias=True, dtype=dtype, context=Ctx(8, policy))
    xd, wd, bd, gd = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (x, w_dev, b_dev, gr))
    y = phx.dense_fwd(xd, wd, bd, desc)
    dw, dx = phx.dense_bwd(xd, wd, gd, desc)
    x64, w64, b64, g64 = (a.astype(np.float64) for a in (x, wt, b, gr))
    want_y = oracle.dense_fwd(x64, w64, b64, "generic", algebra=algebra)
    want_dw, want_dx = oracle.dense_bwd(x64, w64, g64, "generic", algebra=algebra)
    close(y.cpu().numpy(), want_y, dtype, "dense fwd")
    close(dx.cpu().numpy(), want_dx, dtype, "dense dgrad")
    got_dw = dw.cpu().numpy()
    close(got_dw[None] if real else got_dw, want_dw, dtype, "dense wgrad")


@pytest.mark.parametrize("mode", [8, 16])
@pytest.mark.parametrize("layout,filt,fshape", [("OHWI", [1, 1, 1, 0, 0, 2], (2, 1, 1, 3)), ("HWIO", [1, 0, 1, 0, 1, 2], (1, 1, 3, 2))],
                         ids=["ohwi_tests.cpp:440-487", "hwio_tests.cpp:492-547"])
def test_reference_real_channels_last_vectors_as_written(layout, filt, fshape, mode):
    """tests/tests.cpp:440-487 and :492-547 of the reference exactly as they are written there: Algebra::REAL, a 2x2
    image with 3 channels in NHWC, a 1x1 filter with 2 output channels in OHWI / HWIO -> (0,2, 2,4, 3,6, 5,8)."""
    x = [0, -1, 1, 0, 0, 2, 0, 0, 3, 1, 0, 4]
    want = [0, 2, 2, 4, 3, 6, 5, 8]
    for dtype in (torch.float32, torch.float16):
        xd = torch.tensor(x, dtype=dtype, device="cuda").reshape(1, 2, 2, 3)
        wd = torch.tensor(filt, dtype=dtype, device="cuda").reshape(fshape)
        desc = phx.Conv2DDescriptor(xd.shape, wd.shape, 1, 1, "VALID", algebra=phx.REAL, filter_layout=layout, dtype=dtype,
                                    context=Ctx(mode, "full16"), data_format="NHWC")
        assert desc.output_shape == (1, 2, 2, 2)
        y = phx.conv2d_fwd(xd, wd, None, desc)
        assert y.flatten().tolist() == [float(v) for v in want], (layout, mode, dtype)


# name, data format, filter layout, groups
LAYOUTS = [("nhwc_ohwi", "NHWC", "OHWI", 1), ("nchw_hwio", "NCHW", "HWIO", 1), ("nchw_oihw_g2", "NCHW", "OIHW", 2),
           ("nhwc_ohwi_g2", "NHWC", "OHWI", 2), ("nhwc_hwio_g3", "NHWC", "HWIO", 3)]


@pytest.mark.parametrize("dtype,policy", [(torch.float32, "fp32"), (torch.float16, "full16")], ids=["f32", "f16"])
@pytest.mark.parametrize("n", [2, 3, 4])
@pytest.mark.parametrize("variant", LAYOUTS, ids=lambda v: v[0])
@pytest.mark.parametrize("algebra", [phx.REAL, phx.COMPLEX, phx.GA_300], ids=["real", "complex", "ga300"])
def test_conv_layouts_and_groups_against_the_sign_tables(algebra, variant, n, dtype, policy):
    """Channels-last activations, OHWI / HWIO filters and channel groups in the other algebras, as the reference's
    generic path takes them for every algebra (src/conv2d.hpp:237-275; groups go to its scalar convolutions,
    src/backend/onednn/conv2d.hpp:116-137): against the oracle's generic path, group by group, on permuted arrays.
    Batches of 2 and 4 run COMPLEX (and 4: REAL) in place on grouped images, 3 takes the embedding."""
    _, data_format, layout, G = variant
    d = algebras.DIMS[algebra]
    h, w, kh, kw, stride, padding = 9, 7, 3, 3, 1, "SAME"
    ci = 6 if G != 3 else 9
    co = 4 if G == 1 else 2 * G
    cig, cog = ci // G, co // G
    r = np.random.default_rng(1000 * algebra + 10 * G + n)
    npdt = np.float32 if dtype == torch.float32 else np.float16
    scale = 1.0 if dtype == torch.float32 else 0.5
    g = oracle.make_geom(n, cig, cog, h, w, kh, kw, stride, 1, padding)
    x = (scale * r.standard_normal((d * n, ci, h, w))).astype(npdt)
    wt = (scale * r.standard_normal((d, co, cig, kh, kw)) * np.sqrt(2.0 / (cig * kh * kw))).astype(npdt)
    b = (scale * r.standard_normal((d, co))).astype(npdt)
    gr = (scale * r.standard_normal((d * n, co, g.ho, g.wo))).astype(npdt)
    x64, w64, b64, g64 = (a.astype(np.float64) for a in (x, wt, b, gr))
    want_y, want_dx, want_dw = np.empty(gr.shape), np.empty(x.shape), np.empty(wt.shape)
    for k in range(G):
        ic, oc = slice(k * cig, (k + 1) * cig), slice(k * cog, (k + 1) * cog)
        xs, ws, bs, gs = (np.ascontiguousarray(a) for a in (x64[:, ic], w64[:, oc], b64[:, oc], g64[:, oc]))
        want_y[:, oc] = oracle.conv2d_fwd(g, xs, ws, bs, "generic", algebra=algebra)
        want_dw[:, oc], want_dx[:, ic] = oracle.conv2d_bwd(g, xs, ws, gs, "generic", algebra=algebra)
    act = (lambda a: np.ascontiguousarray(a.transpose(0, 2, 3, 1))) if data_format == "NHWC" else np.ascontiguousarray
    act_back = (lambda a: a.transpose(0, 3, 1, 2)) if data_format == "NHWC" else (lambda a: a)
    fperm = {"OIHW": (0, 1, 2, 3, 4), "OHWI": (0, 1, 3, 4, 2), "HWIO": (0, 3, 4, 2, 1)}[layout]
    finv = np.argsort(fperm)
    real = algebra == phx.REAL  # a real filter / bias has no blade axis
    w_l = np.ascontiguousarray(wt.transpose(fperm))
    w_dev, b_dev = (w_l[0], b[0]) if real else (w_l, b)
    desc = phx.Conv2DDescriptor(act(x).shape, w_dev.shape, stride, 1, padding, groups=G, algebra=algebra, filter_layout=layout,
                                use_bias=True, dtype=dtype, context=Ctx(8, policy), data_format=data_format)
    assert desc.output_shape == act(gr).shape
    xd, wd, bd, gd = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (act(x), w_dev, b_dev, act(gr)))
    y = phx.conv2d_fwd(xd, wd, bd, desc)
    dw, dx = phx.conv2d_bwd(xd, wd, gd, desc)
    close(act_back(y.cpu().numpy()), want_y, dtype, "fwd")
    close(act_back(dx.cpu().numpy()), want_dx, dtype, "dgrad")
    got_dw = dw.cpu().numpy()
    close((got_dw[None] if real else got_dw).transpose(finv), want_dw, dtype, "wgrad")


@pytest.mark.parametrize("n", [7, 8])
@pytest.mark.parametrize("algebra", [phx.REAL, phx.COMPLEX, phx.GA_300], ids=["real", "complex", "ga300"])
def test_dense_output_major_filters(algebra, n):
    """Dense filters in OI layout ([blade, out, in]) in the other algebras."""
    d = algebras.DIMS[algebra]
    r = np.random.default_rng(300 + algebra)
    ni, no = 19, 12
    x = r.standard_normal((d * n, ni)).astype(np.float32)
    wt = (r.uniform(-1, 1, (d, ni, no)) * np.sqrt(6.0 / (ni + no))).astype(np.float32)
    b = r.standard_normal((d, no)).astype(np.float32)
    gr = r.standard_normal((d * n, no)).astype(np.float32)
    real = algebra == phx.REAL
    w_oi = np.ascontiguousarray(wt.transpose(0, 2, 1))
    w_dev, b_dev = (w_oi[0], b[0]) if real else (w_oi, b)
    desc = phx.DenseDescriptor(x.shape, w_dev.shape, algebra=algebra, filter_layout="OI", use_bias=True, context=Ctx(8))
    assert desc.output_shape == gr.shape
    xd, wd, bd, gd = (torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in (x, w_dev, b_dev, gr))
    y = phx.dense_fwd(xd, wd, bd, desc)
    dw, dx = phx.dense_bwd(xd, wd, gd, desc)
    x64, w64, b64, g64 = (a.astype(np.float64) for a in (x, wt, b, gr))
    want_y = oracle.dense_fwd(x64, w64, b64, "generic", algebra=algebra)
    want_dw, want_dx = oracle.dense_bwd(x64, w64, g64, "generic", algebra=algebra)
    close(y.cpu().numpy(), want_y, torch.float32, "dense fwd")
    close(dx.cpu().numpy(), want_dx, torch.float32, "dense dgrad")
    got_dw = dw.cpu().numpy()
    close((got_dw[None] if real else got_dw).transpose(0, 2, 1), want_dw, torch.float32, "dense wgrad")
