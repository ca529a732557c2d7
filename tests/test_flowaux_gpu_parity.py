"""GPU parity of the quadratic-fit and median layers against the CPU oracle, through the Python
binding modules (which call the C ABI).

Bars: everything a pixel computes on its own -- both outputs of both forward passes, the gradient
wrt the first feature map, the gradient wrt the histogram -- must be BIT-EQUAL to the oracle.  The
gradient wrt the second feature map is a scatter with float atomics whose summation order is
undefined: max |difference| <= 1e-5 * max |reference| (a few ulps of the largest sum)."""
import numpy as np
import pytest
import torch

from customnetworklayers_amd import workloads

pytestmark = pytest.mark.gpu

SCATTER_TOL = 1e-5


@pytest.fixture(scope="module")
def qf():
    from customnetworklayers_amd.cudaQuadFit import QuadFit_cuda_ext

    return QuadFit_cuda_ext


@pytest.fixture(scope="module")
def med():
    from customnetworklayers_amd.cudaMedian import median_cuda_ext

    return median_cuda_ext


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def random_quadfit(n, c, h, w, seed, fc=2, amp=3.0):
    """Unstructured features and a large random flow: collisions, out-of-image pixels, both branches."""
    rng = np.random.default_rng(seed)
    return dict(feat0=rng.standard_normal((n, c, h, w)).astype(np.float32),
                feat1=rng.standard_normal((n, c, h, w)).astype(np.float32),
                flow=(amp * rng.standard_normal((n, fc, h, w))).astype(np.float32),
                grad=rng.standard_normal((n, 3, h, w)).astype(np.float32))


def check_quadfit(qf, o, d, name):
    print("case", name, flush=True)
    (out,) = qf.forward(dev(d["feat0"]), dev(d["feat1"]), dev(d["flow"]))
    out = out.cpu().numpy()
    rout = o.quadfit_forward(d["feat0"], d["feat1"], d["flow"])
    r0, r1 = o.quadfit_backward(d["grad"], d["feat0"], d["feat1"], d["flow"])
    assert np.array_equal(out, rout)
    for path, atomics in (("gather", False), ("atomic scatter", True)):
        g0, g1 = qf.backward(dev(d["grad"]), dev(d["feat0"]), dev(d["feat1"]), dev(d["flow"]), use_atomics=atomics)
        g0, g1 = g0.cpu().numpy(), g1.cpu().numpy()
        e1 = np.abs(g1 - r1).max() / max(np.abs(r1).max(), 1e-30)
        print("[%s, %s] out bit-equal %.4f, g0 bit-equal %.4f, g1 rel err %.2e; valid x %.2f, outside %.2f"
              % (name, path, (out == rout).mean(), (g0 == r0).mean(), e1, (rout[:, 0] != 0).mean(),
                 (rout[:, 2] == 0).mean()), flush=True)
        assert np.array_equal(g0, r0)
        assert e1 <= SCATTER_TOL
    return out


@pytest.mark.parametrize("n,c,h,w,fc", [
    (1, 4, 9, 11, 2),       # tiny
    (2, 5, 33, 70, 3),      # odd sizes, three flow channels, two samples
    (1, 32, 64, 128, 2),    # many channels: the backward pass keeps every channel's taps in registers, all 32 in use
    (1, 31, 37, 140, 2),    # one channel short of that
    (1, 33, 40, 130, 2),    # one channel too many for it: the second map is read twice
    (3, 7, 17, 300, 2),     # several blocks per row
    (1, 1, 1, 1, 2),        # a single pixel
    (1, 3, 1, 200, 2),      # a single row
    (1, 3, 150, 1, 2),      # a single column
    (1, 1, 12, 70, 2),      # fewer channels than the backward gather's ring of windows holds
    (2, 2, 12, 70, 2),
    (1, 6, 20, 66, 2),      # a channel count that ends in the middle of the ring
])
def test_quadfit_random_inputs_match_oracle(qf, flowaux_oracle, n, c, h, w, fc):
    d = random_quadfit(n, c, h, w, seed=n * 100 + c + h + w, fc=fc)
    check_quadfit(qf, flowaux_oracle, d, "random %dx%dx%dx%d fc=%d" % (n, c, h, w, fc))


@pytest.mark.parametrize("n,c,h,w", [(2, 8, 96, 160), (1, 16, 50, 333), (1, 32, 70, 200),
                                     (1, 32, 384, 1248)])  # one sample of the benchmark's shape: every block of the chip busy at once
def test_quadfit_warped_features_match_oracle(qf, flowaux_oracle, n, c, h, w):
    d = workloads.quadfit_inputs(n, c, h, w, seed=3)
    out = check_quadfit(qf, flowaux_oracle, d, "warped %dx%dx%dx%d" % (n, c, h, w))
    assert (out[:, 0] != 0).mean() > 0.2  # a good share of valid fits


@pytest.mark.parametrize("n,c,h,w", [(2, 6, 40, 90), (1, 3, 9, 200)])
def test_quadfit_one_pixel_per_lane_kernels(qf, flowaux_oracle, n, c, h, w, monkeypatch):
    # INPAINT_QUADFIT_PATH=px: the kernels without LDS windows (a lane reads its taps from memory)
    monkeypatch.setenv("INPAINT_QUADFIT_PATH", "px")
    from customnetworklayers_amd._lib import reload_env
    reload_env()  # the switches are read once per process
    check_quadfit(qf, flowaux_oracle, random_quadfit(n, c, h, w, seed=31 + c), "px path random %dx%dx%dx%d" % (n, c, h, w))
    check_quadfit(qf, flowaux_oracle, workloads.quadfit_inputs(n, c, h, w, seed=32), "px path warped")


@pytest.mark.parametrize("c", [4, 32, 40])
def test_quadfit_flow_that_scatters_the_tile(qf, flowaux_oracle, c):
    # a flow that varies by tens of pixels inside one tile: most taps fall outside the LDS window
    d = random_quadfit(1, c, 64, 256, seed=33, amp=40.0)
    check_quadfit(qf, flowaux_oracle, d, "scattered, %d channels" % c)


@pytest.mark.parametrize("n,c,h,w", [(2, 6, 40, 90), (1, 32, 33, 150)])
def test_quadfit_backward_that_reads_the_second_map_twice(qf, flowaux_oracle, n, c, h, w, monkeypatch):
    # INPAINT_QUADFIT_PATH=reread: the backward kernel of more than 32 channels, forced for fewer
    monkeypatch.setenv("INPAINT_QUADFIT_PATH", "reread")
    from customnetworklayers_amd._lib import reload_env
    reload_env()
    check_quadfit(qf, flowaux_oracle, random_quadfit(n, c, h, w, seed=41 + c), "reread random %dx%dx%dx%d" % (n, c, h, w))
    check_quadfit(qf, flowaux_oracle, workloads.quadfit_inputs(n, c, h, w, seed=42), "reread warped")


def test_quadfit_non_finite_displacements_count_as_outside(qf, flowaux_oracle):
    d = random_quadfit(1, 3, 20, 70, seed=34)
    d["flow"][0, 0, 3, 5] = np.nan
    d["flow"][0, 1, 4, 6] = np.nan
    d["flow"][0, 0, 5, 7] = np.inf
    d["flow"][0, 1, 6, 8] = -np.inf
    out = check_quadfit(qf, flowaux_oracle, d, "non-finite flow")
    for y, x in ((3, 5), (4, 6), (5, 7), (6, 8)):
        assert (out[0, :, y, x] == 0).all()


def test_quadfit_all_pixels_collide(qf, flowaux_oracle):
    # every pixel is sent to one target: its list overflows, and 5 addresses per channel take every atomic
    n, c, h, w = 1, 3, 40, 70
    d = random_quadfit(n, c, h, w, seed=5)
    ys, xs = np.mgrid[0:h, 0:w]
    d["flow"] = np.stack([30 - xs, 20 - ys])[None].astype(np.float32)
    check_quadfit(qf, flowaux_oracle, d, "collide")


def test_quadfit_several_pixels_per_target(qf, flowaux_oracle):
    # the flow folds the image onto itself: two to six pixels land on most targets (lists with several
    # entries, some overflowing), none on others
    n, c, h, w = 2, 5, 30, 64
    d = random_quadfit(n, c, h, w, seed=6)
    ys, xs = np.mgrid[0:h, 0:w]
    fold_x = (xs // 3) * 1.0 + 10 - xs
    fold_y = (ys // 2) * 1.0 + 5 - ys
    d["flow"] = np.broadcast_to(np.stack([fold_x, fold_y])[None], (n, 2, h, w)).astype(np.float32).copy()
    check_quadfit(qf, flowaux_oracle, d, "folded")


def test_quadfit_outputs_are_overwritten_not_accumulated(qf, flowaux_oracle):
    d = random_quadfit(1, 4, 20, 30, seed=8)
    a = qf.backward(dev(d["grad"]), dev(d["feat0"]), dev(d["feat1"]), dev(d["flow"]))
    b = qf.backward(dev(d["grad"]), dev(d["feat0"]), dev(d["feat1"]), dev(d["flow"]))
    assert torch.equal(a[0], b[0])
    assert (a[1] - b[1]).abs().max().item() <= SCATTER_TOL * a[1].abs().max().item()


def test_quadfit_module_and_autograd(qf, flowaux_oracle):
    from customnetworklayers_amd import QuadFittingFromFlow, QuadFittingFromFlowFunction

    d = workloads.quadfit_inputs(1, 6, 24, 40, seed=2, flow_channels=3)
    f0, f1 = dev(d["feat0"]).requires_grad_(True), dev(d["feat1"]).requires_grad_(True)
    sol = QuadFittingFromFlowFunction.apply(f0, f1, dev(d["flow"]))
    (sol * dev(d["grad"])).sum().backward()
    r0, r1 = flowaux_oracle.quadfit_backward(d["grad"], d["feat0"], d["feat1"], d["flow"])
    assert np.array_equal(f0.grad.cpu().numpy(), r0)
    assert np.abs(f1.grad.cpu().numpy() - r1).max() <= SCATTER_TOL * np.abs(r1).max()
    layer = QuadFittingFromFlow(torch.device("cuda:0"))
    hwc = layer(dev(d["feat0"][0].transpose(1, 2, 0)), dev(d["feat1"][0].transpose(1, 2, 0)),
                dev(d["flow"][0].transpose(1, 2, 0)))
    assert tuple(hwc.shape) == (24, 40, 3)
    assert np.array_equal(hwc.cpu().numpy().transpose(2, 0, 1), sol.detach().cpu().numpy()[0])


def test_quadfit_errors(qf):
    d = random_quadfit(1, 2, 6, 7, seed=1)
    f0, f1, fl = dev(d["feat0"]), dev(d["feat1"]), dev(d["flow"])
    with pytest.raises(RuntimeError):
        qf.forward(f0.cpu(), f1, fl)
    with pytest.raises(TypeError):
        qf.forward(f0.double(), f1, fl)
    with pytest.raises(ValueError):
        qf.forward(f0, f1[:, :1].contiguous(), fl)
    with pytest.raises(ValueError):
        qf.forward(f0, f1, fl[:, :1].contiguous())
    with pytest.raises(RuntimeError):
        qf.forward(f0, f1, fl.transpose(2, 3))
    with pytest.raises(ValueError):
        qf.backward(dev(d["grad"])[:, :2].contiguous(), f0, f1, fl)


# ------------------------------------------------------------------------------------------------
# median
# ------------------------------------------------------------------------------------------------
def check_median(med, o, vol, grad, name):
    print("case", name, flush=True)
    (out,) = med.forward(dev(vol))
    (g,) = med.backward(dev(grad), dev(vol))
    out, g = out.cpu().numpy(), g.cpu().numpy()
    rout, rg = o.median_forward(vol), o.median_backward(grad, vol)
    print("[%s] out bit-equal %.4f, grad bit-equal %.4f; no crossing at %.3f of the pixels"
          % (name, (out == rout).mean(), (g == rg).mean(), (rout[:, 1] == 0).mean()), flush=True)
    assert np.array_equal(out, rout)
    assert np.array_equal(g, rg)


@pytest.mark.parametrize("n,h,w,d", [
    (1, 5, 7, 9),
    (2, 16, 20, 33),     # one bin more than a staged chunk
    (1, 9, 31, 32),      # exactly one chunk
    (1, 9, 31, 31),
    (1, 3, 100, 1),      # a single bin
    (2, 13, 40, 64),     # two full chunks
    (1, 7, 50, 100),     # four chunks, the last one ragged
    (3, 1, 1, 5),        # fewer pixels than one wavefront
    (1, 64, 65, 21),     # pixel count not a multiple of the block
    (1, 6, 9, 255),      # the most bins the whole-histogram kernels take
    (1, 6, 9, 300),      # beyond: the chunked kernels
    (2, 5, 7, 2),
    (1, 10, 13, 3),
    (1, 37, 41, 39),     # the most bins the streaming kernel takes; full tiles and a partial one
    (2, 30, 33, 5),      # the fewest
    (3, 7, 11, 21),      # tiles of 64 pixels that straddle samples
    (2, 50, 77, 33),
])
def test_median_matches_oracle(med, flowaux_oracle, n, h, w, d):
    m = workloads.median_inputs(n, h, w, d, seed=n + h + w + d, empty_fraction=0.1)
    check_median(med, flowaux_oracle, m["vol"], m["grad"], "%dx%dx%dx%d" % (n, h, w, d))


@pytest.mark.parametrize("n,h,w,d", [(2, 16, 20, 33), (1, 9, 31, 31), (3, 7, 11, 21)])
def test_median_one_tile_per_wavefront_when_forced(med, flowaux_oracle, n, h, w, d, monkeypatch):
    # odd bin counts up to 39 normally stream their full tiles through a loop that keeps the next tile's loads in flight;
    # INPAINT_MEDIAN_PATH=tile keeps the one-tile-per-wavefront kernel (every other bin count's path) covered for them
    from customnetworklayers_amd._lib import reload_env

    m = workloads.median_inputs(n, h, w, d, seed=n + h + w + d, empty_fraction=0.1)
    monkeypatch.setenv("INPAINT_MEDIAN_PATH", "tile")
    reload_env()
    try:
        check_median(med, flowaux_oracle, m["vol"], m["grad"], "tile path %dx%dx%dx%d" % (n, h, w, d))
    finally:
        monkeypatch.delenv("INPAINT_MEDIAN_PATH")
        reload_env()


def test_median_buffers_without_16_byte_alignment(med, flowaux_oracle):
    m = workloads.median_inputs(1, 9, 14, 21, seed=9)
    flat = torch.zeros(m["vol"].size + 3, dtype=torch.float32, device="cuda")
    for shift in (1, 2, 3):
        v = flat[shift:shift + m["vol"].size].view(m["vol"].shape)
        v.copy_(dev(m["vol"]))
        (out,) = med.forward(v)
        (g,) = med.backward(dev(m["grad"]), v)
        assert np.array_equal(out.cpu().numpy(), flowaux_oracle.median_forward(m["vol"]))
        assert np.array_equal(g.cpu().numpy(), flowaux_oracle.median_backward(m["grad"], m["vol"]))


def test_median_unnormalised_and_signed_histograms(med, flowaux_oracle):
    # the layer does not require a probability vector: masses above one, negative entries, zeros
    rng = np.random.default_rng(3)
    vol = rng.normal(0.05, 0.2, (2, 11, 23, 40)).astype(np.float32)
    vol[0, :3] = 0.0
    vol[1, :2, :, 0] = 1.5
    grad = rng.standard_normal((2, 2, 11, 23)).astype(np.float32)
    check_median(med, flowaux_oracle, vol, grad, "signed")


def test_median_module_and_autograd(med, flowaux_oracle):
    from customnetworklayers_amd import Median, MedianFunction

    m = workloads.median_inputs(1, 12, 18, 21, seed=4)
    v = dev(m["vol"]).requires_grad_(True)
    sol = MedianFunction.apply(v)
    (sol * dev(m["grad"])).sum().backward()
    assert np.array_equal(v.grad.cpu().numpy(), flowaux_oracle.median_backward(m["grad"], m["vol"]))
    layer = Median(torch.device("cuda:0"))
    hw = layer(dev(m["vol"][0]))
    assert tuple(hw.shape) == (12, 18)
    assert np.array_equal(hw.cpu().numpy(), flowaux_oracle.median_forward(m["vol"])[0, 0])


def test_median_errors(med):
    m = workloads.median_inputs(1, 4, 5, 6, seed=1)
    v = dev(m["vol"])
    with pytest.raises(RuntimeError):
        med.forward(v.cpu())
    with pytest.raises(TypeError):
        med.forward(v.double())
    with pytest.raises(ValueError):
        med.forward(v[0])
    with pytest.raises(ValueError):
        med.backward(dev(m["grad"])[:, :1].contiguous(), v)


def test_full_size_workloads_round_trip_properties(qf, med):
    # at the bench sizes: the fit's offsets stay within one pixel and vanish where no fit is valid; the
    # median lies inside the histogram's support; the median's gradient has the sign pattern -,...,-,*,+,...,+
    cfg, d = workloads.config_inputs(5, seed=1)
    (out,) = qf.forward(dev(d["feat0"]), dev(d["feat1"]), dev(d["flow"]))
    assert out[:, :2].abs().max().item() <= 1.0
    assert torch.isfinite(out).all()
    cfg, m = workloads.config_inputs(6, seed=1)
    v = dev(m["vol"])
    (sol,) = med.forward(v)
    found = sol[:, 1] > 0
    assert (sol[:, 0][found] >= -0.5).all() and (sol[:, 0][found] <= cfg["d"] - 0.5).all()
    gin = torch.zeros_like(sol)
    gin[:, 0] = 1.0
    (g,) = med.backward(gin, v)
    k = torch.floor(sol[:, 0] + 0.5).long().clamp(0, cfg["d"] - 1)
    idx = torch.arange(cfg["d"], device=v.device).view(1, 1, 1, -1)
    before, after = idx < k.unsqueeze(-1), idx > k.unsqueeze(-1)
    sel = found.unsqueeze(-1)
    assert (g[before & sel] <= 0).all() and (g[after & sel] >= 0).all()
