"""GPU parity of the TV layer: the HIP path through the C ABI against the CPU oracle on the same
seeded inputs.

Tolerances (the layer's contract): max-abs error / max-abs oracle value <= 1e-4 on the inpainted
flow and <= 1e-3 on the gradients wrt edge weights, confidence, right-hand side and starting point.
The kernels reproduce the oracle's arithmetic operation by operation, so the observed errors are
far smaller (the forward iterates are expected to agree bit for bit); the tests print them.
"""
import numpy as np
import pytest
import torch

from customnetworklayers_amd.workloads import CONFIGS, tv_inputs

pytestmark = pytest.mark.gpu

OUT_TOL = 1e-4
GRAD_TOL = 1e-3


def rel_err(a, ref):
    return float(np.abs(a.astype(np.float64) - ref.astype(np.float64)).max() / max(np.abs(ref).max(), 1e-30))


@pytest.fixture(scope="module")
def ext():
    from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext

    return tvInpaint_cuda_ext


def run_gpu(ext, d, its, pid, fresh=True):
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    if fresh:
        ext.reset_id(pid)
    (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, pid)
    grads = ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, pid)
    torch.cuda.synchronize()
    return sol.cpu().numpy(), [g.cpu().numpy() for g in grads], t["grad"].cpu().numpy()


def run_oracle(o, d, its, pid, fresh=True):
    if fresh:
        o.reset_id(pid)
    sol = o.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], its, pid)
    gin = d["grad"].copy()
    grads = o.backward(gin, d["dx"], d["dy"], d["dc"], d["db"], its, pid)
    return sol, list(grads), gin


def compare(name, got, ref):
    sol, grads, _ = got
    rsol, rgrads, _ = ref
    e_out = rel_err(sol, rsol)
    errs = [rel_err(g, r) for g, r in zip(grads, rgrads)]
    exact = float((sol == rsol).mean())
    print("\n[%s] out rel %.2e (bit-equal %.4f)  gx %.2e gy %.2e gc %.2e gb %.2e gi %.2e"
          % (name, e_out, exact, *errs), flush=True)
    assert e_out <= OUT_TOL, (name, e_out)
    for nm, e in zip(("gx", "gy", "gc", "gb", "gi"), errs):
        assert e <= GRAD_TOL, (name, nm, e)
    return e_out, errs


@pytest.mark.parametrize("n,c,h,w,its", [
    (1, 2, 64, 128, 20),    # the reference's own single-sample case
    (1, 1, 16, 64, 2),      # a single pair of iterations, tile-exact
    (2, 3, 37, 101, 9),     # ragged tiles, odd its, three channels, two samples
    (1, 2, 5, 3, 6),        # smaller than one tile
    (1, 2, 1, 70, 4),       # a single row
    (1, 1, 33, 1, 4),       # a single column
    (3, 2, 130, 200, 50),   # several segments of unequal length
    (2, 2, 45, 508, 14),    # several strips wide, ragged rows
    (1, 1, 9, 63, 8),       # exactly one forward strip wide
    (1, 2, 11, 62, 8),      # exactly one adjoint strip wide
    (1, 2, 21, 64, 6),      # one column more than a strip
    (1, 4, 19, 126, 6),     # four channels, two forward strips
    (1, 3, 40, 125, 10),    # three channels, ragged
])
def test_forward_backward_match_oracle(ext, tv_oracle, n, c, h, w, its):
    d = tv_inputs(n, c, h, w, seed=n * 1000 + h + w + its, conf_density=0.3)
    print("case n=%d c=%d h=%d w=%d its=%d" % (n, c, h, w, its), flush=True)
    compare("%dx%dx%dx%d its=%d" % (n, c, h, w, its), run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2))


@pytest.mark.parametrize("n,c,h,w,its", [
    (1, 5, 20, 64, 6),      # 4 + 1
    (2, 6, 37, 101, 9),     # 4 + 2, ragged, odd its
    (1, 7, 19, 126, 20),    # 4 + 3, several segments
    (2, 8, 45, 130, 12),    # 4 + 4
    (1, 9, 11, 62, 8),      # three groups
])
def test_more_than_four_channels_run_in_channel_groups(ext, tv_oracle, n, c, h, w, its):
    # the strip kernels hold up to four channels; more run as launches over groups of channels, whose shared
    # accumulators (confidence and edge-weight gradients) are summed group after group in the reference's order
    d = tv_inputs(n, c, h, w, seed=300 + c, conf_density=0.3)
    got, ref = run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2)
    compare("%d channels in groups" % c, got, ref)
    assert np.array_equal(got[0], ref[0])
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("n,c,h,w,its", [
    (1, 3, 23, 75, 17),     # odd its: first step, single step and pairs
    (2, 4, 45, 130, 26),    # several strips wide, several segments
    (1, 4, 3, 200, 6),      # fewer rows than the pair kernel's row lag
    (1, 3, 2, 59, 4),
    (1, 3, 70, 61, 8),      # one column more than a strip
    (2, 4, 130, 200, 50),   # several strips high
    (1, 4, 100, 60, 5),
    (1, 3, 33, 1, 4),       # a single column
])
def test_three_and_four_channels_pair_in_two_wavefronts(ext, tv_oracle, n, c, h, w, its):
    # with 3 or 4 channels the two adjoint steps of a launch run in two wavefronts of a workgroup and hand their
    # row results over through LDS; every gradient is bit-equal to the oracle's
    d = tv_inputs(n, c, h, w, seed=500 + c + h + its, conf_density=0.3)
    got, ref = run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2)
    compare("%d channels, two wavefronts" % c, got, ref)
    assert np.array_equal(got[0], ref[0])
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("n,c,h,w,its", [
    (1, 5, 23, 75, 17),     # groups of 3 + 2; odd its: first step, single step and pairs
    (2, 6, 45, 130, 26),    # 3 + 3; several strips wide, several segments
    (1, 7, 3, 200, 6),      # 4 + 3; fewer rows than one interval of the pipeline
    (1, 8, 2, 59, 4),       # 4 + 4
    (1, 5, 70, 61, 8),      # one column more than a strip
    (2, 8, 130, 200, 50),   # several strips high
    (1, 7, 100, 60, 5),
    (1, 6, 33, 1, 4),       # a single column
    (1, 8, 4, 64, 6),       # rows: exactly one block of three after the start-up rows
    (1, 5, 5, 64, 6),
    (1, 6, 6, 64, 6),
])
def test_five_to_eight_channels_pair_in_four_wavefronts(ext, tv_oracle, n, c, h, w, its):
    # two channel groups, step A and step B of each in a wavefront of its own; the shared accumulators travel
    # A(group 0) -> A(group 1) -> B(group 1), which also adds B(group 0)'s terms first: the reference's order
    d = tv_inputs(n, c, h, w, seed=700 + c + h + its, conf_density=0.3)
    got, ref = run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2)
    compare("%d channels, four wavefronts" % c, got, ref)
    assert np.array_equal(got[0], ref[0])
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("c", [2, 3, 4, 5, 8])
@pytest.mark.parametrize("rows", ["1", "3", "8", "13", "64"])
def test_pair_kernels_at_forced_strip_heights(ext, tv_oracle, c, rows, split, monkeypatch):
    # INPAINT_TV_FWD_ROWS / INPAINT_TV_ADJ_ROWS: strips shorter and taller than the image, ragged last strips; all channels
    # per wavefront and one channel per wavefront (forward pairs up to four channels, adjoint pairs at two)
    d = tv_inputs(2, c, 50, 140, seed=610 + c, conf_density=0.3)
    ref = run_oracle(tv_oracle, d, 12, 2)
    monkeypatch.setenv("INPAINT_TV_FWD_ROWS", rows)
    monkeypatch.setenv("INPAINT_TV_ADJ_ROWS", rows)
    monkeypatch.setenv("INPAINT_TV_FWD_SPLIT", split)
    monkeypatch.setenv("INPAINT_TV_ADJ_SPLIT", split)
    from customnetworklayers_amd._lib import reload_env
    reload_env()
    got = run_gpu(ext, d, 12, 2)
    compare("strip height %s, %d channels" % (rows, c), got, ref)
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b)


@pytest.mark.parametrize("keep", ["0", "2"])
@pytest.mark.parametrize("split", ["0", "1"])
@pytest.mark.parametrize("n,c,h,w,its", [(2, 2, 50, 140, 12), (1, 3, 37, 121, 9), (2, 4, 20, 64, 20), (1, 2, 3, 200, 6), (1, 2, 1, 70, 4),
                                         (1, 2, 33, 1, 4), (2, 2, 45, 130, 17)])
def test_forward_pairs_with_one_channel_per_wavefront(ext, tv_oracle, n, c, h, w, its, split, keep, monkeypatch):
    # launches too small to fill the chip run the forward pairs with one channel per wavefront (all channel groups in one
    # launch) and, at two channels, the adjoint pairs likewise (channel 0's accumulator terms handed to channel 1's wavefront
    # through LDS); INPAINT_TV_FWD_SPLIT / INPAINT_TV_ADJ_SPLIT force either layout, with the iterates kept (keep mode 2: the pairs rebuild their input
    # from the x05 rows) and recomputed (keep mode 0)
    d = tv_inputs(n, c, h, w, seed=640 + c + h, conf_density=0.3)
    ref = run_oracle(tv_oracle, d, its, 2)
    monkeypatch.setenv("INPAINT_TV_FWD_SPLIT", split)
    monkeypatch.setenv("INPAINT_TV_ADJ_SPLIT", split)  # (two channels: the adjoint pairs likewise)
    monkeypatch.setenv("INPAINT_KEEP", keep)
    from customnetworklayers_amd._lib import reload_env
    reload_env()
    got = run_gpu(ext, d, its, 2)
    compare("forward split %s, keep %s, %d channels" % (split, keep, c), got, ref)
    assert np.array_equal(got[0], ref[0])
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b)


REGIMES = {
    # name: (scale of the flow, confidence values, edge-weight values)
    "large flows": (1e4, (0.0, 0.3, 1.0), (1e-3, 1.0)),
    "tiny flows": (1e-6, (0.0, 0.3, 1.0), (1e-3, 1.0)),
    "confidence from 1e-8 to 1e3": (8.0, (0.0, 1e-8, 1e-3, 1.0, 1e3), (0.2, 1.0)),
    "weights from 0 to 50": (8.0, (0.0, 0.5), (0.0, 1e-12, 1e-3, 1.0, 50.0)),
    "flat image, no data": (0.0, (0.0,), (1.0,)),
}


@pytest.mark.parametrize("c", [1, 2, 3])
@pytest.mark.parametrize("regime", sorted(REGIMES))
def test_unusual_magnitudes_stay_bit_equal(ext, tv_oracle, regime, c):
    # the short division / reciprocal / square root sequences return the compiler's bits for ordinary operands; inputs far
    # from the benchmark's magnitudes (flows of 1e4 and 1e-6 pixels, confidences and weights over many decades, zero weights,
    # an image without any gradient) must therefore leave every output bit-equal to the oracle
    scale, confs, weights = REGIMES[regime]
    n, h, w, its = 2, 37, 131, 12
    d = tv_inputs(n, c, h, w, seed=900 + c, conf_density=0.5)
    rng = np.random.default_rng(17 + c)
    d["db"] = (d["db"] * np.float32(scale / 8.0)).astype(np.float32)
    d["di"] = d["db"].copy()
    d["dc"] = rng.choice(np.array(confs, np.float32), size=d["dc"].shape).astype(np.float32)
    d["dx"] = rng.choice(np.array(weights, np.float32), size=d["dx"].shape).astype(np.float32)
    d["dy"] = rng.choice(np.array(weights, np.float32), size=d["dy"].shape).astype(np.float32)
    got, ref = run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2)
    compare("%s, %d channels" % (regime, c), got, ref)
    assert np.array_equal(got[0], ref[0], equal_nan=True)
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b, equal_nan=True)


@pytest.mark.parametrize("scale,bit_equal", [(1e-20, True), (1e-30, True), (1e-36, False), (1e20, True), (1e30, True)])
def test_upstream_gradients_of_extreme_magnitude(ext, tv_oracle, scale, bit_equal):
    # The short division (reciprocal refined once, quotient corrected once, no range fix-ups) returns the compiler's bits
    # while the correction's residual stays a normal number.  The adjoint's numerators scale with the upstream gradient:
    # down to 1e-30 and up to 1e30 (where the clamps of the adjoint iterates act) every gradient is the oracle's, bit for
    # bit; at 1e-36 the results (1e-38 and below) are denormal and agree to their last bits only (1e-7 of the largest).
    from customnetworklayers_amd.workloads import tv_inputs as make

    d = make(1, 2, 40, 130, seed=3, conf_density=0.4)
    d["grad"] = (d["grad"].astype(np.float64) * scale).astype(np.float32)
    got, ref = run_gpu(ext, d, 12, 2), run_oracle(tv_oracle, d, 12, 2)
    for a, b in zip(got[1], ref[1]):
        if bit_equal:
            assert np.array_equal(a, b, equal_nan=True)
        else:
            assert float(np.abs(a.astype(np.float64) - b).max()) <= 1e-6 * float(np.abs(b).max())
    ext.reset_id(2)


def test_removed_kernel_path_is_refused(ext, monkeypatch):
    # INPAINT_TV_PATH=tile used to select the LDS-tile kernels written first; the library no longer contains them and
    # says so instead of silently running something else
    d = tv_inputs(1, 2, 20, 64, seed=3, conf_density=0.3)
    t = {k: torch.from_numpy(v).to("cuda:0") for k, v in d.items()}
    monkeypatch.setenv("INPAINT_TV_PATH", "tile")
    try:
        ext.reset_id(2)  # (re-reads the environment)
        with pytest.raises(ValueError, match="no longer contains"):
            ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], 6, 2)
    finally:
        monkeypatch.delenv("INPAINT_TV_PATH")
        ext.reset_id(2)
    ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], 6, 2)
    ext.reset_id(2)


@pytest.mark.parametrize("n,c,h,w,its", [(2, 2, 70, 256, 20), (1, 3, 45, 130, 10)])
def test_single_iteration_strip_kernels(ext, tv_oracle, n, c, h, w, its, monkeypatch):
    # the forward and the recompute normally run two iterations per launch; INPAINT_TV_FUSE=0 keeps
    # the one-iteration strip kernels covered
    d = tv_inputs(n, c, h, w, seed=91 + c, conf_density=0.3)
    ref = run_oracle(tv_oracle, d, its, 2)
    monkeypatch.setenv("INPAINT_TV_FUSE", "0")
    compare("one iteration per launch c=%d" % c, run_gpu(ext, d, its, 2), ref)


@pytest.mark.parametrize("n,c,h,w,its", [(2, 2, 70, 256, 20), (1, 1, 45, 130, 11)])
def test_single_step_adjoint_strip_kernels(ext, tv_oracle, n, c, h, w, its, monkeypatch):
    # the reverse sweep normally runs two adjoint steps per launch; INPAINT_TV_FUSE_ADJ=0 keeps the
    # one-step strip kernels covered (forward and recompute stay fused)
    d = tv_inputs(n, c, h, w, seed=93 + c, conf_density=0.3)
    ref = run_oracle(tv_oracle, d, its, 2)
    monkeypatch.setenv("INPAINT_TV_FUSE_ADJ", "0")
    compare("one adjoint step per launch c=%d" % c, run_gpu(ext, d, its, 2), ref)


@pytest.mark.parametrize("its", [2, 3, 4, 5, 6, 8, 16, 17, 26])
def test_every_pairing_of_the_reverse_sweep(ext, tv_oracle, its):
    # its decides how the sweep splits into the first step, an optional single step and pairs:
    # one segment of 2 (first step + single segment-start step), segments of even and odd remainder
    d = tv_inputs(1, 2, 23, 75, seed=300 + its, conf_density=0.4)
    compare("its=%d" % its, run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2))


@pytest.mark.parametrize("c", [1, 2, 3, 4, 5])
@pytest.mark.parametrize("its", [4, 5, 9, 16, 50])
def test_first_step_of_the_sweep_rides_on_the_second(ext, tv_oracle, c, its, monkeypatch):
    # up to four channels, a last segment of at least four iterations: one launch does the sweep's first two steps
    # (its = 4, 5: the last segment has two iterations, so the two steps stay apart; c = 5 always keeps them apart);
    # INPAINT_TV_FUSE_FIRST=0 keeps the separate launches covered
    d = tv_inputs(2, c, 37, 130, seed=500 + 10 * c + its, conf_density=0.4)
    ref = run_oracle(tv_oracle, d, its, 2)
    a = run_gpu(ext, d, its, 2)
    compare("first two steps in one launch c=%d its=%d" % (c, its), a, ref)
    monkeypatch.setenv("INPAINT_TV_FUSE_FIRST", "0")
    b = run_gpu(ext, d, its, 2)
    compare("first step in its own launch c=%d its=%d" % (c, its), b, ref)
    for x, y in zip(a[1], b[1]):
        np.testing.assert_array_equal(x, y)


@pytest.mark.parametrize("n,c,h,w,its", [
    (1, 1, 9, 60, 8),       # exactly one fused strip wide (60 output columns)
    (1, 2, 11, 61, 8),      # one column more
    (1, 2, 3, 200, 6),      # fewer rows than the fused kernel's row lag
    (1, 2, 2, 59, 4),
    (2, 4, 18, 121, 12),    # four channels, two fused strips and a column
])
def test_fused_forward_strip_edges(ext, tv_oracle, n, c, h, w, its):
    d = tv_inputs(n, c, h, w, seed=n * 100 + h + w, conf_density=0.3)
    compare("%dx%dx%dx%d its=%d" % (n, c, h, w, its), run_gpu(ext, d, its, 2), run_oracle(tv_oracle, d, its, 2))


def test_its_zero_and_one_return_init_and_zero_grads(ext, tv_oracle):
    d = tv_inputs(1, 2, 20, 30, seed=5)
    for its in (0, 1):
        sol, grads, _ = run_gpu(ext, d, its, 3)
        np.testing.assert_array_equal(sol, d["di"])
        rsol, rgrads, _ = run_oracle(tv_oracle, d, its, 3)
        for g, r in zip(grads, rgrads):
            np.testing.assert_array_equal(g, r)
            assert not g.any()


def test_rectangles_and_dense_confidence(ext, tv_oracle):
    # the stress configuration's generators at a size the oracle finishes quickly
    d = tv_inputs(2, 2, 96, 160, seed=4, flow="rectangles", dense_conf=True)
    compare("rectangles", run_gpu(ext, d, 60, 1), run_oracle(tv_oracle, d, 60, 1))


def test_headline_shape_one_sample(ext, tv_oracle):
    # one sample of the headline configuration (2 x 384 x 1248, 100 iterations)
    cfg = CONFIGS[1]
    d = tv_inputs(1, cfg["c"], cfg["h"], cfg["w"], seed=0, **cfg["gen"])
    compare("headline/1", run_gpu(ext, d, cfg["its"], 0), run_oracle(tv_oracle, d, cfg["its"], 0))


def test_upstream_scrub_is_in_place_and_matches(ext, tv_oracle):
    d = tv_inputs(1, 2, 40, 50, seed=6)
    d["grad"][0, 1, 7, 9] = np.nan
    d["grad"][0, 0, 0, 0] = np.inf
    got = run_gpu(ext, d, 12, 4)
    ref = run_oracle(tv_oracle, d, 12, 4)
    np.testing.assert_array_equal(got[2], ref[2])  # scrubbed upstream tensors agree
    assert got[2][0, 1, 7, 9] == 0 and got[2][0, 0, 0, 0] == 0
    compare("scrub", got, ref)


def test_ids_are_independent_and_nest(ext, tv_oracle):
    # forward on ids 0,1,2 then backward 2,1,0 (the hierarchy's calling pattern)
    dev = torch.device("cuda:0")
    cases = [tv_inputs(1, 2, 24 * (i + 1), 40 * (i + 1), seed=30 + i) for i in range(3)]
    its = 10
    tens = [{k: torch.from_numpy(v).to(dev) for k, v in d.items()} for d in cases]
    for i in range(3):
        ext.reset_id(i)
        tv_oracle.reset_id(i)
    sols = [ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, i)[0] for i, t in enumerate(tens)]
    grads = {}
    for i in (2, 1, 0):
        t = tens[i]
        grads[i] = ext.backward(t["grad"], t["dx"], t["dy"], t["dc"], t["db"], its, i)
    torch.cuda.synchronize()
    for i, d in enumerate(cases):
        ref = run_oracle(tv_oracle, d, its, i)
        compare("id%d" % i, (sols[i].cpu().numpy(), [g.cpu().numpy() for g in grads[i]], None), ref)


def test_guard_rescales_and_kills_like_the_oracle(ext, tv_oracle):
    d = tv_inputs(1, 2, 32, 48, seed=8)
    its = 8
    # learn what the plain gradient means are
    base = run_gpu(ext, d, its, 5)
    means = [float(np.abs(g).mean()) for g in base[1]]
    stats = ext.guard_stats(5)
    assert all(row[4] == 0 for row in stats)
    # running means 20x below (C: rescale), 60x below (X: kill), equal (others), after 10 runs.
    # the guard sees the values before the global 0.1 (and the 1/8 of the edge weights)
    f = float(np.float32(0.1))
    pre = [means[2] / f, means[0] / f * 8, means[1] / f * 8, means[3] / f, means[4]]  # C, X, Y, B, I
    state = [10, pre[0] / 20, pre[1] / 60, pre[2], pre[3], pre[4]]
    ext.set_state(5, state)
    tv_oracle.reset_id(5)
    tv_oracle.set_state(5, state)
    got = run_gpu(ext, d, its, 5, fresh=False)
    ref = run_oracle(tv_oracle, d, its, 5, fresh=False)
    stats = ext.guard_stats(5)
    assert [int(r[4]) for r in stats] == [1, 2, 0, 0, 0]
    assert not got[1][0].any()  # gx killed
    np.testing.assert_allclose(got[1][2], base[1][2] * 0.5, rtol=1e-5, atol=0)  # gc halved
    compare("guard", got, ref)
    gs, os_ = ext.get_state(5), tv_oracle.get_state(5)
    np.testing.assert_allclose(gs, os_, rtol=1e-9)
    assert gs[0] == 11


def test_errors(ext):
    dev = torch.device("cuda:0")
    d = {k: torch.from_numpy(v).to(dev) for k, v in tv_inputs(1, 2, 8, 8, seed=1).items()}
    with pytest.raises(IndexError):
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 4, 10)
    with pytest.raises(IndexError):
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 4, -1)
    with pytest.raises(TypeError):
        ext.forward(d["dx"].double(), d["dy"], d["dc"], d["db"], d["di"], 4, 0)
    with pytest.raises(RuntimeError):
        ext.forward(d["dx"].cpu(), d["dy"], d["dc"], d["db"], d["di"], 4, 0)
    with pytest.raises(RuntimeError):
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"].permute(0, 1, 3, 2), d["di"], 4, 0)
    ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 4, 0)
    with pytest.raises(RuntimeError):  # its differs from the forward that filled the slot
        ext.backward(d["grad"], d["dx"], d["dy"], d["dc"], d["db"], 6, 0)
    with pytest.raises(ValueError):
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 10201 + 300, 0)


@pytest.mark.parametrize("its", [2, 3, 20])
def test_forward_in_place_through_the_c_abi(ext, its):
    # a caller of the C ABI may hand the starting point's buffer in as the output: the forward pass then copies the
    # starting point aside before its first launch instead of letting that launch read it while the result is written
    import ctypes

    from customnetworklayers_amd._lib import lib

    dev = torch.device("cuda:0")
    d = tv_inputs(2, 2, 37, 130, seed=77 + its, conf_density=0.3)
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    ext.reset_id(4)
    (ref,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 4)
    gref = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 4)
    buf = t["di"].clone()
    n, c, h, w = d["db"].shape
    p = lambda x: ctypes.c_void_p(x.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    ext.reset_id(4)
    rc = lib.tvinpaint_forward(p(t["dx"]), p(t["dy"]), p(t["dc"]), p(t["db"]), p(buf), p(buf), n, c, h, w, its, 4, stream)
    assert rc == 0
    g = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 4)
    torch.cuda.synchronize()
    assert torch.equal(buf, ref)
    for a, b in zip(g, gref):
        assert torch.equal(a, b)
    ext.reset_id(4)


def test_gradient_mode_is_fixed_by_the_forward_pass(ext):
    # the forward pass latches the id's gradient mode (with every x05 row kept it stores, at each checkpoint, only the
    # half that mode's backward reads); a backward under the other mode says so, and says so in every keep mode
    dev = torch.device("cuda:0")
    d = {k: torch.from_numpy(v).to(dev) for k, v in tv_inputs(1, 2, 24, 70, seed=12).items()}
    try:
        ext.reset_id(3)
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 20, 3)
        ext.gradient_mode(3, 1)
        with pytest.raises(RuntimeError, match="gradient mode"):
            ext.backward(d["grad"].clone(), d["dx"], d["dy"], d["dc"], d["db"], 20, 3)
        ext.gradient_mode(3, 0)
        a = ext.backward(d["grad"].clone(), d["dx"], d["dy"], d["dc"], d["db"], 20, 3)
        ext.reset_id(3)
        ext.keep_iterates(3, 0)
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 20, 3)
        ext.gradient_mode(3, 1)
        with pytest.raises(RuntimeError, match="gradient mode"):  # (both checkpoint halves exist here: same rule)
            ext.backward(d["grad"].clone(), d["dx"], d["dy"], d["dc"], d["db"], 20, 3)
        ext.gradient_mode(3, 0)
        b = ext.backward(d["grad"].clone(), d["dx"], d["dy"], d["dc"], d["db"], 20, 3)
        ext.keep_iterates(3, 1)
        ext.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 20, 3)
        ext.gradient_mode(3, 1)
        with pytest.raises(RuntimeError, match="gradient mode"):
            ext.backward(d["grad"].clone(), d["dx"], d["dy"], d["dc"], d["db"], 20, 3)
        for x, y in zip(a, b):
            assert torch.equal(x, y)
    finally:
        ext.reset_id(3)


def test_module_surface_and_autograd(ext, tv_oracle):
    from customnetworklayers_amd import TVInpaint

    dev = torch.device("cuda:0")
    d = tv_inputs(1, 2, 30, 44, seed=9)
    hwc = lambda a: torch.from_numpy(np.ascontiguousarray(a[0].transpose(1, 2, 0))).to(dev).requires_grad_(True)
    tx, ty, tc, tb, ti = (hwc(d[k]) for k in ("dx", "dy", "dc", "db", "di"))
    layer = TVInpaint(dev, 14, pid=6)
    ext.reset_id(6)
    sol = layer(tx, ty, tc, tb, ti)
    assert tuple(sol.shape) == (30, 44, 2)
    up = torch.from_numpy(np.ascontiguousarray(d["grad"][0].transpose(1, 2, 0))).to(dev)
    sol.backward(up)
    ref = run_oracle(tv_oracle, d, 14, 6)
    got_grads = [t.grad.permute(2, 0, 1).unsqueeze(0).cpu().numpy() for t in (tx, ty, tc, tb, ti)]
    compare("module", (sol.detach().permute(2, 0, 1).unsqueeze(0).cpu().numpy(), got_grads, None), ref)


@pytest.mark.parametrize("n,c,h,w,its", [(2, 2, 40, 130, 20), (1, 1, 30, 70, 9), (1, 3, 20, 64, 6), (1, 7, 25, 64, 12)])
def test_kept_iterates_or_recomputed_segments_give_the_same_bits(ext, tv_oracle, n, c, h, w, its, monkeypatch):
    # keep mode 2 (default) stores every x05 row in the forward and recomputes nothing; mode 1 keeps the last
    # segment's rows, which serve one backward; mode 0 recomputes every segment as the reference does.  A second
    # backward on one forward, a too-small memory budget and the per-call `keep` argument are covered as well.
    d = tv_inputs(n, c, h, w, seed=55, conf_density=0.3)
    ref = run_oracle(tv_oracle, d, its, 2)
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}

    def fwd_bwd(twice=False, **kw):
        ext.reset_id(2)
        if "mode" in kw:
            ext.keep_iterates(2, kw["mode"])
        (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 2, **{k: v for k, v in kw.items() if k == "keep"})
        grads = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 2)
        if twice:
            ext.set_state(2, [0.0] * 6)
            again = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 2)
            for a, b in zip(grads, again):
                assert torch.equal(a, b)
        nbytes = ext.slot_bytes(2) if hasattr(ext, "slot_bytes") else 0
        return sol, grads, nbytes

    sol, first, bytes_all = fwd_bwd(twice=True)
    compare("all kept", (sol.cpu().numpy(), [g.cpu().numpy() for g in first], None), ref)
    runs = {"mode 2": fwd_bwd(mode=2, twice=True), "mode 1": fwd_bwd(mode=1, twice=True),
            "mode 0": fwd_bwd(mode=0, twice=True), "keep=0 once": fwd_bwd(keep=0), "after keep=0": fwd_bwd()}
    monkeypatch.setenv("INPAINT_KEEP_GB", "0.000001")  # the rows do not fit: the last segment's are kept instead
    runs["budget"] = fwd_bwd(twice=True)
    monkeypatch.delenv("INPAINT_KEEP_GB")
    monkeypatch.setenv("INPAINT_KEEP", "0")
    runs["env 0"] = fwd_bwd()
    monkeypatch.delenv("INPAINT_KEEP")
    monkeypatch.setenv("INPAINT_KEEP_LAST", "0")
    runs["env last 0"] = fwd_bwd()
    for name, (s2, grads, _) in runs.items():
        assert torch.equal(sol, s2), name
        for a, b in zip(first, grads):
            assert torch.equal(a, b), name
    if bytes_all:  # a slot that recomputes is smaller than one that keeps every row
        assert runs["mode 0"][2] < bytes_all
    with pytest.raises(ValueError):
        ext.keep_iterates(2, 3)
    ext.reset_id(2)


# the quirk toggles of the oracle that the corrected gradient switches off (clamp and guard stay)
CORRECTED = dict(end_uses_ckpt_y=0, skip_iter0_adjoint=0, getyk_rebuild=0, scale_factors=0, clamp=1, guard=1)


@pytest.mark.parametrize("n,c,h,w,its", [
    (1, 2, 64, 128, 20), (2, 3, 37, 101, 9), (1, 1, 16, 64, 2), (1, 4, 19, 126, 6), (1, 2, 1, 70, 4),
    (1, 1, 33, 1, 4), (3, 2, 130, 200, 50), (1, 2, 21, 64, 3), (1, 6, 23, 70, 10), (2, 8, 40, 126, 16), (1, 5, 9, 64, 7),
])
def test_corrected_gradient_matches_the_oracle_with_the_same_quirks_off(ext, tv_oracle, n, c, h, w, its, monkeypatch):
    # gradient_mode 1: y as the forward pass made it, no checkpoint stand-in at segment starts, iteration 0
    # back-propagated, multipliers 1 -- the oracle with exactly these toggles off is the checker; every keep mode
    d = tv_inputs(n, c, h, w, seed=n * 100 + h + w + its, conf_density=0.3)
    try:
        tv_oracle.set_quirks(**CORRECTED)
        ref = run_oracle(tv_oracle, d, its, 2)
    finally:
        tv_oracle.set_quirks()
    plain = run_oracle(tv_oracle, d, its, 2)
    assert any(not np.array_equal(a, b) for a, b in zip(ref[1], plain[1]))  # the toggles do something
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    try:
        # two channels: also with all channels in one wavefront and with one channel per wavefront forced (small launches
        # pick the latter by themselves)
        for split in ((None, "0", "1") if c == 2 else (None,)):
            for name in ("INPAINT_TV_FWD_SPLIT", "INPAINT_TV_ADJ_SPLIT"):
                if split is None:
                    monkeypatch.delenv(name, raising=False)
                else:
                    monkeypatch.setenv(name, split)
            for keep in (2, 1, 0):
                ext.reset_id(2)  # (reads the switches again)
                ext.gradient_mode(2, 1)
                ext.keep_iterates(2, keep)
                (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 2)
                grads = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 2)
                got = (sol.cpu().numpy(), [g.cpu().numpy() for g in grads], None)
                compare("corrected, keep %d, split %s" % (keep, split), got, ref)
                for a, b in zip(got[1], ref[1]):
                    assert np.array_equal(a, b)
    finally:
        monkeypatch.delenv("INPAINT_TV_FWD_SPLIT", raising=False)
        monkeypatch.delenv("INPAINT_TV_ADJ_SPLIT", raising=False)
        ext.reset_id(2)  # back to the reference's gradient
    compare("plain again", run_gpu(ext, d, its, 2), plain)


def test_corrected_gradient_is_the_gradient_of_the_forward_pass(ext, tv_oracle):
    # with the clamp and the guard idle the corrected gradient is the true one: the float64 oracle with every quirk
    # off (which the CPU pins equate with automatic differentiation of an independent forward pass) agrees to
    # float32 accuracy, and a directional finite difference of the GPU forward pass agrees as well
    n, c, h, w, its = 1, 2, 24, 40, 12
    d = tv_inputs(n, c, h, w, seed=5, conf_density=0.4)
    d64 = {k: v.astype(np.float64) for k, v in d.items()}
    try:
        tv_oracle.set_quirks(0, 0, 0, 0, 0, 0)
        tv_oracle.reset_id(3)
        tv_oracle.forward(d64["dx"], d64["dy"], d64["dc"], d64["db"], d64["di"], its, 3, f64=True)
        true = tv_oracle.backward(d64["grad"].copy(), d64["dx"], d64["dy"], d64["dc"], d64["db"], its, 3, f64=True)
    finally:
        tv_oracle.set_quirks()
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    try:
        ext.reset_id(2)
        ext.gradient_mode(2, 1)
        ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 2)
        grads = [g.cpu().numpy() for g in ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 2)]
    finally:
        ext.reset_id(2)
    errs = [rel_err(g, r) for g, r in zip(grads, true)]
    print("\ncorrected gradient vs float64 true gradient: gx %.2e gy %.2e gc %.2e gb %.2e gi %.2e" % tuple(errs), flush=True)
    for e in errs:
        assert e <= 1e-3
    # the reference's gradient is a different vector: scale factors alone put it a factor 10..100 away
    plain = run_gpu(ext, d, its, 2)[1]
    assert rel_err(plain[3], true[3]) > 0.5


def test_gradient_mode_takes_zero_or_one(ext):
    with pytest.raises(ValueError):
        ext.gradient_mode(2, 2)
    with pytest.raises(ValueError):
        ext.gradient_mode(2, -1)


def test_module_with_the_corrected_gradient(ext, tv_oracle):
    from customnetworklayers_amd import TVInpaint

    dev = torch.device("cuda:0")
    d = tv_inputs(1, 2, 30, 44, seed=9)
    hwc = lambda a: torch.from_numpy(np.ascontiguousarray(a[0].transpose(1, 2, 0))).to(dev).requires_grad_(True)
    tx, ty, tc, tb, ti = (hwc(d[k]) for k in ("dx", "dy", "dc", "db", "di"))
    try:
        ext.reset_id(6)
        layer = TVInpaint(dev, 14, pid=6, corrected_gradient=True)
        sol = layer(tx, ty, tc, tb, ti)
        up = torch.from_numpy(np.ascontiguousarray(d["grad"][0].transpose(1, 2, 0))).to(dev)
        sol.backward(up)
    finally:
        ext.reset_id(6)
    try:
        tv_oracle.set_quirks(**CORRECTED)
        ref = run_oracle(tv_oracle, d, 14, 6)
    finally:
        tv_oracle.set_quirks()
    got_grads = [t.grad.permute(2, 0, 1).unsqueeze(0).cpu().numpy() for t in (tx, ty, tc, tb, ti)]
    compare("module, corrected", (sol.detach().permute(2, 0, 1).unsqueeze(0).cpu().numpy(), got_grads, None), ref)
    for a, b in zip(got_grads, ref[1]):
        assert np.array_equal(a, b)


def test_corrected_gradient_one_step_per_launch(ext, tv_oracle, monkeypatch):
    # two channels normally take the pair kernels; INPAINT_TV_FUSE_ADJ=0 keeps the one-step corrected kernels covered
    n, c, h, w, its = 2, 2, 45, 130, 12
    d = tv_inputs(n, c, h, w, seed=23, conf_density=0.3)
    try:
        tv_oracle.set_quirks(**CORRECTED)
        ref = run_oracle(tv_oracle, d, its, 2)
    finally:
        tv_oracle.set_quirks()
    monkeypatch.setenv("INPAINT_TV_FUSE_ADJ", "0")
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    try:
        ext.reset_id(2)
        ext.gradient_mode(2, 1)
        (sol,) = ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 2)
        grads = ext.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 2)
        got = (sol.cpu().numpy(), [g.cpu().numpy() for g in grads], None)
    finally:
        ext.reset_id(2)
    compare("corrected, one step per launch", got, ref)
    for a, b in zip(got[1], ref[1]):
        assert np.array_equal(a, b)
