"""Writes the fixtures in this folder: small seeded inputs of every layer together with the outputs of
the CPU oracle (fp32, literal reference behaviour), as .npz files of plain arrays.

The reference ships no golden vectors, tests or example data for these layers (its layers cannot be
built or imported here either: CUDA sources with un-vendored headers), so these vectors are NOT
reference outputs.  They freeze the oracle after it was pinned (tests/test_*_oracle_pins.py): the CPU
suite checks that the oracle still reproduces them bit for bit, the GPU suite that the HIP path does
(to the rounding-level bar where a sum's order is undefined).

Run from the repository root:  python tests/golden/make_vectors.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)

from customnetworklayers_amd import workloads  # noqa: E402
from oracle.oracle_lib import FlowAuxOracle, TGVOracle, TVOracle  # noqa: E402


def main():
    tv, tgv, aux = TVOracle(), TGVOracle(), FlowAuxOracle()
    tv.set_quirks()
    tgv.set_quirks()

    d = workloads.tv_inputs(1, 2, 12, 16, seed=41, conf_density=0.3)
    tv.reset_id(0)
    sol = tv.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 8, 0)
    gx, gy, gc, gb, gi = tv.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], 8, 0)
    # the corrected gradient (gradient_mode 1): same forward, the oracle's adjoint with these quirks off
    tv.set_quirks(end_uses_ckpt_y=0, skip_iter0_adjoint=0, getyk_rebuild=0, scale_factors=0, clamp=1, guard=1)
    tv.reset_id(0)
    tv.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 8, 0)
    cx, cy, cc, cb, ci = tv.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], 8, 0)
    tv.set_quirks()
    np.savez_compressed(os.path.join(HERE, "tv_1x2x12x16_its8.npz"), its=8, sol=sol, gx=gx, gy=gy, gc=gc, gb=gb, gi=gi,
                        corrected_gx=cx, corrected_gy=cy, corrected_gc=cc, corrected_gb=cb, corrected_gi=ci, **d)

    d = workloads.tgv_inputs(1, 1, 10, 14, seed=42, conf_density=0.3)
    tgv.reset_id(0)
    sol = tgv.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 6, 0)
    gx, gy, gc, gb, gi = tgv.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], 6, 0)
    tgv.set_quirks(end_uses_ckpt_y=0, skip_iter0_adjoint=0, getyk_rebuild=0, scale_factors=0, clamp=1, guard=1, dw_div=0)
    tgv.reset_id(0)
    tgv.forward(d["dx"], d["dy"], d["dc"], d["db"], d["di"], 6, 0)
    cx, cy, cc, cb, ci = tgv.backward(d["grad"].copy(), d["dx"], d["dy"], d["dc"], d["db"], 6, 0)
    tgv.set_quirks()
    np.savez_compressed(os.path.join(HERE, "tgv_1x1x10x14_its6.npz"), its=6, sol=sol, gx=gx, gy=gy, gc=gc, gb=gb, gi=gi,
                        corrected_gx=cx, corrected_gy=cy, corrected_gc=cc, corrected_gb=cb, corrected_gi=ci, **d)

    d = workloads.quadfit_inputs(1, 4, 12, 18, seed=43, flow_channels=3, amplitude=3.0)
    out = aux.quadfit_forward(d["feat0"], d["feat1"], d["flow"])
    g0, g1 = aux.quadfit_backward(d["grad"], d["feat0"], d["feat1"], d["flow"])
    np.savez_compressed(os.path.join(HERE, "quadfit_1x4x12x18.npz"), out=out, g0=g0, g1=g1, **d)

    d = workloads.median_inputs(1, 6, 9, 11, seed=44, empty_fraction=0.1)
    out = aux.median_forward(d["vol"])
    g = aux.median_backward(d["grad"], d["vol"])
    np.savez_compressed(os.path.join(HERE, "median_1x6x9x11.npz"), out=out, gvol=g, **d)

    rng = np.random.default_rng(45)
    sol = (3 * rng.standard_normal((1, 2, 5, 7))).astype(np.float32)
    img = workloads.smooth_image(rng, 10, 14, sigma=1.5)[None, None].astype(np.float32)
    ga = rng.standard_normal((1, 2, 10, 14)).astype(np.float32)
    gb = rng.standard_normal((1, 2, 10, 14)).astype(np.float32)
    wx, wy = aux.edge_weights(img, 10.0)
    np.savez_compressed(os.path.join(HERE, "hierarchy_1x2x5x7.npz"), sol=sol, img=img, ga=ga, gb=gb,
                        up=aux.upsample2x(sol, 2.0), wx=wx, wy=wy, g_sol=aux.upsample2x_adjoint(ga, gb, 2.0))


if __name__ == "__main__":
    main()
