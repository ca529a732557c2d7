"""The compiled PyTorch bindings (host C++ over the C ABI, the reference's pybind modules with their two calls
swapped) against the ctypes bindings on the same inputs: same library underneath, so the same bits."""
import pytest
import torch

from customnetworklayers_amd.workloads import tgv_inputs, tv_inputs

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("layer", ["tv", "tgv"])
def test_compiled_binding_equals_the_ctypes_binding(layer):
    if layer == "tv":
        from customnetworklayers_amd.cudaTV import tvInpaint_cuda_ext as ref, tvInpaint_hip_ext as ext
        d = tv_inputs(2, 2, 45, 130, seed=5, conf_density=0.3)
    else:
        from customnetworklayers_amd.cudaTGV import tgvInpaint_cuda_ext as ref, tgvInpaint_hip_ext as ext
        d = tgv_inputs(2, 2, 45, 130, seed=5, conf_density=0.3)
    dev = torch.device("cuda:0")
    t = {k: torch.from_numpy(v).to(dev) for k, v in d.items()}
    its = 12
    out = {}
    for name, m in (("ctypes", ref), ("compiled", ext)):
        m.reset_id(1)
        print("binding %s layer %s" % (name, layer), flush=True)
        (sol,) = m.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 1)
        grads = m.backward(t["grad"].clone(), t["dx"], t["dy"], t["dc"], t["db"], its, 1)
        torch.cuda.synchronize()
        out[name] = [sol] + list(grads)
        m.reset_id(1)
    assert len(out["compiled"]) == 6
    for a, b in zip(out["ctypes"], out["compiled"]):
        assert a.shape == b.shape and torch.equal(a, b)
    with pytest.raises(RuntimeError, match="id"):  # a bad id raises (the reference prints and returns an empty list)
        ext.forward(t["dx"], t["dy"], t["dc"], t["db"], t["di"], its, 10)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.forward(t["dx"].transpose(2, 3), t["dy"], t["dc"], t["db"], t["di"], its, 1)
