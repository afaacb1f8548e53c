"""The PyTorch face (extension `fwd`/`bwd` + autograd function) on the GPU: same results as the
C ABI path, reference return lists, and gradients flowing to every differentiable input."""
import numpy as np
import pytest
import torch

from oracle import snd_oracle as O
from test_gpu_fwd import relerr

pytestmark = pytest.mark.gpu


def leaves(d, dev, keys=("u", "delta", "A", "B", "C", "D", "delta_bias")):
    return {k: torch.from_numpy(d[k]).to(dev).requires_grad_(True) for k in keys}


def test_extension_return_lists(gpu_device):
    import selective_nd_scan as s
    d = O.make_inputs(2, 8, 10, 12, N=16, K=2, seed=1, Dd=4)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    res = s.fwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], True, True, None)
    assert len(res) == 4                                   # [out, x, x_v, x_sd]  (host.cpp:282)
    out, x, x_v, x_sd = res
    assert x.dim() == 5 and x_v.dim() == 5 and x_sd.shape == x.shape and x.shape[:3] == (2, 8, 16)
    g = s.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], x, x_v, True, None, x_sd)
    assert len(g) == 8                                     # host.cpp:432
    assert g[1].shape == t["delta"].shape and g[6].shape == (4,)      # group sums, host.cpp:433-438
    assert g[7] is None                                    # undefined tensor for an absent optional
    ref = O.selective_nd_scan_bwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], d["dout"], True)
    for a, b_ in zip(g[:7], ref[:7]):
        assert relerr(a.cpu().numpy(), b_) <= 1e-4
    with pytest.raises(RuntimeError):                      # saved state is mandatory
        s.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], None, x_v, True, None, x_sd)
    with pytest.raises(RuntimeError):                      # wrong shape of saved state
        s.bwd(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], t["dout"], x[:, :, :, :1], x_v, True, None, x_sd)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_autograd_function_matches_oracle(gpu_device, dtype):
    from selective_nd_scan import selective_nd_scan
    d = O.make_inputs(2, 16, 14, 14, N=16, K=4, seed=2)
    L = leaves(d, gpu_device)
    cast = lambda k: L[k].to(dtype) if k in ("u", "delta", "B", "C") else L[k]
    out = selective_nd_scan(cast("u"), cast("delta"), cast("A"), cast("B"), cast("C"), cast("D"), cast("delta_bias"),
                            True, True, None)
    # a non-contiguous upstream gradient exercises the dout.contiguous() path of backward
    w = torch.from_numpy(d["dout"]).to(gpu_device)
    (out * w).sum().backward()
    rd = {k: (L[k].detach().to(dtype).float().cpu().numpy() if k in ("u", "delta", "B", "C") else d[k]) for k in d if k != "dout"}
    ref = O.selective_nd_scan_fwd(rd["u"], rd["delta"], rd["A"], rd["B"], rd["C"], rd["D"], rd["delta_bias"], True)
    gref = O.selective_nd_scan_bwd(rd["u"], rd["delta"], rd["A"], rd["B"], rd["C"], rd["D"], rd["delta_bias"], d["dout"], True)
    tol = 1e-4 if dtype == torch.float32 else 1e-2
    assert relerr(out.detach().float().cpu().numpy(), ref) <= 1e-4
    for key, g in zip(("u", "delta", "A", "B", "C", "D", "delta_bias"), gref):
        assert L[key].grad is not None, key
        assert relerr(L[key].grad.cpu().numpy(), g) <= (tol if key in ("u", "delta", "B", "C") else 1e-4), key


def test_autograd_with_a_decay_and_no_optionals(gpu_device):
    from selective_nd_scan import selective_nd_scan
    d = O.make_inputs(1, 8, 9, 10, N=8, K=2, seed=3)
    L = leaves(d, gpu_device, ("u", "delta", "A", "B", "C"))
    dec = torch.tensor([0.9], device=gpu_device, requires_grad=True)
    delta = L["delta"].abs() + 0.01
    out = selective_nd_scan(L["u"], delta, L["A"], L["B"], L["C"], None, None, False, True, dec)
    out.backward(torch.from_numpy(d["dout"]).to(gpu_device))
    dl = np.abs(d["delta"]) + 0.01
    gref = O.selective_nd_scan_bwd(d["u"], dl, d["A"], d["B"], d["C"], None, None, d["dout"], False, np.array([0.9]))
    assert relerr(dec.grad.cpu().numpy(), gref[7]) <= 1e-4
    assert relerr(L["A"].grad.cpu().numpy(), gref[2]) <= 1e-4
    assert relerr(L["delta"].grad.cpu().numpy(), gref[1] * np.sign(d["delta"])) <= 1e-4


def test_runs_on_the_current_stream(gpu_device):
    from selective_nd_scan import selective_nd_scan
    d = O.make_inputs(1, 8, 9, 10, N=16, K=2, seed=4, with_dout=False)
    t = {k: torch.from_numpy(v).to(gpu_device) for k, v in d.items()}
    ref = O.selective_nd_scan_fwd(d["u"], d["delta"], d["A"], d["B"], d["C"], d["D"], d["delta_bias"], True)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        out = selective_nd_scan(t["u"], t["delta"], t["A"], t["B"], t["C"], t["D"], t["delta_bias"], True)
    side.synchronize()
    assert relerr(out.cpu().numpy(), ref) <= 1e-4
