"""The two bindings over the C ABI: the compiled PyTorch extension (norm_dist_hip_ext, the one the package uses when
it is built; reference: core/cuda/norm_dist.cpp:191-204) and the ctypes route.  On a box with the library built both
must be there, every other GPU test of this suite runs through the extension, and the two give the same bits."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

CHILD = r"""
import json, sys, time, hashlib
sys.path.insert(0, %r); sys.path.insert(0, %r)
import torch
from core import _C
gen = torch.Generator().manual_seed(7)
B, CO, CI = 96, 200, 520
x = torch.randn(B, CI, 1, generator=gen).cuda(); w = (torch.randn(CO, CI, generator=gen) / CI ** 0.5).cuda()
g = torch.randn(B, CO, 1, generator=gen).cuda()
out = torch.empty(B, CO, 1, device="cuda"); pos = torch.empty(B, CO, 1, device="cuda", dtype=torch.int32)
gx, gw = torch.empty_like(x), torch.empty_like(w)
res = {"binding": _C.BINDING}
def digest(*ts):
    h = hashlib.sha256()
    for t in ts: h.update(t.cpu().numpy().tobytes())
    return h.hexdigest()
_C.inf_dist_forward(x, w, out, pos, 1); res["inf_fwd"] = digest(out, pos)
_C.inf_dist_backward_input_weight(g, pos, gx, gw, 1); res["inf_bwd_sum"] = float(gw.double().sum())  # (LDS atomics: no fixed order)
_C.norm_dist_forward(x, w, out, 1, 8.0); res["p8_fwd"] = digest(out)
_C.norm_dist_backward_input_weight(g, x, w, out, gx, gw, 1, 8.0); res["p8_bwd_gw"] = digest(gw)
yl, yu = torch.empty_like(out), torch.empty_like(out)
_C.bound_inf_dist_forward_nograd(x - 0.1, x + 0.1, w, yl, yu, 1); res["bound"] = digest(yl, yu)
img = torch.randn(2, 4, 8, 8, generator=gen).cuda(); cw = torch.randn(6, 36, generator=gen).cuda()
co = torch.empty(2, 6, 64, device="cuda")
_C.conv_inf_dist_forward_nograd(img, cw, co, 1, 3, 1, 1, 1); res["conv"] = digest(co)
# tensors whose sizes do not agree are refused on the host (a kernel would index them out of bounds)
def refused(fn, *a):
    try:
        fn(*a)
    except RuntimeError:
        return True
    return False
short_w = w[:CO - 1].contiguous(); narrow_w = w[:, :CI - 8].contiguous(); small_out = out[:, :CO - 1].contiguous()
res["refusals"] = [
    refused(_C.inf_dist_forward_nograd, x, short_w, out, 1),
    refused(_C.inf_dist_forward_nograd, x, narrow_w, out, 1),
    refused(_C.inf_dist_forward, x, w, out, pos[:, :CO - 1].contiguous(), 1),
    refused(_C.norm_dist_forward, x, w, out, 3, 8.0),
    refused(_C.norm_dist_backward_input_weight, g, x, w, small_out, gx, gw, 1, 8.0),
    refused(_C.norm_dist_backward_input_weight, g, x, w, out, gx[:B - 1].contiguous(), gw, 1, 8.0),
    refused(_C.norm_dist_backward_input_weight, g, x, w, out, gx, gw[:CO - 1].contiguous(), 1, 8.0),
    refused(_C.inf_dist_backward_input_weight, g, pos, gx, gw[:CO - 1].contiguous(), 1),
    refused(_C.bound_inf_dist_forward_nograd, x - 0.1, (x + 0.1)[:B - 1].contiguous(), w, yl, yu, 1),
]
# host cost of queueing one small call (the device is kept busy by the calls themselves)
xs, ws, os_ = x[:8].contiguous(), w[:16].contiguous(), torch.empty(8, 16, 1, device="cuda")
for _ in range(200): _C.inf_dist_forward_nograd(xs, ws, os_, 1)
torch.cuda.synchronize()
t0 = time.perf_counter()
n = 2000
for _ in range(n): _C.inf_dist_forward_nograd(xs, ws, os_, 1)
res["host_us_per_call"] = (time.perf_counter() - t0) / n * 1e6
torch.cuda.synchronize()
print(json.dumps(res))
""" % (ROOT, os.path.join(ROOT, "l_inf-dist-net-v2_amd"))


def _run_child(binding):
    env = dict(os.environ, NORM_DIST_BINDING=binding)
    p = subprocess.run([sys.executable, "-c", CHILD], env=env, capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    return json.loads(p.stdout.strip().splitlines()[-1])


def test_extension_is_the_binding_in_use():
    from core import _C
    assert os.path.exists(_C.EXTENSION_PATH), "norm_dist_hip_ext.so has not been built (make -C l_inf-dist-net-v2_amd/csrc)"
    assert _C.BINDING == "ext"
    assert _C._ext.version() == _C.version()


def test_both_bindings_give_the_same_bits():
    ext, ct = _run_child("ext"), _run_child("ctypes")
    assert ext["binding"] == "ext" and ct["binding"] == "ctypes"
    for k in ("inf_fwd", "p8_fwd", "p8_bwd_gw", "bound", "conv"):
        assert ext[k] == ct[k], k
    assert abs(ext["inf_bwd_sum"] - ct["inf_bwd_sum"]) < 1e-3
    assert all(ext["refusals"]) and all(ct["refusals"]), (ext["refusals"], ct["refusals"])  # mismatched sizes
    print("host microseconds per queued call: extension %.1f, ctypes %.1f" % (ext["host_us_per_call"], ct["host_us_per_call"]))
    assert ext["host_us_per_call"] < 3 * ct["host_us_per_call"] + 20  # sanity only: neither route may stall


def test_extension_checks_like_the_reference_binding():
    from core import _C
    E = _C._ext
    x = torch.randn(4, 8, 1, device="cuda")
    w = torch.randn(5, 8, device="cuda")
    out = torch.empty(4, 5, 1, device="cuda")
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        E.inf_dist_forward_nograd(x.cpu(), w, out, 1)
    with pytest.raises(RuntimeError, match="must be contiguous"):
        E.inf_dist_forward_nograd(torch.randn(4, 16, 1, device="cuda")[:, ::2], w, out, 1)
    with pytest.raises(RuntimeError, match="dtype"):
        E.inf_dist_forward_nograd(x.double(), w, out, 1)
    with pytest.raises(RuntimeError, match="groups"):  # CI not divisible by G
        E.inf_dist_forward_nograd(x, w, out, 3)
    with pytest.raises(RuntimeError, match="status 3"):
        E.norm_dist_forward(x, w, out, 1, -1.0)
    # on a side stream: the extension launches on PyTorch's current stream
    s = torch.cuda.Stream()
    ref = torch.empty_like(out)
    E.inf_dist_forward_nograd(x, w, ref, 1)
    with torch.cuda.stream(s):
        E.inf_dist_forward_nograd(x, w, out, 1)
    s.synchronize()
    torch.cuda.synchronize()
    assert torch.equal(out, ref)
    np.testing.assert_allclose(out.cpu().numpy()[:, :, 0],
                               (x.cpu()[:, None, :, 0] - w.cpu()[None]).abs().amax(-1).clamp(min=1e-10).numpy(), rtol=0, atol=0)
