"""The entry point that allocates nothing: bf_model_forward_static, through the C-ABI.

It runs the four-positions-per-workgroup kernel with the workspace in the library's static device
array instead of a caller-provided buffer.  Checked bit for bit against bf_model_forward on the same
kernel, on two calls in a row (the second with fewer positions, so the array still holds the first
call's contents), and the size limit must be rejected with a clear message.
"""
import ctypes as C

import pytest
import torch

from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet

pytestmark = pytest.mark.gpu


def _outputs(n, dev):
    return (torch.full((n, 32, 64), 7.0, dtype=torch.float16, device=dev),
            torch.full((n, 32, 4), 7.0, dtype=torch.float16, device=dev),
            torch.full((n,), 7.0, dtype=torch.float32, device=dev),
            torch.full((n,), -7, dtype=torch.int32, device=dev))


def test_static_workspace_entry_point_matches_the_allocating_one():
    torch.manual_seed(0)
    net = BrokefishNet().eval().randomise_layers_(seed=5)
    model = encoder_impl("hip")(net, int8=True, kernel="quad")
    lib = model._lib
    lib.bf_model_forward_static.restype = C.c_int
    lib.bf_model_forward_static.argtypes = [C.c_void_p, C.c_void_p]
    stream = C.c_void_p(torch.cuda.current_stream(model.device).cuda_stream)
    # set-up: the first call on a device looks the array's address up, which is when the runtime
    # materialises the library's device globals there; from then on the free memory must not move
    b, c, r, m = (t.cuda() for t in positions.random_positions(4, plies=20, seed=2))
    p, q, v, best = _outputs(4, model.device)
    assert lib.bf_model_forward_static(C.byref(model._args(b, c, r, m, p, q, v, best)), stream) == 0, lib.bf_last_error().decode()
    torch.cuda.synchronize()
    for n, seed in ((1000, 3), (37, 4)):          # the second call is smaller and reuses the array
        b, c, r, m = (t.cuda() for t in positions.random_positions(n, plies=120, seed=seed))
        want = [t.clone() for t in model.forward_masked(b, c, r, m)]
        p, q, v, best = _outputs(n, model.device)
        args = model._args(b, c, r, m, p, q, v, best)
        args.workspace, args.workspace_bytes = None, 0      # ignored by this entry point
        free_before = torch.cuda.mem_get_info(model.device)[0]
        rc = lib.bf_model_forward_static(C.byref(args), stream)
        assert rc == 0, lib.bf_last_error().decode()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info(model.device)[0] == free_before, "the call changed the device's free memory"
        for name, got, ref in zip(("policy", "promo", "value", "best"), (p, q, v, best), want):
            assert torch.equal(got, ref), f"n={n}: {name} differs from bf_model_forward"
    # beyond the static array: rejected, nothing launched
    n = 1025
    b, c, r, m = (t.cuda() for t in positions.random_positions(n, plies=10, seed=1))
    p, q, v, best = _outputs(n, model.device)
    args = model._args(b, c, r, m, p, q, v, best)
    assert lib.bf_model_forward_static(C.byref(args), stream) == -1
    assert b"BF_STATIC_MAX_N" in lib.bf_last_error()
    torch.cuda.synchronize()
    assert (v == 7.0).all()
    # a kernel that has no workspace is not this entry point's business
    args = model._args(b[:8], c[:8], r[:8], m[:8], p[:8], q[:8], v[:8], best[:8])
    args.kernel = 3
    assert lib.bf_model_forward_static(C.byref(args), stream) == -1
