"""The library without Python: tests/abi/c_driver (C++ over include/brokefish_hip.h and the HIP
runtime, built by the build step) reads packed blobs and positions from files, runs move
generation -> evaluator -> expansion through the C-ABI on its own stream and writes the outputs;
they must be the bits the Python binding returns for the same files."""
import os
import subprocess

import numpy as np
import pytest
import torch

from brokefish_amd import encoder_impl, positions
from brokefish_amd.net import BrokefishNet

pytestmark = pytest.mark.gpu
DRIVER = os.path.join(os.path.dirname(os.path.abspath(__file__)), "abi", "c_driver")


@pytest.mark.parametrize("n,n_value", [(77, 1), (700, 3)])
def test_c_host_program_returns_the_python_bindings_bits(tmp_path, n, n_value):
    if not os.path.exists(DRIVER):
        pytest.fail("tests/abi/c_driver is not built: run __graft_entry__.build()")
    torch.manual_seed(0)
    net = BrokefishNet(n_value=n_value).eval().randomise_layers_(seed=6)
    model = encoder_impl("hip")(net, int8=True)
    b, c, r, m = positions.random_positions(n, plies=120, seed=60 + n)
    model.board_wstream.cpu().numpy().tofile(tmp_path / "wstream.bin")
    model.board_fparams.cpu().numpy().tofile(tmp_path / "fparams.bin")
    b.numpy().tofile(tmp_path / "boards.bin")
    c.numpy().tofile(tmp_path / "control.bin")
    r.numpy().tofile(tmp_path / "rep.bin")
    run = subprocess.run([DRIVER, str(tmp_path), str(n), str(n_value)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, run.stderr
    assert f"{n} positions, kernel {4 if n <= 256 else 5}" in run.stdout          # OCTO / DUO by size
    bd, cd, rd = b.cuda(), c.cuda(), r.cuda()
    edges = model.forward_expand(bd, cd, rd)                                      # the mask comes from the device
    assert torch.equal(edges["mask"].cpu(), m)
    p, q, v, best = model.forward_masked(bd, cd, rd, edges["mask"])
    load = lambda name, dtype: np.fromfile(tmp_path / name, dtype=dtype)
    assert (load("mask.bin", np.int64) == m.numpy().ravel()).all()
    assert (load("policy.bin", np.uint16) == p.cpu().numpy().view(np.uint16).ravel()).all()
    assert (load("promo.bin", np.uint16) == q.cpu().numpy().view(np.uint16).ravel()).all()
    assert (load("value.bin", np.uint32) == v.cpu().numpy().view(np.uint32)).all()
    assert (load("best.bin", np.int32) == best.cpu().numpy()).all()
    # the expansion walks the same legal entries whether the policy it is given is masked or raw
    assert (load("n_edges.bin", np.int32) == edges["n_edges"].cpu().numpy()).all()
    assert (load("edge_move.bin", np.int16) == edges["edge_move"].cpu().numpy().ravel()).all()
    assert (load("edge_prior.bin", np.uint16) == edges["edge_prior"].cpu().numpy().view(np.uint16).ravel()).all()


def test_c_host_program_reports_the_librarys_error_text(tmp_path):
    if not os.path.exists(DRIVER):
        pytest.fail("tests/abi/c_driver is not built: run __graft_entry__.build()")
    for name in ("wstream.bin", "fparams.bin", "boards.bin", "control.bin", "rep.bin"):
        (tmp_path / name).write_bytes(b"\0" * 64)
    run = subprocess.run([DRIVER, str(tmp_path), "1", "1"], capture_output=True, text=True, timeout=60)
    assert run.returncode == 1 and "not those of this shape" in run.stderr
