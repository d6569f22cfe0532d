"""The PyTorch extension module over the C-ABI (brokefish_amd._bf_torch): the counterpart of the
reference's pybind module (reference csrc/encoder.cu:1770-1876, :1905-1930)."""
import pytest
import torch

from brokefish_amd import encoder_impl, hip_impl, positions
from brokefish_amd.net import BrokefishNet


def test_extension_module_loads_and_exports_the_reference_modules_functions():
    ext = hip_impl.load_extension()
    for name in ("model_forward", "encoder_forward", "int8_q_max", "fp8_q_max", "profile_phases", "profile_phase_names", "kernel_choice"):
        assert hasattr(ext, name), name
    assert ext.int8_q_max() == (127.0, 255.0) == hip_impl.int8_q_max()
    assert ext.fp8_q_max() == 8.0
    assert ext.profile_phase_names()[-1] == "total" and "attention" in ext.profile_phase_names()
    # AUTO: eight wavefronts per position up to one position per compute unit, the throughput kernel above
    assert ext.kernel_choice(256, 8, 8, 1024, 1, 64, 0, 0, True) == 4
    assert ext.kernel_choice(256, 8, 8, 1024, 1, 4096, 0, 0, True) == 5     # two positions per workgroup
    assert ext.kernel_choice(256, 8, 8, 1024, 1, 4096, 1, 0, True) == 3     # e4m3: one position per workgroup, two workgroups per unit
    assert ext.kernel_choice(512, 16, 16, 2048, 1, 4096, 0, 0, True) == 4
    with pytest.raises(RuntimeError):
        ext.kernel_choice(384, 8, 12, 1536, 1, 64, 0, 0, True)
    # argument errors are Python RuntimeErrors before any device is touched
    z = torch.zeros(4, 32, dtype=torch.int16)
    with pytest.raises(RuntimeError, match="boards must be"):
        ext.model_forward(z, z, z, z, z, z, z, z, 256, 8, 8, 1024, 1e-5)


@pytest.mark.gpu
def test_extension_binding_returns_the_bits_of_the_ctypes_binding_on_the_current_stream():
    torch.manual_seed(0)
    net = BrokefishNet(n_value=3).eval().randomise_layers_(seed=2)
    b, c, r, m = (t.cuda() for t in positions.random_positions(333, plies=120, seed=9))
    act = (torch.arange(333, device="cuda") % 3 != 0)
    for kernel in ("auto", "twin", "octo", "duo", "board", "quad"):
        for fp8 in (False, True):
            kw = dict(fp8=True) if fp8 else dict(int8=True)
            te = encoder_impl("hip")(net, kernel=kernel, binding="torch", **kw)
            ct = encoder_impl("hip")(net, kernel=kernel, binding="ctypes", **kw)
            assert te.binding == "torch" and ct.binding == "ctypes"
            want = [t.clone() for t in ct.forward_masked(b, c, r, m)]
            side = torch.cuda.Stream()
            side.wait_stream(torch.cuda.current_stream())
            with torch.cuda.stream(side):          # the launch follows torch's current stream
                got = [t.clone() for t in te.forward_masked(b, c, r, m)]
            side.synchronize()
            for g, w in zip(got, want):
                assert torch.equal(g, w), (kernel, fp8)
            # the leaf flags reach the kernel through the extension as well
            for mod in (te, ct):
                mod.policy_out.fill_(7.0)
            pa = te.forward_full(b, c, r, active=act)[0].clone()
            pb = ct.forward_full(b, c, r, active=act)[0].clone()
            assert torch.equal(pa, pb) and (pa[~act] == 7.0).all()
    # the default is the extension module when it is built
    assert encoder_impl("hip")(net, int8=True).binding == "torch"
    # errors surface as RuntimeError with the library's message
    ext = hip_impl.load_extension()
    te = encoder_impl("hip")(net, int8=True, kernel="twin", binding="torch")
    te.forward_full(b, c, r)
    bad = torch.empty(10, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError, match="not the blobs of this shape"):
        ext.model_forward(b, c, r, bad, te.board_fparams, te.policy_out, te.promo_out, te.value_out,
                          256, 8, 8, 1024, 1e-5, n_value=3)
    with pytest.raises(RuntimeError, match="policy must be"):
        ext.model_forward(b, c, r, te.board_wstream, te.board_fparams, te.policy_out[:5], te.promo_out[:5], te.value_out[:5],
                          256, 8, 8, 1024, 1e-5)
    # the phase profile through the extension
    cyc = ext.profile_phases(b, c, r, te.board_wstream, te.board_fparams, te.policy_out, te.promo_out, te.value_out,
                             256, 8, 8, 1024, 1e-5, kernel=3, n_value=3)
    torch.cuda.synchronize()
    assert cyc.shape == (12,) and int(cyc[-1]) > 0


@pytest.mark.gpu
def test_encoder_forward_runs_the_stack_alone_in_place_on_every_kernel():
    """reference csrc/encoder.cu:1752-1764: encoder_forward(y, weights, alive, ...) overwrites y with
    the residual stream after the last layer; no board words, no heads, nothing allocated."""
    from oracle import emulated
    torch.manual_seed(0)
    net = BrokefishNet().eval().randomise_layers_(seed=2)
    sd = {k: v.detach() for k, v in net.state_dict().items()}
    ext = hip_impl.load_extension()
    b, c, r, _ = positions.random_positions(300, plies=100, seed=21)
    with torch.no_grad():
        x, alive = emulated.embed(sd, b, c, r)
    xd, ad = x.cuda(), alive.cuda()
    a8 = ad.to(torch.int8)                      # the mask may come as bool or as int8
    bd, cd, rd = b.cuda(), c.cuda(), r.cuda()
    for fp8 in (False, True):
        kw = dict(fp8=True) if fp8 else dict(int8=True)
        want = None
        for kernel in ("auto", "duo", "twin", "octo", "board", "quad"):
            mod = encoder_impl("hip")(net, kernel=kernel, **kw)
            # what the taps of a whole-model launch record after the last layer
            if want is None:
                want = mod.forward_taps(bd, cd, rd, want=["resid"])["resid"][:, -1].clone()
            quad = kernel == "quad"
            y = xd.clone()
            ws = torch.empty(mod._lib.bf_workspace_bytes(hip_impl.C.byref(mod._shape), 300), dtype=torch.uint8, device="cuda") if quad else None
            count = torch.cuda.memory_stats()["allocation.all.allocated"]
            ext.encoder_forward(y, mod.wstream if quad else mod.board_wstream, mod.fparams if quad else mod.board_fparams,
                                a8 if kernel == "duo" else ad, 256, 8, 8, 1024, 1e-5,
                                quant=1 if fp8 else 0, kernel=hip_impl.FusedEncoder.KERNELS[kernel], workspace=ws)
            assert torch.cuda.memory_stats()["allocation.all.allocated"] == count
            torch.cuda.synchronize()
            assert torch.equal(y, want), (kernel, fp8)
            # the class's encoder-only call is the same launch
            assert torch.equal(mod.forward(xd, ad), want)
    # argument errors
    mod = encoder_impl("hip")(net, int8=True)
    with pytest.raises(RuntimeError, match="y must be"):
        ext.encoder_forward(xd.half(), mod.board_wstream, mod.board_fparams, ad, 256, 8, 8, 1024, 1e-5)
    with pytest.raises(RuntimeError, match="alive must be"):
        ext.encoder_forward(xd.clone(), mod.board_wstream, mod.board_fparams, ad[:5], 256, 8, 8, 1024, 1e-5)


@pytest.mark.gpu
def test_two_evaluators_on_two_streams_and_two_host_threads_do_not_disturb_each_other():
    """The library keeps no state between calls but the per-thread error text: launches from two
    host threads on two streams (default priority), overlapping on the GPU, return what each
    evaluator returns alone.  Kernels that need no scratch buffer are used (the four-per-workgroup
    kernel's workspace belongs to its evaluator object, so that one is safe as well and is included)."""
    import threading
    torch.manual_seed(0)
    nets = [BrokefishNet().eval().randomise_layers_(seed=s) for s in (3, 4)]
    inputs = [tuple(t.cuda() for t in positions.random_positions(n, plies=120, seed=50 + i)) for i, n in enumerate((777, 200))]
    for kernel in ("auto", "quad"):
        models = [encoder_impl("hip")(net, int8=True, kernel=kernel) for net in nets]
        alone = [[t.clone() for t in m.forward_masked(*x)] for m, x in zip(models, inputs)]
        torch.cuda.synchronize()
        streams = [torch.cuda.Stream(), torch.cuda.Stream()]
        results, errors = [None, None], []

        def work(i):
            try:
                with torch.cuda.stream(streams[i]):
                    out = None
                    for _ in range(30):                      # long enough for the two loops to overlap
                        out = models[i].forward_masked(*inputs[i])
                    results[i] = [t.clone() for t in out]
                streams[i].synchronize()
            except Exception as e:                            # surfaced in the main thread below
                errors.append(e)
        for s in streams:
            s.wait_stream(torch.cuda.current_stream())
        threads = [threading.Thread(target=work, args=(i,)) for i in range(2)]
        for th in threads:
            th.start()
        for th in threads:
            th.join(timeout=120)
        assert not errors and all(not th.is_alive() for th in threads), errors
        torch.cuda.synchronize()
        for got, want in zip(results, alone):
            for g, w in zip(got, want):
                assert torch.equal(g, w), kernel
