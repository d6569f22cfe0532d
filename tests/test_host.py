"""Host-side logic that needs no GPU: the C-ABI surface, the weight packer, input checks."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

import brokefish_amd
from brokefish_amd import _build, hip_impl
from brokefish_amd.net import BrokefishNet

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_functions():
    text = open(os.path.join(ROOT, "include", "brokefish_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(bf_[a-z0-9_]+)\s*\(", text)))


def test_library_loads_and_exports_every_declared_symbol():
    assert os.path.exists(_build.HIP_LIB), "build first: python -c 'import __graft_entry__ as g; g.build()'"
    lib = ctypes.CDLL(_build.HIP_LIB)
    names = _declared_functions()
    assert {"bf_model_forward", "bf_wstream_bytes", "bf_fparams_floats", "bf_int8_q_max",
            "bf_last_error", "bf_time_kernel_ms", "bf_layer_stride_floats", "bf_workspace_bytes",
            "bf_profile_phases", "bf_profile_phase_count", "bf_profile_phase_name", "bf_fp8_q_max"} <= set(names)
    for n in names:
        assert hasattr(lib, n), f"{n} is declared in include/brokefish_hip.h but not exported"


def test_header_is_plain_c_and_a_c_client_links_and_gets_statuses(tmp_path):
    # a C99 program (no C++, no torch, no Python) built against the header and the library:
    # every argument error must come back as a status before any device is touched
    import shutil
    import subprocess
    if shutil.which("gcc") is None:
        pytest.skip("no gcc")
    exe = tmp_path / "abi_check"
    lib_dir = os.path.dirname(_build.HIP_LIB)
    subprocess.run(["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", "-I", os.path.join(ROOT, "include"),
                    os.path.join(ROOT, "tests", "abi", "abi_check.c"), "-o", str(exe), "-L", lib_dir,
                    "-lbrokefish_hip", f"-Wl,-rpath,{lib_dir}"], check=True, capture_output=True, text=True)
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert run.returncode == 0, (run.returncode, run.stdout, run.stderr)
    assert run.stdout.startswith("abi ok")


def test_interface_tag_ties_the_bindings_to_the_library():
    # a binding built for another version of the header must not reach the library: the ctypes
    # mirror of bf_eval_args is checked on load, the extension module compares its compiled-in tag
    lib = hip_impl.load_library()
    tag = lib.bf_abi_tag()
    header = open(os.path.join(ROOT, "include", "brokefish_hip.h")).read()
    assert tag >> 32 == int(re.search(r"#define BF_ABI_VERSION (\d+)", header).group(1))
    assert tag & 0xFFFFFFFF == ctypes.sizeof(hip_impl._Args)
    if os.path.exists(_build.TORCH_EXT):
        ext = hip_impl.load_extension()
        assert ext.abi_tag() == ext.library_abi_tag() == tag
    # building the library removes an extension module that was built against the previous one
    src = open(os.path.join(os.path.dirname(_build.__file__), "_build.py")).read()
    assert "os.remove(TORCH_EXT)" in src[src.index("def build_hip"):src.index("def build_chessgen")]


def test_constants_agree_between_host_and_library():
    # the counterpart of the reference's Python<->CUDA constant pin (tests/test_quant.py:233-269)
    assert hip_impl.int8_q_max() == (hip_impl.Q_MAX_S8, hip_impl.Q_MAX_U8) == (127.0, 255.0)
    assert hip_impl.fp8_q_max() == hip_impl.Q_MAX_E4M3 == 8.0
    lib = hip_impl.load_library()
    shape = hip_impl._Shape(256, 8, 8, 1024, 1, 1e-5)
    assert lib.bf_wstream_bytes(ctypes.byref(shape)) == (8 * 24 + 3) * 32768
    assert lib.bf_workspace_bytes(ctypes.byref(shape), 4096) == 4096 * 32768
    assert lib.bf_workspace_bytes(ctypes.byref(shape), 5) == 8 * 32768
    bad = hip_impl._Shape(512, 16, 16, 2048, 1, 1e-5)
    assert lib.bf_wstream_bytes(ctypes.byref(bad)) == 0 and lib.bf_fparams_floats(ctypes.byref(bad)) == 0


def test_null_arguments_are_rejected_without_a_launch():
    lib = hip_impl.load_library()
    a = hip_impl._Args()
    a.shape = hip_impl._Shape(256, 8, 8, 1024, 1, 1e-5)
    a.n = 4
    assert lib.bf_model_forward(ctypes.byref(a), None) == -1
    assert b"must not be NULL" in lib.bf_last_error()
    a.shape = hip_impl._Shape(512, 16, 16, 2048, 1, 1e-5)     # carried, but only by the board kernel
    assert lib.bf_model_forward(ctypes.byref(a), None) == -1
    assert b"board_wstream" in lib.bf_last_error()
    a.shape = hip_impl._Shape(384, 8, 12, 1536, 1, 1e-5)
    assert lib.bf_model_forward(ctypes.byref(a), None) == -2
    assert lib.bf_model_forward(None, None) == -1
    # the matrix-pipe probe rejects a missing buffer and a bad format before touching a device
    assert lib.bf_mfma_rate(0, None, 10, 1, None) == -1.0
    assert lib.bf_mfma_rate(7, ctypes.c_void_p(4096), 10, 1, None) == -1.0
    # so does the weight-stream probe: no buffer, a size that is not whole groups of loads
    assert lib.bf_stream_rate(None, 32768, 4, 1, ctypes.c_void_p(4096), None) == -1.0
    assert lib.bf_stream_rate(ctypes.c_void_p(4096), 1000, 4, 1, ctypes.c_void_p(4096), None) == -1.0


def test_kernel_choice_follows_shape_blobs_and_batch_size():
    lib = hip_impl.load_library()
    a = hip_impl._Args()
    a.shape = hip_impl._Shape(256, 8, 8, 1024, 1, 1e-5)
    a.wstream = a.fparams = a.board_wstream = a.board_fparams = 16      # only tested for NULL here
    cut = lib.bf_board_max_n()
    assert cut == 256                                                    # one position per compute unit
    for n, want in ((1, 4), (cut, 4), (cut + 1, 5), (4096, 5)):          # int8: OCTO up to the cut, DUO above
        a.n = n
        assert lib.bf_kernel_choice(ctypes.byref(a)) == want
    for forced in (1, 2, 3, 4, 5):
        a.n, a.kernel = 4096, forced
        assert lib.bf_kernel_choice(ctypes.byref(a)) == forced
    a.kernel, a.quant = 0, 1                                            # e4m3: OCTO up to the cut, TWIN above
    for n, want in ((1, 4), (cut, 4), (cut + 1, 3), (4096, 3)):
        a.n = n
        assert lib.bf_kernel_choice(ctypes.byref(a)) == want
    for forced in (1, 2, 3, 4, 5):
        a.kernel = forced
        assert lib.bf_kernel_choice(ctypes.byref(a)) == forced
    a.kernel, a.quant, a.board_wstream = 0, 0, None                     # no board blobs: always quad
    a.n = 1
    assert lib.bf_kernel_choice(ctypes.byref(a)) == 1
    a.shape = hip_impl._Shape(512, 16, 16, 2048, 1, 1e-5)               # the 512-wide network: OCTO at any size
    a.board_wstream = 16
    for n in (1, 100000):
        a.n = n
        assert lib.bf_kernel_choice(ctypes.byref(a)) == 4
    for forced, want in ((1, -2), (2, 2), (3, -2), (4, 4), (5, -2)):
        a.kernel = forced
        assert lib.bf_kernel_choice(ctypes.byref(a)) == want
    for forced in (0, 2, 4):                                            # ... and in int8 only
        a.kernel, a.quant = forced, 1
        assert lib.bf_kernel_choice(ctypes.byref(a)) < 0
    a.quant = 0
    a.kernel = 7
    assert lib.bf_kernel_choice(ctypes.byref(a)) == -1


def test_timing_experiments_cannot_reach_the_library():
    """The kernels' BF_EXP_* switches give wrong results by construction: the build refuses them,
    and the sources refuse to compile them without BF_TIMING_BUILD."""
    from brokefish_amd import _build
    assert not any("BF_EXP" in f or "BF_TIMING" in f for f in _build.HIPCC_FLAGS)
    for extra in (["-DBF_EXP_NOLOAD"], ["-DBF_TIMING_BUILD"]):
        with pytest.raises(ValueError):
            _build.build_hip(extra=extra)
    src = open(os.path.join(_build.CSRC, "bf_board.hip.h")).read()
    assert '#error "BF_EXP_* switches give wrong results' in src
    import re
    used = set(re.findall(r"BF_EXP_[A-Z0-9]+", src + open(os.path.join(_build.CSRC, "bf_duo.hip.h")).read()))
    guard = src[src.index("#if (defined(BF_EXP_"):src.index("#error")]
    assert used and all(u in guard for u in used), used


def test_board_packing_layout_and_sizes():
    torch.manual_seed(0)
    for d, heads, layers in ((256, 8, 2), (512, 16, 2)):
        f = 4 * d
        net = BrokefishNet(d_model=d, n_heads=heads, d_ff=f, n_layers=layers).eval().randomise_layers_()
        sd = net.state_dict()
        ws, fp = hip_impl.pack_network_board(sd, layers, d, f, 1)
        lib = hip_impl.load_library()
        shape = hip_impl._Shape(d, layers, heads, f, 1, 1e-5)
        assert ws.size == lib.bf_board_wstream_bytes(ctypes.byref(shape))
        assert fp.size == lib.bf_board_fparams_floats(ctypes.byref(shape))
        tw, kc, steps, nt = d // 128, d // 256, f // 512, d // 32
        bpw = 3 * tw * kc + tw * kc + steps * (4 * kc + 2 * tw)
        wave_blocks = layers * bpw + nt // 2 + 1                      # + one block of padding
        assert ws.size == 4 * wave_blocks * 8192
        assert (ws[(3 * wave_blocks - 1) * 8192:3 * wave_blocks * 8192] == 0).all()
        # wave 2, layer 1, first block: Q tile of its first head (tile 2 tw), chunk 0
        q_qkv, s_qkv = hip_impl.quantise_weights_int8(sd["encoder.layers.1.self_attn.in_proj_weight"])
        blk = ws[(2 * wave_blocks + bpw) * 8192:][:8192].view(np.int8).reshape(8, 64, 16)
        assert blk[3, 40, 9] == q_qkv[32 * 2 * tw + 8, 32 * 3 + 8 * 2 + 4 + 1]
        # its last block of the layer: ffn2 tile 2 tw + tw - 1, last chunk
        q_ff2, s_ff2 = hip_impl.quantise_weights_int8(sd["encoder.layers.1.linear2.weight"])
        blk = ws[(2 * wave_blocks + 2 * bpw - 1) * 8192:][:8192].view(np.int8).reshape(8, 64, 16)
        assert blk[0, 1, 0] == q_ff2[32 * (3 * tw - 1) + 1, 256 * (2 * steps - 1)]
        # first feed-forward block of step 1: hidden tile 16 + 4 * 2, chunk 0
        q_ff1, s_ff1 = hip_impl.quantise_weights_int8(sd["encoder.layers.1.linear1.weight"])
        k_ff = 4 * tw * kc + (4 * kc + 2 * tw)
        blk = ws[(2 * wave_blocks + bpw + k_ff) * 8192:][:8192].view(np.int8).reshape(8, 64, 16)
        assert blk[1, 33, 2] == q_ff1[32 * 24 + 1, 32 + 4 + 2]
        # parameter slice of wave 2, layer 1
        cw = 32 * tw
        a_floats = 6 * cw + 16
        b_floats = 3 * cw + 128 * steps + (f // 256) * cw + 32
        pw = a_floats + b_floats
        sl = fp[(2 * layers + 1) * pw:(2 * layers + 2) * pw]
        own = slice(2 * cw, 3 * cw)
        assert (sl[:cw] == sd["encoder.layers.1.norm1.weight"].numpy()[own]).all()
        assert (sl[4 * cw:5 * cw] == sd["encoder.layers.1.self_attn.in_proj_bias"].numpy()[2 * d:][own]).all()
        assert sl[6 * cw + 2 * tw] == s_qkv[(2 * d + 32 * 2 * tw) // 128]            # sw_v of its first head
        # part B: ln2 gamma, ln2 beta, b_ffn2, 32 weight scales, then b_ffn1 and 128 * sum(w)
        pb = sl[a_floats:]
        assert (pb[:cw] == sd["encoder.layers.1.norm2.weight"].numpy()[own]).all()
        assert (pb[2 * cw:3 * cw] == sd["encoder.layers.1.linear2.bias"].numpy()[own]).all()
        assert pb[3 * cw + 5] == s_ff1[(512 + 256 + 32) // 128]                      # step 1, its second hidden tile
        assert pb[3 * cw + 16 + 1] == s_ff2[(32 * (2 * tw + 1)) // 128]
        b1 = sd["encoder.layers.1.linear1.bias"].numpy()
        t0 = 3 * cw + 32
        assert (pb[t0:t0 + 128] == b1[256:384]).all() and (pb[t0 + 128:t0 + 256] == b1[768:896]).all()
        wsum = pb[t0 + 128 * steps:][: (f // 256) * cw].view(np.int32).reshape(f // 256, cw)
        assert (wsum[3] == 128 * q_ff2[own, 768:1024].astype(np.int32).sum(1)).all()
        assert pb.size == b_floats
        tail = fp[4 * layers * pw:]
        assert (tail[:64 * d] == sd["emb_square.weight"].numpy().reshape(-1)).all() and tail.size == (64 + 12 + 4 + 101 + 3 + 2) * d


def test_packed_blocks_decode_back():
    # re-derive the fragment index independently of the packer (the reference does the same for
    # its own layout, tests/test_quant.py::test_the_packed_layout_decodes_back)
    rng = np.random.default_rng(0)
    wq = rng.integers(-127, 128, size=(768, 1024), dtype=np.int8)
    blk = hip_impl.pack_int8_block(wq, n_tile=5, k0=512).view(np.int8)
    assert blk.shape == (8, 64, 16)
    for s, lane, r in [(0, 0, 0), (3, 17, 5), (7, 63, 15), (2, 40, 9), (5, 32, 0)]:
        o, g = lane % 32, lane // 32
        col = 512 + 32 * s + 8 * (r // 4) + 4 * g + (r % 4)
        assert blk[s, lane, r] == wq[32 * 5 + o, col]
    # every element of the 32 x 256 tile appears exactly once
    tile = wq[160:192, 512:768]
    assert sorted(blk.reshape(-1).tolist()) == sorted(tile.reshape(-1).tolist())
    head = rng.standard_normal((96, 256)).astype(np.float32)
    ht = hip_impl.pack_head_tile(head, 2)
    assert ht.shape == (8, 4, 64, 4)
    assert ht[3, 2, 45, 1] == head[64 + 13, 32 * 3 + 8 * 2 + 4 * 1 + 1]


def test_pack_network_layout_and_sizes():
    torch.manual_seed(0)
    net = BrokefishNet(n_layers=2).eval().randomise_layers_()
    sd = net.state_dict()
    ws, fp = hip_impl.pack_network(sd, 2, 256, 1024, 1)
    lib = hip_impl.load_library()
    shape = hip_impl._Shape(256, 2, 8, 1024, 1, 1e-5)
    assert ws.size == lib.bf_wstream_bytes(ctypes.byref(shape)) and ws.dtype == np.uint8
    assert fp.size == lib.bf_fparams_floats(ctypes.byref(shape)) and fp.dtype == np.float32
    layer_floats = (fp.size - (64 + 12 + 4 + 101 + 3 + 2) * 256) // 2
    assert layer_floats == lib.bf_layer_stride_floats(ctypes.byref(shape)) and layer_floats % 1024 == 0
    l1 = fp[layer_floats:2 * layer_floats]
    assert (l1[:256] == sd["encoder.layers.1.norm1.weight"].numpy()).all()
    assert (l1[512:1280] == sd["encoder.layers.1.self_attn.in_proj_bias"].numpy()).all()
    q2, s2 = hip_impl.quantise_weights_int8(sd["encoder.layers.1.linear2.weight"])
    wsum = l1[9 * 256 + 1024: 9 * 256 + 1024 + 4 * 256].view(np.int32).reshape(4, 256)
    assert (wsum[2] == 128 * q2[:, 512:768].astype(np.int32).sum(1)).all()
    sw = l1[9 * 256 + 1024 + 4 * 256:9 * 256 + 1024 + 4 * 256 + 24]
    assert (l1[9 * 256 + 1024 + 4 * 256 + 24:] == 0).all()
    # one ffn2 entry per (128-row block, k-chunk); the int8 scale covers the whole reduction
    assert (sw[16:24] == np.repeat(s2, 4)).all()
    assert (fp[2 * layer_floats:2 * layer_floats + 64 * 256] == sd["emb_square.weight"].numpy().reshape(-1)).all()
    # second block of layer 0 is the K tile of head 0: rows 256..287 of in_proj
    q_qkv, _ = hip_impl.quantise_weights_int8(sd["encoder.layers.0.self_attn.in_proj_weight"])
    assert (ws[8192:16384].view(np.int8).reshape(8, 64, 16)[1, 35, 6] == q_qkv[256 + 3, 32 + 8 * 1 + 4 + 2])


def test_registry_and_input_checks():
    assert brokefish_amd.IMPLEMENTATIONS == ("hip",)
    cls = brokefish_amd.encoder_impl("hip")
    assert cls is hip_impl.FusedEncoder
    with pytest.raises(ValueError):
        brokefish_amd.encoder_impl("cuda")
    chk = cls._check_inputs
    b = torch.zeros(4, 32, dtype=torch.int16)
    c = torch.ones(4, dtype=torch.int16)
    r = torch.zeros(4, dtype=torch.uint8)
    # the rejections the reference pins (tests/test_b2.py:325-343)
    for bad in [(b.int(), c, r), (b[:, :31], c, r), (b, c.int(), r), (b, c[:3], r), (b, c, r.int()),
                (b, c, r[:2]), (b.reshape(-1), c, r), (b[:0], c[:0], r[:0])]:
        with pytest.raises(ValueError):
            chk(*bad)
    with pytest.raises(ValueError, match="GPU"):
        chk(b, c, r)            # right types, wrong device
    with pytest.raises(ValueError):
        chk(b, c, r, mask=torch.zeros(4, 32, dtype=torch.int32))


def test_constructor_rejections_do_not_need_a_gpu():
    net = BrokefishNet(n_layers=1)
    cls = hip_impl.FusedEncoder
    with pytest.raises(ValueError):
        cls(net, fp8=True, int8=True)                    # both quantise the same matmuls
    with pytest.raises(NotImplementedError):
        cls(net, int8=False)                             # the unquantised fp16 evaluator is not carried
    with pytest.raises(ValueError):
        cls(net, acc_dtype="bf16")
    with pytest.raises(ValueError):
        cls(object(), int8=True)                         # neither a network nor an encoder stack
    with pytest.raises(ValueError):
        cls(BrokefishNet(d_model=128, n_heads=4, d_ff=512, n_layers=1), int8=True)
    if not torch.cuda.is_available():
        with pytest.raises(RuntimeError, match="no GPU"):
            cls(net, int8=True)
        with pytest.raises(RuntimeError, match="no GPU"):
            cls(net, fp8=True)


def test_net_matches_reference_parameter_count_and_keys():
    net = BrokefishNet()
    assert sum(p.numel() for p in net.parameters()) == 6_383_360     # docs/reference/spec.md:328-331
    keys = set(net.state_dict())
    for k in ["emb_square.weight", "emb_type_special.weight", "emb_color_turn.weight", "emb_clock.weight",
              "emb_rep.weight", "encoder.layers.7.self_attn.in_proj_weight", "encoder.layers.0.linear2.bias",
              "encoder.layers.3.norm2.weight", "norm_f.bias", "policy.weight", "promo.weight", "value.weight"]:
        assert k in keys
    l0, l7 = net.encoder.layers[0], net.encoder.layers[7]
    assert torch.equal(l0.linear1.weight, l7.linear1.weight)          # deep-copied layers at init
    net.randomise_layers_()
    assert not torch.equal(l0.linear1.weight, l7.linear1.weight)
