"""``FusedEncoder`` for MI355X: the host side of the single-launch int8 evaluator.

Mirrors the reference class of the same name (brokefish/nn/cuda_impl.py:119-531): built
from a network, it snapshots the weights into device blobs once, owns its output
buffers, and ``forward_full(boards, control, rep)`` is one asynchronous kernel launch on
the current stream returning views of those buffers.

Differences from the reference class, all additive or forced by the parity target:

* the arithmetic reproduced is the reference's PyTorch int8 emulation
  (brokefish/nn/quant.py:246-305): fp32 activations, LayerNorm affine applied (not folded
  into the weights), raw weights quantised per 128 output rows, true division;
* ``forward_full`` takes an optional ``mask`` ([n,32] int64 legal-move words): illegal
  policy entries come back as -inf and ``best_move`` holds the masked argmax;
* ``out_dtype=torch.float32`` returns fp32 logits (parity runs); fp16 is the default and
  the contract the search expects (brokefish/search/cuda_impl.py:242-249).

There is no CPU path: if the HIP library is missing or no GPU is present, construction
raises.
"""
from __future__ import annotations

import ctypes as C
import os
from typing import Dict, Optional

import numpy as np
import torch

from . import _build

T, N_POLICY, N_PROMO = 32, 64, 4
BLOCK_N = 128            # weight-scale block, brokefish/nn/quant.py:82
Q_MAX_S8, Q_MAX_U8 = 127.0, 255.0   # brokefish/nn/quant.py:237-241
ROW_K = 256              # k-depth one e4m3 activation scale covers, brokefish/nn/quant.py:92
Q_MAX_E4M3 = 8.0         # what a row's / block's maximum maps to in e4m3, brokefish/nn/quant.py:105
E4M3_MAX = 448.0         # largest finite e4m3 value, brokefish/nn/quant.py:73


class _Shape(C.Structure):
    _fields_ = [("d_model", C.c_int32), ("n_layers", C.c_int32), ("n_heads", C.c_int32),
                ("d_ff", C.c_int32), ("n_value", C.c_int32), ("eps", C.c_float)]


_TAP_PTRS = ["embed", "qa_qkv", "acc_qkv", "qa_out", "acc_out", "qa_ff1", "acc_ff1",
             "qa_ff2", "acc_ff2", "resid", "normed", "resid_last"]


ABI_VERSION = 6     # BF_ABI_VERSION of include/brokefish_hip.h that the structs below mirror


class _Taps(C.Structure):
    _fields_ = ([("x_in", C.c_void_p), ("layer_begin", C.c_int32), ("layer_end", C.c_int32)]
                + [(n, C.c_void_p) for n in _TAP_PTRS] + [("alive", C.c_void_p)])


class _ExpandArgs(C.Structure):
    _fields_ = [("policy", C.c_void_p), ("promo", C.c_void_p), ("value", C.c_void_p), ("mask", C.c_void_p),
                ("boards", C.c_void_p), ("control", C.c_void_p), ("active", C.c_void_p), ("n", C.c_int64),
                ("max_edges", C.c_int32), ("logits_fp32", C.c_int32), ("edge_move", C.c_void_p),
                ("edge_prior", C.c_void_p), ("n_edges", C.c_void_p), ("count", C.c_void_p),
                ("dropped", C.c_void_p), ("node_value", C.c_void_p), ("leaf_index", C.c_void_p), ("leaf_count", C.c_void_p)]


class _Args(C.Structure):
    _fields_ = [("boards", C.c_void_p), ("control", C.c_void_p), ("rep", C.c_void_p),
                ("mask", C.c_void_p), ("n", C.c_int64), ("shape", _Shape),
                ("wstream", C.c_void_p), ("fparams", C.c_void_p),
                ("policy", C.c_void_p), ("promo", C.c_void_p), ("value", C.c_void_p),
                ("best_move", C.c_void_p), ("out_fp32", C.c_int32), ("quant", C.c_int32),
                ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t), ("taps", C.POINTER(_Taps)),
                ("board_wstream", C.c_void_p), ("board_fparams", C.c_void_p), ("active", C.c_void_p),
                ("kernel", C.c_int32), ("value_mode", C.c_int32), ("leaf_index", C.c_void_p), ("leaf_count", C.c_void_p)]


_lib = None


def load_library():
    """The C-ABI library, loaded once.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        path = os.environ.get("BROKEFISH_HIP_LIB", _build.HIP_LIB)   # override: A/B of two builds
        if not os.path.exists(path):
            raise RuntimeError(
                f"{path} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(hipcc, gfx950). There is no fallback path.")
        L = C.CDLL(path)
        L.bf_model_forward.restype = C.c_int
        L.bf_model_forward.argtypes = [C.POINTER(_Args), C.c_void_p]
        L.bf_time_kernel_ms.restype = C.c_double
        L.bf_time_kernel_ms.argtypes = [C.POINTER(_Args), C.c_void_p, C.c_int, C.c_int]
        L.bf_last_error.restype = C.c_char_p
        L.bf_wstream_bytes.restype = C.c_size_t
        L.bf_wstream_bytes.argtypes = [C.POINTER(_Shape)]
        L.bf_fparams_floats.restype = C.c_size_t
        L.bf_fparams_floats.argtypes = [C.POINTER(_Shape)]
        L.bf_workspace_bytes.restype = C.c_size_t
        L.bf_workspace_bytes.argtypes = [C.POINTER(_Shape), C.c_int64]
        L.bf_layer_stride_floats.restype = C.c_size_t
        L.bf_layer_stride_floats.argtypes = [C.POINTER(_Shape)]
        L.bf_profile_phases.restype = C.c_int
        L.bf_profile_phases.argtypes = [C.POINTER(_Args), C.c_void_p, C.c_void_p]
        L.bf_profile_phase_count.restype = C.c_int
        L.bf_profile_phase_name.restype = C.c_char_p
        L.bf_profile_phase_name.argtypes = [C.c_int]
        L.bf_int8_q_max.argtypes = [C.POINTER(C.c_double), C.POINTER(C.c_double)]
        L.bf_fp8_q_max.restype = C.c_double
        L.bf_board_wstream_bytes.restype = C.c_size_t
        L.bf_board_wstream_bytes.argtypes = [C.POINTER(_Shape)]
        L.bf_board_fparams_floats.restype = C.c_size_t
        L.bf_board_fparams_floats.argtypes = [C.POINTER(_Shape)]
        L.bf_expand.restype = C.c_int
        L.bf_expand.argtypes = [C.POINTER(_ExpandArgs), C.c_void_p]
        L.bf_movegen.restype = C.c_int
        L.bf_movegen.argtypes = [C.c_void_p, C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
        L.bf_compact_leaves.restype = C.c_int
        L.bf_compact_leaves.argtypes = [C.c_void_p, C.c_int64, C.c_void_p, C.c_void_p, C.c_void_p]
        L.bf_board_max_n.restype = C.c_int64
        L.bf_kernel_choice.restype = C.c_int
        L.bf_kernel_choice.argtypes = [C.POINTER(_Args)]
        L.bf_mfma_rate.restype = C.c_double
        L.bf_mfma_rate.argtypes = [C.c_int, C.c_void_p, C.c_int, C.c_int, C.c_void_p]
        L.bf_stream_rate.restype = C.c_double
        L.bf_stream_rate.argtypes = [C.c_void_p, C.c_size_t, C.c_int, C.c_int, C.c_void_p, C.c_void_p]
        L.bf_quant_probe.restype = C.c_int
        L.bf_quant_probe.argtypes = [C.c_int, C.c_void_p, C.c_float, C.c_int64, C.c_void_p, C.c_void_p]
        L.bf_abi_tag.restype = C.c_uint64
        # the ctypes mirror of bf_eval_args must be the struct the library was compiled with: a
        # shorter one would make the library read pointers from beyond it
        if (L.bf_abi_tag() >> 32) != ABI_VERSION:
            raise RuntimeError(f"{path} carries interface version {L.bf_abi_tag() >> 32}, this binding is written for "
                               f"{ABI_VERSION}: rebuild the library (`__graft_entry__.build()`)")
        if (L.bf_abi_tag() & 0xFFFFFFFF) != C.sizeof(_Args):
            raise RuntimeError(f"{path} was built with a bf_eval_args of {L.bf_abi_tag() & 0xFFFFFFFF} bytes, this binding "
                               f"passes {C.sizeof(_Args)}: rebuild the library (`__graft_entry__.build()`)")
        _lib = L
    return _lib


_ext = None


def load_extension():
    """The PyTorch extension module over the same library (``brokefish_amd._bf_torch``: tensors in,
    launch on the current stream; the counterpart of the reference's extension module,
    csrc/encoder.cu:1905-1930).  Raises if it has not been built."""
    global _ext
    if _ext is None:
        load_library()
        try:
            from . import _bf_torch
        except ImportError as e:
            raise RuntimeError(f"the PyTorch extension module is not built ({e}); build it with "
                               "`python -c 'import __graft_entry__ as g; g.build()'`") from e
        # the module was compiled against one version of the header and is linked to whatever
        # library file is in the tree now: refuse a pair that does not belong together
        if _bf_torch.abi_tag() != _bf_torch.library_abi_tag():
            raise RuntimeError("brokefish_amd/_bf_torch.so was built for another version of libbrokefish_hip.so "
                               f"(interface tag {_bf_torch.abi_tag():#x} against {_bf_torch.library_abi_tag():#x}): "
                               "rebuild it (`brokefish_amd._build.build_torch_ext()`) or use binding='ctypes'")
        _ext = _bf_torch
    return _ext


def extension_available() -> bool:
    """Whether the default binding is the extension module.  The module is linked against the
    in-tree library, so a ``BROKEFISH_HIP_LIB`` override (another build of the library) selects
    the ctypes binding, which loads the named file."""
    return os.path.exists(_build.TORCH_EXT) and "BROKEFISH_HIP_LIB" not in os.environ


def int8_q_max():
    """(s8, u8) quantisation maxima compiled into the library."""
    a, b = C.c_double(), C.c_double()
    load_library().bf_int8_q_max(C.byref(a), C.byref(b))
    return a.value, b.value


def fp8_q_max() -> float:
    """The e4m3 quantisation maximum compiled into the library."""
    return float(load_library().bf_fp8_q_max())


def mfma_rate(fmt: str = "int8", iters: int = 20000, reps: int = 5, device="cuda") -> float:
    """Measured rate of the matrix pipe in TOP/s for the MFMA instruction of ``fmt`` ("int8" or
    "e4m3"): register-resident independent chains on every compute unit, no memory traffic in
    the loop (the method of reference docs/ledger/perf.md:616-642).  Synchronises."""
    L = load_library()
    scratch = torch.zeros(1024, dtype=torch.int32, device=device)
    with torch.cuda.device(scratch.device):
        rate = L.bf_mfma_rate({"int8": 0, "e4m3": 1}[fmt], scratch.data_ptr(), iters, reps,
                              torch.cuda.current_stream().cuda_stream)
    if rate < 0:
        raise RuntimeError(f"bf_mfma_rate: {L.bf_last_error().decode()}")
    return float(rate)


def stream_rate(nbytes: int, workgroups: int = 4096, reps: int = 3, device="cuda") -> float:
    """Measured rate in TB/s at which ``workgroups`` workgroups can each stream the same ``nbytes``
    (rounded up to a multiple of 32 KiB) out of the cache hierarchy with nothing else to do: the
    ceiling for the evaluator's weight traffic, whose every position reads the whole network.
    Synchronises."""
    L = load_library()
    nbytes = -(-int(nbytes) // 32768) * 32768
    buf = torch.zeros(nbytes // 4, dtype=torch.int32, device=device)
    sink = torch.zeros(64, dtype=torch.int32, device=device)
    with torch.cuda.device(buf.device):
        rate = L.bf_stream_rate(buf.data_ptr(), nbytes, workgroups, reps, sink.data_ptr(),
                                torch.cuda.current_stream().cuda_stream)
    if rate < 0:
        raise RuntimeError(f"bf_stream_rate: {L.bf_last_error().decode()}")
    return float(rate)


def movegen(boards, control, out=None):
    """Legal-move words on the device (the reference's ``env.movegen``, docs/reference/spec.md:152-172):
    ``boards [n,32]`` int16, ``control [n]`` int16 on the GPU -> ``(mask [n,32] int64, in_check [n] bool)``.
    ``out`` reuses a pair returned earlier.  Asynchronous on the current stream."""
    n = boards.shape[0]
    if boards.shape != (n, T) or boards.dtype is not torch.int16 or control.shape != (n,) or control.dtype is not torch.int16:
        raise ValueError("boards must be [n,32] int16 and control [n] int16")
    if not boards.is_cuda or not control.is_cuda:
        raise ValueError("boards and control must be on the GPU")
    if not boards.is_contiguous() or not control.is_contiguous():
        raise ValueError("boards and control must be contiguous")
    if out is None:
        out = (torch.empty(n, T, dtype=torch.int64, device=boards.device),
               torch.empty(n, dtype=torch.bool, device=boards.device))
    mask, chk = out
    if mask.shape != (n, T) or mask.dtype is not torch.int64 or chk.shape != (n,) or chk.dtype is not torch.bool:
        raise ValueError("`out` was made for another n")
    lib = load_library()
    with torch.cuda.device(boards.device):       # the launch goes to the current device
        rc = lib.bf_movegen(boards.data_ptr(), control.data_ptr(), n, mask.data_ptr(), chk.data_ptr(),
                            C.c_void_p(torch.cuda.current_stream(boards.device).cuda_stream))
    if rc:
        raise RuntimeError(f"bf_movegen failed ({rc}): {lib.bf_last_error().decode()}")
    return mask, chk


def _check_leaves(leaves, n, device):
    """(leaf_index [>= n] int32, leaf_count [1] int32) on ``device``, as :func:`compact_leaves` returns them."""
    index, count = leaves
    if index.dtype is not torch.int32 or count.dtype is not torch.int32 or index.dim() != 1 or index.shape[0] < n or \
            count.numel() != 1 or index.device != device or count.device != device or not index.is_contiguous():
        raise ValueError(f"leaves must be (index [{n}] int32, count [1] int32) on {device}")
    return index, count


def quant_probe(x, scale: float, mode: str = "s8"):
    """The kernels' row quantiser on its own (``bf_quant_probe``): ``x`` float32 on the GPU, its
    length a multiple of 4 -> the operand bytes for activation scale ``scale``.  ``mode``: "s8"
    (signed int8), "u8_relu" (the unsigned hidden-row quantiser with the ReLU folded in) or "e4m3"."""
    modes = {"s8": 0, "u8_relu": 1, "e4m3": 2}
    if mode not in modes or x.dtype is not torch.float32 or not x.is_cuda or x.dim() != 1 or x.numel() % 4:
        raise ValueError("x must be a float32 vector on the GPU with a multiple of 4 elements; mode one of " + ", ".join(modes))
    x = x.contiguous()
    out = torch.empty(x.numel(), dtype=torch.uint8, device=x.device)
    lib = load_library()
    with torch.cuda.device(x.device):
        rc = lib.bf_quant_probe(modes[mode], x.data_ptr(), float(scale), x.numel(), out.data_ptr(),
                                C.c_void_p(torch.cuda.current_stream(x.device).cuda_stream))
    if rc:
        raise RuntimeError(f"bf_quant_probe failed ({rc}): {lib.bf_last_error().decode()}")
    return out


def compact_leaves(flags, out=None):
    """The search's leaf flags ([n] uint8 or bool on the GPU, brokefish/search/cuda_impl.py:137-145)
    compacted on the device into ``(leaf_index [n] int32, leaf_count [1] int32)``: the numbers of
    the flagged positions in ascending order and how many there are -- the "compacted list plus a
    count" of the reference's design retrospective (docs/journal/2026-08-09-kernel-design-
    retrospective.md:140-154).  ``forward_full(..., leaves=)`` and ``expand_edges(..., leaves=)``
    take the pair; nothing returns to the host.  ``out`` reuses a pair returned earlier."""
    if flags.dim() != 1 or flags.dtype not in (torch.uint8, torch.bool) or not flags.is_cuda:
        raise ValueError("flags must be [n] uint8 or bool on the GPU")
    n = flags.shape[0]
    flags = flags.contiguous().view(torch.uint8)
    if out is None:
        out = (torch.zeros(n, dtype=torch.int32, device=flags.device), torch.zeros(1, dtype=torch.int32, device=flags.device))
    index, count = _check_leaves(out, n, flags.device)
    lib = load_library()
    with torch.cuda.device(flags.device):
        rc = lib.bf_compact_leaves(flags.data_ptr(), n, index.data_ptr(), count.data_ptr(),
                                   C.c_void_p(torch.cuda.current_stream(flags.device).cuda_stream))
    if rc:
        raise RuntimeError(f"bf_compact_leaves failed ({rc}): {lib.bf_last_error().decode()}")
    return index, count


def expand_edges(policy, promo, value, mask, boards, control, max_edges: int = 96, active=None, out=None, leaves=None):
    """The search's expand step on the device, behind the evaluator (docs/reference/search.md:616-636,
    brokefish/search/torch_impl.py:962-1033): logits + legal-move words -> edges in canonical order.

    ``policy [n,32,64]``, ``promo [n,32,4]`` (fp16 or fp32, as ``forward_full`` returns them),
    ``value [n]`` fp32, ``mask [n,32]`` int64, ``boards [n,32]`` int16, ``control [n]`` int16, all on
    the GPU.  Returns a dict: ``edge_move [n,E]`` int16 (slot*64+square | type << 11), ``edge_prior
    [n,E]`` fp16, ``n_edges [n]`` int32, ``count [n]`` int32 (candidates before truncation to
    ``max_edges``), ``dropped [n]`` fp32 (prior mass truncated away), ``node_value [n]`` fp16 =
    (value+1)/2.  ``active`` ([n] bool/uint8) leaves the rows where it is 0 untouched, and so does
    ``leaves`` (the pair :func:`compact_leaves` returns) for positions not in the list; ``out``
    reuses a dict returned earlier.  The launch is asynchronous on the current stream."""
    n = policy.shape[0]
    if policy.shape != (n, T, N_POLICY) or promo.shape != (n, T, N_PROMO) or policy.dtype != promo.dtype or \
            policy.dtype not in (torch.float16, torch.float32):
        raise ValueError("policy must be [n,32,64] and promo [n,32,4], both fp16 or both fp32")
    if value.shape != (n,) or value.dtype is not torch.float32:
        raise ValueError(f"value must be [{n}] float32")
    if mask.shape != (n, T) or mask.dtype is not torch.int64 or boards.shape != (n, T) or boards.dtype is not torch.int16 \
            or control.shape != (n,) or control.dtype is not torch.int16:
        raise ValueError("mask must be [n,32] int64, boards [n,32] int16, control [n] int16")
    if not 1 <= max_edges <= 255:
        raise ValueError("max_edges must be in [1, 255] (edge indices are uint8 in the search)")
    tensors = [policy, promo, value, mask, boards, control] + ([active] if active is not None else [])
    if any(not t.is_cuda for t in tensors):
        raise ValueError("all inputs must be on the GPU")
    dev = policy.device
    if out is None:
        out = {"edge_move": torch.zeros(n, max_edges, dtype=torch.int16, device=dev),
               "edge_prior": torch.zeros(n, max_edges, dtype=torch.float16, device=dev),
               "n_edges": torch.zeros(n, dtype=torch.int32, device=dev),
               "count": torch.zeros(n, dtype=torch.int32, device=dev),
               "dropped": torch.zeros(n, dtype=torch.float32, device=dev),
               "node_value": torch.zeros(n, dtype=torch.float16, device=dev)}
    elif out["edge_move"].shape != (n, max_edges):
        raise ValueError("`out` was made for another n or max_edges")
    a = _ExpandArgs()
    keep = [t.contiguous() for t in (policy, promo, value, mask, boards, control)]
    a.policy, a.promo, a.value, a.mask, a.boards, a.control = [t.data_ptr() for t in keep]
    if active is not None:
        act = active.to(torch.uint8).contiguous()
        if act.shape != (n,):
            raise ValueError(f"active must be [{n}]")
        a.active = act.data_ptr()
    if leaves is not None:
        if active is not None:
            raise ValueError("a compacted leaf list replaces the active flags: pass one of them")
        index, count = _check_leaves(leaves, n, dev)
        a.leaf_index, a.leaf_count = index.data_ptr(), count.data_ptr()
    a.n, a.max_edges, a.logits_fp32 = n, max_edges, int(policy.dtype is torch.float32)
    a.edge_move, a.edge_prior, a.n_edges = out["edge_move"].data_ptr(), out["edge_prior"].data_ptr(), out["n_edges"].data_ptr()
    a.count, a.dropped, a.node_value = out["count"].data_ptr(), out["dropped"].data_ptr(), out["node_value"].data_ptr()
    lib = load_library()
    with torch.cuda.device(dev):
        rc = lib.bf_expand(C.byref(a), C.c_void_p(torch.cuda.current_stream(dev).cuda_stream))
    if rc:
        raise RuntimeError(f"bf_expand failed ({rc}): {lib.bf_last_error().decode()}")
    # Temporaries made above (contiguous copies, the uint8 view of `active`) were allocated on the
    # current stream, where the launch is queued: the allocator hands their memory out again only
    # to work that this stream runs after the kernel, so no host wait is needed (and none would
    # be legal while a graph is being captured).
    return out


# --------------------------------------------------------------------------- #
# weight packing (host, once per weight generation)
# --------------------------------------------------------------------------- #

def quantise_weights_int8(w: torch.Tensor):
    """[N, K] fp32 -> (int8 [N, K], fp32 scale [N // 128]); one scale per 128 output rows
    over the whole reduction (brokefish/nn/quant.py:263-278)."""
    n, k = w.shape
    if n % BLOCK_N:
        raise ValueError(f"weight {tuple(w.shape)} does not tile into {BLOCK_N} rows")
    blocks = w.detach().float().cpu().reshape(n // BLOCK_N, BLOCK_N * k)
    amax = blocks.abs().amax(dim=1, keepdim=True)
    scale = torch.where(amax > 0, amax / Q_MAX_S8, torch.ones_like(amax))
    q = torch.round(blocks / scale).clamp(-Q_MAX_S8, Q_MAX_S8).to(torch.int8)
    return q.reshape(n, k).numpy(), scale.reshape(-1).numpy().astype(np.float32)


def quantise_weights_e4m3(w: torch.Tensor):
    """[N, K] fp32 -> (e4m3 bytes uint8 [N, K], fp32 scale [N // 128, K // 256]); one scale
    per 128-row x 256-deep block whose largest magnitude lands on 8
    (brokefish/nn/quant.py:208-224 with q_max = Q_MAX, tile_k = ROW_K)."""
    n, k = w.shape
    if n % BLOCK_N or k % ROW_K:
        raise ValueError(f"weight {tuple(w.shape)} does not tile into {BLOCK_N}x{ROW_K} blocks")
    blocks = w.detach().float().cpu().reshape(n // BLOCK_N, BLOCK_N, k // ROW_K, ROW_K)
    amax = blocks.abs().amax(dim=(1, 3), keepdim=True)
    scale = torch.where(amax > 0, amax / Q_MAX_E4M3, torch.ones_like(amax))
    q = (blocks / scale).clamp(-E4M3_MAX, E4M3_MAX).to(torch.float8_e4m3fn).reshape(n, k)
    return q.view(torch.uint8).numpy(), scale.reshape(n // BLOCK_N, k // ROW_K).numpy().astype(np.float32)


def _lane_tables():
    lane = np.arange(64)
    o, g = lane % 32, lane // 32
    r = np.arange(16)
    chan = 8 * (r[None, :] // 4) + 4 * g[:, None] + (r[None, :] % 4)   # [64,16]
    return o, g, chan


def pack_int8_block(wq: np.ndarray, n_tile: int, k0: int) -> np.ndarray:
    """One 8 KiB block: output tile ``n_tile``, the 256-wide k-chunk starting at ``k0``.
    Fragment s, lane 32g+o, byte r  <-  wq[32 n_tile + o][k0 + 32 s + ch(r, g)]."""
    o, _, chan = _lane_tables()
    rows = (32 * n_tile + o)[None, :, None]                       # [1,64,1]
    cols = k0 + 32 * np.arange(8)[:, None, None] + chan[None]     # [8,64,16]
    return np.ascontiguousarray(wq[rows, cols]).view(np.uint8)


def pack_head_tile(head: np.ndarray, m: int) -> np.ndarray:
    """One 32 KiB fp32 head tile: fragment (n, j), lane 32g+o  <-  head[32m+o][32n+8j+4g+0..3]."""
    d = head.shape[1]
    o, g, _ = _lane_tables()
    n = np.arange(d // 32)[:, None, None, None]
    j = np.arange(4)[None, :, None, None]
    i = np.arange(4)[None, None, None, :]
    cols = 32 * n + 8 * j + 4 * g[None, None, :, None] + i         # [NT,4,64,4]
    rows = (32 * m + o)[None, None, :, None]
    return np.ascontiguousarray(head[rows, cols], dtype=np.float32)


def pack_network(sd: Dict[str, torch.Tensor], n_layers: int, d: int, f: int, n_value: int,
                 layer_stride: Optional[int] = None, fmt: str = "int8"):
    """state_dict -> (wstream uint8 [bytes], fparams float32 [floats]) in the layouts of
    include/brokefish_hip.h.  ``layer_stride`` is the per-layer stride of fparams in floats
    (default: what the library reports for this shape); ``fmt`` is "int8" or "e4m3"."""
    if fmt not in ("int8", "e4m3"):
        raise ValueError(f"fmt = {fmt!r}, expected 'int8' or 'e4m3'")
    if layer_stride is None:
        shape = _Shape(d, n_layers, d // 32, f, n_value, 1e-5)
        layer_stride = int(load_library().bf_layer_stride_floats(C.byref(shape)))
        if not layer_stride:
            raise ValueError("the library has no kernel for this shape")
    nt, ft, kcf = d // 32, f // 32, f // 256
    get = lambda k: sd[k].detach().float().cpu()
    stream, fl = [], []
    for l in range(n_layers):
        p = f"encoder.layers.{l}."
        names = ("self_attn.in_proj_weight", "self_attn.out_proj.weight", "linear1.weight", "linear2.weight")
        if fmt == "int8":
            (q_qkv, s_qkv), (q_out, s_out), (q_ff1, s_ff1), (q_ff2, s_ff2) = \
                [quantise_weights_int8(get(p + nm)) for nm in names]
            # the scale table carries one ffn2 entry per (128-row block, k-chunk): the int8
            # scheme scales over the whole reduction, so its value repeats
            s_ff2 = np.repeat(s_ff2[:, None], kcf, axis=1)
            wsum = (128 * q_ff2.astype(np.int32).reshape(d, kcf, 256).sum(axis=2)).T   # [kcf, d]
        else:
            (q_qkv, s_qkv), (q_out, s_out), (q_ff1, s_ff1), (q_ff2, s_ff2) = \
                [quantise_weights_e4m3(get(p + nm)) for nm in names]
            wsum = np.zeros((kcf, d), np.int32)      # no unsigned operand in this format
        for h in range(nt):
            for part in range(3):
                stream.append(pack_int8_block(q_qkv, part * nt + h, 0))
        for n in range(nt):
            stream.append(pack_int8_block(q_out, n, 0))
        for n in range(ft):
            stream.append(pack_int8_block(q_ff1, n, 0))
        for n in range(nt):
            for c in range(kcf):
                stream.append(pack_int8_block(q_ff2, n, 256 * c))
        sw = np.concatenate([np.reshape(x, -1) for x in (s_qkv, s_out, s_ff1, s_ff2)]).astype(np.float32)
        sw = np.concatenate([sw, np.zeros((-len(sw)) % 4, np.float32)])
        layer = [get(p + "norm1.weight").numpy(), get(p + "norm1.bias").numpy(),
                 get(p + "self_attn.in_proj_bias").numpy(), get(p + "self_attn.out_proj.bias").numpy(),
                 get(p + "norm2.weight").numpy(), get(p + "norm2.bias").numpy(),
                 get(p + "linear1.bias").numpy(), get(p + "linear2.bias").numpy(),
                 np.ascontiguousarray(wsum, dtype=np.int32).view(np.float32).reshape(-1), sw]
        used = sum(x.size for x in layer)
        if used > layer_stride:
            raise ValueError("layer parameters do not fit the library's layer stride")
        fl += layer + [np.zeros(layer_stride - used, np.float32)]
    head = np.zeros((96, d), np.float32)
    head[:N_POLICY] = get("policy.weight").numpy()
    head[N_POLICY:N_POLICY + N_PROMO] = get("promo.weight").numpy()
    head[N_POLICY + N_PROMO:N_POLICY + N_PROMO + n_value] = get("value.weight").numpy()
    for m in range(3):
        stream.append(pack_head_tile(head, m).view(np.uint8))
    for name in ("emb_square", "emb_type_special", "emb_color_turn", "emb_clock", "emb_rep"):
        fl.append(get(name + ".weight").numpy())
    fl += [get("norm_f.weight").numpy(), get("norm_f.bias").numpy()]
    wstream = np.concatenate([s.reshape(-1) for s in stream])
    fparams = np.concatenate([np.asarray(x, dtype=np.float32).reshape(-1) for x in fl])
    return wstream, fparams


def pack_network_board(sd: Dict[str, torch.Tensor], n_layers: int, d: int, f: int, n_value: int,
                       fmt: str = "int8"):
    """state_dict -> (board_wstream uint8, board_fparams float32): the network in the order of the
    one-position-per-workgroup kernels (layout at the end of include/brokefish_hip.h), in the
    int8 or (256-wide network only) the e4m3 format.
    Wave w owns tiles tw*w .. tw*w+tw-1 of the width; each wave gets its own weight stream and
    its own slice of the side parameters."""
    if fmt not in ("int8", "e4m3") or (fmt == "e4m3" and d != 256):
        raise ValueError(f"fmt = {fmt!r} at width {d}: expected 'int8', or 'e4m3' at width 256")
    fp8 = fmt == "e4m3"
    nt, tw, kc, kcf = d // 32, d // 128, d // 256, f // 256
    cw = 32 * tw
    get = lambda k: sd[k].detach().float().cpu()
    quant = []
    for l in range(n_layers):
        p = f"encoder.layers.{l}."
        mats = [get(p + nm) for nm in
                ("self_attn.in_proj_weight", "self_attn.out_proj.weight", "linear1.weight", "linear2.weight")]
        if fp8:   # scales [N/128, K/256]: one k-chunk for the three 256-deep matmuls
            qs = [quantise_weights_e4m3(m) for m in mats]
            quant.append([(q, sc[:, 0]) for q, sc in qs[:3]] + [qs[3]])
        else:
            quant.append([quantise_weights_int8(m) for m in mats])
    head = np.zeros((128, d), np.float32)
    head[:N_POLICY] = get("policy.weight").numpy()
    head[N_POLICY:N_POLICY + N_PROMO] = get("promo.weight").numpy()
    head[N_POLICY + N_PROMO:N_POLICY + N_PROMO + n_value] = get("value.weight").numpy()
    stream, fl = [], []
    for w in range(4):
        own = slice(cw * w, cw * (w + 1))
        tiles = [tw * w + i for i in range(tw)]
        for l in range(n_layers):
            p = f"encoder.layers.{l}."
            (q_qkv, s_qkv), (q_out, s_out), (q_ff1, s_ff1), (q_ff2, s_ff2) = quant[l]
            for n in tiles:
                for part in range(3):
                    for c in range(kc):
                        stream.append(pack_int8_block(q_qkv, part * nt + n, 256 * c))
            for n in tiles:
                for c in range(kc):
                    stream.append(pack_int8_block(q_out, n, 256 * c))
            for st in range(f // 512):     # feed-forward in steps of 512 hidden channels, four tiles per wave
                for i in range(4):
                    for c in range(kc):
                        stream.append(pack_int8_block(q_ff1, 16 * st + 4 * w + i, 256 * c))
                for c in range(2 * st, 2 * st + 2):
                    for n in tiles:
                        stream.append(pack_int8_block(q_ff2, n, 256 * c))
            b_qkv = get(p + "self_attn.in_proj_bias").numpy()
            sw_a = np.zeros(16, np.float32)
            for i, n in enumerate(tiles):
                sw_a[i] = s_qkv[(32 * n) // BLOCK_N]
                sw_a[tw + i] = s_qkv[(d + 32 * n) // BLOCK_N]
                sw_a[2 * tw + i] = s_qkv[(2 * d + 32 * n) // BLOCK_N]
                sw_a[3 * tw + i] = s_out[(32 * n) // BLOCK_N]
            part_a = [get(p + "norm1.weight").numpy()[own], get(p + "norm1.bias").numpy()[own],
                      b_qkv[:d][own], b_qkv[d:2 * d][own], b_qkv[2 * d:][own],
                      get(p + "self_attn.out_proj.bias").numpy()[own], sw_a]
            hidden = np.concatenate([np.arange(512 * st + 128 * w, 512 * st + 128 * w + 128) for st in range(f // 512)])
            if fp8:
                wsum = np.zeros((kcf, cw), np.int32)      # no unsigned operand in this format
            else:
                wsum = (128 * q_ff2.astype(np.int32).reshape(d, kcf, 256).sum(axis=2)).T[:, own]   # [kcf, cw]
            sw_b = np.zeros(32, np.float32)
            for st in range(f // 512):
                for i in range(4):
                    sw_b[4 * st + i] = s_ff1[(512 * st + 128 * w + 32 * i) // BLOCK_N]
            for i, n in enumerate(tiles):
                if fp8:   # one scale per (own tile, k-chunk)
                    sw_b[16 + i * kcf:16 + (i + 1) * kcf] = s_ff2[(32 * n) // BLOCK_N]
                else:
                    sw_b[16 + i] = s_ff2[(32 * n) // BLOCK_N]
            part_b = [get(p + "norm2.weight").numpy()[own], get(p + "norm2.bias").numpy()[own],
                      get(p + "linear2.bias").numpy()[own], sw_b, get(p + "linear1.bias").numpy()[hidden],
                      np.ascontiguousarray(wsum, dtype=np.int32).view(np.float32).reshape(-1)]
            fl += part_a + part_b
        stream.append(pack_head_tile(head, w).view(np.uint8))
        stream.append(np.zeros(8192, np.uint8))     # the weight prefetch runs one block past the end
    for name in ("emb_square", "emb_type_special", "emb_color_turn", "emb_clock", "emb_rep"):
        fl.append(get(name + ".weight").numpy())
    fl += [get("norm_f.weight").numpy(), get("norm_f.bias").numpy()]
    wstream = np.concatenate([x.reshape(-1) for x in stream])
    fparams = np.concatenate([np.ascontiguousarray(x, dtype=np.float32).reshape(-1) for x in fl])
    return wstream, fparams


# --------------------------------------------------------------------------- #
# the evaluator object
# --------------------------------------------------------------------------- #

class FusedEncoder:
    """Boards to logits in one launch (see the module docstring)."""

    D, DFF, T, H = 256, 1024, 32, 8
    SHAPES = ((256, 1024, 8), (512, 2048, 16))     # (d_model, d_ff, heads) the library carries
    KERNELS = {"auto": 0, "quad": 1, "board": 2, "twin": 3, "octo": 4, "duo": 5}   # enum bf_kernel
    ACC_DTYPES = ("fp16", "fp32")
    VALUE_HEADS = ("king", "pooled", "prenorm")     # brokefish/nn/model.py:89
    n_value = 1
    vmode = 0
    rj_mode = 0

    def __init__(self, source, acc_dtype: str = "fp16", fp8: bool = False,
                 int8: Optional[bool] = None, two_boards: Optional[bool] = None,
                 int8_scheme: str = "all", out_dtype: torch.dtype = torch.float16,
                 device: Optional[torch.device] = None, kernel: str = "auto", binding: Optional[str] = None):
        if binding not in (None, "torch", "ctypes"):
            raise ValueError(f"binding must be 'torch' (the extension module), 'ctypes' or None, got {binding!r}")
        # how the launch reaches the library: the PyTorch extension module when it is built (the
        # default), else the same C-ABI through ctypes; both are one call into libbrokefish_hip.so
        self.binding = binding or ("torch" if extension_available() else "ctypes")
        if self.binding == "torch":
            load_extension()
        if kernel not in self.KERNELS:
            raise ValueError(f"kernel must be one of {tuple(self.KERNELS)}, got {kernel!r}")
        if acc_dtype not in self.ACC_DTYPES:
            raise ValueError(f"acc_dtype must be one of {self.ACC_DTYPES}, got {acc_dtype!r}")
        if fp8 and int8:
            raise ValueError("fp8 and int8 quantise the same matmuls; pick one")
        if int8 is False and not fp8:
            raise NotImplementedError(
                "this build carries the quantised evaluators only; construct with int8=True "
                "(the default here) or fp8=True")
        if int8_scheme != "all":
            raise NotImplementedError(
                "all four matmuls of every layer are int8 here, which is the reference's 'all' scheme")
        if out_dtype not in (torch.float16, torch.float32):
            raise ValueError(f"out_dtype must be float16 or float32, got {out_dtype}")
        # Like the reference class, this is built either from the whole network (boards in,
        # logits out) or from a bare pre-norm encoder stack (the backbone call only).
        net = source if hasattr(source, "encoder") and hasattr(source, "policy") else None
        if net is None and not hasattr(source, "layers"):
            raise ValueError("source must be a BrokefishNet or an nn.TransformerEncoder stack")
        if net is not None and (getattr(net, "reinject", "none") != "none" or getattr(net, "rule_features", False)):
            raise NotImplementedError("re-injection and rule features are not carried by this evaluator")
        value_head = getattr(net, "value_head", "king") if net is not None else "king"
        if value_head not in self.VALUE_HEADS:
            raise ValueError(f"value_head must be one of {self.VALUE_HEADS}, got {value_head!r}")
        if value_head != "king" and kernel == "quad":
            raise NotImplementedError("the pooled value heads run on the one-position-per-workgroup kernels "
                                      "(kernel='auto', 'twin', 'duo', 'octo' or 'board')")
        # numbering of the reference class (brokefish/nn/cuda_impl.py:141-158): 0 king, 1 pooled, 2 prenorm
        self.value_head, self.vmode = value_head, self.VALUE_HEADS.index(value_head)
        layers = (net.encoder if net is not None else source).layers
        first = layers[0]
        self.n_layers = len(layers)
        self.d_model = first.self_attn.embed_dim
        self.n_heads = first.self_attn.num_heads
        self.d_ff = first.linear1.out_features
        self.d_head = self.d_model // self.n_heads
        self.eps = float(first.norm1.eps)
        if (self.d_model, self.d_ff, self.n_heads) not in self.SHAPES:
            raise ValueError(
                f"kernels are compiled for (d_model, d_ff, heads) in {self.SHAPES}; "
                f"got {self.d_model}, {self.d_ff}, {self.n_heads}")
        wide = self.d_model != self.D
        if wide and fp8:
            raise NotImplementedError("the 512-wide network runs in int8 only")
        if acc_dtype == "fp32":
            # as the reference class (brokefish/nn/cuda_impl.py:170-177): never silently dropped
            raise NotImplementedError("acc_dtype='fp32' names an accumulator of the reference's unquantised fp16 "
                                      "path; the quantised evaluators accumulate in int32 (int8) or fp32 (e4m3)")
        if int8 is None and not fp8:
            import warnings
            warnings.warn("FusedEncoder(net) without int8=True or fp8=True builds the int8 evaluator here; the "
                          "reference class builds its unquantised fp16 path for the same call", stacklevel=2)
        if wide and kernel in ("quad", "twin", "duo"):
            raise NotImplementedError("the 512-wide network runs on the one-position-per-workgroup kernels "
                                      "(kernel='octo', 'board' or 'auto') only")
        if not getattr(first, "norm_first", True) or getattr(first, "activation_relu_or_gelu", 1) != 1:
            raise ValueError("the evaluator implements pre-norm ReLU layers only")
        self.n_value = int(net.value.weight.shape[0]) if net is not None else 1
        if self.n_value not in (1, 3):
            raise ValueError(f"value head must have 1 or 3 rows, got {self.n_value}")
        self.acc_dtype, self.fp8, self.int8 = acc_dtype, bool(fp8), not fp8
        # `quant` keeps the reference's numbering (1: e4m3, 3: int8 on all four matmuls)
        self.int8_scheme, self.quant = int8_scheme, (1 if fp8 else 3)
        # Boards per workgroup is an occupancy detail of this kernel (four); the flag is
        # accepted for signature compatibility and changes no number.
        self.two_boards = True if two_boards is None else bool(two_boards)
        self.out_dtype = out_dtype
        self.net = net

        self._lib = load_library()
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: the evaluator has no CPU path")
        self.device = torch.device(device) if device is not None else torch.device("cuda", torch.cuda.current_device())
        self._shape = _Shape(self.d_model, self.n_layers, self.n_heads, self.d_ff, self.n_value, self.eps)
        if net is not None:
            sd = {k: v.detach() for k, v in net.state_dict().items()}
        else:   # bare stack: inert tables, identity final norm, zero heads (never read back)
            d = self.d_model
            sd = {"encoder." + k: v.detach() for k, v in source.state_dict().items()}
            for name, rows in (("emb_square", 64), ("emb_type_special", 12), ("emb_color_turn", 4),
                               ("emb_clock", 101), ("emb_rep", 3), ("policy", 64), ("promo", 4), ("value", 1)):
                sd[name + ".weight"] = torch.zeros(rows, d)
            sd["norm_f.weight"], sd["norm_f.bias"] = torch.ones(d), torch.zeros(d)
        # Two packings of the same weights (see include/brokefish_hip.h): the one-position-per-
        # workgroup kernels (TWIN / OCTO / BOARD, what kernel="auto" runs) read the board blobs; the
        # four-positions-per-workgroup kernel is packed, and its workspace allocated, only when it
        # is asked for by name.
        self.kernel = kernel
        self.wstream = self.fparams = self.board_wstream = self.board_fparams = None
        if kernel == "quad":
            wstream, fparams = pack_network(sd, self.n_layers, self.d_model, self.d_ff, self.n_value,
                                            fmt="e4m3" if self.fp8 else "int8")
            if wstream.size != self._lib.bf_wstream_bytes(C.byref(self._shape)) or \
                    fparams.size != self._lib.bf_fparams_floats(C.byref(self._shape)):
                raise RuntimeError("packed blob sizes disagree with the library's layout")
            self.wstream = torch.from_numpy(wstream).to(self.device)
            self.fparams = torch.from_numpy(fparams).to(self.device)
        else:
            wstream, fparams = pack_network_board(sd, self.n_layers, self.d_model, self.d_ff, self.n_value,
                                                  fmt="e4m3" if self.fp8 else "int8")
            if wstream.size != self._lib.bf_board_wstream_bytes(C.byref(self._shape)) or \
                    fparams.size != self._lib.bf_board_fparams_floats(C.byref(self._shape)):
                raise RuntimeError("packed blob sizes disagree with the library's layout (board kernel)")
            self.board_wstream = torch.from_numpy(wstream).to(self.device)
            self.board_fparams = torch.from_numpy(fparams).to(self.device)
        self._buffered_full = 0
        self._backbone = None
        self._profile, self._profile_waves, self._profile_kept = None, 0, None
        self.best_move = None

    @property
    def label(self) -> str:
        fmt = "e4m3" if self.fp8 else "int8"
        names = {"quad": "4 boards/workgroup", "board": "1 board/workgroup",
                 "twin": "1 board/workgroup, 2 workgroups/CU", "octo": "1 board/workgroup of 8 wavefronts",
                 "duo": "2 boards/workgroup of 8 wavefronts"}
        if self.kernel != "auto":
            per = names[self.kernel]
        elif self.board_wstream is None:
            per = names["quad"]
        elif self.d_model != self.D:
            per = names["octo"]
        else:
            per = "1 board/workgroup, 1 or 2 workgroups/CU by batch size"
        return f"{fmt} FFN+QKV+out_proj, {per} (gfx950)"

    # -- buffers and checks ---------------------------------------------------

    def _ensure_full_buffers(self, n: int) -> None:
        if self._buffered_full != n:
            self.policy_out = torch.empty(n, T, N_POLICY, device=self.device, dtype=self.out_dtype)
            self.promo_out = torch.empty(n, T, N_PROMO, device=self.device, dtype=self.out_dtype)
            self.value_out = torch.empty(n, device=self.device, dtype=torch.float32)
            self.best_out = torch.empty(n, device=self.device, dtype=torch.int32)
            nbytes = self._lib.bf_workspace_bytes(C.byref(self._shape), n) if self.wstream is not None else 0
            self.workspace = torch.empty(nbytes, device=self.device, dtype=torch.uint8)
            self._buffered_full = n

    @staticmethod
    def _check_inputs(boards, control, rep, mask=None) -> int:
        if boards.dim() != 2 or boards.shape[1] != T:
            raise ValueError(f"boards must be [n, 32], got {tuple(boards.shape)}")
        n = boards.shape[0]
        if n < 1:
            raise ValueError("boards must hold at least one position")
        if boards.dtype is not torch.int16:
            raise ValueError(f"boards must be int16, got {boards.dtype}")
        if control.shape != (n,) or control.dtype is not torch.int16:
            raise ValueError(f"control must be [{n}] int16, got {tuple(control.shape)} {control.dtype}")
        if rep.shape != (n,) or rep.dtype is not torch.uint8:
            raise ValueError(f"rep must be [{n}] uint8, got {tuple(rep.shape)} {rep.dtype}")
        if mask is not None and (mask.shape != (n, T) or mask.dtype is not torch.int64):
            raise ValueError(f"mask must be [{n}, 32] int64, got {tuple(mask.shape)} {mask.dtype}")
        for name, t in (("boards", boards), ("control", control), ("rep", rep), ("mask", mask)):
            if t is not None and not t.is_cuda:
                raise ValueError(f"{name} must be on the GPU")
        return n

    def _args(self, boards, control, rep, mask, policy, promo, value, best, taps=None, active=None, leaves=None) -> _Args:
        for name, t in (("boards", boards), ("control", control), ("rep", rep), ("mask", mask), ("active", active)):
            if t is not None and t.device != self.device:
                raise ValueError(f"{name} is on {t.device}, the evaluator's weights are on {self.device}")
        a = _Args()
        a.active = active.data_ptr() if active is not None else None
        if leaves is not None:
            a.leaf_index, a.leaf_count = leaves[0].data_ptr(), leaves[1].data_ptr()
        a.boards, a.control, a.rep = boards.data_ptr(), control.data_ptr(), rep.data_ptr()
        a.mask = mask.data_ptr() if mask is not None else None
        a.n = boards.shape[0]
        a.shape = self._shape
        if self.wstream is not None:
            a.wstream, a.fparams = self.wstream.data_ptr(), self.fparams.data_ptr()
        if self.board_wstream is not None:
            a.board_wstream, a.board_fparams = self.board_wstream.data_ptr(), self.board_fparams.data_ptr()
        a.kernel = self.KERNELS[self.kernel]
        a.value_mode = self.vmode
        a.policy, a.promo, a.value = policy.data_ptr(), promo.data_ptr(), value.data_ptr()
        a.best_move = best.data_ptr() if (best is not None and mask is not None) else None
        a.out_fp32 = 1 if policy.dtype is torch.float32 else 0
        a.quant = 1 if self.fp8 else 0
        need = self._lib.bf_workspace_bytes(C.byref(self._shape), a.n) if self.wstream is not None else 0
        if getattr(self, "workspace", None) is None or self.workspace.numel() < need:
            self.workspace = torch.empty(need, device=self.device, dtype=torch.uint8)
        if need:
            a.workspace, a.workspace_bytes = self.workspace.data_ptr(), self.workspace.numel()
        a.taps = C.pointer(taps) if taps is not None else None
        return a

    def kernel_choice(self, n: int) -> str:
        """Which kernel a call with ``n`` positions runs ("quad", "board", "twin", "octo" or "duo")."""
        a = _Args()
        a.n, a.shape, a.quant, a.kernel = n, self._shape, (1 if self.fp8 else 0), self.KERNELS[self.kernel]
        a.wstream = a.fparams = 16 if self.wstream is not None else None        # only tested for NULL
        a.board_wstream = a.board_fparams = 16 if self.board_wstream is not None else None
        rc = self._lib.bf_kernel_choice(C.byref(a))
        if rc < 0:
            raise RuntimeError(f"bf_kernel_choice failed ({rc}): {self._lib.bf_last_error().decode()}")
        return {1: "quad", 2: "board", 3: "twin", 4: "octo", 5: "duo"}[rc]

    def forward_expand(self, boards, control, rep, mask=None, max_edges: int = 96, active=None, out=None, leaves=None):
        """``forward_full`` followed on the same stream by the search's expand step
        (:func:`expand_edges`), with the legal-move words generated on the device
        (:func:`movegen`) when ``mask`` is not given: two or three launches, no host round trip.
        Returns the edge dict (plus ``mask`` / ``in_check`` when generated here); the logits stay
        available as ``policy_out`` / ``promo_out`` / ``value_out`` until the next call."""
        extra = {}
        if mask is None:
            mask, chk = movegen(boards, control)
            extra = {"mask": mask, "in_check": chk}
        policy, promo, value = self.forward_full(boards, control, rep, active=active, leaves=leaves)
        edges = expand_edges(policy, promo, value, mask, boards, control, max_edges, active, out, leaves)
        edges.update(extra)
        return edges

    def _call(self, args: _Args) -> None:
        with torch.cuda.device(self.device):     # the launch goes to the current device
            rc = self._lib.bf_model_forward(C.byref(args), C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream))
        if rc:
            raise RuntimeError(f"bf_model_forward failed ({rc}): {self._lib.bf_last_error().decode()}")

    # -- the call ----------------------------------------------------------------

    def _require_net(self, what: str):
        if self.net is None:
            raise ValueError(f"{what} needs the whole model: build this from a BrokefishNet, not "
                             "from a bare nn.TransformerEncoder")
        return self.net

    def forward(self, x, alive=None, out=None):
        """The encoder stack alone (reference brokefish/nn/cuda_impl.py:447-463):
        ``x [n, 32, d]`` tokens and ``alive [n, 32]`` (bool or int8; dead tokens are masked
        out of attention as keys) to the residual stream after the last layer, in ``x``'s
        dtype.  The arithmetic inside is the same fp32 / int8 path as ``forward_full``.
        """
        n, t, d = x.shape
        if d != self.d_model or t != T:
            raise ValueError(f"expected [n, {T}, {self.d_model}], got {tuple(x.shape)}")
        if not x.is_cuda:
            raise ValueError("x must be on the GPU")
        if alive is not None:
            if alive.shape != (n, t):
                raise ValueError(f"alive must be [{n}, {t}], got {tuple(alive.shape)}")
            if alive.dtype not in (torch.bool, torch.int8):
                raise ValueError(f"alive must be bool or int8, got {alive.dtype}")
        if out is not None and (out.shape != x.shape or out.device != x.device):
            raise ValueError(f"out must be {tuple(x.shape)} on {x.device}")
        # An encoder-only launch (reference csrc/encoder.cu:1752-1764): the residual stream goes in
        # and comes out through the tap table, the token mask replaces the board words, no heads
        # run.  What is needed beyond x, alive and out is kept between calls, so a repeated call
        # with out= given (fp32, contiguous) allocates nothing.
        bb = self._backbone
        if bb is None or bb["cap"] < n:
            bb = self._backbone = {"cap": n, "ones": torch.ones(n, T, dtype=torch.int8, device=self.device),
                                   "x": None, "y": None}
        alive8 = bb["ones"][:n] if alive is None else alive.contiguous()      # bool or int8: one byte, non-zero = live
        if x.dtype is torch.float32 and x.is_contiguous():
            x32 = x
        else:
            if bb["x"] is None or bb["x"].shape[0] < n:
                bb["x"] = torch.empty(bb["cap"], T, d, dtype=torch.float32, device=self.device)
            x32 = bb["x"][:n]
            x32.copy_(x)
        direct = out is not None and out.dtype is torch.float32 and out.is_contiguous()
        if direct:
            y32 = out
        else:
            if bb["y"] is None or bb["y"].shape[0] < n:
                bb["y"] = torch.empty(bb["cap"], T, d, dtype=torch.float32, device=self.device)
            y32 = bb["y"][:n]
        for name, t_ in (("x", x), ("alive", alive), ("out", out)):
            if t_ is not None and t_.device != self.device:
                raise ValueError(f"{name} is on {t_.device}, the evaluator's weights are on {self.device}")
        taps = _Taps()
        taps.x_in, taps.resid_last, taps.alive = x32.data_ptr(), y32.data_ptr(), alive8.data_ptr()
        taps.layer_begin, taps.layer_end = 0, self.n_layers
        a = _Args()
        a.n, a.shape = n, self._shape
        if self.wstream is not None:
            a.wstream, a.fparams = self.wstream.data_ptr(), self.fparams.data_ptr()
            need = self._lib.bf_workspace_bytes(C.byref(self._shape), n)
            if getattr(self, "workspace", None) is None or self.workspace.numel() < need:
                self.workspace = torch.empty(need, device=self.device, dtype=torch.uint8)
            a.workspace, a.workspace_bytes = self.workspace.data_ptr(), self.workspace.numel()
        if self.board_wstream is not None:
            a.board_wstream, a.board_fparams = self.board_wstream.data_ptr(), self.board_fparams.data_ptr()
        a.kernel, a.quant, a.value_mode = self.KERNELS[self.kernel], (1 if self.fp8 else 0), self.vmode
        a.taps = C.pointer(taps)      # the library copies the table at launch
        self._call(a)
        if direct:
            return out
        if out is not None:
            out.copy_(y32)
            return out
        return y32.to(x.dtype, copy=True)

    __call__ = forward

    def forward_full(self, boards, control, rep, mask=None, active=None, leaves=None):
        """Boards to ``(policy_logits, promo, value)`` in one launch.

        Without ``mask`` the policy is raw, as the reference evaluator returns it.  With
        ``mask`` illegal entries are ``-inf`` and ``self.best_move`` ([n] int32) is the
        masked argmax.  Returns views on internal buffers, which the next call overwrites.
        ``active`` ([n] uint8 or bool on the GPU, e.g. the search's leaf flags) skips the
        positions where it is 0: their rows of the output buffers keep what they held.
        ``leaves`` (the pair :func:`compact_leaves` returns) does the same from a compacted list
        with a device-side count: only the listed positions are evaluated.
        """
        self._require_net("forward_full")
        n = self._check_inputs(boards, control, rep, mask)
        self._ensure_full_buffers(n)
        boards, control, rep = boards.contiguous(), control.contiguous(), rep.contiguous()
        mask = mask.contiguous() if mask is not None else None
        if active is not None:
            if active.shape != (n,) or active.dtype not in (torch.uint8, torch.bool) or not active.is_cuda:
                raise ValueError(f"active must be [{n}] uint8 or bool on the GPU")
            active = active.contiguous().view(torch.uint8)
        if leaves is not None:
            if active is not None:
                raise ValueError("a compacted leaf list replaces the active flags: pass one of them")
            leaves = _check_leaves(leaves, n, self.device)
        if self._profile is not None:
            # set_profile(True): the launch goes through the phase-accounting build, which adds
            # into the counters that read_profile returns
            args = self._args(boards, control, rep, mask, self.policy_out, self.promo_out,
                              self.value_out, self.best_out, active=active, leaves=leaves)
            with torch.cuda.device(self.device):
                rc = self._lib.bf_profile_phases(C.byref(args), C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream),
                                                 C.c_void_p(self._profile.data_ptr()))
            if rc:
                raise RuntimeError(f"bf_profile_phases failed ({rc}): {self._lib.bf_last_error().decode()}")
            self._profile_waves += self._launch_waves(n)
        elif self.binding == "torch":
            for name, t in (("boards", boards), ("control", control), ("rep", rep), ("mask", mask), ("active", active)):
                if t is not None and t.device != self.device:
                    raise ValueError(f"{name} is on {t.device}, the evaluator's weights are on {self.device}")
            quad = self.wstream is not None
            if quad:
                need = self._lib.bf_workspace_bytes(C.byref(self._shape), n)
                if getattr(self, "workspace", None) is None or self.workspace.numel() < need:
                    self.workspace = torch.empty(need, device=self.device, dtype=torch.uint8)
            none = None
            load_extension().model_forward(
                boards, control, rep, self.wstream if quad else self.board_wstream,
                self.fparams if quad else self.board_fparams, self.policy_out, self.promo_out, self.value_out,
                self.d_model, self.n_layers, self.n_heads, self.d_ff, self.eps, 1 if self.fp8 else 0,
                self.KERNELS[self.kernel], self.n_value, self.vmode,
                mask if mask is not None else none, self.best_out if mask is not None else none,
                active if active is not None else none, self.workspace if quad else none,
                leaves[0] if leaves is not None else none, leaves[1] if leaves is not None else none)
        else:
            self._call(self._args(boards, control, rep, mask, self.policy_out, self.promo_out,
                                  self.value_out, self.best_out, active=active, leaves=leaves))
        self.best_move = self.best_out if mask is not None else None
        return self.policy_out, self.promo_out, self.value_out

    def forward_masked(self, boards, control, rep, mask):
        """``(policy_logits, promo, value, best_move)`` with the legal-move AND fused in."""
        p, q, v = self.forward_full(boards, control, rep, mask)
        return p, q, v, self.best_out

    def time_kernel_ms(self, boards, control, rep, mask=None, warmup: int = 3, iters: int = 20) -> float:
        """Average device time of one launch, from HIP events on the current stream."""
        n = self._check_inputs(boards, control, rep, mask)
        self._ensure_full_buffers(n)
        args = self._args(boards.contiguous(), control.contiguous(), rep.contiguous(),
                          mask.contiguous() if mask is not None else None,
                          self.policy_out, self.promo_out, self.value_out, self.best_out)
        with torch.cuda.device(self.device):
            ms = self._lib.bf_time_kernel_ms(C.byref(args), C.c_void_p(torch.cuda.current_stream(self.device).cuda_stream),
                                             warmup, iters)
        if ms < 0:
            raise RuntimeError(f"bf_time_kernel_ms failed ({ms}): {self._lib.bf_last_error().decode()}")
        return ms

    def _launch_waves(self, n: int) -> int:
        """Wavefronts in a launch of ``n`` positions of the kernel such a call runs."""
        kind = self.kernel_choice(n)
        return {"board": 4 * n, "twin": 4 * n, "octo": 8 * n, "duo": 8 * ((n + 1) // 2), "quad": 4 * ((n + 3) // 4)}[kind]

    def profile_phase_names(self):
        """Names of the counters of :meth:`read_profile`, in order (reference csrc/encoder.cu:1910)."""
        return [self._lib.bf_profile_phase_name(i).decode() for i in range(self._lib.bf_profile_phase_count())]

    def set_profile(self, on: bool) -> None:
        """Phase accounting on or off for the ``forward_full`` calls that follow (reference
        csrc/encoder.cu:1886, 1907): while on, each call runs the phase-accounting build of the
        kernel it would run anyway (same outputs) and adds its shader-clock cycles per phase to the
        counters.  Turning it on keeps counters already collected; ``reset_profile`` zeroes them."""
        if on and self._profile is None:
            self._profile = torch.zeros(self._lib.bf_profile_phase_count(), dtype=torch.int64, device=self.device)
            self._profile_waves = 0
        elif not on and self._profile is not None:
            self._profile_kept = (self._profile, self._profile_waves)
            self._profile = None

    def reset_profile(self) -> None:
        """Zero the cycle counters (reference csrc/encoder.cu:1888, 1908)."""
        self._profile_kept = None
        if self._profile is not None:
            self._profile.zero_()
            self._profile_waves = 0

    def read_profile(self):
        """``(cycles, wavefronts)``: the [phases] int64 cycle counters summed over all wavefronts
        of the profiled launches since the last reset, and how many wavefronts that was (reference
        csrc/encoder.cu:1894, 1909 returns the all-warps sum and warp 0's; here the sum and the
        divisor).  Synchronises with the evaluator's stream."""
        cyc, waves = (self._profile, self._profile_waves) if self._profile is not None else \
            (self._profile_kept or (torch.zeros(self._lib.bf_profile_phase_count(), dtype=torch.int64), 0))
        if cyc.is_cuda:
            torch.cuda.current_stream(self.device).synchronize()
        return cyc.cpu(), waves

    def profile_phases(self, boards, control, rep, mask=None) -> Dict[str, float]:
        """Shader-clock cycles per phase, averaged over the wavefronts of one launch of the
        profiling build of the kernel this call would run: ``set_profile`` / one call /
        ``read_profile`` in one step.  ``sync_wait`` (time at workgroup barriers) is also
        contained in the phases around it; ``total`` is a wavefront's lifetime.  The outputs it
        writes are the normal ones."""
        saved = (self._profile, self._profile_waves, self._profile_kept)
        self._profile = None
        self.set_profile(True)
        try:
            self.forward_full(boards, control, rep, mask)
            cyc, waves = self.read_profile()
        finally:
            self._profile, self._profile_waves, self._profile_kept = saved
        return {name: cyc[i].item() / waves for i, name in enumerate(self.profile_phase_names())}

    # -- debug taps (the counterpart of the reference's forward_stage) ------------

    def forward_stage(self, boards, control, rep, stage: int):
        """Activations at an intermediate stage, as reference nn/cuda_impl.py:512-531:
        stage 9 is the embedding sum alone, stage 8 the output of ``norm_f``; both come back as
        [n, 32, d] float32.  Stages 1-7 name points inside the reference's own kernel (its
        staging buffers between phases) and have no counterpart here: ``forward_taps`` exposes
        this kernel's intermediates (operand bytes, accumulators, residual stream) instead.
        """
        self._require_net("forward_stage")
        if stage not in (8, 9):
            raise NotImplementedError(f"stage {stage}: only 9 (embeddings) and 8 (after norm_f) exist; "
                                      "see forward_taps for the per-layer intermediates")
        key = "embed" if stage == 9 else "normed"
        return self.forward_taps(boards, control, rep, want=[key])[key]

    def forward_taps(self, boards, control, rep, mask=None, x_in=None, layer_begin: int = 0,
                     layer_end: Optional[int] = None, want=None):
        """Run with intermediate outputs.  Returns a dict of fresh fp32-output tensors:
        policy, promo, value, [best], plus the taps named in ``want`` (default: all).
        With ``fp8=True`` the operand taps come back as float8_e4m3fn and the accumulator
        taps as float32.

        ``x_in`` ([n,32,d] fp32) replaces the embedding as the residual stream entering
        layer ``layer_begin``; layers ``[layer_begin, layer_end)`` run, then the heads.
        """
        n = self._check_inputs(boards, control, rep, mask)
        d, f = self.d_model, self.d_ff
        layer_end = self.n_layers if layer_end is None else layer_end
        lr = layer_end - layer_begin
        kd, kf = d // 256, f // 256
        dev = self.device
        shapes = {"embed": ((n, T, d), torch.float32),
                  "qa_qkv": ((n, lr, T, d), torch.int8), "acc_qkv": ((n, lr, kd, T, 3 * d), torch.int32),
                  "qa_out": ((n, lr, T, d), torch.int8), "acc_out": ((n, lr, kd, T, d), torch.int32),
                  "qa_ff1": ((n, lr, T, d), torch.int8), "acc_ff1": ((n, lr, kd, T, f), torch.int32),
                  "qa_ff2": ((n, lr, T, f), torch.uint8), "acc_ff2": ((n, lr, kf, T, d), torch.int32),
                  "resid": ((n, lr, T, d), torch.float32), "normed": ((n, T, d), torch.float32),
                  "resid_last": ((n, T, d), torch.float32)}
        want = list(shapes) if want is None else list(want)
        out = {k: torch.zeros(shapes[k][0], dtype=shapes[k][1], device=dev) for k in want}
        taps = _Taps()
        if x_in is not None:
            if x_in.shape != (n, T, d) or x_in.dtype is not torch.float32 or not x_in.is_cuda:
                raise ValueError(f"x_in must be [{n}, 32, {d}] float32 on the GPU")
            x_in = x_in.contiguous()
            taps.x_in = x_in.data_ptr()
        taps.layer_begin, taps.layer_end = layer_begin, layer_end
        if layer_begin == 0 and layer_end == 0:
            raise ValueError("empty layer range")
        for k in want:
            setattr(taps, k, out[k].data_ptr())
        out["policy"] = torch.empty(n, T, N_POLICY, device=dev, dtype=torch.float32)
        out["promo"] = torch.empty(n, T, N_PROMO, device=dev, dtype=torch.float32)
        out["value"] = torch.empty(n, device=dev, dtype=torch.float32)
        best = torch.empty(n, device=dev, dtype=torch.int32) if mask is not None else None
        if best is not None:
            out["best"] = best
        self._call(self._args(boards.contiguous(), control.contiguous(), rep.contiguous(),
                              mask.contiguous() if mask is not None else None,
                              out["policy"], out["promo"], out["value"], best, taps))
        torch.cuda.current_stream(dev).synchronize()   # taps/x_in must outlive the launch
        if self.fp8:   # the accumulators are fp32 and the operand bytes e4m3 in this format
            for k in want:
                if k.startswith("acc_"):
                    out[k] = out[k].view(torch.float32)
                elif k.startswith("qa_"):
                    out[k] = out[k].view(torch.float8_e4m3fn)
        return out
