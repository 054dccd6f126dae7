"""torch.library custom ops over the C-ABI HIP library, with autograd and fake (meta) kernels.

Op graph (names under the ``flexsae_amd::`` namespace):

    hier_fwd(indices, weight, vals, bias, target) -> (loss, resid)
    hier_bwd(grad_out, indices, weight, vals, resid) -> (dW, dvals, dbias)
    topk_fwd(indices, weight, vals, bias, target) -> (loss, resid)
    topk_bwd(grad_out, indices, weight, vals, resid) -> (dW, dvals, dbias)
    hier_train_sliced(indices, weight, vals, bias, target) -> (loss, dvals, dbias, dW)   [unit gradient]
    scale_(x, grad_out), scale_by(x, grad_out) -> x * grad_out
    hier_train(indices, weight, vals, bias, target, stage) -> (loss, dvals, dbias)       [unit gradient; fills stage]
    hier_finish(grad_out, indices, weight, vals, stage) -> dW

``resid[B,D]`` (fp32) is the reconstruction error of the full row, the only state the first four
keep between forward and backward.  The hierarchical loss, when gradients are needed, goes
through ``hier_train_sliced`` instead (forward and reverse walk sharing one gather; the backward
only scales), or through ``hier_train`` / ``hier_finish`` when a stage budget lets all per-pair
contributions wait for the backward.  The ops take the place of the reference's two ``autograd.Function``
classes (reference torch-ext/flex_sae/hierarchical_kernels.py:273-299 and
torch-ext/flex_sae/topk_kernels.py:188-223) and keep their contract: gradients for ``weight``,
``vals`` and ``bias`` only (plus ``target`` for TopK, whose loss tail is differentiable there),
``indices`` never, an arbitrary scalar upstream gradient, no autocast of the inputs.

Everything runs on the current stream of the tensors' device; nothing synchronises unless
index checking is switched on.
"""
from __future__ import annotations

import contextlib
import ctypes
import os
from typing import Tuple

import torch
from torch import Tensor

from . import _lib

_DTYPES = {torch.float32: _lib.F32, torch.bfloat16: _lib.BF16, torch.float16: _lib.F16}

# device index -> int32[1] status flag the kernels OR error bits into (never reset by the ops)
_status_flags = {}
_check_indices = os.environ.get("FLEXSAE_CHECK_INDICES", "0") not in ("", "0")


def set_index_checking(enabled: bool) -> None:
    """When enabled every fused call synchronises and raises on an out-of-range index.

    Off by default (the reference never checks; here such an index is neutralised on the
    device -- treated as latent 0 with value 0 -- and recorded in a flag instead of reading
    out of bounds)."""
    global _check_indices
    _check_indices = bool(enabled)


def _flag_for(device: torch.device) -> Tensor:
    key = device.index if device.index is not None else torch.cuda.current_device()
    flag = _status_flags.get(key)
    if flag is None:
        flag = torch.zeros(1, dtype=torch.int32, device=device)
        _status_flags[key] = flag
    return flag


def check_index_flag(device=None) -> None:
    """Synchronise and raise IndexError if any fused call since the last check saw an index
    outside ``[0, F)``; clears the flag."""
    dev = torch.device("cuda", torch.cuda.current_device()) if device is None else torch.device(device)
    flag = _flag_for(dev)
    bits = int(flag.item())
    if bits:
        flag.zero_()
        if bits & _lib.FLAG_INDEX_RANGE:
            raise IndexError("flexsae_amd: an entry of `indices` was outside [0, F)")
        raise RuntimeError(f"flexsae_amd: device status flag {bits:#x}")


def _validate(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor, target: Tensor):
    """Shape/dtype/device checks the reference leaves to undefined behaviour."""
    if indices.dim() != 2 or weight.dim() != 2 or vals.dim() != 2 or bias.dim() != 1 or target.dim() != 2:
        raise ValueError("expected indices[B,K], weight[F,D], vals[B,K], bias[D], target[B,D]")
    B, K = indices.shape
    F, D = weight.shape
    if tuple(vals.shape) != (B, K) or tuple(bias.shape) != (D,) or tuple(target.shape) != (B, D):
        raise ValueError(
            f"shape mismatch: indices{tuple(indices.shape)} weight{tuple(weight.shape)} "
            f"vals{tuple(vals.shape)} bias{tuple(bias.shape)} target{tuple(target.shape)}")
    if B == 0 or K == 0 or F == 0 or D == 0:
        raise ValueError("empty inputs are not supported (B, K, F, D must all be >= 1)")
    if indices.dtype != torch.int64:
        raise TypeError(f"indices must be int64 (int32 is widened by the public functions), got {indices.dtype}")
    for name, t in (("weight", weight), ("vals", vals), ("bias", bias), ("target", target)):
        if t.dtype not in _DTYPES:
            raise TypeError(f"{name} must be float32, bfloat16 or float16, got {t.dtype}")
    dev = weight.device
    if dev.type != "cuda":
        raise RuntimeError(
            "flexsae_amd fused ops run on an AMD GPU only (tensors must live on a 'cuda' device); "
            "use flexsae_amd.topk_sae_loss / hierarchical_sae_loss for the eager torch definition")
    for name, t in (("indices", indices), ("vals", vals), ("bias", bias), ("target", target)):
        if t.device != dev:
            raise RuntimeError(f"{name} is on {t.device}, weight on {dev}")
    if B * K >= 2 ** 32 or F >= 2 ** 31 or D >= 2 ** 29:
        raise ValueError("sizes beyond the kernels' index range: need B*K < 2^32, F < 2^31, D < 2^29")
    return B, K, F, D


def _shape(B, K, F, D, weight: Tensor, vals: Tensor, bias_dtype, target_dtype) -> _lib.Shape:
    return _lib.Shape(B, K, F, D, _DTYPES[weight.dtype], _DTYPES[vals.dtype], _DTYPES[bias_dtype],
                      _DTYPES[target_dtype])


def _prep(t: Tensor) -> Tensor:
    """Contiguous and 16-byte aligned, as the vector accesses of the kernels need: a view into a
    larger buffer that starts at an odd element (``flat[1:1 + D]``) is copied."""
    t = t.contiguous()
    return t.clone() if t.data_ptr() % 16 else t


def _ptr(t: Tensor) -> ctypes.c_void_p:
    return ctypes.c_void_p(t.data_ptr())


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _forward(entry: str, indices, weight, vals, bias, target) -> Tuple[Tensor, Tensor]:
    B, K, F, D = _validate(indices, weight, vals, bias, target)
    lib = _lib.load()
    indices, weight, vals, bias, target = (_prep(t) for t in (indices, weight, vals, bias, target))
    dev = weight.device
    with torch.cuda.device(dev):
        shape = _shape(B, K, F, D, weight, vals, bias.dtype, target.dtype)
        ws_bytes = lib.flexsae_fwd_workspace_bytes(ctypes.byref(shape))
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        resid = torch.empty((B, D), dtype=torch.float32, device=dev)
        flag = _flag_for(dev)
        rc = getattr(lib, entry)(ctypes.byref(shape), _ptr(indices), _ptr(weight), _ptr(vals), _ptr(bias),
                                 _ptr(target), _ptr(loss), _ptr(resid), _ptr(workspace), ws_bytes,
                                 _ptr(flag), _stream())
        _lib.check(rc, entry)
        if _check_indices:
            check_index_flag(dev)
    return loss, resid


def _grad_scalar(grad_out: Tensor, dev) -> Tensor:
    return grad_out.detach().to(device=dev, dtype=torch.float32).reshape(1).contiguous()


@torch.library.custom_op("flexsae_amd::hier_fwd", mutates_args=())
def hier_fwd(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor,
             target: Tensor) -> Tuple[Tensor, Tensor]:
    return _forward("flexsae_hier_fwd", indices, weight, vals, bias, target)


@torch.library.custom_op("flexsae_amd::topk_fwd", mutates_args=())
def topk_fwd(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor,
             target: Tensor) -> Tuple[Tensor, Tensor]:
    return _forward("flexsae_topk_fwd", indices, weight, vals, bias, target)


def _fwd_fake(indices, weight, vals, bias, target):
    B, _ = indices.shape
    D = weight.shape[1]
    return (weight.new_empty((), dtype=torch.float32), weight.new_empty((B, D), dtype=torch.float32))


hier_fwd.register_fake(_fwd_fake)
topk_fwd.register_fake(_fwd_fake)


# Scratch the hierarchical backward may use for the per-pair contributions of one slice of D
# columns.  More scratch = wider slices = fewer passes; 0 selects the atomic single-pass fallback;
# None (the default) sizes it from the problem, see _hier_scratch_budget.
_hier_scratch_bytes = (int(os.environ["FLEXSAE_HIER_SCRATCH_MB"]) << 20) if "FLEXSAE_HIER_SCRATCH_MB" in os.environ else None
_HIER_SCRATCH_CAP = 256 << 20


# Narrowest slice the scratch budget may lead to on its own; a budget that gives fewer columns is
# exceeded up to this width.  None (the default): 256 columns -- narrower slices measured slower at
# B*K = 2^19 pairs of bf16 rows (more launches, each too short to overlap its gather, arithmetic
# and store phases) -- except for fp32 rows of more than 64 steps, whose training-step kernel works
# on 64-column tiles and measured fastest one tile at a time (B = 2048, K = 256: 1.20 ms with
# 64-column slices, 1.25 with 128, 1.22 with 256).
_hier_min_slice_cols = (int(os.environ["FLEXSAE_HIER_MIN_SLICE_COLS"])
                        if "FLEXSAE_HIER_MIN_SLICE_COLS" in os.environ else None)


def set_hier_min_slice_cols(cols) -> None:
    """Narrowest column slice of the sliced hierarchical step (``None``: 256, or 64 for fp32 rows of
    more than 64 steps).  128 (16-bit weights) halves the scratch of large problems at a cost of
    5-10 % of the step time."""
    global _hier_min_slice_cols
    _hier_min_slice_cols = None if cols is None else max(1, int(cols))


def _train_tile_cols(K: int, weight_dtype) -> int:
    """Columns per tile of the training-step kernel (train_tile_cols() of the library)."""
    return 64 if (weight_dtype == torch.float32 and K > 64) else 128


def _hier_scratch_budget(B: int, K: int, F: int, D: int, weight_dtype) -> int:
    """Bytes the contributions of one slice may take.  Unless set explicitly: 0.45 of the weight
    matrix, at most 256 MiB -- memory above the inputs then stays within about 1.25 of the TopK
    loss's (whose peak is the dense gradient plus the residual) whatever K is, at 4-5 % of the step
    time where that is less than the 256 MiB that measured fastest (B = 4096, F = 65536, D = 2304,
    bf16: K = 32 0.483 instead of 0.463 ms, K = 64 0.751 instead of 0.717 ms; K = 128 unchanged)."""
    if _hier_scratch_bytes is not None:
        return _hier_scratch_bytes
    sw = 4 if weight_dtype == torch.float32 else 2
    return min(_HIER_SCRATCH_CAP, int(0.45 * F * D * sw))


def _hier_slice_cols(B: int, K: int, F: int, D: int, weight_dtype) -> int:
    p_size = 2 if weight_dtype == torch.bfloat16 else 4
    tile = _train_tile_cols(K, weight_dtype)
    floor = _hier_min_slice_cols if _hier_min_slice_cols is not None else (64 if tile == 64 else 256)
    cols = _hier_scratch_budget(B, K, F, D, weight_dtype) // (B * K * p_size)
    if cols >= tile:
        cols -= cols % tile  # whole tiles: the library rounds up, the budget is an upper bound
    return max(floor, cols, 1)


def set_hier_scratch_bytes(nbytes) -> None:
    """Upper bound on the scratch of the hierarchical backward (bytes): the per-pair contributions
    of one slice of columns.  0 = use the atomic scatter fallback, which needs no scratch but an
    fp32 [F,D] accumulator.  ``None`` (the default) sizes it from the problem: 0.45 of the weight
    matrix, at most 256 MiB.  A slice is never narrower than ``set_hier_min_slice_cols``, so with
    many pairs the scratch can exceed the bound by a large factor (B*K*256 contributions).  Slices
    of 256 columns measured fastest at B*K = 2^19 pairs; wider ones are not faster."""
    global _hier_scratch_bytes
    _hier_scratch_bytes = None if nbytes is None else int(nbytes)


# Hot-latent accumulators of the sliced training step (FLEXSAE_BWD_HOT_LATENTS of the library): the
# most frequent latents of the batch are summed in the LDS by blocks of 128 rows instead of being
# staged pair by pair.  That pays where indices are skewed (a few latents in most rows) and costs
# where they are not (its blocks hold the LDS of a whole compute unit: half the wavefronts of the
# plain kernel), and only the device knows which it is.  "auto" therefore measures: every sliced step
# leaves, in pinned host memory, how many of its pairs belong to latents with more than 64 pairs
# (flexsae_hier_pair_stats; no synchronisation: an event is polled), and the next step of the same
# shape on the same device takes the accumulators when that was a quarter of the pairs or more.  The
# first step of a shape, and steps traced by a compiler, run the plain kernel.
# "on" takes them wherever the shape is supported (16-bit weights, K <= 64); "off" never.
#
# The same measurement serves a second decision (FLEXSAE_BWD_DENSE_LATENTS of the library).  Shapes
# with at most two pairs per latent on average (B*K <= 2F) reduce, by default, from a list of the
# latents ordered by pair count and zero the rows of latents without pairs in one pass: a sixth faster
# where two thirds of the latents are empty (skewed indices), 8 % slower where an eighth is (uniform
# ones; B = 4096, K = 32, F = 65536: 0.441 instead of 0.477 ms without the list).  The step therefore
# also leaves the number of latents without pairs, and the next one drops the list when that was less
# than 40 % of the latents (with uniform indices the two ways break even at one pair per latent, 37 %
# empty).
_hot_latents = os.environ.get("FLEXSAE_HOT_LATENTS", "auto").lower()
_dense_latents = os.environ.get("FLEXSAE_DENSE_LATENTS", "auto").lower()
_HOT_ROWS_PER_BLOCK = 128   # kHotRowsPerBlock of the library
_HOT_AUTO_FRACTION = 0.25   # of the pairs in latents with more than 64 pairs
_DENSE_AUTO_FRACTION = 0.40  # of the latents without a pair
_hot_auto = {}              # (device index, B, K, F, D, dtype) -> {"hot", "dense", "pinned", "event"}


def set_hot_latents(mode) -> None:
    """``"auto"`` (default), ``"on"``/``True`` or ``"off"``/``False``: whether the sliced hierarchical
    training step sums the most frequent latents of the batch in LDS accumulators (bit-reproducible
    fixed-point sums; skewed indices stage about half as many contributions then).  ``"auto"``
    decides from the previous step of the same shape (see the module's comment)."""
    global _hot_latents
    if isinstance(mode, bool):
        mode = "on" if mode else "off"
    mode = "auto" if mode is None else str(mode).lower()
    if mode not in ("auto", "on", "off"):
        raise ValueError("set_hot_latents: expected 'auto', 'on' or 'off'")
    _hot_latents = mode
    _hot_auto.clear()


def set_dense_latents(mode) -> None:
    """``"auto"`` (default), ``"on"``/``True`` or ``"off"``/``False``: whether the sliced hierarchical
    step of a shape with at most two pairs per latent (B*K <= 2F) reduces WITHOUT the list of latents
    ordered by pair count (``"on"``: most latents have pairs).  The results are the same bits either
    way.  ``"auto"`` decides from the previous step of the same shape (see the module's comment)."""
    global _dense_latents
    if isinstance(mode, bool):
        mode = "on" if mode else "off"
    mode = "auto" if mode is None else str(mode).lower()
    if mode not in ("auto", "on", "off"):
        raise ValueError("set_dense_latents: expected 'auto', 'on' or 'off'")
    _dense_latents = mode
    _hot_auto.clear()


def _hot_latents_supported(B: int, K: int, F: int, D: int, weight_dtype) -> bool:
    """flexsae_hier_hot_latents_supported() of the library, restated so that a compiler trace can
    follow it: 16-bit weights, at most 64 steps, rows the piece reduction can serve."""
    if weight_dtype not in (torch.bfloat16, torch.float16) or K > 64 or B * K >= 2 ** 31:
        return False
    return D % (8 if weight_dtype == torch.bfloat16 else 4) == 0


def _hot_key(device, B, K, F, D, weight_dtype):
    return (device.index if device.index is not None else torch.cuda.current_device(), B, K, F, D, weight_dtype)


def _use_hot_latents(B: int, K: int, F: int, D: int, weight_dtype, device=None, traced: bool = False) -> bool:
    if _hot_latents == "off" or not _hot_latents_supported(B, K, F, D, weight_dtype):
        return False
    if _hot_latents == "on":
        return True
    if traced or device is None or torch.cuda.is_current_stream_capturing():
        return False  # (a graph under capture keeps whatever kernel it captured)
    st = _index_stats(_hot_key(device, B, K, F, D, weight_dtype), B, K, F)
    return st is not None and st["hot"]


def _use_dense_latents(B: int, K: int, F: int, D: int, weight_dtype, device=None, traced: bool = False) -> bool:
    if B * K > 2 * F or _dense_latents == "off":
        return False  # (with more pairs than that the library never uses the list)
    if _dense_latents == "on":
        return True
    if traced or device is None or torch.cuda.is_current_stream_capturing():
        return False
    st = _index_stats(_hot_key(device, B, K, F, D, weight_dtype), B, K, F)
    return st is not None and st["dense"]


def _index_stats(key, B, K, F):
    """What the last measured step of the shape said about its indices (None: nothing yet)."""
    st = _hot_auto.get(key)
    if st is None:
        return None
    if st["event"] is not None and st["event"].query():  # the previous step's measurement has arrived
        long_pairs = int(st["pinned"][1]) * 64
        st["hot"] = long_pairs >= _HOT_AUTO_FRACTION * B * K
        st["dense"] = int(st["pinned"][2]) < _DENSE_AUTO_FRACTION * F
        st["event"] = None
    return st


def _hot_measure(lib, shape, workspace: Tensor, B, K, F, D, weight_dtype) -> None:
    """Leave the skew of this step's indices where the next step of the shape finds it."""
    wanted = ((_hot_latents == "auto" and _hot_latents_supported(B, K, F, D, weight_dtype))
              or (_dense_latents == "auto" and B * K <= 2 * F))
    if not wanted or torch.cuda.is_current_stream_capturing():
        return
    key = _hot_key(workspace.device, B, K, F, D, weight_dtype)
    st = _hot_auto.get(key)
    if st is None:
        st = _hot_auto[key] = {"hot": False, "dense": False,
                               "pinned": torch.zeros(3, dtype=torch.int32, pin_memory=True), "event": None}
    if st["event"] is not None:
        return  # a measurement is still on its way
    rc = lib.flexsae_hier_pair_stats(ctypes.byref(shape), _ptr(workspace), _ptr(st["pinned"]), _stream())
    _lib.check(rc, "flexsae_hier_pair_stats")
    ev = torch.cuda.Event()
    ev.record()
    st["event"] = ev


def _hot_slice_cols(B: int, cols: int, device) -> int:
    """Slice width for the hot-latent kernel: one block per (128 rows, 128 columns), so a slice
    should hold a whole number of rounds of one block per compute unit; never narrower than `cols`
    unless that already is such a width."""
    n_cu = torch.cuda.get_device_properties(device).multi_processor_count
    row_blocks = -(-B // _HOT_ROWS_PER_BLOCK)
    tiles = max(1, round(n_cu / row_blocks))
    want = 128 * tiles
    return want if cols <= want else (cols // want) * want


# Memory the fused training step may hold between forward and backward: all B*K*D per-pair
# contributions (2 bytes each for bf16 weights, else 4) plus the pair list.  The default is 0:
# memory stays flat (the step runs slice by slice inside the scratch above, and only the weight
# gradient itself waits for the backward).  A budget that covers the contributions makes the step
# about 5 % faster at the price of that memory.
_hier_stage_bytes = (int(os.environ["FLEXSAE_HIER_STAGE_MB"]) << 20) if "FLEXSAE_HIER_STAGE_MB" in os.environ else 0


def set_hier_stage_bytes(nbytes) -> None:
    """Upper bound (bytes) on what the fused training step may keep alive from forward to
    backward beyond the gradients themselves.  0 or None (the default): nothing, the step runs
    slice by slice in the scratch of ``set_hier_scratch_bytes`` and memory stays flat.  A budget
    that holds all B*K*D per-pair contributions (2 bytes each for bf16 weights, else 4) lets the
    step write them once and reduce them in the backward, which is a little faster."""
    global _hier_stage_bytes
    _hier_stage_bytes = 0 if nbytes is None else int(nbytes)


def hier_stage_bytes(device=None) -> int:
    """The stage budget in force (the same for every device)."""
    return _hier_stage_bytes


# ---- one pair list for both losses ---------------------------------------------------------
# While a `shared_pair_list()` block is active, the latent-major pair list (begin[F+1], map[B*K])
# of an `indices` tensor is built by the first backward that needs it and reused by the others.
_pair_cache = None


@contextlib.contextmanager
def shared_pair_list():
    """Share the latent-major pair list between losses evaluated on the same ``indices`` tensor.

    Inside the block, the first TopK or hierarchical call that needs the list of an ``indices``
    tensor builds it; later calls on the same tensor (same storage, unmodified) reuse it instead
    of rebuilding it, e.g. when a training step evaluates both losses.  Results do not change.
    The cached lists (and the ``indices`` tensors they belong to) are released when the block ends."""
    global _pair_cache
    outer = _pair_cache
    if outer is None:
        _pair_cache = {}
    try:
        yield
    finally:
        _pair_cache = outer


def _pair_key(indices: Tensor, F: int):
    return (indices.data_ptr(), indices._version, tuple(indices.shape), F, indices.device.index)


def _pair_lookup(indices: Tensor, F: int):
    if _pair_cache is None:
        return None
    hit = _pair_cache.get(_pair_key(indices, F))
    return None if hit is None else hit[1:]


def _pair_store(indices: Tensor, F: int, begin: Tensor, pair_map: Tensor) -> None:
    if _pair_cache is not None:
        # the entry keeps `indices` alive, so its address cannot be handed to another tensor
        _pair_cache[_pair_key(indices, F)] = (indices, begin, pair_map)


def _pair_import(lib, shape, workspace: Tensor, cached) -> None:
    begin, pair_map = cached
    rc = lib.flexsae_hier_import_pair_list(ctypes.byref(shape), _ptr(begin), _ptr(pair_map), _ptr(workspace),
                                           workspace.numel(), _stream())
    _lib.check(rc, "flexsae_hier_import_pair_list")


def _pair_export(lib, shape, workspace: Tensor, indices: Tensor, F: int) -> None:
    if _pair_cache is None:
        return
    ob, om = ctypes.c_size_t(), ctypes.c_size_t()
    _lib.check(lib.flexsae_hier_pair_list_layout(ctypes.byref(shape), ctypes.byref(ob), ctypes.byref(om)),
               "flexsae_hier_pair_list_layout")
    n_pairs = indices.numel()
    begin = workspace[ob.value: ob.value + (F + 1) * 4].view(torch.int32).clone()
    pair_map = workspace[om.value: om.value + n_pairs * 4].view(torch.int32).clone()
    _pair_store(indices, F, begin, pair_map)


@torch.library.custom_op("flexsae_amd::hier_bwd", mutates_args=())
def hier_bwd(grad_out: Tensor, indices: Tensor, weight: Tensor, vals: Tensor,
             resid: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    lib = _lib.load()
    B, K = indices.shape
    F, D = weight.shape
    dev = weight.device
    indices, weight, vals, resid = (_prep(t) for t in (indices, weight, vals, resid))
    with torch.cuda.device(dev):
        g = _grad_scalar(grad_out, dev)
        shape = _shape(B, K, F, D, weight, vals, torch.float32, torch.float32)
        dvals = torch.empty((B, K), dtype=torch.float32, device=dev)
        dbias = torch.empty((D,), dtype=torch.float32, device=dev)
        if _hier_scratch_budget(B, K, F, D, weight.dtype) > 0:
            slice_cols = _hier_slice_cols(B, K, F, D, weight.dtype)
            ws_bytes = lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(shape), slice_cols)
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            dW = torch.empty_like(weight)
            cached = _pair_lookup(indices, F)
            if cached is not None:
                _pair_import(lib, shape, workspace, cached)
            rc = lib.flexsae_hier_bwd(ctypes.byref(shape), _ptr(indices), _ptr(weight), _ptr(vals), _ptr(resid),
                                      _ptr(g), _ptr(dW), _DTYPES[weight.dtype], _ptr(dvals), _ptr(dbias),
                                      _ptr(workspace), ws_bytes,
                                      _lib.BWD_REUSE_PAIR_LIST if cached is not None else 0,
                                      _ptr(_flag_for(dev)), _stream())
            _lib.check(rc, "flexsae_hier_bwd")
            if cached is None:
                _pair_export(lib, shape, workspace, indices, F)
            return dW, dvals, dbias
        dW_acc = torch.empty((F, D), dtype=torch.float32, device=dev)
        rc = lib.flexsae_hier_bwd_atomic(ctypes.byref(shape), _ptr(indices), _ptr(weight), _ptr(vals),
                                         _ptr(resid), _ptr(g), _ptr(dW_acc), _ptr(dvals), _ptr(dbias), 0,
                                         _ptr(_flag_for(dev)), _stream())
        _lib.check(rc, "flexsae_hier_bwd_atomic")
        if weight.dtype == torch.float32:
            dW = dW_acc
        else:
            dW = torch.empty_like(weight)
            rc = lib.flexsae_cast_from_f32(_ptr(dW), _DTYPES[weight.dtype], _ptr(dW_acc), F * D, _stream())
            _lib.check(rc, "flexsae_cast_from_f32")
    return dW, dvals, dbias


# With bf16 weights the TopK backward gathers a bf16 copy of the residual (half the cache footprint;
# the reference's backward also receives the residual gradient in the weight dtype, reference
# torch-ext/flex_sae/topk_kernels.py:52).  That rounding shows in `vals.grad` (about 4e-3 normwise
# instead of 1e-6); switching it off gathers the fp32 residual instead, a little slower.
_topk_residual_bf16 = os.environ.get("FLEXSAE_TOPK_RESIDUAL_BF16", "1") not in ("", "0")


def set_topk_residual_bf16(enabled: bool) -> None:
    """bf16 weights only: whether the TopK backward reads a bf16 copy of the residual (default,
    faster) or the fp32 residual itself (``vals.grad`` then carries fp32 rounding only)."""
    global _topk_residual_bf16
    _topk_residual_bf16 = bool(enabled)


@torch.library.custom_op("flexsae_amd::topk_bwd", mutates_args=())
def topk_bwd(grad_out: Tensor, indices: Tensor, weight: Tensor, vals: Tensor,
             resid: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    lib = _lib.load()
    B, K = indices.shape
    F, D = weight.shape
    dev = weight.device
    indices, weight, vals, resid = (_prep(t) for t in (indices, weight, vals, resid))
    with torch.cuda.device(dev):
        g = _grad_scalar(grad_out, dev)
        shape = _shape(B, K, F, D, weight, vals, torch.float32, torch.float32)
        cached = _pair_lookup(indices, F)
        if cached is not None:
            begin, pair_map = cached
        else:
            begin = torch.empty(F + 1, dtype=torch.int32, device=dev)   # uint32 payload
            pair_map = torch.empty(B * K, dtype=torch.int32, device=dev)  # uint32 payload
            ws_bytes = lib.flexsae_csr_workspace_bytes(B, K, F)
            workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
            rc = lib.flexsae_csr_build(_ptr(indices), B, K, F, _ptr(begin), _ptr(pair_map), _ptr(workspace),
                                       ws_bytes, _ptr(_flag_for(dev)), _stream())
            _lib.check(rc, "flexsae_csr_build")
            _pair_store(indices, F, begin, pair_map)
        dW = torch.empty_like(weight)
        dvals = torch.empty((B, K), dtype=torch.float32, device=dev)
        dbias = torch.empty((D,), dtype=torch.float32, device=dev)
        # the slice width only sizes the partial sums of hot latents; one launch over all of D is
        # fastest, so allow them 256 MiB before slicing
        slice_cols = max(1, (256 << 20) // max(1, (B * K // 32) * 4))
        bws_bytes = lib.flexsae_topk_bwd_workspace_bytes(ctypes.byref(shape), slice_cols)
        bws = torch.empty(bws_bytes, dtype=torch.uint8, device=dev)
        rc = lib.flexsae_topk_bwd(ctypes.byref(shape), _ptr(begin), _ptr(pair_map), _ptr(indices), _ptr(weight),
                                  _ptr(vals), _ptr(resid), _ptr(g), _ptr(dW), _DTYPES[weight.dtype], _ptr(dvals),
                                  _ptr(dbias), _ptr(bws), bws_bytes,
                                  0 if _topk_residual_bf16 else _lib.TOPK_BWD_FP32_RESIDUAL, _stream())
        _lib.check(rc, "flexsae_topk_bwd")
    return dW, dvals, dbias


def _bwd_fake(grad_out, indices, weight, vals, resid):
    return (torch.empty_like(weight), vals.new_empty(vals.shape, dtype=torch.float32),
            weight.new_empty((weight.shape[1],), dtype=torch.float32))


hier_bwd.register_fake(_bwd_fake)
topk_bwd.register_fake(_bwd_fake)


def _setup_context(ctx, inputs, output):
    indices, weight, vals, bias, target = inputs
    _, resid = output
    ctx.save_for_backward(indices, weight, vals, resid)
    ctx.leaf_dtypes = (vals.dtype, bias.dtype, target.dtype)
    ctx.set_materialize_grads(False)  # no zero-filled gradient for the saved residual


# Training-step fusion: when gradients will be needed, compute loss and (unit-gradient) gradients
# in one pass that gathers the weight rows once; the backward then only scales by grad_out.
_fused_training = os.environ.get("FLEXSAE_FUSED_TRAINING", "1") not in ("", "0")


def set_fused_training(enabled: bool) -> None:
    """Enable/disable the fused forward + reverse walk of the hierarchical loss (default on).

    When gradients are required, loss and gradients come out of one pass that gathers the weight
    rows once per training step instead of twice; the gradients are those of a unit upstream
    gradient and the backward only scales them.  By default the pass runs slice by slice with an
    immediate segment reduction (flat memory); with a stage budget (``set_hier_stage_bytes``)
    that holds all per-pair contributions, they are written once and reduced in the backward.
    Code that evaluates the loss with gradients enabled but never calls ``backward()`` pays for
    the reverse walk anyway: switch it off there or use ``torch.no_grad()``."""
    global _fused_training
    _fused_training = bool(enabled)


def _train_supported(weight: Tensor, K: int) -> bool:
    D = weight.shape[1]
    return D % 4 == 0 and K <= 256


def _stage_fits(indices: Tensor, weight: Tensor) -> bool:
    """Staging keeps one contribution per (b, k, d) alive until the backward; it is chosen only
    when the stage budget covers that."""
    B, K = indices.shape
    D = weight.shape[1]
    p_size = 2 if weight.dtype == torch.bfloat16 else 4
    return B * K * (-(-D // 256) * 256) * p_size <= hier_stage_bytes(weight.device)


def _single_slice_workspace_bytes(lib, shape, D: int) -> int:
    return lib.flexsae_hier_bwd_workspace_bytes(ctypes.byref(shape), D)


def hier_train_stage(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor, target: Tensor) -> Tensor:
    """A fresh (uninitialised) stage for ``hier_train``: the workspace that holds the pair list and
    all per-pair contributions of one step of these shapes.  Eager mode only: the size comes from
    the library (a host-side query through ctypes, which a compiler trace cannot follow)."""
    B, K, F, D = _validate(indices, weight, vals, bias, target)
    shape = _shape(B, K, F, D, weight, vals, bias.dtype, target.dtype)
    return torch.empty(_single_slice_workspace_bytes(_lib.load(), shape, D), dtype=torch.uint8, device=weight.device)


@torch.library.custom_op("flexsae_amd::hier_train", mutates_args=("stage",))
def hier_train(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor, target: Tensor,
               stage: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """Fused forward + reverse walk with the segment reduction deferred.

    Returns (loss, dvals, dbias), dvals/dbias for a unit upstream gradient, and fills ``stage``
    (from ``hier_train_stage``; scratch that the op mutates, not an output: its bytes are of no
    meaning to the caller and partly unwritten) with the pair list and all per-pair
    contributions, from which ``hier_finish`` produces dW with the upstream gradient folded in."""
    B, K, F, D = _validate(indices, weight, vals, bias, target)
    lib = _lib.load()
    indices, weight, vals, bias, target = (_prep(t) for t in (indices, weight, vals, bias, target))
    dev = weight.device
    if stage.dtype != torch.uint8 or stage.device != dev or not stage.is_contiguous():
        raise ValueError("stage must be a contiguous uint8 tensor on the weight's device (see hier_train_stage)")
    with torch.cuda.device(dev):
        shape = _shape(B, K, F, D, weight, vals, bias.dtype, target.dtype)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dvals = torch.empty((B, K), dtype=torch.float32, device=dev)
        dbias = torch.empty((D,), dtype=torch.float32, device=dev)
        flag = _flag_for(dev)
        cached = _pair_lookup(indices, F)
        if cached is not None:
            _pair_import(lib, shape, stage, cached)
        flags = _lib.BWD_SWEEP_ONLY | (_lib.BWD_REUSE_PAIR_LIST if cached is not None else 0)
        rc = lib.flexsae_hier_fwd_bwd(ctypes.byref(shape), _ptr(indices), _ptr(weight), _ptr(vals), _ptr(bias),
                                      _ptr(target), _ptr(loss), None, _DTYPES[weight.dtype], _ptr(dvals),
                                      _ptr(dbias), _ptr(stage), stage.numel(), flags, _ptr(flag), _stream())
        _lib.check(rc, "flexsae_hier_fwd_bwd (stage too small or misaligned?)" if rc == _lib.ERR_WORKSPACE
                   else "flexsae_hier_fwd_bwd")
        if cached is None:
            _pair_export(lib, shape, stage, indices, F)
        if _check_indices:
            check_index_flag(dev)
    return loss, dvals, dbias


@hier_train.register_fake
def _(indices, weight, vals, bias, target, stage):
    return (weight.new_empty((), dtype=torch.float32), vals.new_empty(vals.shape, dtype=torch.float32),
            weight.new_empty((weight.shape[1],), dtype=torch.float32))


@torch.library.custom_op("flexsae_amd::hier_finish", mutates_args=())
def hier_finish(grad_out: Tensor, indices: Tensor, weight: Tensor, vals: Tensor, stage: Tensor) -> Tensor:
    """dW = grad_out * (segment sums of the contributions staged by ``hier_train``)."""
    lib = _lib.load()
    B, K = indices.shape
    F, D = weight.shape
    dev = weight.device
    with torch.cuda.device(dev):
        g = _grad_scalar(grad_out, dev)
        shape = _shape(B, K, F, D, weight, vals, torch.float32, torch.float32)
        dW = torch.empty((F, D), dtype=weight.dtype, device=dev)
        flags = _lib.BWD_REUSE_PAIR_LIST | _lib.BWD_REDUCE_ONLY | _lib.BWD_SCALE_BY_GRAD_OUT
        rc = lib.flexsae_hier_bwd(ctypes.byref(shape), None, None, None, None, _ptr(g), _ptr(dW),
                                  _DTYPES[weight.dtype], None, None, _ptr(stage), stage.numel(), flags, None,
                                  _stream())
        _lib.check(rc, "flexsae_hier_bwd (deferred reduction)")
    return dW


@hier_finish.register_fake
def _(grad_out, indices, weight, vals, stage):
    return torch.empty_like(weight)


class _HierTrainStaged(torch.autograd.Function):
    """Autograd glue of the staged step (eager mode): ``hier_train`` fills a fresh stage in the
    forward, ``hier_finish`` reduces it with the upstream gradient folded in (the counterpart of
    reference torch-ext/flex_sae/hierarchical_kernels.py:273-299).  ``hier_train`` mutates its stage
    argument, so it carries no autograd formula of its own."""

    @staticmethod
    def forward(ctx, indices, weight, vals, bias, target):
        stage = hier_train_stage(indices, weight, vals, bias, target)
        loss, dvals, dbias = hier_train(indices, weight, vals, bias, target, stage)
        ctx.save_for_backward(indices, weight, vals, dvals, dbias, stage)
        ctx.leaf_dtypes = (vals.dtype, bias.dtype)
        return loss

    @staticmethod
    def backward(ctx, grad_loss):
        indices, weight, vals, dvals, dbias, stage = ctx.saved_tensors
        g = grad_loss.to(torch.float32)
        vdt, bdt = ctx.leaf_dtypes
        dW = hier_finish(g, indices, weight, vals, stage) if ctx.needs_input_grad[1] else None
        return None, dW, (dvals * g).to(vdt), (dbias * g).to(bdt), None


@torch.library.custom_op("flexsae_amd::hier_train_sliced", mutates_args=())
def hier_train_sliced(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor,
                      target: Tensor, need_dw: bool = True, hot: bool = False,
                      dense: bool = False) -> Tuple[Tensor, Tensor, Tensor, Tensor]:
    """Fused forward + reverse walk in column slices, each reduced right away (flat memory).

    Used when the contributions of a whole step do not fit the stage budget: the scratch is one
    slice of them (``set_hier_scratch_bytes``), and every slice gathers its weight-row pieces once
    for both walks.  Returns (loss, dvals, dbias, dW), the gradients for a unit upstream gradient;
    the backward scales them.  With ``need_dw`` false (a decoder whose weight takes no gradient)
    the segment reductions are left out and the returned dW is empty.  ``hot`` and ``dense`` are the
    library's FLEXSAE_BWD_HOT_LATENTS and FLEXSAE_BWD_DENSE_LATENTS hints."""
    B, K, F, D = _validate(indices, weight, vals, bias, target)
    lib = _lib.load()
    indices, weight, vals, bias, target = (_prep(t) for t in (indices, weight, vals, bias, target))
    dev = weight.device
    with torch.cuda.device(dev):
        shape = _shape(B, K, F, D, weight, vals, bias.dtype, target.dtype)
        slice_cols = _hier_slice_cols(B, K, F, D, weight.dtype)
        hot_flag = _lib.BWD_HOT_LATENTS if (hot and need_dw) else 0
        if hot_flag:
            slice_cols = _hot_slice_cols(B, slice_cols, dev)
        ws_bytes = lib.flexsae_hier_fwd_bwd_workspace_bytes_flags(ctypes.byref(shape), slice_cols, hot_flag)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dw_dtype = _unit_dw_dtype(weight.dtype)
        dW = torch.empty((F, D), dtype=dw_dtype, device=dev) if need_dw else weight.new_empty((0, D), dtype=dw_dtype)
        dvals = torch.empty((B, K), dtype=torch.float32, device=dev)
        dbias = torch.empty((D,), dtype=torch.float32, device=dev)
        flag = _flag_for(dev)
        cached = _pair_lookup(indices, F)
        if cached is not None:
            _pair_import(lib, shape, workspace, cached)
        flags = ((_lib.BWD_REUSE_PAIR_LIST if cached is not None else 0) | (0 if need_dw else _lib.BWD_NO_DW) |
                 hot_flag | (_lib.BWD_DENSE_LATENTS if dense else 0))
        rc = lib.flexsae_hier_fwd_bwd(ctypes.byref(shape), _ptr(indices), _ptr(weight), _ptr(vals), _ptr(bias),
                                      _ptr(target), _ptr(loss), _ptr(dW) if need_dw else None,
                                      _DTYPES[dw_dtype], _ptr(dvals),
                                      _ptr(dbias), _ptr(workspace), ws_bytes, flags, _ptr(flag), _stream())
        _lib.check(rc, "flexsae_hier_fwd_bwd")
        if cached is None:
            _pair_export(lib, shape, workspace, indices, F)
        if need_dw:
            _hot_measure(lib, shape, workspace, B, K, F, D, weight.dtype)
        if _check_indices:
            check_index_flag(dev)
    return loss, dvals, dbias, dW


def _unit_dw_dtype(weight_dtype):
    """dtype of the unit-gradient dW of the sliced step: the weight's, but fp32 for fp16 weights."""
    return torch.float32 if weight_dtype == torch.float16 else weight_dtype


@hier_train_sliced.register_fake
def _(indices, weight, vals, bias, target, need_dw=True, hot=False, dense=False):
    dw_dtype = _unit_dw_dtype(weight.dtype)
    return (weight.new_empty((), dtype=torch.float32), vals.new_empty(vals.shape, dtype=torch.float32),
            weight.new_empty((weight.shape[1],), dtype=torch.float32),
            weight.new_empty(weight.shape, dtype=dw_dtype) if need_dw
            else weight.new_empty((0, weight.shape[1]), dtype=dw_dtype))


@torch.library.custom_op("flexsae_amd::hier_sgd_step", mutates_args=("weight",))
def hier_sgd_step(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor, target: Tensor,
                  step: Tensor) -> Tuple[Tensor, Tensor, Tensor]:
    """HierarchicalTopK training step with the plain-SGD decoder update fused in.

    ``weight[f] -= step * dL/dW[f]`` for every latent f that ``indices`` touches, in place (fp32
    arithmetic, one rounding to the weight's dtype); no dense gradient is formed and rows of
    untouched latents are neither read nor written.  ``step`` is a 0-dim tensor: learning rate
    times the upstream gradient of the loss.  Returns (loss, dvals, dbias) for a unit upstream
    gradient and the weights as they were on entry: feed ``dvals`` to the encoder's backward
    (``vals.backward(dvals * upstream)``) and apply ``dbias`` to the bias.
    Takes the place of ``loss.backward(); torch.optim.SGD.step()`` for the decoder weight in a loop
    written like reference example.py:76-77; with momentum or weight decay untouched rows change
    too, and the dense gradient of ``triton_hierarchical_sae_loss`` is the interface to use.
    ``weight`` must be contiguous and 16-byte aligned, D a multiple of 8 (16-bit) or 4 (fp32),
    K <= 256."""
    B, K, F, D = _validate(indices, weight, vals, bias, target)
    if not weight.is_contiguous() or weight.data_ptr() % 16:
        raise ValueError("hier_sgd_step updates weight in place: it must be contiguous and 16-byte aligned")
    if not _train_supported(weight, K):
        raise ValueError("hier_sgd_step needs D % 4 == 0 and K <= 256")
    lib = _lib.load()
    indices, vals, bias, target = (_prep(t) for t in (indices, vals, bias, target))
    dev = weight.device
    with torch.cuda.device(dev):
        shape = _shape(B, K, F, D, weight, vals, bias.dtype, target.dtype)
        slice_cols = _hier_slice_cols(B, K, F, D, weight.dtype)
        # hot-latent accumulators: the same decision as the loss takes (set_hot_latents)
        hot_flag = _lib.BWD_HOT_LATENTS if _use_hot_latents(B, K, F, D, weight.dtype, dev, _is_traced(weight)) else 0
        dense_flag = (_lib.BWD_DENSE_LATENTS
                      if _use_dense_latents(B, K, F, D, weight.dtype, dev, _is_traced(weight)) else 0)
        if hot_flag:
            slice_cols = _hot_slice_cols(B, slice_cols, dev)
        ws_bytes = lib.flexsae_hier_fwd_bwd_workspace_bytes_flags(ctypes.byref(shape), slice_cols, hot_flag)
        workspace = torch.empty(ws_bytes, dtype=torch.uint8, device=dev)
        loss = torch.empty((), dtype=torch.float32, device=dev)
        dvals = torch.empty((B, K), dtype=torch.float32, device=dev)
        dbias = torch.empty((D,), dtype=torch.float32, device=dev)
        g = _grad_scalar(step, dev)
        flag = _flag_for(dev)
        cached = _pair_lookup(indices, F)
        if cached is not None:
            _pair_import(lib, shape, workspace, cached)
        rc = lib.flexsae_hier_sgd_step(ctypes.byref(shape), _ptr(indices), _ptr(weight), _ptr(vals), _ptr(bias),
                                       _ptr(target), _ptr(g), _ptr(loss), _ptr(dvals), _ptr(dbias),
                                       _ptr(workspace), ws_bytes,
                                       (_lib.BWD_REUSE_PAIR_LIST if cached is not None else 0) | hot_flag | dense_flag,
                                       _ptr(flag),
                                       _stream())
        _lib.check(rc, "flexsae_hier_sgd_step")
        if cached is None:
            _pair_export(lib, shape, workspace, indices, F)
        if not _is_traced(weight):
            _hot_measure(lib, shape, workspace, B, K, F, D, weight.dtype)
        if _check_indices:
            check_index_flag(dev)
    return loss, dvals, dbias


@hier_sgd_step.register_fake
def _(indices, weight, vals, bias, target, step):
    return (weight.new_empty((), dtype=torch.float32), vals.new_empty(vals.shape, dtype=torch.float32),
            weight.new_empty((weight.shape[1],), dtype=torch.float32))


def hierarchical_sae_sgd_step(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor, target: Tensor,
                              lr: float, grad_out=1.0) -> Tuple[Tensor, Tensor, Tensor]:
    """``hier_sgd_step`` with a learning rate and an optional upstream gradient (float or 0-dim
    tensor).  Runs without autograd: ``weight`` may be a leaf that requires grad; it is updated through
    ``weight.data`` semantics (under ``torch.no_grad()``).  Returns (loss, dvals, dbias), unit upstream gradient."""
    with torch.no_grad():
        if isinstance(grad_out, Tensor):
            step = (grad_out.detach().to(device=weight.device, dtype=torch.float32) * lr).reshape(())
        else:
            step = torch.tensor(float(lr) * float(grad_out), dtype=torch.float32, device=weight.device)
        return hier_sgd_step(indices, weight, vals.detach(), bias.detach(), target, step)


@torch.library.custom_op("flexsae_amd::scale_by", mutates_args=())
def scale_by(x: Tensor, grad_out: Tensor) -> Tensor:
    """x * grad_out (a 0-dim scalar on the device), in x's dtype; replaces the reference's
    ``dW.mul_(grad)`` (hierarchical_kernels.py:294-297) after a unit-gradient pass."""
    lib = _lib.load()
    dev = x.device
    with torch.cuda.device(dev):
        g = _grad_scalar(grad_out, dev)
        x = _prep(x)
        out = torch.empty_like(x)
        rc = lib.flexsae_scale(_ptr(out), _ptr(x), _DTYPES[x.dtype], x.numel(), _ptr(g), _stream())
        _lib.check(rc, "flexsae_scale")
    return out


@scale_by.register_fake
def _(x, grad_out):
    return torch.empty_like(x)


@torch.library.custom_op("flexsae_amd::scale_to", mutates_args=())
def scale_to(x: Tensor, grad_out: Tensor, dtype: torch.dtype) -> Tensor:
    """(x * grad_out) rounded once to ``dtype``; x is fp32.  For fp16 weights: the unit-gradient dW is
    kept in fp32 and takes the upstream gradient (a loss scale, typically) before it is rounded, like
    the reference's fp32 ``mul_`` followed by the engine's cast (hierarchical_kernels.py:294-299)."""
    if x.dtype != torch.float32:
        raise TypeError("scale_to expects a float32 tensor")
    lib = _lib.load()
    dev = x.device
    with torch.cuda.device(dev):
        g = _grad_scalar(grad_out, dev)
        x = _prep(x)
        out = torch.empty(x.shape, dtype=dtype, device=dev)
        rc = lib.flexsae_scale_from_f32(_ptr(out), _DTYPES[dtype], _ptr(x), x.numel(), _ptr(g), _stream())
        _lib.check(rc, "flexsae_scale_from_f32")
    return out


@scale_to.register_fake
def _(x, grad_out, dtype):
    return x.new_empty(x.shape, dtype=dtype)


@torch.library.custom_op("flexsae_amd::scale_", mutates_args=("x",))
def scale_(x: Tensor, grad_out: Tensor) -> None:
    """x *= grad_out in place (x contiguous); a grad_out of exactly one costs an empty launch."""
    lib = _lib.load()
    dev = x.device
    if not x.is_contiguous():
        raise ValueError("scale_ needs a contiguous tensor")
    with torch.cuda.device(dev):
        g = _grad_scalar(grad_out, dev)
        rc = lib.flexsae_scale(_ptr(x), _ptr(x), _DTYPES[x.dtype], x.numel(), _ptr(g), _stream())
        _lib.check(rc, "flexsae_scale")


@scale_.register_fake
def _(x, grad_out):
    return None


def _is_traced(t: Tensor) -> bool:
    """True while a compiler traces the call (fake or functional tensors instead of real ones)."""
    return type(t) is not torch.Tensor or torch.compiler.is_compiling()


def _train_sliced_setup_context(ctx, inputs, output):
    indices, weight, vals, bias, target, need_dw, hot, dense = inputs
    ctx.need_dw = need_dw
    ctx.hot = hot
    ctx.dense = dense
    _, dvals, dbias, dW = output
    ctx.mark_non_differentiable(dvals, dbias, dW)
    ctx.leaf_dtypes = (vals.dtype, bias.dtype)
    ctx.set_materialize_grads(False)
    # The unit-gradient dW is as large as the weight.  In eager mode it is kept outside the saved
    # tensors so that the backward can scale it in place and hand the very buffer on as the weight
    # gradient (it carries no autograd history, so keeping it on ctx forms no reference cycle).
    ctx.dw_in_place = not _is_traced(dW)
    if ctx.dw_in_place:
        ctx.save_for_backward(indices, weight, vals, bias, target, dvals, dbias)
        ctx.dw_unit = dW if ctx.needs_input_grad[1] else None
    else:
        ctx.save_for_backward(indices, weight, vals, bias, target, dvals, dbias, dW)


def _train_sliced_backward(ctx, grad_loss, grad_dvals, grad_dbias, grad_dw):
    if grad_loss is None:
        return None, None, None, None, None, None, None, None
    if ctx.needs_input_grad[1] and not ctx.need_dw:
        raise RuntimeError("hier_train_sliced was called with need_dw=False but weight requires a gradient")
    g = grad_loss.to(torch.float32)
    vdt, bdt = ctx.leaf_dtypes
    if not ctx.dw_in_place:
        indices, weight, vals, bias, target, dvals, dbias, dW_unit = ctx.saved_tensors
        dW = None
        if ctx.needs_input_grad[1]:
            dW = scale_by(dW_unit, g) if dW_unit.dtype == weight.dtype else scale_to(dW_unit, g, weight.dtype)
    else:
        indices, weight, vals, bias, target, dvals, dbias = ctx.saved_tensors
        dW = None
        if ctx.needs_input_grad[1]:
            dW = ctx.dw_unit
            ctx.dw_unit = None  # the buffer now belongs to whoever receives the gradient
            if dW is None:
                # a second backward through a retained graph: the buffer went with the first one
                with torch.no_grad():
                    _, dvals, dbias, dW = hier_train_sliced(indices, weight, vals, bias, target, True, ctx.hot, ctx.dense)
            if dW.dtype == weight.dtype:
                scale_(dW, g)
            else:  # fp16 weights: the fp32 unit gradient meets the upstream gradient before its only rounding
                dW = scale_to(dW, g, weight.dtype)
    return None, dW, (dvals * g).to(vdt), (dbias * g).to(bdt), None, None, None, None


hier_train_sliced.register_autograd(_train_sliced_backward, setup_context=_train_sliced_setup_context)


def _hier_backward(ctx, grad_loss, grad_resid):
    indices, weight, vals, resid = ctx.saved_tensors
    if grad_loss is None:
        return None, None, None, None, None
    dW, dvals, dbias = hier_bwd(grad_loss, indices, weight, vals, resid)
    vdt, bdt, _ = ctx.leaf_dtypes
    # no gradient for target on this path (reference hierarchical_kernels.py:299)
    return None, dW, dvals.to(vdt), dbias.to(bdt), None


def _topk_backward(ctx, grad_loss, grad_resid):
    indices, weight, vals, resid = ctx.saved_tensors
    if grad_loss is None:
        return None, None, None, None, None
    dW, dvals, dbias = topk_bwd(grad_loss, indices, weight, vals, resid)
    vdt, bdt, tdt = ctx.leaf_dtypes
    dtarget = None
    if ctx.needs_input_grad[4]:
        # the reference's eager loss tail is differentiable w.r.t. target (topk_kernels.py:221)
        B, D = resid.shape
        dtarget = (resid * (grad_loss.to(torch.float32) * (-2.0 / (B * D)))).to(tdt)
    return None, dW, dvals.to(vdt), dbias.to(bdt), dtarget


hier_fwd.register_autograd(_hier_backward, setup_context=_setup_context)
topk_fwd.register_autograd(_topk_backward, setup_context=_setup_context)


def triton_hierarchical_sae_loss(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor,
                                 target: Tensor) -> Tensor:
    """Fused HierarchicalTopK decoder loss (0-dim fp32), differentiable w.r.t. weight, vals, bias.

    Same name, argument order and meaning as the reference entry point
    (torch-ext/flex_sae/hierarchical_kernels.py:302-309); the kernels underneath are HIP."""
    if indices.dtype == torch.int32:
        indices = indices.to(torch.int64)
    needs_grad = torch.is_grad_enabled() and (weight.requires_grad or vals.requires_grad or bias.requires_grad)
    if (needs_grad and _fused_training and weight.dim() == 2 and indices.dim() == 2
            and _train_supported(weight, indices.shape[1])):
        # (a compiler trace cannot follow the stage's size query: traced calls take the sliced step,
        # which gives the same bits)
        if _stage_fits(indices, weight) and not _is_traced(weight):
            return _HierTrainStaged.apply(indices, weight, vals, bias, target)
        # (fp16 weights: the step's unit-gradient dW is fp32, of magnitude 2/(B*K*D), and is scaled by the
        # upstream gradient before its only rounding, like reference hierarchical_kernels.py:294-299)
        if _hier_scratch_bytes != 0:
            B, K = indices.shape
            F, D = weight.shape
            hot = bool(weight.requires_grad) and _use_hot_latents(B, K, F, D, weight.dtype, weight.device,
                                                                   _is_traced(weight))
            dense = bool(weight.requires_grad) and _use_dense_latents(B, K, F, D, weight.dtype, weight.device,
                                                                       _is_traced(weight))
            return hier_train_sliced(indices, weight, vals, bias, target, bool(weight.requires_grad), hot, dense)[0]
    return hier_fwd(indices, weight, vals, bias, target)[0]


def triton_topk_sae_loss(indices: Tensor, weight: Tensor, vals: Tensor, bias: Tensor,
                         target: Tensor) -> Tensor:
    """Fused TopK decoder loss (0-dim fp32), differentiable w.r.t. weight, vals, bias, target.

    Same name, argument order and meaning as the reference entry point
    (torch-ext/flex_sae/topk_kernels.py:213-223); the kernels underneath are HIP."""
    if indices.dtype == torch.int32:
        indices = indices.to(torch.int64)
    return topk_fwd(indices, weight, vals, bias, target)[0]
