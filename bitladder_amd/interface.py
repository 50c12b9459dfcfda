"""Python entry points of the low-bit KV-cache decode path, drop-in for the reference's
`bit_decode/bit_decode_interface.py`: same names, positional order, defaults, tensor shapes and
dtypes.  Host code is PyTorch (device memory, streams); all device work goes through the C ABI
of libbitdecode.so (hand-written HIP for gfx950).  Keyword-only arguments are extensions.
"""
from __future__ import annotations

import ctypes
import threading
from typing import Optional, Union

import torch

from . import _lib

_PACK_DTYPES = (torch.uint16, torch.int16)
_PARAM_DTYPES = (torch.float32,)
CHUNK = 128


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float16:
        return _lib.FP16
    if t.dtype == torch.bfloat16:
        return _lib.BF16
    # decode_api.cpp:531-533: "only support fp16 and bf16 data type"
    raise RuntimeError("bit_decode only supports fp16 and bf16 data type")


def _check_quant(quant_mode: str, group_size: int, num_bits: int) -> int:
    """Returns the C ABI's code of the quantization mode."""
    if quant_mode not in ("k-channel", "k-tensor"):
        raise ValueError(f"quant_mode must be 'k-channel' or 'k-tensor', got {quant_mode!r}")
    if num_bits not in (2, 4):
        raise ValueError(f"num_bits must be 2 or 4, got {num_bits}")
    if group_size not in (32, 64, 128):
        raise ValueError(f"group_size must be 32, 64 or 128, got {group_size}")
    if quant_mode == "k-tensor" and num_bits != 4:
        # the reference's quantizer for this mode is 4-bit only (qpack.h:385)
        raise NotImplementedError("quant_mode 'k-tensor' is implemented for num_bits=4 only")
    return _lib.K_TENSOR if quant_mode == "k-tensor" else _lib.K_CHANNEL


def _check_block_table(block_table, b, device):
    """Paged cache (decode_api.cpp:328-335): int32 [batch, max_pages_per_seq], last dim contiguous."""
    if block_table.dtype != torch.int32:
        raise RuntimeError("block_table must have dtype torch.int32")
    if block_table.dim() != 2 or block_table.shape[0] != b:
        raise RuntimeError("block_table must be [batch, max_pages_per_seq]")
    if block_table.stride(-1) != 1:
        raise RuntimeError("block_table must have contiguous last dimension")
    if block_table.device != device:
        raise RuntimeError(f"block_table must be on {device}")
    return block_table


def _set_paging(a, block_table, num_pages):
    a.block_table = block_table.data_ptr()
    a.block_table_stride = block_table.stride(0)
    a.max_pages_per_seq = block_table.shape[1]
    a.num_pages = num_pages


def _check_cache(k_pack, k_params, v_pack, v_params, num_bits, group_size, device, k_tensor=False):
    """Validates the caller-allocated packed tensors (evaluation/test.py:74-83) and returns
    (batch, capacity_tokens, h_k).  In "k-tensor" mode K has one (scale, zero) per token and channel
    group, and k_params has v_params' shape."""
    pn = 16 // num_bits
    if v_pack.dim() != 4 or k_pack.dim() != 4 or k_params.dim() != 4 or v_params.dim() != 4:
        raise RuntimeError("k_pack, k_params, v_pack, v_params must be 4-dimensional")
    b, S, h_k, dp = v_pack.shape
    d = dp * pn
    if d != 128:
        raise RuntimeError(f"head dimension {d} is not supported (only 128)")
    if S % CHUNK:
        raise RuntimeError(f"packed cache capacity {S} must be a multiple of {CHUNK} tokens")
    k_params_shape = (b, d // group_size, h_k, S) if k_tensor else (b, S // group_size, h_k, d)
    for name, t, want, dtypes in (("k_pack", k_pack, (b, S // pn, h_k, d), _PACK_DTYPES),
                                  ("k_params", k_params, k_params_shape, _PARAM_DTYPES),
                                  ("v_pack", v_pack, (b, S, h_k, dp), _PACK_DTYPES),
                                  ("v_params", v_params, (b, d // group_size, h_k, S), _PARAM_DTYPES)):
        if t.shape != want:
            raise RuntimeError(f"{name} must have shape {want}, got {tuple(t.shape)}")
        if t.device != device:
            raise RuntimeError(f"{name} must be on {device}")
        if not t.is_contiguous():
            raise RuntimeError(f"{name} must be contiguous")
        if t.dtype not in dtypes:
            if dtypes is _PACK_DTYPES:
                raise RuntimeError(f"{name} must have dtype torch.uint16")
            raise RuntimeError(f"{name} must have dtype torch.float32 (each element holds two 16-bit values)")
    return b, S, h_k


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream_ptr(device) -> int:
    """Handle of torch's current stream on `device` (hipStream_t as an integer)."""
    if _raw_stream is not None:
        return _raw_stream(device.index)
    return torch.cuda.current_stream(device).cuda_stream


class _on_device:
    """`with _on_device(device):` makes `device` current for the block; free when it already is."""

    def __init__(self, device):
        self._ctx = None if torch.cuda.current_device() == device.index else torch.cuda.device(device)

    def __enter__(self):
        if self._ctx is not None:
            self._ctx.__enter__()

    def __exit__(self, *exc):
        if self._ctx is not None:
            self._ctx.__exit__(*exc)
        return False


# Split workspaces of the plain entry points, one per (device, stream, kind, batch, heads, splits): a call
# leaves its workspace ready for the next call of the same shape (counters at zero, the records it used marked
# "not written" again by the call after it), so the next call on the same stream takes the same buffer without
# refilling it (calls on one stream run one after the other; two streams never share a buffer, and neither do
# two shapes).  Plans own their workspace instead: they may be replayed from anywhere.
_WORKSPACES: "dict[tuple, torch.Tensor]" = {}
_MAX_WORKSPACES = 64


def _stream_workspace(device, kind: str, b: int, h: int, ns: int, nbytes: int) -> torch.Tensor:
    key = (device.index, _stream_ptr(device), kind, b, h, ns)
    ws = _WORKSPACES.get(key)
    if ws is None or ws.numel() < nbytes:
        if len(_WORKSPACES) >= _MAX_WORKSPACES:
            _WORKSPACES.pop(next(iter(_WORKSPACES)))
        # zero-filled once: the whole workspace must be 0 before its first call
        ws = torch.zeros(nbytes, dtype=torch.uint8, device=device)
        _WORKSPACES[key] = ws
    return ws


_SPLIT_PLANS: "dict[tuple, tuple]" = {}


def _split_plan(dev_index, b, h, h_k, max_seqlen, max_res, ragged, bits, gs, num_splits):
    """(split count, workspace bytes) of a decode call on the current device; both are pure functions of
    these arguments (and of the device's compute-unit count), so the two library calls are made once.
    `ragged`: the call takes per-sequence packed lengths from the device."""
    key = (dev_index, b, h, h_k, max_seqlen, max_res, ragged, bits, gs, num_splits)
    hit = _SPLIT_PLANS.get(key)
    if hit is None:
        L = _lib.lib()
        ns = num_splits or L.bitdecode_num_splits_for(b, h_k, max_seqlen, max_res, 0, bits, gs, int(ragged))
        hit = (ns, L.bitdecode_fwd_workspace_bytes(b, h, ns))
        if len(_SPLIT_PLANS) >= 4096:
            _SPLIT_PLANS.clear()
        _SPLIT_PLANS[key] = hit
    return hit


# A decode loop over a model makes one distinct call per attention layer and token, each over its layer's own
# cache: the kept argument blocks must cover all layers (a block is a few hundred bytes plus a reference to
# the stream's shared workspace), or every call of the loop would miss.
_MAX_PLANS = 512
_tls = threading.local()


def _plan_cache() -> dict:
    """Argument blocks of this thread's last distinct drop-in calls (a thread of its own each: a block is
    patched with the call's output pointer before it is handed to the library)."""
    c = getattr(_tls, "plans", None)
    if c is None:
        c = _tls.plans = {}
    return c


def _call_key(tensors, scalars, kwargs):
    """Hashable key of a drop-in call: a tensor counts by address, shape, strides and element type (the argument
    block holds nothing else of it), everything else by value; the current stream is part of the key because
    the workspace belongs to it."""
    parts = []
    for t in tensors:
        parts.append(None if t is None else (t.data_ptr(), t.shape, t.stride(), t.dtype))
    for name in sorted(kwargs):
        v = kwargs[name]
        parts.append((name, v.data_ptr(), v.shape, v.stride(), v.dtype) if isinstance(v, torch.Tensor) else (name, v))
    dev = tensors[0].device
    return (tuple(parts), scalars, dev.index, _stream_ptr(dev) if dev.type == "cuda" else 0)


def _run_kept(key, q, kwargs, make_plan):
    """Runs a plain (non-plan) decode call.  A decode loop makes such a call again and again over the same
    memory: the validated argument block of a thread's last distinct calls (up to 512) is kept and found again by the
    address, shape, strides and element type of every tensor, which saves 40 % of the host's time per call."""
    return_lse = kwargs.get("return_lse", False)
    if q.is_cuda and torch.cuda.is_current_stream_capturing():
        # Recorded into a HIP graph: the graph bakes the workspace address in and may be replayed on any stream,
        # at any time.  The call gets a workspace of its own, allocated (and zero-filled by a fill kernel) inside
        # the capture, so it lives in the graph's memory pool for as long as the graph does; none of the caches is used.
        plan = make_plan(False)
        with _on_device(plan.device):
            plan.run()
        return (plan.out, plan.lse) if return_lse else plan.out
    cache = _plan_cache()
    plan = cache.get(key)
    if plan is None:
        plan = make_plan(True)
        out, lse = plan.out, plan.lse
        # a kept plan must not keep the caller's tensors alive: it holds addresses, and its workspace
        fwd = plan.args.fwd if isinstance(plan.args, _lib.FwdAppendArgs) else plan.args
        plan._keep = plan._keep[-1:] if fwd.workspace else ()
        plan.out = plan.lse = None
        if len(cache) >= _MAX_PLANS:
            cache.pop(next(iter(cache)))
        cache[key] = plan
    else:
        fwd = plan.args.fwd if isinstance(plan.args, _lib.FwdAppendArgs) else plan.args
        out = kwargs.get("out")
        if out is None:         # a new output (and LSE) tensor per call, as the reference returns
            out = torch.empty_like(q)
            fwd.out = out.data_ptr()
        lse = None
        if return_lse:
            lse = torch.empty((fwd.b, fwd.h), dtype=torch.float32, device=q.device)
            fwd.softmax_lse = lse.data_ptr()
    with _on_device(plan.device):
        plan.run()
    return (out, lse) if return_lse else out


def _i32_dev(x, b, device, name):
    if not isinstance(x, torch.Tensor):
        raise TypeError(f"{name} must be a tensor")
    if x.dtype != torch.int32 or x.device != device or not x.is_contiguous() or x.numel() != b:
        raise RuntimeError(f"{name} must be a contiguous int32 tensor of {b} elements on {device}")
    return x


def kvcache_pack_int(k_cache: torch.Tensor, k_pack: torch.Tensor, k_params: torch.Tensor,
                     v_cache: torch.Tensor, v_pack: torch.Tensor, v_params: torch.Tensor,
                     opt_block_table: Optional[torch.Tensor] = None,
                     cu_seqlens_k: torch.Tensor = None,
                     seqlen_k: int = 0,
                     quant_mode: str = "k-channel",
                     group_size: int = 128,
                     num_bits: int = 4,
                     *,
                     dst_offset: int = 0,
                     dst_offsets: Optional[torch.Tensor] = None) -> None:
    """Quantize-pack `k_cache`/`v_cache` [b, n, h_k, 128] into the caller-allocated packed cache
    (reference: bit_decode_interface.py:10-41).  K is quantized per channel, V per token.

    As in the reference `seqlen_k` is ignored in favour of `k_cache.shape[1]` and `cu_seqlens_k`
    is only validated (decode_api.cpp:537-541, 585).  Extensions: `dst_offset` (int) or
    `dst_offsets` (int32 [b] device tensor) give the token position, a multiple of 128, at which
    the n new tokens are written, so a full fp16 residual block can be appended to the cache.
    """
    mode = _check_quant(quant_mode, group_size, num_bits)
    if k_cache.dim() != 4 or v_cache.shape != k_cache.shape:
        raise RuntimeError("k_cache and v_cache must both be [batch, seqlen, nheads_k, head_dim]")
    if not k_cache.is_cuda:
        raise RuntimeError("k_cache must be on a GPU device")
    if v_cache.dtype != k_cache.dtype or v_cache.device != k_cache.device:
        raise RuntimeError("k_cache and v_cache must have the same dtype and device")
    dtype = _dtype_code(k_cache)
    device = k_cache.device
    b, n, h_k, d = k_cache.shape
    cb, S, ch_k = _check_cache(k_pack, k_params, v_pack, v_params, num_bits, group_size, device, mode == _lib.K_TENSOR)
    paged = opt_block_table is not None
    if paged:      # the cache tensors are page pools: leading dimension = pages, S = page size
        _check_block_table(opt_block_table, b, device)
    if (not paged and cb != b) or ch_k != h_k or d != 128:
        raise RuntimeError("packed cache shape does not match k_cache")
    if cu_seqlens_k is not None:
        if cu_seqlens_k.dtype != torch.int32:
            raise RuntimeError("cu_seqlens_k must have dtype int32")
        if not cu_seqlens_k.is_contiguous():
            raise RuntimeError("cu_seqlens_k must be contiguous")
    if k_cache.stride(3) != 1 or v_cache.stride(3) != 1:
        raise RuntimeError("Input tensor must have contiguous last dimension")
    if n % CHUNK:
        raise RuntimeError(f"number of tokens to pack ({n}) must be a multiple of {CHUNK}; "
                           "keep the remainder in the fp16 residual window")

    a = _lib.QpackArgs()
    a.k, a.v = k_cache.data_ptr(), v_cache.data_ptr()
    a.k_stride_b, a.k_stride_t, a.k_stride_h = k_cache.stride(0), k_cache.stride(1), k_cache.stride(2)
    a.v_stride_b, a.v_stride_t, a.v_stride_h = v_cache.stride(0), v_cache.stride(1), v_cache.stride(2)
    a.k_pack, a.k_params = k_pack.data_ptr(), k_params.data_ptr()
    a.v_pack, a.v_params = v_pack.data_ptr(), v_params.data_ptr()
    a.b, a.n_tokens, a.h_k, a.d = b, n, h_k, d
    a.cache_tokens = S
    a.dst_offset = int(dst_offset)
    a.dst_offsets = None if dst_offsets is None else _i32_dev(dst_offsets, b, device, "dst_offsets").data_ptr()
    a.bits, a.group_size, a.dtype = num_bits, group_size, dtype
    a.quant_mode = mode
    if paged:
        _set_paging(a, opt_block_table, cb)
    with _on_device(device):
        _lib.check(_lib.lib().bitdecode_qpack(ctypes.byref(a), _stream_ptr(device)))


class DecodePlan:
    """A validated decode call with its argument block and workspace held ready, so that
    `run()` is one C-ABI call with no allocation (serving loops, HIP-graph capture).
    Built by `plan_fwd_kvcache_int`; the tensors it was built from must stay alive and in place.
    """

    def __init__(self, args, out: torch.Tensor, lse: Optional[torch.Tensor],
                 keep: tuple, device: torch.device):
        self.args = args            # FwdArgs, or FwdAppendArgs for a decode step with append
        self.out = out
        self.lse = lse
        self._keep = keep
        self.device = device
        step = isinstance(args, _lib.FwdAppendArgs)
        self.num_splits = args.fwd.num_splits if step else args.num_splits
        self._fn = _lib.lib().bitdecode_fwd_append if step else _lib.lib().bitdecode_fwd
        self._ref = ctypes.byref(args)

    def run(self, stream: Optional[int] = None) -> torch.Tensor:
        rc = self._fn(self._ref, _stream_ptr(self.device) if stream is None else stream)
        if rc:
            _lib.check(rc)
        return self.out


def plan_fwd_kvcache_int(q: torch.Tensor,
                         k_pack: torch.Tensor, k_params: torch.Tensor,
                         v_pack: torch.Tensor, v_params: torch.Tensor,
                         opt_block_table: Optional[torch.Tensor] = None,
                         softmax_scale: float = 1.0,
                         quant_mode: str = "k-channel",
                         group_size: int = 128,
                         num_bits: int = 4,
                         *,
                         seqlen_k: Optional[int] = None,
                         seqlens_k: Optional[torch.Tensor] = None,
                         max_seqlen_k: Optional[int] = None,
                         k_residual: Optional[torch.Tensor] = None,
                         v_residual: Optional[torch.Tensor] = None,
                         residual_len: Union[int, torch.Tensor, None] = None,
                         max_residual_len: Optional[int] = None,
                         num_splits: int = 0,
                         out: Optional[torch.Tensor] = None,
                         return_lse: bool = False,
                         _stream_ws: bool = False) -> DecodePlan:
    """Validates a decode call and returns a `DecodePlan`; see `fwd_kvcache_int`."""
    mode = _check_quant(quant_mode, group_size, num_bits)
    if q.dim() != 4 or q.shape[1] != 1:
        raise RuntimeError("q must be [batch, 1, nheads, head_dim] (one query token per sequence)")
    if not q.is_cuda:
        raise RuntimeError("q must be on a GPU device")
    dtype = _dtype_code(q)
    device = q.device
    b, _, h, d = q.shape
    cb, S, h_k = _check_cache(k_pack, k_params, v_pack, v_params, num_bits, group_size, device, mode == _lib.K_TENSOR)
    paged = opt_block_table is not None
    if paged:      # page pools: cb pages of S tokens; a sequence holds up to max_pages_per_seq * S tokens
        _check_block_table(opt_block_table, b, device)
    elif cb != b:
        raise RuntimeError(f"batch size of q ({b}) and of the packed cache ({cb}) differ")
    if d != 128:
        raise RuntimeError("head dimension must be 128")
    if h % h_k:
        raise RuntimeError("Number of heads in key/value must divide number of heads in query")
    if q.stride(3) != 1:
        raise RuntimeError("Input tensor must have contiguous last dimension")

    a = _lib.FwdArgs()
    keep = [q, k_pack, k_params, v_pack, v_params]
    a.q, a.q_stride_b, a.q_stride_h = q.data_ptr(), q.stride(0), q.stride(2)
    a.k_pack, a.k_params = k_pack.data_ptr(), k_params.data_ptr()
    a.v_pack, a.v_params = v_pack.data_ptr(), v_params.data_ptr()
    a.cache_tokens = S
    capacity = S
    if paged:
        keep.append(opt_block_table)
        _set_paging(a, opt_block_table, cb)
        capacity = opt_block_table.shape[1] * S        # as the reference: seqlen_k = pages per sequence * page size
    a.seqlen_k = capacity if seqlen_k is None else int(seqlen_k)
    a.max_seqlen_k = a.seqlen_k
    if seqlens_k is not None:
        keep.append(_i32_dev(seqlens_k, b, device, "seqlens_k"))
        a.seqlens_k = seqlens_k.data_ptr()
        a.max_seqlen_k = capacity if max_seqlen_k is None else int(max_seqlen_k)
    if (k_residual is None) != (v_residual is None):
        raise RuntimeError("k_residual and v_residual must be given together")
    if k_residual is not None:
        for name, t in (("k_residual", k_residual), ("v_residual", v_residual)):
            if t.dim() != 4 or t.shape[0] != b or t.shape[2] != h_k or t.shape[3] != d:
                raise RuntimeError(f"{name} must be [batch, R, nheads_k, head_dim]")
            if t.dtype != q.dtype or t.device != device:
                raise RuntimeError(f"{name} must have the dtype and device of q")
            if t.stride(3) != 1:
                raise RuntimeError(f"{name} must have contiguous last dimension")
        if v_residual.shape[1] != k_residual.shape[1]:
            raise RuntimeError("k_residual and v_residual must hold the same number of tokens")
        R = k_residual.shape[1]
        keep += [k_residual, v_residual]
        a.k_res, a.v_res = k_residual.data_ptr(), v_residual.data_ptr()
        a.kres_stride_b, a.kres_stride_t, a.kres_stride_h = (k_residual.stride(0), k_residual.stride(1),
                                                               k_residual.stride(2))
        a.vres_stride_b, a.vres_stride_t, a.vres_stride_h = (v_residual.stride(0), v_residual.stride(1),
                                                               v_residual.stride(2))
        if isinstance(residual_len, torch.Tensor):
            keep.append(_i32_dev(residual_len, b, device, "residual_len"))
            a.res_lens = residual_len.data_ptr()
            a.res_len = R
            a.max_res_len = R if max_residual_len is None else int(max_residual_len)
        else:
            a.res_len = R if residual_len is None else int(residual_len)
            a.max_res_len = a.res_len
        if a.max_res_len > R or a.res_len > R or a.res_len < 0:
            raise RuntimeError("residual_len exceeds the residual window")
    elif residual_len is not None:
        raise RuntimeError("residual_len given without k_residual / v_residual")

    if out is None:
        out = torch.empty_like(q)
    else:
        if out.shape != q.shape or out.dtype != q.dtype or out.device != device or out.stride(3) != 1:
            raise RuntimeError("out must match q in shape, dtype and device")
    keep.append(out)
    a.out, a.out_stride_b, a.out_stride_h = out.data_ptr(), out.stride(0), out.stride(2)
    lse = None
    if return_lse:
        lse = torch.empty((b, h), dtype=torch.float32, device=device)
        keep.append(lse)
        a.softmax_lse = lse.data_ptr()
    a.b, a.h, a.h_k, a.d = b, h, h_k, d
    a.bits, a.group_size, a.dtype = num_bits, group_size, dtype
    a.quant_mode = mode
    a.softmax_scale = float(softmax_scale)
    with _on_device(device):
        ns, nbytes = _split_plan(device.index, b, h, h_k, a.max_seqlen_k, a.max_res_len, seqlens_k is not None,
                                 num_bits, group_size, int(num_splits))
        a.num_splits = ns
        if nbytes:
            # zero-filled: the arrival counters at its head must be 0 before the first call
            # (every call leaves them at 0 again)
            ws = (_stream_workspace(device, "fwd", b, h, ns, nbytes) if _stream_ws
                  else torch.zeros(nbytes, dtype=torch.uint8, device=device))
            keep.append(ws)
            a.workspace, a.workspace_bytes = ws.data_ptr(), nbytes
    return DecodePlan(a, out, lse, tuple(keep), device)


def fwd_kvcache_int(q: torch.Tensor,
                    k_pack: torch.Tensor, k_params: torch.Tensor,
                    v_pack: torch.Tensor, v_params: torch.Tensor,
                    opt_block_table: Optional[torch.Tensor] = None,
                    softmax_scale: float = 1.0,
                    quant_mode: str = "k-channel",
                    group_size: int = 128,
                    num_bits: int = 4,
                    **kwargs):
    """Decode attention of one query token per sequence over the packed cache
    (reference: bit_decode_interface.py:43-86; non-causal, no softcap, heuristic split count).

    q [b, 1, h, 128] fp16/bf16; returns a new tensor of the same shape.  `softmax_scale`
    defaults to 1.0 as in the reference; callers pass 1/sqrt(d).  q [b, m, h, 128] with m > 1 rows per sequence is
    accepted too (every row attends every key, as with the reference's fixed is_causal = False): see
    _fwd_query_rows.

    Keyword-only extensions:
      seqlen_k          valid packed tokens (multiple of 128); default = capacity of the cache
      seqlens_k         int32 [b] device tensor of per-sequence packed lengths (ragged batch)
      max_seqlen_k      host upper bound of seqlens_k (default: capacity)
      k_residual, v_residual   fp16 window of recent tokens [b, R, h_k, 128], attended after the
                        packed prefix; residual_len = valid tokens (int or int32 [b] tensor)
      num_splits        0 = choose; out = preallocated output; return_lse -> (out, lse [b, h])
    """
    if q.dim() == 4 and q.shape[1] > 1:
        return _fwd_query_rows(q, k_pack, k_params, v_pack, v_params, opt_block_table, softmax_scale, quant_mode,
                               group_size, num_bits, **kwargs)
    key = _call_key((q, k_pack, k_params, v_pack, v_params, opt_block_table),
                    (softmax_scale, quant_mode, group_size, num_bits), kwargs)
    # the split workspace comes from a per-stream cache: no allocation and no fill after the first call
    # (the reference allocates its accumulators per call, decode_api.cpp:292-295, 375-390)
    return _run_kept(key, q, kwargs, lambda shared: plan_fwd_kvcache_int(
        q, k_pack, k_params, v_pack, v_params, opt_block_table, softmax_scale, quant_mode, group_size, num_bits,
        _stream_ws=shared, **kwargs))


def _fwd_query_rows(q, k_pack, k_params, v_pack, v_params, opt_block_table, softmax_scale, quant_mode, group_size,
                    num_bits, out=None, return_lse=False, **kwargs):
    """Several query rows per sequence, q [b, m, h, 128] (the reference admits them, decode_api.cpp:341, 358-368:
    rows of the M tile; its interface fixes is_causal = False, so every row attends every key).  The kernel's
    16 columns hold up to eight (query head, row) pairs of a kv head: the rows are folded into the head dimension,
    8 // (h / h_k) rows per launch, and unfolded again.  Returns [b, m, h, 128] (and lse [b, m, h])."""
    b, m, h, d = q.shape
    h_k = v_pack.shape[2]
    if h_k <= 0 or h % h_k or h // h_k > 8:
        raise ValueError(f"q has {h} heads for {h_k} kv heads: need a multiple, at most 8 per kv head")
    g = h // h_k
    per = max(1, 8 // g)
    res = out if out is not None else torch.empty_like(q)
    if res.shape != q.shape or res.dtype != q.dtype or res.device != q.device:
        raise ValueError("out must match q in shape, dtype and device")
    lse = torch.empty((b, m, h), dtype=torch.float32, device=q.device) if return_lse else None
    for r0 in range(0, m, per):
        mr = min(per, m - r0)
        # (kv head, query head in the group, row) -> one head index
        qv = q[:, r0:r0 + mr].reshape(b, mr, h_k, g, d).permute(0, 2, 3, 1, 4).reshape(b, 1, h_k * g * mr, d).contiguous()
        got = fwd_kvcache_int(qv, k_pack, k_params, v_pack, v_params, opt_block_table, softmax_scale, quant_mode,
                              group_size, num_bits, return_lse=return_lse, **kwargs)
        ov, lv = got if return_lse else (got, None)
        res[:, r0:r0 + mr] = ov.reshape(b, h_k, g, mr, d).permute(0, 3, 1, 2, 4).reshape(b, mr, h, d)
        if return_lse:
            lse[:, r0:r0 + mr] = lv.reshape(b, h_k, g, mr).permute(0, 3, 1, 2).reshape(b, mr, h)
    return (res, lse) if return_lse else res


def plan_fwd_kvcache_int_append(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                                k_pack: torch.Tensor, k_params: torch.Tensor,
                                v_pack: torch.Tensor, v_params: torch.Tensor,
                                k_residual: torch.Tensor, v_residual: torch.Tensor,
                                lengths: torch.Tensor, max_len: int,
                                opt_block_table: Optional[torch.Tensor] = None,
                                softmax_scale: float = 1.0,
                                quant_mode: str = "k-channel",
                                group_size: int = 128,
                                num_bits: int = 4,
                                *,
                                num_splits: int = 0,
                                out: Optional[torch.Tensor] = None,
                                return_lse: bool = False,
                                _stream_ws: bool = False) -> DecodePlan:
    """Validates a decode step with append and returns its `DecodePlan`; see `fwd_kvcache_int_append`."""
    if k_residual is None or v_residual is None or k_residual.dim() != 4 or k_residual.shape[1] < CHUNK:
        raise RuntimeError(f"the residual window must hold at least {CHUNK} tokens")
    max_len = int(max_len)
    if max_len < 0:
        raise RuntimeError("max_len must not be negative")
    inner = plan_fwd_kvcache_int(q, k_pack, k_params, v_pack, v_params, opt_block_table, softmax_scale, quant_mode,
                                 group_size, num_bits, seqlen_k=0, k_residual=k_residual, v_residual=v_residual,
                                 residual_len=CHUNK, num_splits=1, out=out, return_lse=return_lse)
    device, b, h, h_k = inner.device, q.shape[0], q.shape[2], v_pack.shape[2]
    for name, t in (("k_new", k_new), ("v_new", v_new)):
        if t.dim() != 4 or tuple(t.shape) != (b, 1, h_k, 128):
            raise RuntimeError(f"{name} must be [batch, 1, nheads_k, head_dim]")
        if t.dtype != q.dtype or t.device != device:
            raise RuntimeError(f"{name} must have the dtype and device of q")
        if t.stride(3) != 1:
            raise RuntimeError(f"{name} must have contiguous last dimension")
    a = _lib.FwdAppendArgs()
    a.fwd = inner.args
    a.fwd.max_res_len = k_residual.shape[1]
    a.lengths = _i32_dev(lengths, b, device, "lengths").data_ptr()
    a.k_new, a.knew_stride_b, a.knew_stride_h = k_new.data_ptr(), k_new.stride(0), k_new.stride(2)
    a.v_new, a.vnew_stride_b, a.vnew_stride_h = v_new.data_ptr(), v_new.stride(0), v_new.stride(2)
    a.max_len = max_len
    L = _lib.lib()
    with _on_device(device):
        ns = int(num_splits)
        if ns == 0:
            ns = L.bitdecode_num_splits(b, h_k, max_len // CHUNK * CHUNK, CHUNK, 0, num_bits, group_size)
        a.fwd.num_splits = ns
        nbytes = L.bitdecode_fwd_append_workspace_bytes(b, h, ns)
        # zero-filled: the arrival counters must be 0 before the first call (every call leaves them at 0)
        ws = (_stream_workspace(device, "step", b, h, ns, nbytes) if _stream_ws
              else torch.zeros(nbytes, dtype=torch.uint8, device=device))
        a.fwd.workspace, a.fwd.workspace_bytes = ws.data_ptr(), nbytes
    keep = inner._keep + (k_new, v_new, lengths, ws)
    return DecodePlan(a, inner.out, inner.lse, keep, device)


def fwd_kvcache_int_append(q: torch.Tensor, k_new: torch.Tensor, v_new: torch.Tensor,
                           k_pack: torch.Tensor, k_params: torch.Tensor,
                           v_pack: torch.Tensor, v_params: torch.Tensor,
                           k_residual: torch.Tensor, v_residual: torch.Tensor,
                           lengths: torch.Tensor, max_len: int,
                           opt_block_table: Optional[torch.Tensor] = None,
                           softmax_scale: float = 1.0,
                           quant_mode: str = "k-channel",
                           group_size: int = 128,
                           num_bits: int = 4,
                           **kwargs):
    """One decode step in one launch (the "residual kernel" of the reference's figures,
    imgs/overview.png and imgs/scheme.png; no code for it in the reference's main branch).

    Sequence i holds `lengths[i]` tokens (int32 device tensor): whole blocks of 128 in the packed cache,
    the remainder in rows 0.. of `k_residual / v_residual [b, >=128, h_k, 128]`.  The call attends
    q [b, 1, h, 128] over all of them plus the new token `k_new / v_new [b, 1, h_k, 128]`, stores the
    new token in the window, quantize-packs a window that reaches 128 tokens behind the prefix, and
    advances `lengths` on the device.  `max_len` is a host upper bound of `lengths` before the step (it
    sizes the grid; the capacity of the cache always works).  Keyword-only: num_splits, out, return_lse.
    """
    key = _call_key((q, k_new, v_new, k_pack, k_params, v_pack, v_params, k_residual, v_residual, lengths,
                     opt_block_table), ("step", max_len, softmax_scale, quant_mode, group_size, num_bits), kwargs)
    return _run_kept(key, q, kwargs, lambda shared: plan_fwd_kvcache_int_append(
        q, k_new, v_new, k_pack, k_params, v_pack, v_params, k_residual, v_residual, lengths, max_len,
        opt_block_table, softmax_scale, quant_mode, group_size, num_bits, _stream_ws=shared, **kwargs))
