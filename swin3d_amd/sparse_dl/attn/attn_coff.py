"""All-in-one sparse window self-attention operator on the swin3d_amd HIP library.

Same Python surface as Swin3D/sparse_dl/attn/attn_coff.py (SelfAttnAIOFunction
:155-232 and the enums :20-40), so WindowAttention (Swin3D/modules/swin3d_layers.py:554-567)
can call it unchanged.  Differences in mechanism, not in result:
  * one fused HIP pass (s3d_attn_fwd) instead of cal_max_coffs + self_attn_forward + divide;
  * slots 0 and 2 of `indices` (the O(pairs) m2w / w2m arrays) are ignored and may be None;
  * only the combination the model uses is implemented (PosEmb.SEPARATE, TableDims.D0,
    IndexMode.INDIRECT);
  * q, k, v may be strided views of the qkv projection output (read in place).
"""
import ctypes
import enum

import torch
from torch.autograd.function import Function

from ... import _lib


class PosEmb(enum.Enum):
    NONE = 1
    LINEAR = 2
    SEPARATE = 3


class TableDims(enum.Enum):
    WHCD = 1
    DWHC = 2
    D0 = 3


class IndexMode(enum.Enum):
    DIRECT = 1
    INDIRECT = 2


class PrecisionMode(enum.Enum):
    HALF_ALL = 1
    HALF_FORWARD = 2
    HALF_NONE = 3


_DTYPE_CODE = {torch.float32: _lib.S3D_DTYPE_F32, torch.float16: _lib.S3D_DTYPE_F16}

# the backward keeps dL and P of every (pair, head) in its workspace when the window set's pair count is known
# (window_attention_backward): switch, and the size above which it runs the fused sweeps instead
BWD_PAIR_STORE = True
BWD_PAIR_STORE_MAX_BYTES = 32 << 30
# s3d_attn_bwd keeps a head's table gradients in registers where they fit: at most 64 rows per axis on average and
# head_dim 8 or 16.  Beyond that (and at head_dim 32) the library runs its general form, which adds with global
# atomics as the reference does and is many times slower.
BWD_MAX_ROWS_PER_AXIS = 64
BWD_HEAD_DIMS = (8, 16, 32)


def _require_cuda(name, t, device=None, strided_rows=False):
    if not isinstance(t, torch.Tensor):
        raise TypeError(f"{name} must be a torch.Tensor, got {type(t).__name__}")
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA (HIP) tensor")
    if device is not None and t.device != device:
        raise RuntimeError(f"{name} is on {t.device}, expected {device}")
    if strided_rows and _row_stride(t) is not None:
        return
    if not t.is_contiguous():
        raise RuntimeError(f"{name} must be contiguous")


def _row_stride(t):
    """Row stride (elements) of an [N,H,D] tensor whose (H,D) block is dense and whose rows are a multiple
    of 8 elements apart with 16-byte aligned storage: what the forward kernels read in place, e.g. the
    q / k / v slices of the [N, 3*H*D] output of the qkv projection.  None for any other layout."""
    if t.dim() != 3:
        return None
    n, h, d = t.shape
    s0, s1, s2 = t.stride()
    if n <= 1:
        s0 = max(s0, h * d)
    if s2 != 1 or s1 != d or s0 < h * d or s0 % 8 or (t.storage_offset() * t.element_size()) % 16:
        return None
    return s0


def _as_int32(name, t, device):
    """Index tensors arrive as int64 from torch ops (the reference's caller builds every one of them with
    torch.long, Swin3D/modules/swin3d_layers.py:96-140); the kernels read int32.  The int32 copy of an int64 CUDA
    tensor is kept on the tensor object, with its version counter and address, so a caller that hands the same
    index tensors to block after block pays the cast kernels once per window set and not once per call."""
    if not isinstance(t, torch.Tensor):
        t = torch.as_tensor(t)
    if t.dtype not in (torch.int32, torch.int64):
        raise TypeError(f"{name} must be an int32/int64 tensor, got {t.dtype}")
    if t.device != device:
        if t.is_cuda:
            raise RuntimeError(f"{name} is on {t.device}, expected {device}")
        t = t.to(device)
    if t.dtype == torch.int32:
        return t.contiguous()
    stamp = (t._version, t.data_ptr(), tuple(t.shape), tuple(t.stride()))
    kept = getattr(t, "_s3d_int32", None)
    if kept is None or kept[0] != stamp:
        kept = (stamp, t.to(torch.int32).contiguous())
        try:
            t._s3d_int32 = kept
        except (AttributeError, RuntimeError):     # an object that takes no attributes: cast on every call
            pass
    return kept[1]


def _host_table_sizes(table_sizes):
    """The per-axis table sizes as a host list (the backward needs them there).  A CUDA
    tensor costs one synchronising device-to-host copy; the values are then kept on the tensor object (with
    its version counter), so a module that keeps its table_offsets tensor pays the copy once."""
    if isinstance(table_sizes, torch.Tensor):
        if not table_sizes.is_cuda:
            return [int(x) for x in table_sizes.reshape(-1).tolist()]
        kept = getattr(table_sizes, "_s3d_host_sizes", None)
        if kept is None or kept[0] != table_sizes._version:
            kept = (table_sizes._version, [int(x) for x in table_sizes.reshape(-1).tolist()])
            table_sizes._s3d_host_sizes = kept
        return list(kept[1])
    return [int(x) for x in table_sizes]


# keep the sweep kernel's work list ("plan") on the w_sizes tensor between calls (False: build it in every call)
REUSE_PLANS = True

# a CUDA table_sizes tensor whose values the host has not seen yet goes to the sweep kernel as it is, and the
# host never waits for it (False: always copy it to the host, which checks the values there)
DEVICE_TABLE_SIZES = True


def _sizes_stay_on_device(table_sizes):
    """True for the reference caller's table_offsets (a new CUDA tensor on every call, Swin3D/modules/
    swin3d_layers.py:511) in a forward that does not need the values on the host."""
    if not DEVICE_TABLE_SIZES or not isinstance(table_sizes, torch.Tensor) or not table_sizes.is_cuda:
        return False
    kept = getattr(table_sizes, "_s3d_host_sizes", None)
    return kept is None or kept[0] != table_sizes._version


def _plan_for(lib, w_sizes_in, w2n_in, w_sizes, w2n, c_sizes, sizes, nd, table_len, n, h, d, code, stream):
    """The plan buffer (s3d_attn_plan) of this window set and shape, built on first use and kept as an attribute
    of the caller's w_sizes tensor; None when there is no tensor object to keep it on.  A plan is valid for the
    contents it was built from (the tensors' version counters are checked) and for one stream (it holds the work
    counters of the launch that uses it)."""
    if not isinstance(w_sizes_in, torch.Tensor) or not isinstance(w2n_in, torch.Tensor) or w_sizes.numel() == 0 or n == 0:
        return None
    plans = getattr(w_sizes_in, "_s3d_attn_plans", None)
    if plans is None:
        plans = w_sizes_in._s3d_attn_plans = {}
    key = (h, d, code, tuple(sizes) if sizes is not None else None, n, stream)
    stamp = (w_sizes_in._version, w2n_in._version, w2n_in.data_ptr())
    kept = plans.get(key)
    if kept is not None and kept[0] == stamp:
        return kept[1]
    num_w = w_sizes.numel()
    nbytes = lib.s3d_attn_plan_bytes(h, n, num_w)
    plan = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=w_sizes.device)
    # the work list depends on the tables through their total length only: no sizes are passed when they are
    # on the device
    status = lib.s3d_attn_plan(c_sizes if sizes is not None else None, nd, table_len, w_sizes.data_ptr(),
                               w2n.data_ptr(), n, h, d, num_w, code, plan.data_ptr(), nbytes, stream)
    _lib.check(status, "s3d_attn_plan")
    plans[key] = (stamp, plan)
    return plan


def window_attention_forward(q, k, v, table_q, table_k, table_v, table_sizes, w_sizes, w2n, n2n,
                             n_coords, return_stats=False):
    """softmax-normalised window attention, [N,H,D] in the dtype of q.

    q, k, v        [N,H,D] fp16 or fp32 CUDA tensors (q already scaled by D**-0.5); dense, or views with
                   a dense (H,D) block and one common row stride (slices of a [N,3*H*D] projection output)
    table_*        flat [sum(table_sizes)] tensors, layout [axis][row][h][c], dtype of q
    table_sizes    int tensor / list [nd], per-axis element counts rows*H*D.  A list or CPU tensor is read on
                   the host; a CUDA tensor stays on the device and the kernel reads it (no host wait, no
                   check of the values beyond clipping them to the table) unless DEVICE_TABLE_SIZES = False
    w_sizes, w2n   [W] voxels per window and their exclusive prefix sum (int32, or int64 as torch ops give them)
    n2n            [N] window-sorted position -> row of q/k/v, or None when the rows are in window-sorted
                   order already (the kernel then reads and writes them without the indirection)
    n_coords       [N,nd] fp32 signals in window-sorted order (already quant-scaled)
    return_stats   also return (max logit [N,H] fp32, sum exp(logit - max) [N,H] fp32)
    """
    _require_cuda("query", q, strided_rows=True)
    dev = q.device
    if q.dim() != 3:
        raise ValueError(f"query must be [N,H,D], got {tuple(q.shape)}")
    n, h, d = q.shape
    if q.dtype not in _DTYPE_CODE:
        raise TypeError(f"unsupported feature dtype {q.dtype} (float16 or float32)")
    for name, t in (("key", k), ("value", v)):
        _require_cuda(name, t, dev, strided_rows=True)
        if t.shape != q.shape or t.dtype != q.dtype:
            raise ValueError(f"{name} must match query: {tuple(t.shape)} {t.dtype}")
    # q, k, v are read in place when they share one row stride (views of one projection output)
    strides = {_row_stride(t) for t in (q, k, v)}
    if len(strides) != 1 or None in strides:
        q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
    row_stride = _row_stride(q)
    if d not in (8, 16, 32):
        raise ValueError(f"head_dim must be 8, 16 or 32, got {d}")
    if _sizes_stay_on_device(table_sizes):
        sizes = None
        sizes_dev = _as_int32("table_sizes", table_sizes.reshape(-1), dev)
        nd = sizes_dev.numel()
        c_sizes = sizes_dev.data_ptr()
    else:
        sizes = _host_table_sizes(table_sizes)
        nd = len(sizes)
    if nd not in (3, 6, 9):
        raise ValueError(f"table_sizes must have 3, 6 or 9 entries, got {nd}")
    if sizes is not None:
        if any(sz <= 0 or sz % (h * d) for sz in sizes) or sum(sizes) != table_q.numel():
            raise ValueError(f"table_sizes {sizes} must be positive multiples of H*D = {h * d} that sum "
                             f"to the table length {table_q.numel()}")
        c_sizes = (ctypes.c_int32 * nd)(*sizes)
    table_len = table_q.numel()
    for name, t in (("query_table", table_q), ("key_table", table_k), ("value_table", table_v)):
        _require_cuda(name, t, dev)
        if t.dtype != q.dtype:
            raise TypeError(f"{name} must have the dtype of the features ({q.dtype}), got {t.dtype}")
        if t.numel() != table_len:
            raise ValueError("the three tables must have the same number of elements")
    if table_len == 0 or table_len % (h * d) != 0:
        raise ValueError(f"table length {table_len} is not a positive multiple of H*D = {h * d}")
    w_sizes_in, w2n_in = w_sizes, w2n
    w_sizes = _as_int32("w_sizes", w_sizes, dev)
    w2n = _as_int32("w2n_indices", w2n, dev)
    if n2n is not None:
        n2n = _as_int32("n2n_indices", n2n, dev)
        if n2n.shape != (n,):
            raise ValueError(f"n2n_indices must be [{n}], got {tuple(n2n.shape)}")
    if w_sizes.shape != w2n.shape or w_sizes.dim() != 1:
        raise ValueError("w_sizes and w2n_indices must be 1-D of equal length")
    _require_cuda("n_coords", n_coords, dev)
    if n_coords.dtype != torch.float32 or n_coords.shape != (n, nd):
        raise ValueError(f"n_coords must be float32 [{n},{nd}], got {n_coords.dtype} {tuple(n_coords.shape)}")

    out = torch.empty((n, h, d), dtype=q.dtype, device=dev)
    omax = torch.empty((n, h), dtype=torch.float32, device=dev) if return_stats else None
    osum = torch.empty((n, h), dtype=torch.float32, device=dev) if return_stats else None
    lib = _lib.lib()
    code = _DTYPE_CODE[q.dtype]
    num_w = w_sizes.numel()
    flags = _lib.S3D_ATTN_SIZES_ON_DEVICE if sizes is None else 0
    with torch.cuda.device(dev):
        stream = torch.cuda.current_stream(dev).cuda_stream
        # the work list depends on the window set only: it is built once and kept on the caller's w_sizes
        # tensor, so the blocks that share a window set share it
        plan = None if not REUSE_PLANS else _plan_for(lib, w_sizes_in, w2n_in, w_sizes, w2n, c_sizes, sizes,
                                                      nd, table_len, n, h, d, code, stream)
        if plan is not None:
            workspace, ws_bytes, flags = plan, plan.numel(), flags | _lib.S3D_ATTN_PLANNED
        else:
            ws_bytes = lib.s3d_attn_fwd_workspace_bytes(h, n, num_w)
            workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
        status = lib.s3d_attn_fwd(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), table_q.data_ptr(), table_k.data_ptr(),
            table_v.data_ptr(), c_sizes, nd, table_len, w_sizes.data_ptr(),
            w2n.data_ptr(), n2n.data_ptr() if n2n is not None else None, n_coords.data_ptr(), out.data_ptr(),
            omax.data_ptr() if return_stats else None, osum.data_ptr() if return_stats else None,
            n, h, d, num_w, row_stride, code, flags, workspace.data_ptr(), ws_bytes, stream)
    _lib.check(status, "s3d_attn_fwd")
    if return_stats:
        return out, omax, osum
    return out


def _pairs_of(w_sizes_in, w_sizes):
    """M = sum of w_sizes^2, the pairs of the window set (one host read, kept on the caller's tensor)."""
    if isinstance(w_sizes_in, torch.Tensor):
        kept = getattr(w_sizes_in, "_s3d_pairs", None)
        if kept is not None and kept[0] == w_sizes_in._version:
            return kept[1]
    pairs = int((w_sizes.long() ** 2).sum().item()) if w_sizes.numel() else 0
    if isinstance(w_sizes_in, torch.Tensor):
        w_sizes_in._s3d_pairs = (w_sizes_in._version, pairs)
    return pairs


def window_attention_backward(q, k, v, table_q, table_k, table_v, table_sizes, w_sizes, w2n, n2n, n_coords,
                              out, out_max, out_sum, dout, pairs=None):
    """Gradients of window_attention_forward -> (dq, dk, dv [N,H,D] in the dtype of q,
    dtable_q, dtable_k, dtable_v flat fp32).  out / out_max / out_sum are the forward's results
    (return_stats=True) for the same inputs; arithmetic is fp32 for both dtypes.  The tables have the dtype of q, or
    are fp32 beside fp16 features: the backward of an fp16 forward computed in fp32 (PrecisionMode.HALF_FORWARD,
    attn_coff.py:206-215), whose results are those of fp32 copies of the features with dq, dk, dv rounded to fp16
    (to the rounding of the fp32 sums).

    pairs: M = sum(w_sizes^2) of the window set (the reference's index arrays have this length,
    swin3d_layers.py:96-103); None = read it from w_sizes once and keep it on that tensor.  With it the library
    runs the pair sweeps, which keep dL and P of every (pair, head) in the workspace (12 bytes each); 0, or a
    store above BWD_PAIR_STORE_MAX_BYTES, selects the fused sweeps, which need no such store and take about a
    third longer.  head_dim 32 and tables of more than BWD_MAX_ROWS_PER_AXIS rows per axis on average run in the
    library's general form (atomic adds, as the reference works): correct, some fifty times slower per pair."""
    w_sizes_in = w_sizes
    _require_cuda("query", q)
    dev = q.device
    if q.dim() != 3:
        raise ValueError(f"query must be [N,H,D], got {tuple(q.shape)}")
    n, h, d = q.shape
    if q.dtype not in _DTYPE_CODE:
        raise TypeError(f"unsupported feature dtype {q.dtype} (float16 or float32)")
    for name, t in (("key", k), ("value", v), ("out", out), ("dout", dout)):
        _require_cuda(name, t, dev)
        if t.shape != q.shape or t.dtype != q.dtype:
            raise ValueError(f"{name} must match query: {tuple(t.shape)} {t.dtype}")
    if d not in BWD_HEAD_DIMS:
        raise NotImplementedError(f"attention backward supports head_dim 8, 16 and 32, got {d}")
    sizes = _host_table_sizes(table_sizes)
    nd = len(sizes)
    if nd not in (3, 6, 9):
        raise ValueError(f"table_sizes must have 3, 6 or 9 entries, got {nd}")
    table_len = table_q.numel()
    if any(sz <= 0 or sz % (h * d) for sz in sizes) or sum(sizes) != table_len:
        raise ValueError(f"table_sizes {sizes} must be positive multiples of H*D = {h * d} that sum "
                         f"to the table length {table_len}")
    general = d == 32 or sum(sizes) // (h * d) > BWD_MAX_ROWS_PER_AXIS * nd     # the library's general form
    mixed = q.dtype == torch.float16 and table_q.dtype == torch.float32
    for name, t in (("query_table", table_q), ("key_table", table_k), ("value_table", table_v)):
        _require_cuda(name, t, dev)
        if t.dtype != table_q.dtype or (t.dtype != q.dtype and not mixed) or t.numel() != table_len:
            raise ValueError(f"{name} must have the dtype of the features (or float32 beside float16 features) "
                             f"and {table_len} elements")
    for name, t in (("out_max", out_max), ("out_sum", out_sum)):
        _require_cuda(name, t, dev)
        if t.dtype != torch.float32 or t.shape != (n, h):
            raise ValueError(f"{name} must be float32 [{n},{h}]")
    w_sizes = _as_int32("w_sizes", w_sizes, dev)
    w2n = _as_int32("w2n_indices", w2n, dev)
    # None: rows in window-sorted order already (the forward took no row map); the library then reads the identity
    # map that it writes into its workspace
    n2n = None if n2n is None else _as_int32("n2n_indices", n2n, dev)
    _require_cuda("n_coords", n_coords, dev)
    if n_coords.dtype != torch.float32 or n_coords.shape != (n, nd):
        raise ValueError(f"n_coords must be float32 [{n},{nd}]")
    c_sizes = (ctypes.c_int32 * nd)(*sizes)
    if pairs is None:
        pairs = _pairs_of(w_sizes_in, w_sizes) if BWD_PAIR_STORE else 0
    pairs = int(pairs)
    if pairs < 0:
        raise ValueError(f"pairs = {pairs}")
    if 12 * pairs * h > BWD_PAIR_STORE_MAX_BYTES:
        pairs = 0
    code = _lib.S3D_DTYPE_F32_F16_ROWS if mixed else _DTYPE_CODE[q.dtype]
    if mixed and pairs == 0 and not general:
        # the fused sweeps take one dtype: fp32 copies of the features, the gradients rounded afterwards
        q, k, v, out, dout = (t.float() for t in (q, k, v, out, dout))
        code = _lib.S3D_DTYPE_F32
    dq, dk, dv = torch.empty_like(q), torch.empty_like(q), torch.empty_like(q)
    dtq, dtk, dtv = (torch.empty(table_len, dtype=torch.float32, device=dev) for _ in range(3))
    lib = _lib.lib()
    tensors = [t.contiguous() for t in (q, k, v, table_q, table_k, table_v)]
    out, dout, out_max, out_sum, n_coords = (t.contiguous() for t in (out, dout, out_max, out_sum, n_coords))
    with torch.cuda.device(dev):
        ws_bytes = lib.s3d_attn_bwd_workspace_bytes(h, d, nd, table_len, n, w_sizes.numel(), pairs)
        workspace = torch.empty(max(ws_bytes, 1), dtype=torch.uint8, device=dev)
        stream = torch.cuda.current_stream(dev).cuda_stream
        status = lib.s3d_attn_bwd(
            *(t.data_ptr() for t in tensors), c_sizes, nd, table_len, w_sizes.data_ptr(), w2n.data_ptr(),
            None if n2n is None else n2n.data_ptr(), n_coords.data_ptr(), out.data_ptr(), out_max.data_ptr(),
            out_sum.data_ptr(), dout.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(), dtq.data_ptr(), dtk.data_ptr(),
            dtv.data_ptr(), n, h, d, w_sizes.numel(), pairs, code, workspace.data_ptr(), ws_bytes,
            stream)
    _lib.check(status, "s3d_attn_bwd")
    if mixed and code == _lib.S3D_DTYPE_F32:
        dq, dk, dv = dq.half(), dk.half(), dv.half()
    return dq, dk, dv, dtq, dtk, dtv


def _compute_dtype(precision):
    """fp32 unless autocast is on and the precision mode allows half (attn_coff.py:172-175)."""
    if torch.is_autocast_enabled() and precision != PrecisionMode.HALF_NONE:
        return torch.get_autocast_dtype("cuda")
    return torch.float32


class SelfAttnAIOFunction(Function):
    """Function of all-in-one self-attention (Swin3D/sparse_dl/attn/attn_coff.py:155-232)."""

    @staticmethod
    def forward(ctx, raw_query_feats, raw_key_feats, raw_value_feats, query_table, key_table,
                value_table, table_offsets, indices, pe, table_dim, mode, precision):
        if table_dim != TableDims.D0:
            raise NotImplementedError("only TableDims.D0 tables are supported")
        if pe != PosEmb.SEPARATE or mode != IndexMode.INDIRECT:
            raise NotImplementedError("only PosEmb.SEPARATE with IndexMode.INDIRECT is implemented")
        if len(indices) != 6:
            raise ValueError("indices must be [m2w, w_sizes, w2m, w2n, n2n, n_coords]")
        c_dtype = _compute_dtype(precision)
        if c_dtype not in _DTYPE_CODE:
            raise NotImplementedError(f"compute dtype {c_dtype} is not supported (float16 / float32)")
        _, w_sizes, _, w2n, n2n, n_coords = indices
        raw = (raw_query_feats, raw_key_feats, raw_value_feats, query_table, key_table, value_table)
        feats = [t.to(c_dtype) for t in raw[:3]]
        feats = [t if _row_stride(t) is not None else t.contiguous() for t in feats]
        tables = [t.to(c_dtype).contiguous() for t in raw[3:]]
        n_coords = n_coords.to(torch.float32).contiguous()
        needs_grad = any(ctx.needs_input_grad[:6])
        if needs_grad:
            # the backward's limits, reported where the op is called and not from inside autograd
            if raw_query_feats.shape[2] not in BWD_HEAD_DIMS:
                raise NotImplementedError(
                    f"attention backward supports head_dim 8, 16 and 32, got {raw_query_feats.shape[2]}; run the "
                    "forward under torch.no_grad()")
        res = window_attention_forward(*feats, *tables, table_offsets, w_sizes, w2n, n2n, n_coords,
                                       return_stats=needs_grad)
        if not needs_grad:
            return res
        out, omax, osum = res
        ctx.precision = precision
        ctx.table_sizes = _host_table_sizes(table_offsets)
        # the window set's pair count, for the backward's pair store: on the tensor when the window index of this
        # package built it, else read from w_sizes once (and kept on it)
        ctx.pairs = _pairs_of(w_sizes, w_sizes) if BWD_PAIR_STORE else 0
        ctx.save_for_backward(out, omax, osum, *raw, w_sizes, w2n, n2n, n_coords)
        return out

    @staticmethod
    def backward(ctx, *grad_outputs):
        """Compute dtype as in the reference (attn_coff.py:206-215): the gradient's dtype for HALF_ALL,
        fp32 otherwise; the statistics saved by the forward are reused either way."""
        (dout,) = grad_outputs
        out, omax, osum = ctx.saved_tensors[:3]
        raw = ctx.saved_tensors[3:9]
        w_sizes, w2n, n2n, n_coords = ctx.saved_tensors[9:]
        c_dtype = dout.dtype if ctx.precision == PrecisionMode.HALF_ALL else torch.float32
        if c_dtype not in _DTYPE_CODE:
            raise NotImplementedError(f"compute dtype {c_dtype} is not supported (float16 / float32)")
        # fp32 arithmetic on fp16 tensors (HALF_FORWARD under autocast): the library widens the rows as it loads
        # them, where the reference makes fp32 copies
        f_dtype = c_dtype
        if c_dtype == torch.float32 and dout.dtype == torch.float16 and out.dtype == torch.float16 \
                and all(t.dtype == torch.float16 for t in raw[:3]):
            f_dtype = torch.float16
        feats = [t.to(f_dtype).contiguous() for t in raw[:3]]
        tables = [t.to(c_dtype).contiguous() for t in raw[3:]]
        grads = window_attention_backward(*feats, *tables, ctx.table_sizes, w_sizes, w2n, n2n, n_coords,
                                          out.to(f_dtype), omax, osum, dout.to(f_dtype).contiguous(),
                                          pairs=ctx.pairs)
        grads = [g.to(t.dtype).reshape(t.shape) if need else None
                 for g, t, need in zip(grads, raw, ctx.needs_input_grad[:6])]
        return (*grads, None, None, None, None, None, None)
