"""Fused window attention: one autograd Function around the token-plan and the fused MFMA
block products of ``libsswin3d.so``.

Numerically this is the same computation as the operator-by-operator composition in
:mod:`sparseswin3d_amd.window_attention` (reference ``sparse_swin/swin3d_base.py:654-675``):

    S = (scale*Q) K^T + bias + mask  ->  P = sparse softmax(S)  ->  O = P V  (in voxel order)

but Q, K, V token rows are read straight from the dense ``qkv`` tensor through the token order
and the output is written straight into voxel order, so the sorted COO copies, the bias/mask
gather passes, the permute and the un-sort never exist.  The attention values S and P are still
materialised in HBM (P is needed by the backward pass).
"""
from __future__ import annotations

import ctypes as C

import torch
from torch.autograd import Function
from torch.autograd.function import once_differentiable

from . import _lib
from . import custom_ops as ops

_DTYPE_CODE = {torch.float32: 0, torch.float16: 1, torch.bfloat16: 2}


def _ptr(t):
    return C.c_void_p(t.data_ptr() if t is not None else 0)


_PINNED_TOTALS = []      # pinned host buffers of finished plans, reused


class TokenPlan:
    """Token order and per-group table of one set of (window, pos) voxel indices.

    With ``defer=True`` the constructor only enqueues the kernels and the copy of the totals;
    work enqueued afterwards (the qkv projection) overlaps the host round trip, and
    :meth:`finish` waits for the totals when they are needed.  :meth:`finish` raises if an index
    lies outside ``[0, batch_size) x [0, n)`` or a (window, pos) pair occurs twice."""

    MAX_BATCH = 4            # plans per sswin_token_plan_batch call

    def __init__(self, indices: torch.Tensor, batch_size: int, n: int, num_heads: int, defer: bool = False,
                 tasks: bool = True, order_only: bool = False):
        self._allocate(indices, batch_size, n, num_heads, tasks, order_only)
        if order_only:
            self._enqueue([self])                    # the flag exists in the batch entry point only
        else:
            lib = _lib.load()
            d = self.device
            with _lib.on_device(d):
                stream = _lib.stream_handle(d)
                _lib.check(lib.sswin_token_plan(_ptr(self._indices), self.N, self.B, self.n, self.H, _ptr(self.tokens),
                                                _ptr(self.plan), self.g_cap, _ptr(self.tasks),
                                                C.c_void_p(self._totals.data_ptr()), _ptr(self._ws), self._ws.numel(),
                                                0, stream))
                self._event = torch.cuda.Event()
                self._event.record(torch.cuda.current_stream(d))
        if not defer:
            self.finish()

    def _allocate(self, indices, batch_size, n, num_heads, tasks, order_only=False):
        lib = _lib.load()
        if indices.device.type != "cuda":
            raise RuntimeError("TokenPlan runs on the GPU only; there is no CPU fallback")
        if indices.dtype != torch.int32 or indices.dim() != 2 or indices.shape[1] != 2:
            raise RuntimeError("TokenPlan: indices must be int32 [N, 2]")
        indices = indices.contiguous()
        d = indices.device
        N = indices.shape[0]
        self.N, self.H, self.n, self.B = N, int(num_heads), int(n), int(batch_size)
        self.g_cap = max(1, min(N, self.B) * self.H)
        # order_only: the plan of a stride-2 merge, whose consumers read the voxel of every rank and nothing else
        self.order_only = bool(order_only)
        self.tokens = torch.empty((1 if order_only else 5) * max(N, 1), dtype=torch.int32, device=d)
        self.plan = torch.empty(5 * self.g_cap, dtype=torch.int32, device=d)
        # group descriptors of the window-resident kernels, bucketed by ceil(c / 32)
        # (and behind them the token records, one per window and tile of 32 tokens)
        self.tasks = (torch.empty(int(lib.sswin_token_plan_task_ints(N, self.g_cap, self.H)), dtype=torch.int32, device=d)
                      if tasks else None)
        self.device = d
        self._totals = _PINNED_TOTALS.pop() if _PINNED_TOTALS else torch.zeros(9, dtype=torch.int64, pin_memory=True)
        self._indices = indices                      # kept alive until the kernels have run
        with _lib.on_device(d):
            nbytes = lib.sswin_token_plan_workspace_bytes(N, self.B, self.n)
            self._ws = torch.empty(int(nbytes), dtype=torch.uint8, device=d)

    @classmethod
    def batch(cls, specs):
        """Deferred plans for several index sets on one device, built by shared launches (the regular and the
        shifted block of a stage).  ``specs``: tuples ``(indices, batch_size, n, num_heads)``,
        ``(..., tasks)`` or ``(..., tasks, order_only)``; returns the plans in the same order, each to be completed
        with :meth:`finish`."""
        plans = []
        for spec in specs:
            p = cls.__new__(cls)
            p._allocate(*spec[:4], spec[4] if len(spec) > 4 else True, spec[5] if len(spec) > 5 else False)
            plans.append(p)
        if plans:
            cls._enqueue(plans)
        return plans

    @staticmethod
    def _enqueue(plans):
        """Launch allocated plans through the batch entry point, MAX_BATCH per call; they share one event."""
        d = plans[0].device
        if any(p.device != d for p in plans):
            raise RuntimeError("TokenPlan.batch: all index sets must live on one device")
        lib = _lib.load()
        with _lib.on_device(d):
            stream = torch.cuda.current_stream(d)
            for k in range(0, len(plans), TokenPlan.MAX_BATCH):
                chunk = plans[k:k + TokenPlan.MAX_BATCH]
                descs = (_lib.TokenPlanDesc * len(chunk))()
                for desc, p in zip(descs, chunk):
                    desc.indices, desc.N, desc.B, desc.n, desc.H = p._indices.data_ptr(), p.N, p.B, p.n, p.H
                    desc.flags = 1 if p.order_only else 0
                    desc.tokens, desc.plan, desc.g_cap = p.tokens.data_ptr(), p.plan.data_ptr(), p.g_cap
                    desc.tasks = p.tasks.data_ptr() if p.tasks is not None else None
                    desc.totals_out, desc.ws, desc.ws_bytes = p._totals.data_ptr(), p._ws.data_ptr(), p._ws.numel()
                _lib.check(lib.sswin_token_plan_batch(descs, len(chunk), C.c_void_p(stream.cuda_stream)))
            event = torch.cuda.Event()
            event.record(stream)
        for p in plans:
            p._event = event

    def finish(self):
        """Wait for the totals (once) and decode them."""
        if self._event is None:
            return self
        self._event.synchronize()
        self._event = None
        if self.N > 0:
            _lib.check(_lib.load().sswin_token_plan_totals(C.c_void_p(self._totals.data_ptr()), self.H, self.g_cap))
        totals = self._totals.tolist()
        if len(_PINNED_TOTALS) < 64:                 # the pinned buffer goes back for the next plan (allocating one costs
            _PINNED_TOTALS.append(self._totals)      # the host tens of microseconds); the library writes all nine entries
        self._totals = None
        self.G, self.windows, self.A, self.c_max = (int(totals[i]) for i in range(4))
        self.bucket_counts = (C.c_int64 * 4)(*(int(totals[4 + b]) for b in range(4)))
        self.oversize_groups = int(totals[8])
        self._ws = self._indices = None
        return self


def _tokens_to_sq(tp, dtype, epilogue, a, a_stride, a_col0, b, b_stride, b_col0, hd, scale, bias, mask, out, rows):
    lib = _lib.load()
    stream = _lib.stream_handle(tp.device)
    _lib.check(lib.sswin_fused_tokens_to_sq(
        _DTYPE_CODE[dtype], 1 if epilogue else 0, _ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, tp.H, hd,
        _ptr(a), a_stride, a_col0, _ptr(b), b_stride, b_col0, C.c_float(scale), _ptr(bias), tp.n, _ptr(mask),
        0 if mask is None else mask.shape[0], _ptr(out), _ptr(rows), stream))


def _sq_to_tokens(tp, dtype, a_kmajor, sq, b, b_stride, b_col0, o, o_stride, o_col0, hd, scale):
    lib = _lib.load()
    stream = _lib.stream_handle(tp.device)
    _lib.check(lib.sswin_fused_sq_to_tokens(
        _DTYPE_CODE[dtype], 1 if a_kmajor else 0, _ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, tp.H, hd,
        _ptr(sq), _ptr(b), b_stride, b_col0, _ptr(o), o_stride, o_col0, C.c_float(scale), stream))


def _score_grad(tp, dtype, d_o, do_stride, do_col0, v, v_stride, v_col0, o, o_stride, o_col0, hd, p, ds):
    """dS = P (dO V^T - D), D_i = dO_i . O_i: the product dP and the softmax backward in one launch."""
    _lib.check(_lib.load().sswin_fused_score_grad(
        _DTYPE_CODE[dtype], _ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, tp.H, hd, tp.c_max, _ptr(d_o), do_stride,
        do_col0, _ptr(v), v_stride, v_col0, _ptr(o), o_stride, o_col0, _ptr(p), _ptr(ds), _lib.stream_handle(tp.device)))


def _group_softmax(tp, backward, x_or_y, grad, out):
    """Row softmax (or its backward) over the [c x c] blocks of the plan's groups; ``out`` may be one of the inputs."""
    _lib.check(_lib.load().sswin_group_softmax(
        1 if backward else 0, _ptr(tp.plan), tp.g_cap, tp.G, tp.N, tp.H, tp.c_max, _ptr(x_or_y), _ptr(grad), _ptr(out),
        _lib.stream_handle(tp.device)))


def _bias32(bias, table_index, H, n, d):
    """The fp32 [H, n, n] bias the kernels read: ``bias`` itself, or gathered from the [rows, H] table."""
    if table_index is None:
        return bias.detach().to(torch.float32).contiguous()
    table32 = bias.detach().to(torch.float32).contiguous()
    bias32 = torch.empty((H, n, n), dtype=torch.float32, device=d)
    with _lib.on_device(d):
        _lib.check(_lib.load().sswin_bias_from_table(
            _ptr(table32), table32.shape[0], H, _ptr(table_index.code), table_index.offset0, n, _ptr(bias32),
            _lib.stream_handle(d)))
    return bias32


def _bias_gradient(tp, H, d_s, bias_meta, table_index):
    """Gradient of the [H, n, n] bias, or of the [rows, H] table when ``table_index`` is given, from dS
    (one [c x c] block per group)."""
    lib = _lib.load()
    d = d_s.device
    bias_dtype, bias_shape = bias_meta
    stream = _lib.stream_handle(d)
    if table_index is None:
        d_bias32 = torch.zeros(bias_shape, dtype=torch.float32, device=d)
        nbytes = lib.sswin_fused_bias_grad_workspace_bytes(tp.G, H, tp.n)
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=d)
        _lib.check(lib.sswin_fused_bias_grad(_ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, H, tp.n,
                                             _ptr(d_s), _ptr(d_bias32), _ptr(ws), nbytes, stream))
    else:
        rows = bias_shape[0]
        d_bias32 = torch.empty(bias_shape, dtype=torch.float32, device=d)
        nbytes = lib.sswin_bias_table_grad_workspace_bytes(tp.G, H, rows)
        ws = torch.empty(int(nbytes), dtype=torch.uint8, device=d)
        if tp.tasks is not None and tp.n <= 128 and sum(tp.bucket_counts) == tp.G:
            # every group has a task descriptor: the batches of dS are dealt evenly from the descriptor lists
            _lib.check(lib.sswin_bias_table_grad_tasks(_ptr(tp.tasks), tp.g_cap, tp.bucket_counts, tp.G, _ptr(tp.tokens), tp.N,
                                                       H, tp.n, _ptr(table_index.code), table_index.offset0, rows,
                                                       _ptr(d_s), _ptr(d_bias32), _ptr(ws), nbytes, stream))
        else:
            _lib.check(lib.sswin_bias_table_grad(_ptr(tp.plan), tp.g_cap, tp.G, _ptr(tp.tokens), tp.N, H, tp.n,
                                                 _ptr(table_index.code), table_index.offset0, rows, _ptr(d_s),
                                                 _ptr(d_bias32), _ptr(ws), nbytes, stream))
    return d_bias32.to(bias_dtype)


class _FusedWindowAttention(Function):
    @staticmethod
    def forward(ctx, qkv, bias, indices, mask, batch_size, n, scale, plan, table_index):
        # qkv [N, 3, H, hd]; bias fp32 [H, n, n], or with ``table_index`` the [rows, H] bias table; indices int32
        # [N, 2]; mask int8 [nW, n] or None
        qkv = qkv.contiguous()
        N, _, H, hd = qkv.shape
        D = H * hd
        dtype = qkv.dtype
        tp = (plan or TokenPlan(indices, batch_size, n, H)).finish()
        d = qkv.device
        bias32 = _bias32(bias, table_index, H, n, d)
        if mask is not None:
            mask = mask.to(torch.int8).contiguous()
        with _lib.on_device(d):
            p = torch.empty(tp.A, dtype=torch.float32, device=d)
            _tokens_to_sq(tp, dtype, True, qkv, 3 * D, 0, qkv, 3 * D, D, hd, scale, bias32, mask, p, None)
            _group_softmax(tp, False, p, None, p)                  # S -> P in place, rows from the group table
            out = torch.empty((N, D), dtype=dtype, device=d)
            _sq_to_tokens(tp, dtype, False, p, qkv, 3 * D, 2 * D, out, D, 0, hd, 1.0)
        ctx.save_for_backward(qkv, p, out)
        ctx.tp, ctx.scale, ctx.bias_meta, ctx.table_index = tp, scale, (bias.dtype, bias.shape), table_index
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        qkv, p, out = ctx.saved_tensors
        tp, scale = ctx.tp, ctx.scale
        N, _, H, hd = qkv.shape
        D = H * hd
        dtype = qkv.dtype
        d = qkv.device
        grad_out = grad_out.contiguous().to(dtype)
        lib = _lib.load()
        with _lib.on_device(d):
            d_qkv = torch.empty_like(qkv)
            d_s = torch.empty(tp.A, dtype=torch.float32, device=d)
            # dS = P (dO V^T - dO . O): the softmax backward is the epilogue of the product ; dV = P^T dO
            _score_grad(tp, dtype, grad_out, D, 0, qkv, 3 * D, 2 * D, out, D, 0, hd, p, d_s)
            _sq_to_tokens(tp, dtype, True, p, grad_out, D, 0, d_qkv, 3 * D, 2 * D, hd, 1.0)
            # dQ = scale * dS K ; dK = scale * dS^T Q
            _sq_to_tokens(tp, dtype, False, d_s, qkv, 3 * D, D, d_qkv, 3 * D, 0, hd, scale)
            _sq_to_tokens(tp, dtype, True, d_s, qkv, 3 * D, 0, d_qkv, 3 * D, D, hd, scale)
            d_bias = _bias_gradient(tp, H, d_s, ctx.bias_meta, ctx.table_index) if ctx.needs_input_grad[1] else None
        return d_qkv, d_bias, None, None, None, None, None, None, None


def _token_args(t, stride, col0):
    return _ptr(t), stride, col0


class _ResidentWindowAttention(Function):
    """Window-resident kernels: the attention matrix never reaches HBM.  Saved for backward:
    qkv, the attention output and one log-sum-exp per attention row."""

    @staticmethod
    def forward(ctx, qkv, bias, indices, mask, batch_size, n, scale, plan, table_index):
        # ``bias`` is the gathered [H, n, n] bias, or, with ``table_index`` (a BiasTableIndex), the
        # [rows, H] bias table itself: then the backward returns the table's gradient directly
        qkv = qkv.contiguous()
        N, _, H, hd = qkv.shape
        D = H * hd
        dtype = qkv.dtype
        d = qkv.device
        tp = (plan or TokenPlan(indices, batch_size, n, H)).finish()
        if tp.oversize_groups:
            raise RuntimeError(f"window-resident attention: {tp.oversize_groups} groups hold more than 128 tokens")
        bias32 = _bias32(bias, table_index, H, n, d)
        if mask is not None:
            mask = mask.to(torch.int8).contiguous()
        lib = _lib.load()
        with _lib.on_device(d):
            out = torch.empty((N, D), dtype=dtype, device=d)
            lse = torch.empty(max(H * N, 1), dtype=torch.float32, device=d)
            stream = _lib.stream_handle(d)
            _lib.check(lib.sswin_window_attention_forward(
                _DTYPE_CODE[dtype], _ptr(tp.tasks), tp.g_cap, tp.bucket_counts, _ptr(tp.tokens), N, H, hd,
                *_token_args(qkv, 3 * D, 0), *_token_args(qkv, 3 * D, D), *_token_args(qkv, 3 * D, 2 * D),
                C.c_float(scale), _ptr(bias32), n, _ptr(mask), 0 if mask is None else mask.shape[0],
                *_token_args(out, D, 0), _ptr(lse), stream))
        ctx.save_for_backward(qkv, out, lse, bias32, mask)
        ctx.tp, ctx.scale, ctx.bias_meta, ctx.table_index = tp, scale, (bias.dtype, bias.shape), table_index
        return out

    @staticmethod
    @once_differentiable
    def backward(ctx, grad_out):
        qkv, out, lse, bias32, mask = ctx.saved_tensors
        tp, scale = ctx.tp, ctx.scale
        N, _, H, hd = qkv.shape
        D = H * hd
        dtype = qkv.dtype
        d = qkv.device
        grad_out = grad_out.contiguous().to(dtype)
        lib = _lib.load()
        with _lib.on_device(d):
            d_qkv = torch.empty_like(qkv)
            want_bias = ctx.needs_input_grad[1]
            d_s = torch.empty(max(tp.A, 1), dtype=torch.float32, device=d) if want_bias else None
            stream = _lib.stream_handle(d)
            _lib.check(lib.sswin_window_attention_backward(
                _DTYPE_CODE[dtype], _ptr(tp.tasks), tp.g_cap, tp.bucket_counts, _ptr(tp.tokens), N, H, hd,
                *_token_args(qkv, 3 * D, 0), *_token_args(qkv, 3 * D, D), *_token_args(qkv, 3 * D, 2 * D),
                C.c_float(scale), _ptr(bias32), tp.n, _ptr(mask), 0 if mask is None else mask.shape[0],
                *_token_args(out, D, 0), *_token_args(grad_out, D, 0), _ptr(lse),
                *_token_args(d_qkv, 3 * D, 0), *_token_args(d_qkv, 3 * D, D), *_token_args(d_qkv, 3 * D, 2 * D),
                _ptr(d_s), 3, stream))
            d_bias = _bias_gradient(tp, H, d_s, ctx.bias_meta, ctx.table_index) if want_bias else None
        return d_qkv, d_bias, None, None, None, None, None, None, None


class BiasTableIndex:
    """The relative position index [n, n] of a bias table in the form the library uses:
    ``index[p, q] = code[p] - code[q] + offset0`` (true for the index arithmetic of
    sparse_swin/swin3d_base.py:630-647).  :meth:`build` returns None if an index is not of
    that form or the table is too large for the table-gradient kernel."""

    def __init__(self, flat, code, offset0):
        self.flat, self.code, self.offset0 = flat, code, offset0

    @staticmethod
    def build(index: torch.Tensor, table_rows: int):
        n = index.shape[0]
        if index.dim() != 2 or index.shape[1] != n or n > 384 or table_rows > 4096 or n == 0:
            return None
        idx = index.to(torch.int64)
        code = idx[:, 0]
        offset0 = int(idx[0, 0]) - 0
        # index[p, q] = code[p] - code[q] + offset0 with code[0] carrying offset0 out again
        code = code - int(code[0])
        if not torch.equal(idx, code[:, None] - code[None, :] + offset0):
            return None
        if int(idx.min()) < 0 or int(idx.max()) >= table_rows:
            return None
        return BiasTableIndex(idx.reshape(-1).contiguous(), code.to(torch.int32).contiguous(), offset0)


def fused_window_attention(qkv, bias, indices, mask, batch_size, n, scale, resident=None, plan=None,
                           table_index=None):
    """``qkv`` [N,3,H,hd], ``bias`` [H,n,n], ``indices`` int32 [N,2] (window,pos), ``mask`` int8
    [nW,n] or None -> attention output [N, H*hd] in the caller's voxel order.

    ``resident`` selects the window-resident kernels (default: whenever they apply, i.e. heads
    of 32 channels); otherwise the block products with the attention matrix in HBM are used.
    ``plan``: a :class:`TokenPlan` of ``indices`` made earlier (possibly still in flight).
    ``table_index``: a :class:`BiasTableIndex`; ``bias`` is then the [rows, H] bias table and its
    gradient is computed without the [H, n, n] detour."""
    if resident is None:
        resident = supports_resident(qkv, n)
    fn = _ResidentWindowAttention if resident else _FusedWindowAttention
    return fn.apply(qkv, bias, indices, mask, batch_size, n, scale, plan, table_index)


def supports_resident(qkv: torch.Tensor, n: int) -> bool:
    return supports(qkv, n) and qkv.shape[-1] == 32 and n <= 128


def supports(qkv: torch.Tensor, n: int, table: bool = False) -> bool:
    """The fused path covers fp32/fp16/bf16 on the GPU.  Windows: at most 128 positions when the bias gradient is
    formed as an [H, n, n] array (its LDS table), at most 384 (7^3 = 343 included) when it goes straight to the
    relative position table (``table``: the module has a :class:`BiasTableIndex`).  Everything else takes the
    operator-by-operator path."""
    return qkv.is_cuda and qkv.dtype in _DTYPE_CODE and (n <= 384 if table else n * n * 4 <= 64 * 1024)
