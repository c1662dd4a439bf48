"""Tensor-level wrappers over the C ABI: argument checks, workspace and stream plumbing.

Every function here enqueues HIP kernels on torch's current stream and returns
without synchronising.  Tensors must live on the GPU; there is no CPU path.
"""
from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

import torch
from torch import Tensor

from . import _lib
from ._lib import BGX_BF16, BGX_F16, BGX_F32, BlockDesc, ModuleDesc

SCAN_KMAX = 65536  # largest k of the scan's fused top-k selection (sorted in LDS up to 2048, in global memory beyond)

DTYPE_CODE = {torch.float32: BGX_F32, torch.float16: BGX_F16, torch.bfloat16: BGX_BF16}


def dtype_code(dtype: torch.dtype) -> int:
    try:
        return DTYPE_CODE[dtype]
    except KeyError:
        raise TypeError(f"unsupported dtype {dtype}; the kernels take float32, float16 and bfloat16") from None


def _need_gpu(t: Tensor, name: str) -> None:
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a GPU tensor: bergson_amd has no CPU path (got device {t.device})")


def _stream() -> C.c_void_p:
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t: Tensor | None) -> C.c_void_p | None:
    return None if t is None else C.c_void_p(t.data_ptr())


_workspaces: dict[tuple[int, int, str], Tensor] = {}

# When set to a list, every collection launch appends (start_event, stop_event, algorithmic_bytes): the
# events bracket the launch on the stream it runs on.  Used by the benchmark; None costs nothing.
collect_timer: list | None = None


def _workspace(device: torch.device, nbytes: int, tag: str) -> Tensor:
    """Scratch buffer per (device, stream, purpose), grown on demand and reused between calls.  One per stream:
    launches on different streams may overlap, and a buffer that is replaced by a larger one goes back to the
    allocator, which only orders its reuse against the stream it was allocated on."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    key = (index, torch.cuda.current_stream(device).cuda_stream, tag)
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < nbytes:
        ws = torch.empty(max(nbytes, 1 << 20), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


def collect_timing_start(max_launches: int) -> None:
    """Record an event pair around the collection kernel of the next `max_launches` launches."""
    _lib.check(_lib.load().bgx_collect_timing_enable(max_launches), "bgx_collect_timing_enable")


def collect_timing_stop() -> list[float]:
    """Kernel-only durations (ms) of the launches recorded since `collect_timing_start`."""
    lib = _lib.load()
    cap = 1 << 16
    buf = (C.c_float * cap)()
    n = C.c_int32(0)
    _lib.check(lib.bgx_collect_timing_read(buf, cap, C.byref(n)), "bgx_collect_timing_read")
    out = [float(buf[i]) for i in range(n.value)]
    _lib.check(lib.bgx_collect_timing_enable(0), "bgx_collect_timing_enable")
    return out


def adafactor_scales(row: Tensor | None, col: Tensor | None, dtype: torch.dtype) -> tuple[Tensor | None, Tensor | None]:
    """(row_scale [O], col_scale [I]) fp32 vectors of Adafactor factors rounded to `dtype`."""
    lib = _lib.load()
    ref = row if row is not None else col
    assert ref is not None
    _need_gpu(ref, "row/col")
    row32 = row.detach().to(torch.float32).contiguous() if row is not None else None
    col32 = col.detach().to(torch.float32).contiguous() if col is not None else None
    row_scale = torch.empty_like(row32) if row32 is not None else None
    col_scale = torch.empty_like(col32) if col32 is not None else None
    rc = lib.bgx_adafactor_scales(
        _ptr(row32), 0 if row32 is None else row32.numel(), _ptr(col32), 0 if col32 is None else col32.numel(),
        dtype_code(dtype), _ptr(row_scale), _ptr(col_scale), _stream(),
    )
    _lib.check(rc, "bgx_adafactor_scales")
    return row_scale, col_scale


@dataclass
class ModuleInput:
    """One hooked module of one batch, as the collection kernels see it."""

    a: Tensor  # [N, S, I]
    g: Tensor  # [N, S, O]
    r_in: Tensor  # [p, I], dtype of a
    r_out: Tensor  # [p, O]
    out_col: int
    col_scale: Tensor | None = None  # [I] fp32
    row_scale: Tensor | None = None  # [O] fp32
    bias_col: Tensor | None = None  # [p] fp32: column I of the [p, I+1] right projection
    bias_scale: Tensor | None = None  # [O] fp32: factor of g for the bias column (None = 1)


def _check_batch_vectors(lengths: Tensor | None, rows: Tensor | None, N: int, device: torch.device) -> None:
    """`lengths` (int32 [N]) and `rows` (int64 [N]: store rows or first-row offsets) as every kernel reads them.
    A wrong dtype would make a kernel read garbage lengths, a wrong size an out-of-range scatter: both are
    refused before anything is launched."""
    for t, name, dt in ((lengths, "lengths", torch.int32), (rows, "row indices / offsets", torch.int64)):
        if t is None:
            continue
        if t.dtype != dt or t.dim() != 1 or t.numel() != N or not t.is_contiguous():
            raise ValueError(f"{name} must be a contiguous {str(dt).removeprefix('torch.')} vector of N={N} elements, "
                             f"got {str(t.dtype).removeprefix('torch.')} {tuple(t.shape)}")
        _need_gpu(t, name)
        if t.device != device:
            raise ValueError(f"{name} live on {t.device}, the output on {device}")


def _rows_view(t: Tensor, name: str) -> Tensor:
    if t.dim() != 3:
        raise ValueError(f"{name} must be [N, S, features], got {tuple(t.shape)}")
    return t if t.stride(2) == 1 else t.contiguous()


def _collect(per_token: bool, modules: list[ModuleInput], p: int, out: Tensor, lengths: Tensor | None,
             rows: Tensor | None, lo: float, hi: float, static_scratch: bool = False) -> None:
    lib = _lib.load()
    if not modules:
        raise ValueError("no modules to collect")
    _need_gpu(out, "out")
    if out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("out must be a 2-D tensor with contiguous rows")
    N, S = modules[0].a.shape[:2]
    in_dtype = modules[0].a.dtype
    keep = []  # tensors that must stay alive until the launch is enqueued
    descs = (ModuleDesc * len(modules))()
    for d, m in zip(descs, modules):
        a = _rows_view(m.a, "a")
        g = _rows_view(m.g, "g")
        _need_gpu(a, "a")
        _need_gpu(g, "g")
        if a.shape[:2] != (N, S) or g.shape[:2] != (N, S):
            raise ValueError(f"all modules of a launch share [N, S]; got a {tuple(a.shape)} g {tuple(g.shape)}")
        if a.dtype != in_dtype or g.dtype != in_dtype:
            raise TypeError(f"all a/g of a launch share one dtype; got {a.dtype} and {g.dtype} vs {in_dtype}")
        I, O = a.shape[2], g.shape[2]
        r_in = m.r_in.contiguous()
        r_out = m.r_out.contiguous()
        if r_in.shape != (p, I) or r_out.shape != (p, O):
            raise ValueError(f"projection shapes {tuple(r_in.shape)} / {tuple(r_out.shape)} do not match p={p} I={I} O={O}")
        if r_in.dtype != in_dtype or r_out.dtype != in_dtype:
            raise TypeError("projection matrices must have the dtype of the activations")
        for s, n, k in ((m.col_scale, "col_scale", I), (m.row_scale, "row_scale", O)):
            if s is not None and (s.dtype != torch.float32 or s.numel() != k or not s.is_contiguous()):
                raise ValueError(f"{n} must be a contiguous fp32 vector of {k} elements")
        keep += [a, g, r_in, r_out]
        d.a, d.g, d.r_in, d.r_out = a.data_ptr(), g.data_ptr(), r_in.data_ptr(), r_out.data_ptr()
        d.col_scale = None if m.col_scale is None else m.col_scale.data_ptr()
        d.row_scale = None if m.row_scale is None else m.row_scale.data_ptr()
        for t_, n_, k_ in ((m.bias_col, "bias_col", p), (m.bias_scale, "bias_scale", O)):
            if t_ is not None and (t_.dtype != torch.float32 or t_.numel() != k_ or not t_.is_contiguous()):
                raise ValueError(f"{n_} must be a contiguous fp32 vector of {k_} elements")
        d.bias_col = None if m.bias_col is None else m.bias_col.data_ptr()
        d.bias_scale = None if m.bias_scale is None else m.bias_scale.data_ptr()
        d.a_seq_stride, d.a_tok_stride = a.stride(0), a.stride(1)
        d.g_seq_stride, d.g_tok_stride = g.stride(0), g.stride(1)
        d.out_col = m.out_col
        d.I, d.O = I, O
    _check_batch_vectors(lengths, rows, N, out.device)
    if static_scratch:
        rc = lib.bgx_collect_seq_static(descs, len(modules), N, S, p, dtype_code(in_dtype), _ptr(lengths), _ptr(rows),
                                        _ptr(out), out.stride(0), dtype_code(out.dtype), lo, hi, _stream())
        _lib.check(rc, "bgx_collect_seq_static")
        return
    nbytes = lib.bgx_collect_workspace_bytes_for(descs, len(modules), N, S, p, dtype_code(in_dtype))
    ws = _workspace(out.device, nbytes, "collect")
    fn = lib.bgx_collect_tok if per_token else lib.bgx_collect_seq
    timer = collect_timer
    if timer is not None:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
    rc = fn(descs, len(modules), N, S, p, dtype_code(in_dtype), _ptr(lengths), _ptr(rows), _ptr(out),
            out.stride(0), dtype_code(out.dtype), lo, hi, _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "bgx_collect_tok" if per_token else "bgx_collect_seq")
    if timer is not None:
        ev1.record()
        esz = 4 if in_dtype == torch.float32 else 2
        timer.append((ev0, ev1, sum(int(N) * int(S) * (d.I + d.O) * esz for d in descs)))
    del keep


class PreparedModule:
    """The batch-independent part of a module's descriptor, validated once.

    `fill` completes a descriptor with the (a, g) of one batch; only what can change between batches is
    checked there.
    """

    def __init__(self, m: ModuleInput, p: int):
        I, O = m.a.shape[2], m.g.shape[2]
        self.dtype = m.a.dtype
        self.I, self.O, self.p, self.out_col = I, O, p, m.out_col
        self.r_in = m.r_in.contiguous()
        self.r_out = m.r_out.contiguous()
        if self.r_in.shape != (p, I) or self.r_out.shape != (p, O):
            raise ValueError(f"projection shapes {tuple(self.r_in.shape)} / {tuple(self.r_out.shape)} do not match "
                             f"p={p} I={I} O={O}")
        if self.r_in.dtype != self.dtype or self.r_out.dtype != self.dtype or m.g.dtype != self.dtype:
            raise TypeError("activations, gradients and projection matrices must share one dtype")
        for s, n, k in ((m.col_scale, "col_scale", I), (m.row_scale, "row_scale", O)):
            if s is not None and (s.dtype != torch.float32 or s.numel() != k or not s.is_contiguous()):
                raise ValueError(f"{n} must be a contiguous fp32 vector of {k} elements")
        for t in (m.a, m.g, self.r_in, self.r_out):
            _need_gpu(t, "module operand")
        for s, n, k in ((m.bias_col, "bias_col", p), (m.bias_scale, "bias_scale", O)):
            if s is not None and (s.dtype != torch.float32 or s.numel() != k or not s.is_contiguous()):
                raise ValueError(f"{n} must be a contiguous fp32 vector of {k} elements")
        self.col_scale, self.row_scale = m.col_scale, m.row_scale
        self.bias_col, self.bias_scale = m.bias_col, m.bias_scale
        d = ModuleDesc()
        d.r_in, d.r_out = self.r_in.data_ptr(), self.r_out.data_ptr()
        d.col_scale = None if m.col_scale is None else m.col_scale.data_ptr()
        d.row_scale = None if m.row_scale is None else m.row_scale.data_ptr()
        d.bias_col = None if m.bias_col is None else m.bias_col.data_ptr()
        d.bias_scale = None if m.bias_scale is None else m.bias_scale.data_ptr()
        d.out_col, d.I, d.O = m.out_col, I, O
        self.template = d


def collect_prepared(per_token: bool, items: list, p: int, out: Tensor, lengths: Tensor | None,
                     rows: Tensor | None, lo: float, hi: float) -> None:
    """Fused launch over `items` = [(PreparedModule, a, g), ...] of one batch."""
    lib = _lib.load()
    _need_gpu(out, "out")
    if out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("out must be a 2-D tensor with contiguous rows")
    n = len(items)
    N, S = items[0][1].shape[:2]
    in_dtype = items[0][0].dtype
    descs = (ModuleDesc * n)()
    keep = []
    nbytes_alg = 0
    for i, (pm, a, g) in enumerate(items):
        if a.stride(2) != 1:
            a = a.contiguous()
        if g.stride(2) != 1:
            g = g.contiguous()
        if a.shape != (N, S, pm.I) or g.shape != (N, S, pm.O) or a.dtype != in_dtype or g.dtype != in_dtype \
                or pm.p != p:
            raise ValueError(f"module {i}: a {tuple(a.shape)} {a.dtype} / g {tuple(g.shape)} {g.dtype} do not match "
                             f"[N={N}, S={S}], I={pm.I}, O={pm.O}, {in_dtype}")
        keep.append(a)
        keep.append(g)
        C.memmove(C.byref(descs[i]), C.byref(pm.template), C.sizeof(ModuleDesc))
        d = descs[i]
        d.a, d.g = a.data_ptr(), g.data_ptr()
        d.a_seq_stride, d.a_tok_stride = a.stride(0), a.stride(1)
        d.g_seq_stride, d.g_tok_stride = g.stride(0), g.stride(1)
        nbytes_alg += pm.I + pm.O
    _check_batch_vectors(lengths, rows, N, out.device)
    ws = _workspace(out.device, lib.bgx_collect_workspace_bytes_for(descs, n, N, S, p, dtype_code(in_dtype)), "collect")
    fn = lib.bgx_collect_tok if per_token else lib.bgx_collect_seq
    timer = collect_timer
    if timer is not None:
        ev0, ev1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        ev0.record()
    rc = fn(descs, n, N, S, p, dtype_code(in_dtype), _ptr(lengths), _ptr(rows), _ptr(out), out.stride(0),
            dtype_code(out.dtype), lo, hi, _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "bgx_collect_tok" if per_token else "bgx_collect_seq")
    if timer is not None:
        ev1.record()
        timer.append((ev0, ev1, int(N) * int(S) * nbytes_alg * (4 if in_dtype == torch.float32 else 2)))
    del keep


adam_table_budget_bytes: int | None = None
"""Device memory the Adam tables of all modules may hold together; None = a quarter of the device's memory."""
_tables_in_use: dict = {}  # id(prep) -> weak reference to it; insertion order = least recently used first


def _touch_table(prep: "AdamPrepared") -> None:
    """Marks `prep`'s table as just used and drops the least recently used tables beyond the budget."""
    import weakref

    _tables_in_use.pop(id(prep), None)
    _tables_in_use[id(prep)] = weakref.ref(prep)
    budget = adam_table_budget_bytes
    if budget is None:
        budget = torch.cuda.get_device_properties(prep.r_in.device).total_memory // 4
    live = {}
    for key, ref in list(_tables_in_use.items()):
        q = ref()
        if q is None or q._table is None:
            del _tables_in_use[key]  # the module's state is gone, or its table was dropped
        else:
            live[key] = q
    held = sum(q._table.numel() * q._table.element_size() for q in live.values())
    for key, q in live.items():
        if held <= budget or key == id(prep):
            break
        held -= q._table.numel() * q._table.element_size()
        q._table = None
        del _tables_in_use[key]


class AdamPrepared:
    """Per-module state of the Adam path: the [(O*p), I] table built from the right projection and the
    second moments, and the left projection."""

    def __init__(self, r_in: Tensor, r_out: Tensor, weight_avg_sq: Tensor, out_col: int,
                 bias_col: Tensor | None = None, bias_avg_sq: Tensor | None = None):
        lib = _lib.load()
        _need_gpu(r_in, "r_in")
        p, I = r_in.shape
        O = r_out.shape[1]
        if r_out.shape[0] != p or tuple(weight_avg_sq.shape) != (O, I):
            raise ValueError(f"Adam shapes: r_in {tuple(r_in.shape)}, r_out {tuple(r_out.shape)}, "
                             f"weight_avg_sq {tuple(weight_avg_sq.shape)}")
        self.dtype = r_in.dtype
        self.p, self.I, self.O, self.out_col = p, I, O, out_col
        self.r_in = r_in.contiguous()
        self.r_out = r_out.contiguous()
        self.bias_col = self.bias_scale = None
        if bias_col is not None:
            if bias_avg_sq is None:
                raise ValueError("the bias column needs bias_avg_sq")
            self.bias_col = bias_col.detach().to(device=r_in.device, dtype=torch.float32).contiguous()
            # 1 / (sqrt(bias_avg_sq) + 1e-8): eps outside the root
            self.bias_scale = (bias_avg_sq.detach().to(device=r_in.device, dtype=torch.float32).sqrt() + 1e-8
                               ).reciprocal().contiguous()
        self.v = weight_avg_sq.detach().to(device=r_in.device, dtype=torch.float32).contiguous()
        self._table: Tensor | None = None
        self._seq_state = None

    @property
    def table(self) -> Tensor:
        """[(O*p), I] table of the per-token path: p times the bytes of the weight matrix, so the tables of all
        modules of a large model do not fit beside it.  Built on first use and kept while the tables of the
        process stay within `adam_table_budget_bytes` (least recently used go first, rebuilt when needed again:
        one pass over the second moments)."""
        if self._table is None:
            lib = _lib.load()
            bias = int(self.bias_col is not None)
            nbytes = lib.bgx_adam_table_bytes(self.O, self.I, self.p, dtype_code(self.dtype), bias)
            self._table = torch.empty(nbytes // self.r_in.element_size(), dtype=self.dtype, device=self.r_in.device)
            rc = lib.bgx_adam_prepare(_ptr(self.r_in), _ptr(self.v), _ptr(self.bias_col), _ptr(self.bias_scale), self.O,
                                      self.I, self.p, dtype_code(self.dtype), _ptr(self._table), _stream())
            _lib.check(rc, "bgx_adam_prepare")
        _touch_table(self)
        # the table may be dropped and its memory handed out again while this stream still reads it
        self._table.record_stream(torch.cuda.current_stream(self._table.device))
        return self._table

    def seq_state(self):
        """Operands of the per-sequence path that do not change between batches: the normaliser module of
        the weight-shaped gradient, the right projection over [grad | bias] and L^T with an identity
        projection (see collect_adam)."""
        if self._seq_state is None:
            dev = self.r_in.device
            bias = self.bias_col is not None
            full = FullGradModule(O=self.O, I=self.I, out_col=0, collect_bias=bias, adam_v=self.v,
                                  bias_scale=self.bias_scale)
            r_in = self.r_in
            if bias:
                r_in = torch.cat([self.r_in, self.bias_col.to(self.dtype).unsqueeze(1)], dim=1).contiguous()
            lt = self.r_out.t().contiguous()  # [O, p]: row o is what output feature o contributes to every P[i, :]
            eye = torch.eye(self.p, dtype=self.dtype, device=dev)
            self._seq_state = (full, r_in, lt, eye)
        return self._seq_state


def collect_adam(prep: AdamPrepared, a: Tensor, g: Tensor, out: Tensor, *, per_token: bool, lengths: Tensor | None,
                 rows: Tensor | None, lo: float, hi: float, chunk_tokens: int = 0) -> None:
    """One module with an Adam normaliser: writes its p*p block of every output row (see bgx_collect_adam)."""
    lib = _lib.load()
    for t, name in ((a, "a"), (g, "g"), (out, "out")):
        _need_gpu(t, name)
    if a.dim() != 3 or g.dim() != 3 or a.shape[:2] != g.shape[:2]:
        raise ValueError(f"a {tuple(a.shape)} / g {tuple(g.shape)} must be [N, S, I] and [N, S, O]")
    N, S, I = a.shape
    O = g.shape[2]
    if (I, O) != (prep.I, prep.O) or a.dtype != prep.dtype or g.dtype != prep.dtype:
        raise ValueError("a / g do not match the prepared module")
    if a.stride(2) != 1 or a.stride(0) != S * a.stride(1):
        a = a.contiguous()
    if g.stride(2) != 1:
        g = g.contiguous()
    if out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("out must be a 2-D tensor with contiguous rows")
    if per_token and (lengths is None or rows is None):
        raise ValueError("per-token collection needs lengths and row offsets")
    _check_batch_vectors(lengths, rows, N, out.device)
    if not per_token and chunk_tokens == 0:
        # Two ways to the per-sequence rows.  Normalising the summed gradient costs ~ N * S * O * I flops for the
        # product over the tokens plus a projection per 64 x 64 tile and sequence; summing per-token results costs
        # ~ N * S * p * O * I flops on the fused kernel, whatever the sequences' length.  Measured per layer of
        # Pythia-160m shapes on 4096 tokens, first against second: 0.27 / 0.88 ms (4 x 1024, p = 16), 0.44 / 0.83
        # (16 x 256), 0.64 / 0.82 (32 x 128), 1.08 / 0.82 (64 x 64); at p = 32: 0.74 / 1.63 (32 x 128), 1.33 / 1.66
        # (64 x 64), 2.56 / 1.66 (128 x 32) -- the second wins once sequences are shorter than about 1500 / p tokens.
        fused_ok = a.dtype != torch.float32 and prep.p <= 32   # the shapes the fused per-token kernels take
        if not (fused_ok and S * prep.p < 1500):
            _collect_adam_seq(prep, a, g, out, lengths, rows, lo, hi)
            return
    nbytes = lib.bgx_collect_adam_workspace_bytes(N, S, I, O, prep.p, dtype_code(prep.dtype),
                                                  int(prep.bias_col is not None), chunk_tokens)
    ws = _workspace(out.device, nbytes, "adam")
    rc = lib.bgx_collect_adam(_ptr(a), _ptr(g), a.stride(0), a.stride(1), g.stride(0), g.stride(1), N, S, I, O, prep.p,
                              dtype_code(prep.dtype), _ptr(prep.table), _ptr(prep.r_out), _ptr(prep.bias_col),
                              _ptr(prep.bias_scale), int(per_token), _ptr(lengths),
                              _ptr(rows), _ptr(out), out.stride(0), prep.out_col, dtype_code(out.dtype), lo, hi,
                              _ptr(ws), ws.numel(), chunk_tokens, _stream())
    _lib.check(rc, "bgx_collect_adam")


@dataclass
class FullGradModule:
    """Per-module state of the unprojected path: the normaliser's vectors on the device and the output column."""

    O: int
    I: int
    out_col: int
    collect_bias: bool = False
    row_scale: Tensor | None = None   # Adafactor, from adafactor_scales
    col_scale: Tensor | None = None
    adam_v: Tensor | None = None      # [O, I] fp32
    bias_scale: Tensor | None = None  # [O] fp32, None = 1

    @property
    def width(self) -> int:
        return self.O * (self.I + int(self.collect_bias))


def full_gradient(mod: FullGradModule, a: Tensor, g: Tensor, out: Tensor, *, per_token: bool,
                  lengths: Tensor | None, rows: Tensor | None, lo: float, hi: float) -> None:
    """Weight-shaped gradient of one module written to its columns of `out` (see bgx_fullgrad_seq / _tok).

    per_token=False: out[rows[n] (or n)] gets flatten(normalise(g[n]^T a[n])), the sum running over the
    tokens s < lengths[n] - 1 when lengths are given (all of them otherwise) -- one kernel, GEMM on the matrix
    cores with the normalisation behind it; per_token=True: out[rows[n] + s] gets
    flatten(normalise(g[n, s] (x) a[n, s])) for s < lengths[n] - 1.
    """
    lib = _lib.load()
    for t, name in ((a, "a"), (g, "g"), (out, "out")):
        _need_gpu(t, name)
    if a.dim() != 3 or g.dim() != 3 or a.shape[:2] != g.shape[:2]:
        raise ValueError(f"a {tuple(a.shape)} / g {tuple(g.shape)} must be [N, S, I] and [N, S, O]")
    N, S, I = a.shape
    O = g.shape[2]
    if (I, O) != (mod.I, mod.O) or a.dtype != g.dtype:
        raise ValueError("a / g do not match the prepared module")
    if out.dim() != 2 or out.stride(1) != 1:
        raise ValueError("out must be a 2-D tensor with contiguous rows")
    if a.stride(2) != 1:
        a = a.contiguous()
    if g.stride(2) != 1:
        g = g.contiguous()
    code = dtype_code(a.dtype)
    if per_token and (lengths is None or rows is None):
        raise ValueError("per-token collection needs lengths and row offsets")
    _check_batch_vectors(lengths, rows, N, out.device)
    if per_token:
        rc = lib.bgx_fullgrad_tok(_ptr(a), _ptr(g), a.stride(0), a.stride(1), g.stride(0), g.stride(1), N, S, I, O, code,
                                  _ptr(mod.row_scale), _ptr(mod.col_scale), _ptr(mod.adam_v), int(mod.collect_bias),
                                  _ptr(mod.bias_scale), _ptr(lengths), _ptr(rows), _ptr(out), out.stride(0),
                                  mod.out_col, dtype_code(out.dtype), lo, hi, _stream())
        _lib.check(rc, "bgx_fullgrad_tok")
        return
    rc = lib.bgx_fullgrad_seq_gemm(_ptr(a), _ptr(g), a.stride(0), a.stride(1), g.stride(0), g.stride(1), N, S, I, O,
                                   code, _ptr(mod.row_scale), _ptr(mod.col_scale), _ptr(mod.adam_v),
                                   int(mod.collect_bias), _ptr(mod.bias_scale), _ptr(lengths), _ptr(rows), _ptr(out),
                                   out.stride(0), mod.out_col, dtype_code(out.dtype), lo, hi, _stream())
    _lib.check(rc, "bgx_fullgrad_seq_gemm")


def project_rows(rows: Tensor, proj: Tensor, acc: Tensor) -> None:
    """acc[m, j] += sum_k rows[m, k] * proj[j, k]: one module's share of the global projection
    (collector.py:364-390).  rows [M, W] and proj [P, W] in the model dtype, acc [M, P] fp32, added to."""
    lib = _lib.load()
    for t, name in ((rows, "rows"), (proj, "proj"), (acc, "acc")):
        _need_gpu(t, name)
    if rows.dim() != 2 or proj.dim() != 2 or rows.shape[1] != proj.shape[1] or rows.dtype != proj.dtype:
        raise ValueError(f"rows {tuple(rows.shape)} {rows.dtype} / proj {tuple(proj.shape)} {proj.dtype} do not match")
    if acc.dtype != torch.float32 or acc.shape != (rows.shape[0], proj.shape[0]) or acc.stride(1) != 1:
        raise ValueError("acc must be fp32 [rows, P] with contiguous rows")
    if rows.stride(1) != 1:
        rows = rows.contiguous()
    proj = proj.contiguous()
    M, W = rows.shape
    P = proj.shape[0]
    if M == 0:
        return
    code = dtype_code(rows.dtype)
    ws = _workspace(rows.device, lib.bgx_project_rows_workspace_bytes(M, W, P, code), "project")
    rc = lib.bgx_project_rows(_ptr(rows), M, W, rows.stride(0), code, _ptr(proj), P, _ptr(acc), acc.stride(0),
                              _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "bgx_project_rows")


def _collect_adam_seq(prep: AdamPrepared, a: Tensor, g: Tensor, out: Tensor, lengths: Tensor | None,
                      rows: Tensor | None, lo: float, hi: float, through_memory: bool = False) -> None:
    """Per-sequence Adam without anything per token: the normalisation is applied to the summed gradient, as
    the reference does (collector.py:634-644):
        Q[n] = (g[n]^T a[n]) / (sqrt(v) + 1e-8)  [| bias column],   P[n] = L Q[n] R^T.
    16-bit models with p <= 32: one launch forms Q tile by tile and projects every tile where it is
    (bgx_collect_seq_weight).  Otherwise Q goes through memory: bgx_fullgrad_seq_gemm, then bgx_collect_seq with
    the output features in the role of tokens -- "a" = Q[n] ([O, I(+1)] rows), projected by R; "g" = L^T ([O, p],
    shared by all n, sequence stride 0) with an identity projection; the token reduction is the sum over output
    features.
    """
    N, S, _ = a.shape
    full, r_in, lt, eye = prep.seq_state()
    if prep.dtype != torch.float32 and prep.p <= 32 and not through_memory:
        lib = _lib.load()
        ws = _workspace(out.device, lib.bgx_collect_seq_weight_workspace_bytes(N, prep.I, prep.O, prep.p), "adam_seq")
        rc = lib.bgx_collect_seq_weight(_ptr(a), _ptr(g), a.stride(0), a.stride(1), g.stride(0), g.stride(1), N, S,
                                        prep.I, prep.O, prep.p, dtype_code(prep.dtype), None, None, _ptr(full.adam_v),
                                        _ptr(prep.r_out), _ptr(prep.r_in), prep.r_in.stride(0), _ptr(prep.bias_col),
                                        _ptr(full.bias_scale), _ptr(lengths), _ptr(rows), _ptr(out), out.stride(0),
                                        prep.out_col, dtype_code(out.dtype), lo, hi, _ptr(ws), ws.numel(), _stream())
        _lib.check(rc, "bgx_collect_seq_weight")
        return
    q = torch.empty((N, full.width), dtype=prep.dtype, device=a.device)
    # positions from len-1 on carry no label: the kernel leaves them out of the sum
    full_gradient(full, a, g, q, per_token=False, lengths=lengths, rows=None, lo=float("-inf"), hi=float("inf"))
    Iw = full.width // prep.O
    m = ModuleInput(a=q.view(N, prep.O, Iw), g=lt.unsqueeze(0).expand(N, prep.O, prep.p), r_in=r_in, r_out=eye,
                    out_col=prep.out_col)
    _collect(False, [m], prep.p, out, None, rows, lo, hi)


def collect_seq(modules: list[ModuleInput], p: int, out: Tensor, *, lengths: Tensor | None = None,
                out_rows: Tensor | None = None, lo: float = float("-inf"), hi: float = float("inf")) -> None:
    """out[row(n), m.out_col : m.out_col + p*p] = clamp(sum_s g'[n,s] (x) a'[n,s]) for every module m."""
    _collect(False, modules, p, out, lengths, out_rows, lo, hi)


def collect_seq_static(modules: list[ModuleInput], p: int, out: Tensor, *, lengths: Tensor | None = None,
                       out_rows: Tensor | None = None, lo: float = float("-inf"), hi: float = float("inf")) -> None:
    """`collect_seq` through the entry point that allocates nothing: no workspace tensor, the library's own
    static scratch array instead (16 MiB per GPU; larger launches are refused).  Calls that could overlap on
    one GPU must not use it at the same time."""
    _collect(False, modules, p, out, lengths, out_rows, lo, hi, static_scratch=True)


def collect_tok(modules: list[ModuleInput], p: int, out: Tensor, *, lengths: Tensor, row_offsets: Tensor,
                lo: float = float("-inf"), hi: float = float("inf")) -> None:
    """out[row_offsets[n] + s, block(m)] = clamp(g'[n,s] (x) a'[n,s]) for s < lengths[n] - 1."""
    _collect(True, modules, p, out, lengths, row_offsets, lo, hi)


def unit_normalize_rows_(rows: Tensor) -> Tensor:
    """In-place g * rsqrt(max(sum g^2, eps^2)) per row."""
    lib = _lib.load()
    _need_gpu(rows, "rows")
    if rows.dim() != 2 or rows.stride(1) != 1:
        raise ValueError("rows must be 2-D with contiguous rows")
    rc = lib.bgx_unit_normalize_rows(_ptr(rows), rows.shape[0], rows.shape[1], rows.stride(0), dtype_code(rows.dtype),
                                     _stream())
    _lib.check(rc, "bgx_unit_normalize_rows")
    return rows


def _block_descs(blocks: list[tuple[Tensor, int]], width: int) -> "C.Array":
    """(matrix [d, d] fp32 on the GPU, first column) per module -> bgx_block_desc array."""
    descs = (BlockDesc * len(blocks))()
    for d, (h, col0) in zip(descs, blocks):
        _need_gpu(h, "block matrix")
        if h.dtype != torch.float32 or h.dim() != 2 or h.shape[0] != h.shape[1] or not h.is_contiguous():
            raise ValueError("a block matrix must be a contiguous square fp32 tensor")
        if col0 < 0 or col0 + h.shape[0] > width:
            raise ValueError(f"block columns {col0}..{col0 + h.shape[0]} outside a row of {width}")
        d.h_dev, d.col0, d.dim, d.reserved = h.data_ptr(), col0, h.shape[0], 0
    return descs


def block_gemm(rows: Tensor, blocks: list[tuple[Tensor, int]], out_dtype: torch.dtype = torch.float32,
               out: Tensor | None = None) -> Tensor:
    """out[:, c0:c0+d] = rows[:, c0:c0+d].float() @ H for every (H [d, d] fp32, c0) in `blocks`.

    Columns that belong to no block are copied (cast) from `rows`, so that `out` is a complete row
    block (DensePreconditioner.apply passes modules without a matrix through unchanged)."""
    lib = _lib.load()
    _need_gpu(rows, "rows")
    if rows.dim() != 2 or rows.stride(1) != 1:
        raise ValueError("rows must be 2-D with contiguous rows")
    if out is None:
        out = torch.empty(rows.shape, dtype=out_dtype, device=rows.device)
    elif out.shape != rows.shape or out.stride(1) != 1 or out.data_ptr() == rows.data_ptr():
        raise ValueError("out must be a separate [rows, width] tensor with contiguous rows")
    covered = sum(h.shape[0] for h, _ in blocks)
    if covered != rows.shape[1]:
        out.copy_(rows)
    if not blocks or rows.shape[0] == 0:
        return out
    descs = _block_descs(blocks, rows.shape[1])
    nbytes = lib.bgx_precond_workspace_bytes(len(blocks))
    ws = _workspace(rows.device, nbytes, "precond")
    rc = lib.bgx_block_gemm(_ptr(rows), dtype_code(rows.dtype), rows.stride(0), _ptr(out), dtype_code(out.dtype),
                            out.stride(0), rows.shape[0], descs, len(blocks), _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "bgx_block_gemm")
    return out


def gram_accumulate(rows: Tensor, blocks: list[tuple[Tensor, int]]) -> None:
    """H += rows[:, c0:c0+d].float().T @ rows[:, c0:c0+d].float() for every (H, c0) in `blocks`, in place."""
    lib = _lib.load()
    _need_gpu(rows, "rows")
    if rows.dim() != 2 or rows.stride(1) != 1:
        raise ValueError("rows must be 2-D with contiguous rows")
    if not blocks or rows.shape[0] == 0:
        return
    descs = _block_descs(blocks, rows.shape[1])
    nbytes = lib.bgx_precond_workspace_bytes(len(blocks))
    ws = _workspace(rows.device, nbytes, "precond")
    rc = lib.bgx_gram_accumulate(_ptr(rows), dtype_code(rows.dtype), rows.stride(0), rows.shape[0], descs, len(blocks),
                                 _ptr(ws), ws.numel(), _stream())
    _lib.check(rc, "bgx_gram_accumulate")


def row_sumsq(store: Tensor) -> Tensor:
    """fp32 [n] sums of squares of the rows of `store` in one HBM-bound pass: the values a scan's own `sumsq`
    holds, bit for bit (see bgx_row_sumsq), so `scan(..., row_sumsq=row_sumsq(store))` equals a plain scan."""
    lib = _lib.load()
    _need_gpu(store, "store")
    if store.dim() != 2 or store.stride(1) != 1:
        raise ValueError("store must be 2-D with contiguous rows")
    out = torch.empty((store.shape[0],), dtype=torch.float32, device=store.device)
    if store.shape[0]:
        rc = lib.bgx_row_sumsq(_ptr(store), store.shape[0], store.shape[1], store.stride(0), dtype_code(store.dtype),
                               _ptr(out), _stream())
        _lib.check(rc, "bgx_row_sumsq")
    return out


@dataclass
class ScanResult:
    topk_values: Tensor | None = None  # [Q, k] fp32
    topk_indices: Tensor | None = None  # [Q, k] int64
    row_max: Tensor | None = None  # [n_rows] fp32
    row_mean: Tensor | None = None  # [n_rows] fp32
    scores: Tensor | None = None  # [n_rows, Q] fp32
    sumsq: Tensor | None = None  # [n_rows] fp32


def scan(store: Tensor, queries: Tensor, *, unit_norm: bool, k: int = 0, query_scale: float = 1.0, row_base: int = 0,
         want_row_max: bool = False, want_row_mean: bool = False, want_scores: bool = False,
         want_sumsq: bool = False, chunk_rows: int = 0, row_sumsq: Tensor | None = None) -> ScanResult:
    """Score store rows [n, D] against queries [Q, D] (same dtype); see bgx_scan in include/bergson_amd.h.
    `row_sumsq` [n] fp32: the `sumsq` of an earlier scan of the same rows (bgx_scan_known_norms): kernels then
    leave the row norms out of their inner loops."""
    lib = _lib.load()
    _need_gpu(store, "store")
    _need_gpu(queries, "queries")
    if store.dim() != 2 or store.stride(1) != 1:
        raise ValueError("store must be 2-D with contiguous rows")
    if queries.dim() != 2 or queries.shape[1] != store.shape[1]:
        raise ValueError(f"queries {tuple(queries.shape)} do not match store {tuple(store.shape)}")
    if queries.dtype != store.dtype:
        raise TypeError("queries must have the store dtype")
    queries = queries.contiguous()
    n, D = store.shape
    Q = queries.shape[0]
    dev = store.device
    res = ScanResult()
    if k:
        res.topk_values = torch.empty((Q, k), dtype=torch.float32, device=dev)
        res.topk_indices = torch.empty((Q, k), dtype=torch.int64, device=dev)
    if want_row_max:
        res.row_max = torch.empty((n,), dtype=torch.float32, device=dev)
    if want_row_mean:
        res.row_mean = torch.empty((n,), dtype=torch.float32, device=dev)
    if want_scores:
        res.scores = torch.empty((n, Q), dtype=torch.float32, device=dev)
    if want_sumsq and row_sumsq is None:
        res.sumsq = torch.empty((n,), dtype=torch.float32, device=dev)
    ws = None
    if k or want_row_mean or Q <= 96:  # few queries: the streaming kernel keeps its query fragments there
        ws = _workspace(dev, lib.bgx_scan_workspace_bytes_for(Q, k, chunk_rows, D, dtype_code(store.dtype)), "scan")
    if row_sumsq is not None:
        _need_gpu(row_sumsq, "row_sumsq")
        if row_sumsq.dtype != torch.float32 or row_sumsq.shape != (n,) or not row_sumsq.is_contiguous():
            raise ValueError("row_sumsq must be a contiguous fp32 vector with one entry per store row")
        if want_sumsq:
            res.sumsq = row_sumsq
        rc = lib.bgx_scan_known_norms(_ptr(store), n, D, store.stride(0), dtype_code(store.dtype), _ptr(queries), Q,
                                      query_scale, int(unit_norm), k, row_base, _ptr(row_sumsq),
                                      _ptr(res.topk_values), _ptr(res.topk_indices), _ptr(res.row_max),
                                      _ptr(res.row_mean), _ptr(res.scores), _ptr(ws), 0 if ws is None else ws.numel(),
                                      chunk_rows, _stream())
        _lib.check(rc, "bgx_scan_known_norms")
        return res
    rc = lib.bgx_scan(_ptr(store), n, D, store.stride(0), dtype_code(store.dtype), _ptr(queries), Q, query_scale,
                      int(unit_norm), k, row_base, _ptr(res.topk_values), _ptr(res.topk_indices), _ptr(res.row_max),
                      _ptr(res.row_mean), _ptr(res.scores), _ptr(res.sumsq), _ptr(ws), 0 if ws is None else ws.numel(), chunk_rows,
                      _stream())
    _lib.check(rc, "bgx_scan")
    return res
