"""Python faces of the HIP kernels: they check shapes and types on the host, then launch.

Every function takes torch tensors that live on the GPU, launches on torch's current stream
and returns its output tensor.  There is no other implementation behind these functions: a
missing library or a refused size raises :class:`~gesso_amd.errors.KernelError`.
"""
from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long

import torch

from ..errors import KernelError
from . import build as _build

F32, BF16 = 0, 1
_DT = {torch.float32: F32, torch.bfloat16: BF16}

_lib = None


def lib():
    global _lib
    if _lib is None:
        _lib = _build.load()
    return _lib


def _dt(t: torch.Tensor) -> int:
    d = t.dtype
    if d is torch.bfloat16:
        return BF16
    if d is torch.float32:
        return F32
    raise KernelError(f"kernels take float32 or bfloat16, got {d}")


def _p(t):
    """A tensor's address as the library's entry points take it (their argument types are declared when the library is
    loaded, so a plain integer or None is all a pointer argument needs)."""
    return None if t is None else t.data_ptr()


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream():
    """The current stream of the current device as a raw handle (a launch asks for it every time: the short way;
    ``torch.cuda.current_device`` alone costs a microsecond a call, and a step of prompt portions asks 150 times)."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _check(rc: int):
    if rc != 0:
        raise KernelError(lib().gs_last_error().decode())


def _need(cond: bool, msg: str):
    if not cond:
        raise KernelError(msg)


def _dev(*ts):
    # (the messages are made only when a check fails: these run before every launch)
    for t in ts:
        if t is not None and not (t.is_cuda and t.is_contiguous()):
            raise KernelError("kernel operands must live on the GPU" if not t.is_cuda else "kernel operands must be contiguous")


def _i32(t, n=None, what="index"):
    if t.dtype != torch.int32:
        raise KernelError(f"{what} must be int32, got {t.dtype}")
    if n is not None and t.numel() < n:
        raise KernelError(f"{what} holds {t.numel()} entries, {n} needed")


# ---------------------------------------------------------------------- tiled rows

class TiledRows:
    """Rows of bfloat16 that feed a weight-streaming product, kept in the order the matrix cores take them.

    ``(M, K)`` with K a multiple of 32; the buffer holds, for each step of 32 columns and each tile of 16 rows,
    64 lanes x 16 bytes: lane ``l`` has row ``l % 16``, columns ``8 (l / 16) ... + 7`` of the step.  A product reads
    such a tile with one contiguous kilobyte per wavefront instead of sixteen pieces of rows.  Kernels that write
    rows for a product (embedding, the SwiGLU, convolution and residual epilogues, decode attention) write this
    order when handed one of these; the products read it.  ``rows()`` gives the ordinary tensor.
    """

    __slots__ = ("buf", "shape", "dtype", "device")

    def __init__(self, M: int, K: int, device):
        _need(K % 32 == 0, f"tiled rows are a multiple of 32 wide, not {K}")
        self.buf = torch.empty(((M + 15) // 16) * 16 * K, dtype=torch.bfloat16, device=device)
        self.shape = (M, K)
        self.dtype = torch.bfloat16
        self.device = self.buf.device

    @staticmethod
    def fits(K: int) -> bool:
        return K % 32 == 0

    @classmethod
    def of(cls, x: torch.Tensor) -> "TiledRows":
        """The tiled copy of a bfloat16 tensor ``(M, K)``."""
        _need(x.dim() == 2 and x.dtype == torch.bfloat16 and x.stride(1) == 1, "tiled rows are made from bfloat16 (M, K)")
        M, K = x.shape
        t = cls(M, K, x.device)
        t.buf.zero_()
        _check(lib().gs_retile_rows(_p(x), _p(t.buf), c_int(M), c_int(K), c_int(x.stride(0) if M > 1 else K), c_int(1),
                                    _stream()))
        return t

    def rows(self) -> torch.Tensor:
        M, K = self.shape
        out = torch.empty((M, K), dtype=torch.bfloat16, device=self.device)
        _check(lib().gs_retile_rows(_p(self.buf), _p(out), c_int(M), c_int(K), c_int(K), c_int(0), _stream()))
        return out


def _rows_out(out, M, N, device, dtype=torch.bfloat16):
    """An output of rows ``(M, N)``: a tensor, or tiled rows when ``out`` is True (made here) or a TiledRows."""
    if out is True:
        out = TiledRows(M, N, device)
    if isinstance(out, TiledRows):
        _need(out.shape == (M, N), f"tiled rows of shape {out.shape}, expected {(M, N)}")
        return out, out.buf, 1
    if out is None or out is False:
        out = torch.empty((M, N), dtype=dtype, device=device)
    return out, out, 0


# ---------------------------------------------------------------------- elementwise

def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor = None, ssq: torch.Tensor = None,
          next_weight: torch.Tensor = None, xs: torch.Tensor = None, scale: float = 1.0) -> torch.Tensor:
    """``out[t] = table[ids[t]] * scale`` as float32 ``(T, H)``; with ``ssq (T, 1)`` also each row's sum of squares;
    with ``next_weight (H,)`` and ``xs (T, H)`` bfloat16 also ``xs = out * next_weight``."""
    _dev(ids, table, out, ssq, next_weight, None if isinstance(xs, TiledRows) else xs)
    _i32(ids, what="token ids")
    V, H = table.shape
    T = ids.numel()
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.shape == (T, H), "embed: out must be float32 (T, H)")
    _need(ssq is None or (ssq.dtype == torch.float32 and ssq.numel() == T), "embed: ssq must be float32 (T, 1)")
    _need((next_weight is None) == (xs is None), "embed: next_weight and xs come together")
    xs_buf, xs_tiled = xs, 0
    if xs is not None:
        if isinstance(xs, TiledRows):
            xs_buf, xs_tiled = xs.buf, 1
        _need(next_weight.dtype == torch.float32 and next_weight.shape == (H,) and xs.dtype == torch.bfloat16
              and tuple(xs.shape) == (T, H) and xs_buf.is_contiguous(), "embed: next_weight float32 (H,), xs bfloat16 (T, H)")
    _check(lib().gs_embed(_p(ids), _p(table), _dt(table), _p(out), _p(ssq), _p(next_weight), _p(xs_buf), c_int(xs_tiled),
                          c_int(T), c_int(H), c_int(V), c_float(scale), _stream()))
    return out


def add_rmsnorm(res: torch.Tensor, delta, weight: torch.Tensor, eps: float, out_dtype, rows=None,
                out: torch.Tensor = None) -> torch.Tensor:
    """``res += delta`` (when given and no ``rows``), then ``out = rmsnorm(res) * weight``.

    ``rows`` (int32) picks source rows; then ``res`` is not written.
    """
    f32 = torch.float32
    if not (res.is_cuda and res.is_contiguous() and res.dtype is f32 and res.dim() == 2):
        raise KernelError("add_rmsnorm: the residual stream is float32 (T, H), contiguous, on the GPU")
    T, H = res.shape
    if not (weight.is_cuda and weight.dtype is f32 and weight.shape == (H,) and weight.is_contiguous()):
        raise KernelError("add_rmsnorm: weight must be float32 (H,)")
    if delta is not None and not (delta.is_cuda and delta.is_contiguous() and delta.shape == res.shape):
        raise KernelError("add_rmsnorm: delta must have the stream's shape")
    n_out = T
    if rows is not None:
        _dev(rows)
        _i32(rows, what="rows")
        n_out = rows.numel()
    if out is None:
        out = torch.empty((n_out, H), dtype=out_dtype, device=res.device)
    elif not (out.is_cuda and out.is_contiguous() and out.shape == (n_out, H) and out.dtype == out_dtype):
        raise KernelError("add_rmsnorm: out has the wrong shape or type")
    rc = lib().gs_add_rmsnorm(res.data_ptr(), None if delta is None else delta.data_ptr(),
                              _dt(delta) if delta is not None else _dt(out), weight.data_ptr(), eps, out.data_ptr(),
                              _dt(out), None if rows is None else rows.data_ptr(), n_out, H, _stream())
    if rc != 0:
        _check(rc)
    return out


def residual_add(res: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _dev(res, delta)
    _need(res.dtype == torch.float32 and delta.shape == res.shape, "residual_add: shapes or types differ")
    _check(lib().gs_residual_add(_p(res), _p(delta), c_int(_dt(delta)), c_long(res.numel()), _stream()))
    return res


def swiglu(x: torch.Tensor, out: torch.Tensor = None) -> torch.Tensor:
    """``x (T, 2F)`` = gate | up  ->  ``silu(gate) * up (T, F)``."""
    if not (x.is_cuda and x.is_contiguous() and x.dim() == 2):
        raise KernelError("swiglu: rows (T, 2F), contiguous, on the GPU")
    T, F2 = x.shape
    if F2 % 2:
        raise KernelError("swiglu: the input holds gate and up side by side")
    F = F2 // 2
    if out is None:
        out = torch.empty((T, F), dtype=x.dtype, device=x.device)
    elif not (out.is_cuda and out.is_contiguous() and out.shape == (T, F) and out.dtype == x.dtype):
        raise KernelError("swiglu: out has the wrong shape or type")
    rc = lib().gs_swiglu(x.data_ptr(), out.data_ptr(), _dt(x), T, F, _stream())
    if rc != 0:
        _check(rc)
    return out


def add_bias(y: torch.Tensor, bias: torch.Tensor, out_dtype=None, out: torch.Tensor = None) -> torch.Tensor:
    """``y + bias`` row by row: ``y`` float32 ``(M, N)`` contiguous (a product's sums), ``bias`` float32 ``(N,)``;
    the result in ``out_dtype``, rounded once."""
    _dev(y, bias)
    _need(out is None or out.is_cuda, "kernel operands must live on the GPU")
    _need(y.dtype == torch.float32 and y.dim() == 2 and y.is_contiguous(), "add_bias: y must be float32 (M, N), contiguous")
    M, N = y.shape
    _need(bias.dtype == torch.float32 and bias.shape == (N,) and bias.is_contiguous(), "add_bias: bias must be float32 (N,)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or torch.float32, device=y.device)
    _need(out.shape == (M, N) and out.stride(1) == 1 and out.dtype in (torch.float32, torch.bfloat16),
          "add_bias: out has the wrong shape or type")
    _check(lib().gs_add_bias(_p(y), _p(bias), _p(out), c_int(_dt(out)), c_int(M), c_int(N),
                             c_long(out.stride(0) if M > 1 else N), _stream()))
    return out


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """``cap * tanh(logits / cap)`` in place (float32)."""
    _dev(logits)
    _need(logits.dtype == torch.float32, "softcap takes float32 logits")
    _check(lib().gs_softcap(_p(logits), c_float(cap), c_long(logits.numel()), _stream()))
    return logits


def stream_read(buf: torch.Tensor, blocks: int = 2048, contiguous: bool = True, sink: torch.Tensor = None) -> None:
    """Read ``buf`` once from memory with a plain streaming kernel (a measurement, see ``bench.py``): each block its
    own contiguous share, or the grid sweeping the buffer together."""
    _dev(buf, sink)
    nbytes = buf.numel() * buf.element_size()
    if sink is None:
        sink = torch.zeros(blocks, dtype=torch.int32, device=buf.device)
    _need(sink.dtype == torch.int32 and sink.numel() >= blocks, "stream_read: sink holds an int32 per block")
    _check(lib().gs_stream_read(_p(buf), c_long(nbytes), _p(sink), c_int(blocks), c_int(1 if contiguous else 0), _stream()))


FILL_MAX = 65535


def fill_rows(pool: torch.Tensor, ids: torch.Tensor, value: float, planes: int = 1) -> None:
    """``pool[..., id, ...] = value`` for each id in ``ids`` (int32): ``pool`` is ``(planes..., rows, *row shape)`` with
    ``planes`` leading axes flattened into one (1: ``(rows, ...)``), float32 or bfloat16.  A fresh state slot gets its
    initial value this way; with poisoning on, so do the pages and slots a request gave back (NaN)."""
    _dev(pool, ids)
    _i32(ids, what="row ids")
    lead = pool.shape[:planes - 1] if planes > 1 else ()
    outer = 1
    for n in lead:
        outer *= n
    rows = pool.shape[len(lead)]
    row = pool[(0,) * (len(lead) + 1)].numel() if pool.numel() else 0
    _need(outer <= FILL_MAX, f"fill_rows: {outer} planes are more than a launch takes ({FILL_MAX})")
    for at in range(0, ids.numel(), FILL_MAX):            # a launch takes 65,535 ids: many freed pages go in turns
        part = ids[at:at + FILL_MAX]
        _check(lib().gs_fill_rows(_p(pool), c_int(_dt(pool)), _p(part), c_int(part.numel()), c_long(row), c_int(outer),
                                  c_long(rows), c_float(value), _stream()))


# ---------------------------------------------------------------------- short convolution

def short_conv(bcx, taps, bias, state, seq_of_token, q_start, slots, nseq: int, all_single: bool,
               out: torch.Tensor = None) -> torch.Tensor:
    """Gated short convolution over segments; ``state (num_slots, H, W-1)`` is read and advanced."""
    _dev(bcx, taps, bias, state, seq_of_token, q_start, slots, out)
    T, H3 = bcx.shape
    _need(H3 % 3 == 0, "short_conv: bcx holds B, C, X side by side")
    H = H3 // 3
    W = taps.shape[1]
    _need(taps.dtype == torch.float32 and taps.shape == (H, W), "short_conv: taps must be float32 (H, W)")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (H,)), "short_conv: bias must be float32 (H,)")
    _need(state.dtype == torch.float32 and state.dim() == 3 and state.shape[1:] == (H, W - 1),
          "short_conv: state must be float32 (slots, H, W-1)")
    _i32(seq_of_token, T, "seq_of_token")
    _i32(q_start, nseq + 1, "q_start")
    _i32(slots, nseq, "slots")
    if out is None:
        out = torch.empty((T, H), dtype=bcx.dtype, device=bcx.device)
    _need(out.shape == (T, H) and out.dtype == bcx.dtype, "short_conv: out has the wrong shape or type")
    _check(lib().gs_short_conv(_p(bcx), c_int(_dt(bcx)), _p(taps), _p(bias), _p(state), _p(seq_of_token),
                               _p(q_start), _p(slots), _p(out), c_int(T), c_int(nseq), c_int(H), c_int(W),
                               c_int(1 if all_single else 0), _stream()))
    return out


# ---------------------------------------------------------------------- attention

ROPE_LAYOUTS = ("half", "interleaved")


def _value_tables(vcos, vsin, vd):
    """Checks the tables by which values are turned (``(P, vd/2)`` float32, both or neither)."""
    _need((vcos is None) == (vsin is None), "the value tables come together")
    if vcos is not None:
        _dev(vcos, vsin)
        _need(vd % 2 == 0 and vcos.dtype == torch.float32 and vsin.dtype == torch.float32 and vcos.shape == vsin.shape
              and vcos.dim() == 2 and vcos.shape[1] == vd // 2, "value tables must be float32 (P, value width / 2)")


def qknorm_rope_kv(qkv, q_weight, k_weight, eps, cos, sin, rotary_dim, positions, seq_of_token, block_table,
                   page_size, kcache, vcache, nh, nkv, d, write_kv=True, layout: str = "half", vd: int = None,
                   vcos=None, vsin=None, plain_norm: bool = False, v_first=None, mix=None) -> None:
    """Head norm and rotation of q (in place) and k; k and v written into the pages.  ``layout``: which features
    form a rotation pair, ``"half"`` (i, i + rotary_dim/2) or ``"interleaved"`` (2i, 2i + 1).  ``vd``: the width of
    a value head where it is not ``d``; ``vcos``, ``vsin`` ``(P, vd/2)``: the values are cached turned by their
    position over their whole width.  The rows may hold more columns behind q|k|v.  ``plain_norm``: q and k are divided
    by their root mean square, no weight.  ``v_first (T, >= nkv vd)`` (a range of columns of wider rows will do) with
    ``mix`` (one float32 on the device): the values are cached as ``(1 - mix) v + mix v_first``."""
    _need(layout in ROPE_LAYOUTS, f"qknorm_rope_kv: pairs are laid out 'half' or 'interleaved', not {layout!r}")
    _dev(qkv, q_weight, k_weight, cos, sin, positions, seq_of_token, block_table, kcache, vcache, mix)
    vd = d if vd is None else int(vd)
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] >= (nh + nkv) * d + nkv * vd, "qknorm_rope_kv: rows hold at least (nh + nkv) d + nkv vd values")
    _need(not (plain_norm and q_weight is not None), "qknorm_rope_kv: a head norm has a weight or none")
    _need((v_first is None) == (mix is None), "qknorm_rope_kv: the other values and their share come together")
    ldf = 0
    if v_first is not None:
        _need(v_first.is_cuda and v_first.dim() == 2 and v_first.shape == (T, nkv * vd) and v_first.stride(1) == 1
              and v_first.dtype == qkv.dtype and mix.dtype == torch.float32 and mix.numel() == 1,
              "qknorm_rope_kv: the other values are (T, nkv vd) of the rows' type, their share one float32")
        ldf = v_first.stride(0) if T > 1 else nkv * vd
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.shape == (d,)), "qknorm_rope_kv: head norm weight must be float32 (d,)")
    max_pos = 0
    if rotary_dim:
        _need(cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.dim() == 2 and cos.shape[1] == rotary_dim // 2, "qknorm_rope_kv: tables must be float32 (P, rotary_dim/2)")
        max_pos = cos.shape[0]
    _value_tables(vcos, vsin, vd)
    if vcos is not None:
        max_pos = vcos.shape[0] if not max_pos else min(max_pos, vcos.shape[0])
    _i32(positions, T, "positions")
    _i32(seq_of_token, T, "seq_of_token")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    _need(kcache.dtype == qkv.dtype and vcache.dtype == qkv.dtype, "cache and activations differ in type")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape[:3] + (vd,),
          "caches must be (pages, nkv, page_size, d) and (pages, nkv, page_size, vd)")
    _check(lib().gs_qknorm_rope_kv(_p(qkv), c_int(_dt(qkv)), _p(q_weight), _p(k_weight), c_float(eps), _p(cos),
                                   _p(sin), c_int(rotary_dim), c_int(1 if layout == "interleaved" else 0), c_int(max_pos),
                                   _p(positions), _p(seq_of_token),
                                   _p(block_table), c_int(block_table.shape[1]), c_int(page_size), _p(kcache),
                                   _p(vcache), c_int(T), c_int(nh), c_int(nkv), c_int(d),
                                   c_int(1 if write_kv else 0), c_int(vd), _p(vcos), _p(vsin), c_int(qkv.shape[1]),
                                   c_int(1 if plain_norm else 0), _p(v_first), c_int(ldf), _p(mix), _stream()))


def attention_generic(q, q_stride, kcache, vcache, positions, seq_of_token, block_table, page_size, window, scale,
                      nh, nkv, d, ntok, out: torch.Tensor = None, vd: int = None, chunk: int = None, sink: bool = False,
                      vcos=None, vsin=None, layout: str = "half", softcap: float = None, keep_first: int = 0,
                      sinks=None) -> torch.Tensor:
    """Causal GQA over the paged cache, any sizes; ``q`` rows are ``q_stride`` apart.  ``vd``: the width of a value
    head where it is not ``d``; ``chunk``: a query sees only the keys of its own run of ``chunk`` positions;
    ``sink``: one more term ``exp(0)`` in the softmax's denominator; ``vcos``, ``vsin``: the cached values are turned
    by their positions, and a head's sum is turned back by the query's (pairs laid out as ``layout`` says);
    ``softcap``: scores become ``softcap tanh(score / softcap)``; ``keep_first``: with a window, the sequence's first
    positions that stay visible beyond it; ``sinks (nh,)`` float32: the extra term is ``exp(sinks[h])``."""
    _dev(q, kcache, vcache, positions, seq_of_token, block_table, out, sinks)
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.shape == (nh,)), "attention: sinks must be float32 (nh,)")
    vd = d if vd is None else int(vd)
    _need(q.numel() >= (ntok - 1) * q_stride + nh * d if ntok else True, "attention: q is too small")
    _need(kcache.dtype == q.dtype and vcache.dtype == q.dtype, "cache and activations differ in type")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape[:3] + (vd,),
          "caches must be (pages, nkv, page_size, d) and (pages, nkv, page_size, vd)")
    _value_tables(vcos, vsin, vd)
    _need(layout in ROPE_LAYOUTS, f"attention: pairs are laid out 'half' or 'interleaved', not {layout!r}")
    _i32(positions, ntok, "positions")
    _i32(seq_of_token, ntok, "seq_of_token")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, nh * vd), dtype=q.dtype, device=q.device)
    _need(out.shape == (ntok, nh * vd) and out.dtype == q.dtype, "attention: out has the wrong shape or type")
    _check(lib().gs_attention_generic(_p(q), c_int(q_stride), _p(kcache), _p(vcache), c_int(_dt(q)), _p(positions),
                                      _p(seq_of_token), _p(block_table), c_int(block_table.shape[1]),
                                      c_int(page_size), c_int(window or 0), c_float(scale), _p(out), c_int(ntok),
                                      c_int(nh), c_int(nkv), c_int(d), c_int(vd), c_int(chunk or 0),
                                      c_int(1 if sink else 0), _p(vcos), _p(vsin),
                                      c_int(1 if layout == "interleaved" else 0), c_float(softcap or 0.0),
                                      c_int(keep_first or 0), _p(sinks), _stream()))
    return out


# ---------------------------------------------------------------------- linear attention

_ACTS = {None: 0, "none": 0, "silu": 1}
_GATES = {"sigmoid": 0, "silu": 1}
GATED_ACTS = {"silu": 0, "gelu_tanh": 1}
LINEAR_ATTENTION_MAX_KEY = 512
LINEAR_ATTENTION_CHUNKS_MAX_KEY = 128


def linear_attention_scan(x, oq: int, ok: int, ov: int, H: int, n: int, m: int, decay, state, q_start, slots, positions,
                          nseq: int, activation=None, cos=None, sin=None, rotary_dim: int = 0, key_scale: float = 1.0,
                          out: torch.Tensor = None, below: int = 0, chunks_from: int = 0, segment: int = 0,
                          longest: int = 0) -> torch.Tensor:
    """Linear attention through a fading state: per sequence and head ``S <- decay_h S + k_t v_t^T``, ``o_t = S^T q_t``.

    ``x (T, ld)`` holds q of head h at columns ``[oq + h n, ...)``, k at ``[ok + h n, ...)``, v at ``[ov + h m, ...)``;
    ``activation`` (None or ``"silu"``) is applied to all three, q and k are turned by ``positions`` over their first
    ``rotary_dim`` features (half-split pairs, tables ``(P, rotary_dim/2)``), k is multiplied by ``key_scale``.
    ``state (slots, H, n, m)`` float32 is read and advanced for the sequences' ``slots``.  Returns ``(T, H m)`` float32.

    ``below`` > 0: only the sequences that bring fewer tokens than that (the rows of the others are left as they are).
    ``chunks_from`` > 0: the kernel on the matrix cores instead (bfloat16 rows, keys up to
    ``LINEAR_ATTENTION_CHUNKS_MAX_KEY`` wide), for the sequences that bring at least that many tokens; with
    ``segment`` > 0 (a multiple of 32) those sequences are cut into segments of that many tokens, each a block of its
    own, in three launches (``longest``: the most tokens a sequence brings)."""
    _dev(x, decay, state, q_start, slots, positions, cos, sin, out)
    _need(x.dim() == 2, "linear_attention: rows (T, ld)")
    T, ld = x.shape
    _need(activation in _ACTS, f"linear_attention: activation is None or 'silu', not {activation!r}")
    _need(decay.dtype == torch.float32 and decay.shape == (H,), "linear_attention: decay must be float32 (H,)")
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.shape[1:] == (H, n, m),
          "linear_attention: state must be float32 (slots, H, n, m)")
    _need(n <= LINEAR_ATTENTION_MAX_KEY, f"linear_attention: keys of {n} features, the kernel holds up to {LINEAR_ATTENTION_MAX_KEY}")
    _i32(q_start, nseq + 1, "q_start")
    _i32(slots, nseq, "slots")
    _i32(positions, T, "positions")
    max_pos = 0
    if rotary_dim:
        _need(cos is not None and cos.dtype == torch.float32 and sin.dtype == torch.float32 and cos.shape == sin.shape
              and cos.dim() == 2 and cos.shape[1] == rotary_dim // 2, "linear_attention: tables must be float32 (P, rotary_dim/2)")
        max_pos = cos.shape[0]
    if out is None:
        out = torch.empty((T, H * m), dtype=torch.float32, device=x.device)
    _need(out.shape == (T, H * m) and out.dtype == torch.float32, "linear_attention: out must be float32 (T, H m)")
    if chunks_from > 0:
        _need(x.dtype == torch.bfloat16 and n <= LINEAR_ATTENTION_CHUNKS_MAX_KEY,
              "linear_attention: the kernel on the matrix cores takes bfloat16 rows and keys up to 128 wide")
        ws, maxseg = None, 0
        if segment > 0:
            _need(segment % 32 == 0 and longest > 0, "linear_attention: segments are whole runs of 32 tokens")
            maxseg = -(-longest // segment)
            ws = torch.empty(nseq * maxseg * H * n * m, dtype=torch.float32, device=x.device)
        _check(lib().gs_linear_attention_chunks(_p(x), c_int(ld), c_int(oq), c_int(ok), c_int(ov), c_int(_ACTS[activation]),
                                                _p(cos) if rotary_dim else None, _p(sin) if rotary_dim else None,
                                                c_int(rotary_dim), c_int(max_pos), c_float(key_scale), _p(decay), _p(state),
                                                _p(q_start), _p(slots), _p(positions), _p(out), c_int(nseq), c_int(H),
                                                c_int(n), c_int(m), c_int(chunks_from), _p(ws), c_int(maxseg),
                                                c_int(segment), _stream()))
        return out
    _check(lib().gs_linear_attention_scan(_p(x), c_int(_dt(x)), c_int(ld), c_int(oq), c_int(ok), c_int(ov),
                                          c_int(_ACTS[activation]), _p(cos) if rotary_dim else None,
                                          _p(sin) if rotary_dim else None, c_int(rotary_dim), c_int(max_pos),
                                          c_float(key_scale), _p(decay), _p(state), _p(q_start), _p(slots), _p(positions),
                                          _p(out), c_int(nseq), c_int(H), c_int(n), c_int(m), c_int(below), _stream()))
    return out


def gated_outnorm(o, gate_rows, og: int, weight, eps: float, H: int, m: int, joint: bool, gate: str, out_dtype) -> torch.Tensor:
    """``o (T, H m)`` float32 normed (``joint``: all heads as one row, times ``weight``; else each head by its own root
    mean square) and multiplied by ``sigmoid`` or ``silu`` of the gate, which stands in ``gate_rows (T, ldg)`` from
    column ``og`` on.  Returns ``(T, H m)`` in ``out_dtype``."""
    _dev(o, gate_rows, weight)
    T = o.shape[0]
    _need(o.dtype == torch.float32 and o.shape == (T, H * m), "gated_outnorm: o must be float32 (T, H m)")
    _need(gate_rows.dim() == 2 and gate_rows.shape[0] == T and gate_rows.dtype == out_dtype,
          "gated_outnorm: the gate's rows are (T, ldg) in the result's type")
    _need(weight is None or (weight.dtype == torch.float32 and weight.shape == (H * m,)), "gated_outnorm: weight must be float32 (H m,)")
    _need(gate in _GATES, f"gated_outnorm: the gate is 'sigmoid' or 'silu', not {gate!r}")
    out = torch.empty((T, H * m), dtype=out_dtype, device=o.device)
    _check(lib().gs_gated_outnorm(_p(o), _p(gate_rows), c_int(_dt(gate_rows)), c_int(gate_rows.shape[1]), c_int(og),
                                  _p(weight), c_float(eps), c_int(1 if joint else 0), c_int(_GATES[gate]), _p(out),
                                  c_int(_dt(out)), c_int(T), c_int(H), c_int(m), _stream()))
    return out


def add_rmsnorm_pair(res, d1, d2, w1, w2, eps: float, out_dtype, bias=None):
    """``res += d1 + d2 + bias`` (each where given; ``bias (H,)`` float32 is added to every row), then
    ``(rmsnorm(res) * w1, rmsnorm(res) * w2)``; ``w2`` None: one result."""
    _dev(res, d1, d2, w1, w2, bias)
    _need(res.dtype == torch.float32 and res.dim() == 2, "add_rmsnorm_pair: the residual stream is float32 (T, H)")
    T, H = res.shape
    for w in (w1, w2, bias):
        _need(w is None or (w.dtype == torch.float32 and w.shape == (H,)), "add_rmsnorm_pair: weights and bias must be float32 (H,)")
    _need(w1 is not None, "add_rmsnorm_pair: a first weight")
    ds = [d for d in (d1, d2) if d is not None]
    for d in ds:
        _need(d.shape == res.shape and d.dtype == ds[0].dtype, "add_rmsnorm_pair: deltas have the stream's shape and one type")
    out1 = torch.empty((T, H), dtype=out_dtype, device=res.device)
    out2 = torch.empty((T, H), dtype=out_dtype, device=res.device) if w2 is not None else None
    _check(lib().gs_add_rmsnorm_pair(_p(res), _p(ds[0]) if ds else None, _p(ds[1]) if len(ds) > 1 else None,
                                     c_int(_dt(ds[0]) if ds else _dt(out1)), _p(w1), _p(w2), c_float(eps), _p(out1),
                                     _p(out2), c_int(_dt(out1)), c_int(T), c_int(H), _p(bias), _stream()))
    return out1, out2


def scaled_sum(a, sa: float, b, sb: float, out_dtype) -> torch.Tensor:
    """``sa * a + sb * b`` in float32, rounded once to ``out_dtype``; ``a`` and ``b`` of one shape and type."""
    _dev(a, b)
    _need(a.shape == b.shape and a.dtype == b.dtype, "scaled_sum: operands of one shape and type")
    out = torch.empty(a.shape, dtype=out_dtype, device=a.device)
    _check(lib().gs_scaled_sum(_p(a), c_float(sa), _p(b), c_float(sb), c_int(_dt(a)), _p(out), c_int(_dt(out)),
                               c_long(a.numel()), _stream()))
    return out


def gated_act(x, bias, activation: str, out_dtype) -> torch.Tensor:
    """``x (T, 2F)`` = gate | up, ``bias (2F,)`` float32 or None -> ``act(gate + b) * (up + b) (T, F)`` in ``out_dtype``."""
    _dev(x, bias)
    _need(x.dim() == 2 and x.shape[1] % 2 == 0, "gated_act: rows hold gate and up side by side")
    T, F2 = x.shape
    F = F2 // 2
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (F2,)), "gated_act: bias must be float32 (2F,)")
    _need(activation in GATED_ACTS, f"gated_act: the activation is one of {sorted(GATED_ACTS)}, not {activation!r}")
    out = torch.empty((T, F), dtype=out_dtype, device=x.device)
    _check(lib().gs_gated_act(_p(x), c_int(_dt(x)), _p(bias), _p(out), c_int(_dt(out)), c_int(T), c_int(F),
                              c_int(GATED_ACTS[activation]), _stream()))
    return out


# ---------------------------------------------------------------------- matrix products

def gemm_tiled(x: torch.Tensor, w: torch.Tensor, bias=None, out_dtype=None, out: torch.Tensor = None) -> torch.Tensor:
    """``y = x @ w.T (+ bias)`` by float32 FMAs; any sizes, any mix of float32/bfloat16 storage."""
    _dev(w, bias, out)
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1, "gemm: x must be (M, K) with unit column stride")
    M, K = x.shape
    N = w.shape[0]
    if w.shape != (N, K):
        raise KernelError(f"gemm: weight is {tuple(w.shape)}, expected ({N}, {K})")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (N,)), "gemm: bias must be float32 (N,)")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or x.dtype, device=x.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "gemm: out has the wrong shape")
    ldx = x.stride(0) if M > 1 else K
    if (x.dtype == torch.float32 and w.dtype == torch.float32 and w.is_contiguous()
            and lib().gs_gemv_f32_supports(c_int(M), c_int(K), c_int(ldx), _p(x), _p(w))):
        # few rows: the weights are streamed once, each output summed in an order that depends on K alone
        _check(lib().gs_gemv_f32(_p(x), c_int(ldx), _p(w), _p(bias), _p(out), c_int(_dt(out)),
                                 c_int(out.stride(0) if M > 1 else N), c_int(M), c_int(N), c_int(K), _stream()))
        return out
    _check(lib().gs_gemm_tiled(_p(x), c_int(_dt(x)), c_int(x.stride(0) if M > 1 else K), _p(w), c_int(_dt(w)),
                               _p(bias), _p(out), c_int(_dt(out)), c_int(out.stride(0) if M > 1 else N), c_int(M),
                               c_int(N), c_int(K), _stream()))
    return out


def mfma_ok(x, w: torch.Tensor) -> bool:
    """Whether the matrix-core product for many rows takes these operands (bfloat16, K a multiple of 8, aligned)."""
    return (isinstance(x, torch.Tensor) and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2
            and x.shape[0] > 0 and x.shape[1] % 8 == 0 and x.stride(1) == 1
            and (x.shape[0] <= 1 or x.stride(0) % 8 == 0) and x.data_ptr() % 16 == 0 and w.is_contiguous()
            and w.data_ptr() % 16 == 0)


def gemm_mfma(x: torch.Tensor, w: torch.Tensor, out_dtype=None, out: torch.Tensor = None, swiglu: bool = False):
    """``x @ w.T`` for many rows on the matrix cores (bfloat16 in, float32 sums, bfloat16 or float32 out); with
    ``swiglu`` the weight holds gate rows then up rows and the result is ``silu(gate) * up``, half as wide."""
    _dev(w, out)
    _need(mfma_ok(x, w), "gemm_mfma: operands must be bfloat16, K a multiple of 8, 16-byte aligned")
    M, K = x.shape
    N = w.shape[0]
    if w.shape != (N, K):
        raise KernelError(f"gemm_mfma: weight is {tuple(w.shape)}, expected ({N}, {K})")
    _need(not swiglu or N % 2 == 0, "gemm_mfma: SwiGLU needs gate and up rows")
    cols = N // 2 if swiglu else N
    if out is None:
        out = torch.empty((M, cols), dtype=out_dtype or torch.bfloat16, device=w.device)
    _need(out.shape == (M, cols) and out.stride(1) == 1, "gemm_mfma: out has the wrong shape")
    _need(not swiglu or out.dtype == torch.bfloat16, "gemm_mfma: the SwiGLU epilogue stores bfloat16")
    _check(lib().gs_gemm_mfma(_p(x), c_int(x.stride(0) if M > 1 else K), _p(w), _p(out), c_int(_dt(out)),
                              c_int(out.stride(0) if M > 1 else cols), c_int(M), c_int(N), c_int(K),
                              c_int(1 if swiglu else 0), _stream()))
    return out


def library_gemm(x: torch.Tensor, w: torch.Tensor, workspace: torch.Tensor, out: torch.Tensor = None, tune: bool = True,
                 checked: bool = False):
    """``x @ w.T`` for many rows by the vendor's library, called directly (bfloat16 in and out, float32 sums).  The
    first call of a shape makes its plan, with ``tune`` by measuring the library's two dozen best guesses on these
    operands (a few milliseconds), else by taking its first choice.
    ``workspace``: device bytes the library's kernels may use.  Not to be recorded into a graph.
    ``checked``: the caller has asked :func:`library_gemm_ok` about ``x`` and ``w`` (and ``out`` is None or fits): the
    operands are not looked at again here (a step of prompt portions makes 64 such calls; the entry point still
    refuses misaligned or missing operands)."""
    bf = torch.bfloat16
    M, K = x.shape
    N = w.shape[0]
    if not checked:
        if not (x.is_cuda and x.dim() == 2 and x.dtype is bf and w.dtype is bf and x.stride(1) == 1 and w.is_cuda
                and w.is_contiguous() and workspace.is_cuda):
            raise KernelError("library_gemm: bfloat16 (M, K) rows and a contiguous bfloat16 weight on the GPU")
        if w.shape != (N, K):
            raise KernelError(f"library_gemm: weight is {tuple(w.shape)}, expected ({N}, {K})")
        if out is not None and not (out.is_cuda and out.shape == (M, N) and out.dtype is bf and out.stride(1) == 1):
            raise KernelError("library_gemm: out is bfloat16 (M, N) on the GPU")
    if out is None:
        out = torch.empty((M, N), dtype=bf, device=w.device)
    rc = lib().gs_library_gemm(x.data_ptr(), x.stride(0) if M > 1 else K, w.data_ptr(), out.data_ptr(),
                               out.stride(0) if M > 1 else N, M, N, K, workspace.data_ptr(),
                               workspace.numel() * workspace.element_size(), 1 if tune else 0, _stream())
    if rc != 0:
        _check(rc)
    return out


def library_gemm_ok(x, w: torch.Tensor) -> bool:
    """Whether :func:`library_gemm` takes these operands (bfloat16 on the GPU, a weight ``(N, K)`` for rows of K, K and
    the row stride multiples of 8, aligned)."""
    bf = torch.bfloat16
    if not (isinstance(x, torch.Tensor) and x.dtype is bf and w.dtype is bf and x.dim() == 2 and w.dim() == 2):
        return False
    M, K = x.shape
    return (M > 0 and K % 8 == 0 and w.shape[1] == K and w.shape[0] % 8 == 0 and x.stride(1) == 1
            and (M <= 1 or x.stride(0) % 8 == 0) and x.is_cuda and w.is_cuda and w.is_contiguous()
            and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def library_gemm_plan(M: int, N: int, K: int):
    """``(plans kept in all, candidates measured for this shape, the best one's microseconds)``."""
    cand, best = c_int(0), c_float(0.0)
    n = lib().gs_library_gemm_plans(c_int(M), c_int(N), c_int(K), ctypes.byref(cand), ctypes.byref(best))
    return n, cand.value, best.value


# ---------------------------------------------------------------------- sampling

def argmax_rows(logits: torch.Tensor):
    """``(ids int32 (rows,), bad int32 (rows,))``: first maximum per row; bad = a non-finite logit."""
    _dev(logits)
    _need(logits.dtype == torch.float32 and logits.dim() == 2, "argmax: logits are float32 (rows, V)")
    rows, V = logits.shape
    ids = torch.empty(rows, dtype=torch.int32, device=logits.device)
    bad = torch.empty(rows, dtype=torch.int32, device=logits.device)
    _check(lib().gs_argmax_rows(_p(logits), c_int(rows), c_int(V), _p(ids), _p(bad), _stream()))
    return ids, bad


def sample_temperature(logits: torch.Tensor, temperature: torch.Tensor, u: torch.Tensor):
    """One id per row from ``softmax(logits / temperature)`` by inverse CDF at ``u`` (float64 each)."""
    return choose_rows(logits, temperature, torch.ones_like(temperature), u)


def sample_top_p(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, u: torch.Tensor):
    """Nucleus sampling: one id per row from the shortest descending-weight prefix whose mass reaches ``top_p``."""
    return choose_rows(logits, temperature, top_p, u)


def choose_rows(logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, u: torch.Tensor):
    """One id per row, each row in its own manner: ``temperature <= 0`` greedy, else a draw at ``u`` from the whole row
    or (``top_p < 1``) from its nucleus; float64 ``(rows,)`` each.  ``(ids, bad)`` int32 as :func:`argmax_rows`.  The
    weights are made by many blocks a row (the kernels of the decode loop's choice)."""
    _dev(logits, temperature, top_p, u)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "choose: logits are float32 (rows, V)")
    rows, V = logits.shape
    for name, t in (("temperature", temperature), ("top_p", top_p), ("u", u)):
        _need(t.dtype == torch.float64 and t.numel() == rows, f"choose: {name} is float64 (rows,)")
    dev = logits.device
    zeros = torch.zeros((5, rows), dtype=torch.int32, device=dev)      # counter, next id, position, key count, live
    out = torch.empty((2, 1, rows), dtype=torch.int32, device=dev)
    nucleus = bool((top_p < 1).any())
    wide = (torch.empty(rows * choice_parts(V), dtype=torch.float64, device=dev), torch.empty(rows, dtype=torch.int32, device=dev),
            torch.empty(rows, dtype=torch.int32, device=dev), torch.empty(rows * choice_hist(), dtype=torch.int64, device=dev))
    decode_choose(logits, temperature, u.reshape(1, rows), zeros[0], zeros[1], out[0], out[1], zeros[2], zeros[3], zeros[4],
                  wide, top_p=top_p if nucleus else None,
                  wbuf=torch.empty(rows * V, dtype=torch.float64, device=dev) if nucleus else None)
    return out[0, 0], out[1, 0]


# ---------------------------------------------------------------------- decoding

SKINNY_MAX_ROWS = 64


def skinny_ok(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether the weight-streaming kernel takes this product (few rows, bfloat16, aligned rows)."""
    if isinstance(x, TiledRows):
        return (w.dtype == torch.bfloat16 and x.shape[0] <= SKINNY_MAX_ROWS and w.is_contiguous()
                and w.data_ptr() % 16 == 0)
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and x.shape[0] <= SKINNY_MAX_ROWS
            and x.shape[1] % 8 == 0 and x.stride(1) == 1 and (x.shape[0] <= 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0 and w.is_contiguous() and w.data_ptr() % 16 == 0)


class LazyNorm:
    """An RMSNorm not yet applied: the float32 stream, its rows' sums of squares as partial sums, weight and eps.

    The weight-streaming products take it in place of a tensor and norm on the fly; ``materialize``
    runs a light norm kernel for everything else.  ``xs``, when given, holds ``res * weight`` in bfloat16,
    written by whatever last added to the stream: then a product reads ``xs`` and multiplies its result by the
    row's inverse root mean square, and the norm costs nothing of its own.
    """

    __slots__ = ("res", "ssq", "weight", "eps", "dtype", "xs", "ready")

    def __init__(self, res, ssq, weight, eps, dtype, xs=None, ready=None):
        self.res, self.ssq, self.weight, self.eps, self.dtype, self.xs = res, ssq, weight, eps, dtype, xs
        self.ready = ready            # the normed rows themselves, where whatever wrote the stream last made them

    @property
    def shape(self):
        return self.res.shape

    def materialize(self) -> torch.Tensor:
        """The normed rows as a tensor; the sums of squares are at hand, so one light pass does it."""
        if self.ready is not None:
            return self.ready
        T, H = self.res.shape
        out = torch.empty((T, H), dtype=self.dtype, device=self.res.device)
        _check(lib().gs_norm_from_ssq(_p(self.res), _p(self.ssq), c_int(self.ssq.shape[1]), _p(self.weight),
                                      c_float(self.eps), _p(out), c_int(_dt(out)), c_int(T), c_int(H), _stream()))
        return out


def lazy_ok(x, w: torch.Tensor) -> bool:
    return (isinstance(x, LazyNorm) and x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16
            and x.res.shape[0] <= SKINNY_MAX_ROWS and x.res.shape[1] % 8 == 0 and x.res.is_contiguous()
            and w.is_contiguous() and w.data_ptr() % 16 == 0 and x.res.data_ptr() % 16 == 0)


def _lazy_args(x):
    if isinstance(x, LazyNorm):
        if x.xs is not None:
            return _x_args(x.xs) + (None, _p(x.ssq), c_int(x.ssq.shape[1]), None, c_float(x.eps))
        return (None, c_int(x.res.shape[1]), c_int(0), _p(x.res), _p(x.ssq), c_int(x.ssq.shape[1]), _p(x.weight),
                c_float(x.eps))
    return _x_args(x) + (None, None, c_int(0), None, c_float(0.0))


def _x_args(x):
    """Pointer, row stride and layout flag of a product's rows."""
    M, K = x.shape
    if isinstance(x, TiledRows):
        return (_p(x.buf), c_int(K), c_int(1))
    return (_p(x), c_int(x.stride(0) if M > 1 else K), c_int(0))


def tile_major(w: torch.Tensor) -> torch.Tensor:
    """The tile-major copy of a bfloat16 weight ``(N, K)``, N a multiple of 16 and K of 32, that the
    weight-streaming kernels read fastest: each 16 x 32 tile as 64 lanes x 16 bytes, in the MFMA operand's order."""
    _dev(w)
    N, K = w.shape
    _need(w.dtype == torch.bfloat16 and N % 16 == 0 and K % 32 == 0, "tile_major: bfloat16 (N, K), N % 16 == 0, K % 32 == 0")
    out = torch.empty_like(w)
    _check(lib().gs_tile_major(_p(w), _p(out), c_int(N), c_int(K), _stream()))
    return out


def gemm_skinny(x, w: torch.Tensor, out_dtype=None, out=None, swiglu: bool = False, wt=None):
    """``x @ w.T`` for at most 64 rows, streaming the weights once; optionally ``silu(gate) * up`` of the result.

    ``x`` is a bfloat16 tensor, :class:`TiledRows` or a :class:`LazyNorm`.  With ``swiglu`` the weight holds gate
    rows then up rows and the output is half as wide, and ``out`` may be True or a :class:`TiledRows` for tiled rows.
    """
    _dev(w, out if isinstance(out, torch.Tensor) else None)
    lazy = isinstance(x, LazyNorm)
    _need(lazy_ok(x, w) if lazy else skinny_ok(x, w),
          "gemm_skinny: operands must be bfloat16, at most 64 rows, K a multiple of 8, aligned")
    M, K = x.shape
    N = w.shape[0]
    if w.shape != (N, K):
        raise KernelError(f"gemm_skinny: weight is {tuple(w.shape)}, expected ({N}, {K})")
    cols = N // 2 if swiglu else N
    out, buf, tiled = _rows_out(out, M, cols, w.device, out_dtype or torch.bfloat16)
    _need(not tiled or swiglu, "gemm_skinny: only the SwiGLU epilogue writes tiled rows")
    _need(tiled or (out.shape == (M, cols) and out.stride(1) == 1), "gemm_skinny: out has the wrong shape")
    _check(lib().gs_gemm_skinny(*_lazy_args(x), _p(w), _p(wt), _p(buf), c_int(_dt(out)),
                                c_int(cols if tiled or M <= 1 else out.stride(0)), c_int(M), c_int(N), c_int(K),
                                c_int(1 if swiglu else 0), c_int(tiled), _stream()))
    return out


def gemm_skinny_residual(x: torch.Tensor, w: torch.Tensor, res: torch.Tensor, wt=None, next_weight=None,
                         xs: torch.Tensor = None) -> torch.Tensor:
    """``res += x @ w.T`` in place (float32); returns the new rows' sums of squares as partial sums ``(M, nb)``.
    With ``next_weight (N,)`` and ``xs (M, N)`` bfloat16 also ``xs = res * next_weight``."""
    _dev(w, res, next_weight, None if isinstance(xs, TiledRows) else xs)
    _need(skinny_ok(x, w), "gemm_skinny_residual: operands must be bfloat16, at most 64 rows, K a multiple of 8, aligned")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape == (N, K) and res.shape == (M, N) and res.dtype == torch.float32, "gemm_skinny_residual: shapes")
    nb = lib().gs_gemm_skinny_residual_blocks(c_int(N), c_int(0 if wt is None else 1))
    ssq = torch.empty((M, nb), dtype=torch.float32, device=res.device)
    _need((next_weight is None) == (xs is None), "gemm_skinny_residual: next_weight and xs come together")
    xs_buf, xs_tiled = xs, 0
    if xs is not None:
        if isinstance(xs, TiledRows):
            xs_buf, xs_tiled = xs.buf, 1
        _need(next_weight.dtype == torch.float32 and next_weight.shape == (N,) and xs.dtype == torch.bfloat16
              and tuple(xs.shape) == (M, N) and xs_buf.is_contiguous(), "gemm_skinny_residual: next_weight float32 (N,), xs bfloat16 (M, N)")
    _check(lib().gs_gemm_skinny_residual(*_x_args(x), _p(w), _p(wt), _p(res), _p(ssq), _p(next_weight), _p(xs_buf),
                                         c_int(xs_tiled), c_int(M), c_int(N), c_int(K), _stream()))
    return ssq


def gemm_skinny_residual_parts(x, w: torch.Tensor, res: torch.Tensor, parts: int, wt=None,
                               next_weight=None, eps: float = 0.0, out_dtype=None, tiled: bool = False):
    """``res += x @ w.T`` for up to 64 rows in two kernels: partial sums over ``parts`` parts of K from many blocks,
    then one pass that adds them to the stream.  Returns ``(ssq (M, 1), normed)``: the new rows' sums of squares and,
    with ``next_weight``, the rows normed with that weight and ``eps`` (else None; as :class:`TiledRows` with ``tiled``)."""
    _dev(w, res, next_weight)
    _need(skinny_ok(x, w), "gemm_skinny_residual_parts: operands must be bfloat16, at most 64 rows, K a multiple of 8, aligned")
    M, K = x.shape
    N = w.shape[0]
    _need(w.shape == (N, K) and res.shape == (M, N) and res.dtype == torch.float32 and res.is_contiguous(),
          "gemm_skinny_residual_parts: shapes")
    _need(1 <= parts <= 64, "gemm_skinny_residual_parts: 1 to 64 parts")
    part = torch.empty((parts, M, N), dtype=torch.float32, device=res.device)
    _check(lib().gs_gemm_skinny_parts(*_x_args(x), _p(w), _p(wt), _p(part), c_int(parts), c_int(M), c_int(N), c_int(K),
                                      _stream()))
    ssq = torch.empty((M, 1), dtype=torch.float32, device=res.device)
    normed = None
    if next_weight is not None:
        _need(next_weight.dtype == torch.float32 and next_weight.shape == (N,), "next_weight must be float32 (N,)")
        normed, nbuf, ntiled = _rows_out(bool(tiled), M, N, res.device, out_dtype or torch.bfloat16)
    else:
        nbuf, ntiled = None, 0
    _check(lib().gs_residual_from_parts(_p(part), c_int(parts), _p(res), _p(ssq), _p(next_weight), c_float(eps),
                                        _p(nbuf), c_int(_dt(normed) if normed is not None else 1), c_int(ntiled),
                                        c_int(M), c_int(N), _stream()))
    return ssq, normed


def gemm_skinny_conv(x, w_in, taps, bias, state, slots, wt=None, tiled: bool = False):
    """A decode step's gated short convolution fused into its input product; ``state`` is advanced.
    With ``tiled`` the mixed rows come as :class:`TiledRows`."""
    _dev(w_in, taps, bias, state, slots)
    _need(lazy_ok(x, w_in) if isinstance(x, LazyNorm) else skinny_ok(x, w_in),
          "gemm_skinny_conv: needs bfloat16 rows or a lazy norm, and a bfloat16 weight")
    M, K = x.shape
    H, W = taps.shape
    _need(w_in.shape == (3 * H, K), "gemm_skinny_conv: the input weight must be (3H, K)")
    _need(taps.dtype == torch.float32 and state.dtype == torch.float32 and state.shape[1:] == (H, W - 1),
          "gemm_skinny_conv: taps float32 (H, W), state float32 (slots, H, W-1)")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (H,)), "gemm_skinny_conv: bias float32 (H,)")
    _i32(slots, M, "slots")
    out, buf, otiled = _rows_out(bool(tiled), M, H, w_in.device)
    _check(lib().gs_gemm_skinny_conv(*_lazy_args(x), _p(w_in), _p(wt), _p(taps), _p(bias), _p(state), _p(slots), c_int(W),
                                     _p(buf), c_int(otiled), c_int(M), c_int(H), c_int(K), _stream()))
    return out


def choice_parts(V: int) -> int:
    """Partial sums a row of ``V`` logits has in the many-block form of the decode loop's choice."""
    return int(lib().gs_choice_parts(c_int(V)))


def choice_hist() -> int:
    """64-bit sums a row has in the ready-made histograms of the many-block choice."""
    return int(lib().gs_choice_hist())


def _choice_rows(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live):
    _dev(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live)
    _need(logits.dtype == torch.float32 and logits.dim() == 2 and logits.is_contiguous(), "decode_choose: logits are float32 (rows, V)")
    rows, V = logits.shape
    for t in (counter, next_ids, positions, kv_len, live):
        _i32(t, rows)
    for t in (ring, bad_ring):
        _i32(t)
    _need(ring.dim() == 2 and ring.shape[1] == rows and bad_ring.shape == ring.shape, "decode_choose: rings are (steps, rows)")
    return rows, V


def decode_choose_greedy(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live) -> None:
    """The decode loop's choice while every row is greedy, one kernel: per row the first maximum into the loop's buffers
    (``ring[counter[row], row]``, the flag of a non-finite row beside it, the id fed back); then the row's counter counts
    up and a live row moves one position on.  A counter at or beyond the rings' step count writes into their last row
    and marks the step bad."""
    rows, V = _choice_rows(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live)
    _check(lib().gs_decode_choose(_p(logits), c_int(rows), c_int(V), _p(counter), _p(next_ids), _p(ring), _p(bad_ring),
                                  _p(positions), _p(kv_len), _p(live), c_int(ring.shape[0]), _stream()))


def decode_choose(logits, temperature, u, counter, next_ids, ring, bad_ring, positions, kv_len, live, wide, top_p=None,
                  wbuf=None) -> None:
    """The decode loop's choice when rows draw, three kernels (the rows' weights by many blocks: one block weighs a row
    of 65,536 logits in some 40 us).  Per row: greedy (temperature <= 0) or a draw with ``u[counter[row], row]``, from
    the whole row or, where ``top_p[row] < 1``, from its nucleus (``wbuf``: float64 scratch of at least ``rows * V``);
    results and the rows' advance as in :func:`decode_choose_greedy`.

    ``wide``: ``(part, amax, bad0, hist)``, float64 ``rows * choice_parts(V)``, int32 ``rows`` twice and int64
    ``rows * choice_hist()``: scratch."""
    rows, V = _choice_rows(logits, counter, next_ids, ring, bad_ring, positions, kv_len, live)
    _dev(temperature, u, top_p, wbuf)
    _need(temperature.dtype == torch.float64 and temperature.numel() == rows, "decode_choose: temperature float64 (rows,)")
    _need(u.dtype == torch.float64 and u.shape == ring.shape, "decode_choose: u is float64 (steps, rows)")
    _need((top_p is None) == (wbuf is None), "decode_choose: top_p and its scratch come together")
    if top_p is not None:
        _need(top_p.dtype == torch.float64 and top_p.numel() == rows, "decode_choose: top_p float64 (rows,)")
        _need(wbuf.dtype == torch.float64 and wbuf.numel() >= rows * V, "decode_choose: wbuf float64, rows * V at least")
    part, amax, bad0, hist = wide
    _dev(part, amax, bad0, hist)
    _need(part.dtype == torch.float64 and part.numel() >= rows * choice_parts(V), "decode_choose: part float64, rows * choice_parts(V) at least")
    _need(hist.dtype == torch.int64 and hist.numel() >= rows * choice_hist(), "decode_choose: hist int64, rows * choice_hist() at least")
    _i32(amax, rows)
    _i32(bad0, rows)
    _check(lib().gs_decode_choose_wide(_p(logits), c_int(rows), c_int(V), _p(temperature), _p(top_p), _p(wbuf), _p(part),
                                       _p(amax), _p(bad0), _p(hist), _p(u), _p(counter), _p(next_ids), _p(ring), _p(bad_ring),
                                       _p(positions), _p(kv_len), _p(live), c_int(u.shape[0]), _stream()))


def attention_decode_supports(nh: int, nkv: int, d: int) -> bool:
    return bool(lib().gs_attention_decode_supports(c_int(nh), c_int(nkv), c_int(d)))


_decode_ws = {}


def _decode_workspace(device, nseq, nh, nkv, d, nsplit):
    key = (device, nseq, nh, nkv, d, nsplit)
    ws = _decode_ws.get(key)
    if ws is None:
        n = lib().gs_attention_decode_workspace
        n.restype = c_long
        floats = n(c_int(nseq), c_int(nh), c_int(nkv), c_int(d), c_int(nsplit))
        ws = _decode_ws[key] = torch.empty(max(1, floats), dtype=torch.float32, device=device)
    return ws


def attention_decode(q, q_stride, kcache, vcache, positions, block_table, page_size, window, scale, nh, nkv, d, nseq,
                     nsplit: int, out=None, chunk: int = None, sink: bool = False, softcap: float = None,
                     keep_first: int = 0, sinks=None):
    """One query per sequence over its paged keys (bfloat16), keys split over ``nsplit`` blocks per key head.
    ``out``: a tensor, or True / a :class:`TiledRows` for tiled rows.  ``chunk``: the query sees only the keys of its
    own run of ``chunk`` positions; ``sink``: one more term ``exp(0)`` in the softmax's denominator; ``softcap``: scores
    become ``softcap tanh(score / softcap)``; ``keep_first``: with a window, the sequence's first positions that stay
    visible beyond it; ``sinks (nh,)`` float32: the extra term is ``exp(sinks[h])``."""
    _dev(q, kcache, vcache, positions, block_table, out if isinstance(out, torch.Tensor) else None, sinks)
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.shape == (nh,)), "attention_decode: sinks must be float32 (nh,)")
    _need(q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_decode takes bfloat16")
    _need(q.numel() >= (nseq - 1) * q_stride + nh * d if nseq else True, "attention_decode: q is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, nseq, "positions")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= nseq,
          "block_table must be int32 (nseq, max_blocks)")
    ws = _decode_workspace(q.device, nseq, nh, nkv, d, nsplit)
    out, buf, tiled = _rows_out(out, nseq, nh * d, q.device, q.dtype)
    _need(tuple(out.shape) == (nseq, nh * d) and out.dtype == q.dtype, "attention_decode: out has the wrong shape or type")
    if softcap or keep_first or sinks is not None:
        _check(lib().gs_attention_decode_rules(_p(q), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(block_table),
                                               c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0),
                                               c_float(scale), _p(buf), c_int(tiled), _p(ws), c_int(nseq), c_int(nh),
                                               c_int(nkv), c_int(d), c_int(nsplit), c_int(chunk or 0),
                                               c_int(1 if sink else 0), c_float(softcap or 0.0), c_int(keep_first or 0),
                                               _p(sinks), _stream()))
        return out
    if chunk or sink:
        _check(lib().gs_attention_decode_runs(_p(q), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(block_table),
                                              c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0),
                                              c_float(scale), _p(buf), c_int(tiled), _p(ws), c_int(nseq), c_int(nh),
                                              c_int(nkv), c_int(d), c_int(nsplit), c_int(chunk or 0),
                                              c_int(1 if sink else 0), _stream()))
        return out
    _check(lib().gs_attention_decode(_p(q), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(block_table),
                                     c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0), c_float(scale),
                                     _p(buf), c_int(tiled), _p(ws), c_int(nseq), c_int(nh), c_int(nkv), c_int(d),
                                     c_int(nsplit), _stream()))
    return out


def attention_decode_raw_supports(nh: int, nkv: int, d: int, rotary_dim: int) -> bool:
    return bool(lib().gs_attention_decode_raw_supports(c_int(nh), c_int(nkv), c_int(d), c_int(rotary_dim)))


def attention_decode_raw(qkv, q_stride, kcache, vcache, positions, block_table, page_size, window, scale, q_weight,
                         k_weight, head_eps, cos, sin, nh, nkv, d, nseq, nsplit: int, write_kv: bool = True,
                         out=None):
    """Decode attention straight from the rows of q|k|v as their product left them: the kernel norms and rotates
    the queries and the new key, writes the new key and value into their pages, and attends."""
    _dev(qkv, kcache, vcache, positions, block_table, q_weight, k_weight, cos, sin,
         out if isinstance(out, torch.Tensor) else None)
    _need(qkv.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_decode_raw takes bfloat16")
    _need(qkv.numel() >= (nseq - 1) * q_stride + (nh + 2 * nkv) * d if nseq else True, "attention_decode_raw: qkv is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    for w in (q_weight, k_weight):
        _need(w is None or (w.dtype == torch.float32 and w.shape == (d,)), "head norm weight float32 (d,)")
    _need(cos.dtype == torch.float32 and cos.shape == sin.shape and cos.dim() == 2 and cos.shape[1] == d // 2
          and cos.is_contiguous() and sin.is_contiguous(), "rotation tables (positions, d/2) float32")
    _i32(positions, nseq, "positions")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.shape[0] >= nseq,
          "block_table must be int32 (nseq, max_blocks)")
    ws = _decode_workspace(qkv.device, nseq, nh, nkv, d, nsplit)
    out, buf, tiled = _rows_out(out, nseq, nh * d, qkv.device, qkv.dtype)
    _need(tuple(out.shape) == (nseq, nh * d) and out.dtype == qkv.dtype, "attention_decode_raw: out has the wrong shape or type")
    _check(lib().gs_attention_decode_raw(_p(qkv), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(block_table),
                                         c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0),
                                         c_float(scale), _p(q_weight), _p(k_weight), c_float(head_eps), _p(cos), _p(sin),
                                         c_int(d), c_int(1 if write_kv else 0), _p(buf), c_int(tiled), _p(ws), c_int(nseq),
                                         c_int(nh), c_int(nkv), c_int(d), c_int(nsplit), _stream()))
    return out


def attention_prefill_supports(nh: int, nkv: int, d: int) -> bool:
    return bool(lib().gs_attention_prefill_supports(c_int(nh), c_int(nkv), c_int(d)))


def turn_heads(x, cos, sin, positions, nh: int, w: int, sign: float = 1.0, layout: str = "half") -> torch.Tensor:
    """``x (T, nh w)`` in place: every head turned over its whole width by its token's position (``sign`` < 0:
    backwards); tables ``(P, w/2)``."""
    _dev(x, cos, sin, positions)
    T = x.shape[0]
    _need(x.dim() == 2 and x.shape[1] == nh * w, "turn_heads: rows (T, nh w)")
    _value_tables(cos, sin, w)
    _need(cos is not None, "turn_heads: no tables")
    _need(layout in ROPE_LAYOUTS, f"turn_heads: pairs are laid out 'half' or 'interleaved', not {layout!r}")
    _i32(positions, T, "positions")
    _check(lib().gs_turn_heads(_p(x), c_int(_dt(x)), _p(cos), _p(sin), c_int(cos.shape[0]), _p(positions),
                               c_int(1 if layout == "interleaved" else 0), c_float(sign), c_int(T), c_int(nh), c_int(w),
                               _stream()))
    return x


def attention_prefill(q, q_stride, kcache, vcache, positions, tiles, block_table, page_size, window, scale, nh, nkv, d,
                      ntok, out: torch.Tensor = None, tile_rows: int = 16, chunk: int = None, sink: bool = False,
                      softcap: float = None, keep_first: int = 0, sinks=None) -> torch.Tensor:
    """Causal GQA of many queries per sequence on the matrix cores (bfloat16).  ``chunk``: a query sees only the keys
    of its own run of ``chunk`` positions; ``sink``: one more term ``exp(0)`` in the softmax's denominator;
    ``softcap``: scores become ``softcap tanh(score / softcap)``; ``keep_first``: with a window, the sequence's first
    positions that stay visible beyond it; ``sinks (nh,)`` float32: the extra term is ``exp(sinks[h])``.

    ``tiles``: int32 ``(3, ntiles)``: sequence, first row and number of rows (at most ``tile_rows``, 16 or
    32) of each tile of consecutive queries of one sequence.
    """
    _dev(q, kcache, vcache, positions, tiles, block_table, out, sinks)
    _need(sinks is None or (sinks.dtype == torch.float32 and sinks.shape == (nh,)), "attention_prefill: sinks must be float32 (nh,)")
    _need(q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_prefill takes bfloat16")
    _need(q.numel() >= (ntok - 1) * q_stride + nh * d if ntok else True, "attention_prefill: q is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, ntok, "positions")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[0] == 3, "tiles must be int32 (3, ntiles)")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, nh * d), dtype=q.dtype, device=q.device)
    _need(out.shape == (ntok, nh * d) and out.dtype == q.dtype, "attention_prefill: out has the wrong shape or type")
    nt = tiles.shape[1]
    _check(lib().gs_attention_prefill(_p(q), c_int(q_stride), _p(kcache), _p(vcache), _p(positions), _p(tiles[0]),
                                      _p(tiles[1]), _p(tiles[2]), c_int(nt), _p(block_table),
                                      c_int(block_table.shape[1]), c_int(page_size), c_int(window or 0), c_float(scale),
                                      _p(out), c_int(nh), c_int(nkv), c_int(d), c_int(tile_rows), c_int(chunk or 0),
                                      c_int(1 if sink else 0), c_float(softcap or 0.0), c_int(keep_first or 0), _p(sinks),
                                      _stream()))
    return out


def attention_prefill_wide_supports(nh: int, nkv: int, d: int) -> bool:
    return bool(lib().gs_attention_prefill_wide_supports(c_int(nh), c_int(nkv), c_int(d)))


def attention_prefill_wide_rows(nh: int, nkv: int) -> int:
    """The most queries a block of :func:`attention_prefill_wide` holds for these head counts when it walks the keys
    whole (half as many with the keys in two halves)."""
    return int(lib().gs_attention_prefill_wide_rows(c_int(nh), c_int(nkv)))


def attention_prefill_wide(q, q_stride, kcache, vcache, positions, tiles, block_table, page_size, window, scale, nh, nkv,
                           d, ntok, out: torch.Tensor = None, key_splits: int = 1) -> torch.Tensor:
    """Causal GQA of long prompt portions (bfloat16, heads of 64): 32 queries a wavefront, keys and values shared by a
    block through LDS.  ``tiles``: int32 ``(3, blocks * wq)``, the sequence, first row and row count (at most 32; 0: none)
    of every sub-tile, ``wq = attention_prefill_wide_rows(nh, nkv) // 32 // key_splits`` of them a block, all of
    one sequence, neighbours or not (``BatchContext.query_subtiles`` pairs late ones with early ones).  With
    ``key_splits = 2`` (groups of up to four heads) a block holds half as many queries and two wavefronts walk half
    of the keys each: twice the blocks, half the longest walk."""
    _dev(q, kcache, vcache, positions, tiles, block_table, out)
    _need(q.dtype == torch.bfloat16 and kcache.dtype == torch.bfloat16 and vcache.dtype == torch.bfloat16,
          "attention_prefill_wide takes bfloat16")
    _need(q.numel() >= (ntok - 1) * q_stride + nh * d if ntok else True, "attention_prefill_wide: q is too small")
    _need(kcache.dim() == 4 and kcache.shape[1:] == (nkv, page_size, d) and vcache.shape == kcache.shape,
          "cache must be (pages, nkv, page_size, d)")
    _i32(positions, ntok, "positions")
    _need(key_splits in (1, 2) and (key_splits == 1 or attention_prefill_wide_rows(nh, nkv) >= 64),
          "attention_prefill_wide: the keys in two halves only for groups of up to four heads")
    rows = attention_prefill_wide_rows(nh, nkv) // key_splits
    wq = rows // 32
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[0] == 3 and wq > 0 and tiles.shape[1] % wq == 0,
          "tiles must be int32 (3, blocks * sub-tiles a block)")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, nh * d), dtype=q.dtype, device=q.device)
    _need(out.shape == (ntok, nh * d) and out.dtype == q.dtype, "attention_prefill_wide: out has the wrong shape or type")
    nt = tiles.shape[1] // wq
    _check(lib().gs_attention_prefill_wide(_p(q), q_stride, _p(kcache), _p(vcache), _p(positions), _p(tiles[0]),
                                           _p(tiles[1]), _p(tiles[2]), nt, _p(block_table),
                                           block_table.shape[1], page_size, kcache.shape[0],
                                           window or 0, scale, _p(out), nh, nkv, d, rows, key_splits, _stream()))
    return out


# ---------------------------------------------------------------------- blocks with their norm on the output

def norm_scaled_add(res: torch.Tensor, y, weight, eps: float, mult: float, rows_dtype=None) -> torch.Tensor:
    """``res += mult * rmsnorm(y) * weight`` row by row (``y = None``: nothing is added); returns the stream's new rows
    in ``rows_dtype`` (what the next sub-layer's products read), or None when no type is given."""
    _dev(res, y, weight)
    _need(res.dtype == torch.float32 and res.dim() == 2, "norm_scaled_add: the residual stream is float32 (T, H)")
    T, H = res.shape
    _need(y is None or (y.shape == res.shape and weight is not None and weight.dtype == torch.float32
                        and weight.shape == (H,)), "norm_scaled_add: y has the stream's shape, weight is float32 (H,)")
    rows = None if rows_dtype is None else torch.empty((T, H), dtype=rows_dtype, device=res.device)
    _check(lib().gs_norm_scaled_add(_p(res), _p(y), _dt(y) if y is not None else _dt(rows), _p(weight), float(eps),
                                    float(mult), _p(rows), _dt(rows) if rows is not None else _dt(y), T, H, _stream()))
    return rows


# ---------------------------------------------------------------------- attention through a cached latent row

def latent_prep(down, q_off, q_rank, kv_off, c, r, q_weight, kv_weight, eps, cos, sin, positions, seq_of_token,
                block_table, page_size, cache, write_kv: bool = True) -> torch.Tensor:
    """Per token of ``down (T, ld)``: the columns ``[q_off, q_off + q_rank)`` RMS-normed with ``q_weight`` are
    returned as ``(T, q_rank)``; the columns ``[kv_off, kv_off + c)`` RMS-normed with ``kv_weight`` and the ``r``
    columns behind them, rotated by the token's position, are written into the token's cache row ``[c | r]``.
    ``cache (pages, 1, page_size, c + r)``."""
    _dev(down, q_weight, kv_weight, positions, seq_of_token, block_table, cache)
    T, ld = down.shape
    _need(cache.dtype == down.dtype and cache.dim() == 4 and cache.shape[1:] == (1, page_size, c + r),
          "latent_prep: the cache is (pages, 1, page_size, c + r) in the activations' type")
    _need(q_weight.dtype == torch.float32 and q_weight.shape == (q_rank,) and kv_weight.dtype == torch.float32
          and kv_weight.shape == (c,), "latent_prep: norm weights are float32 (q_rank,), (c,)")
    if r:
        _dev(cos, sin)
        _need(cos.dtype == torch.float32 and sin.shape == cos.shape and cos.dim() == 2 and cos.shape[1] == r // 2,
              "latent_prep: cos and sin are float32 (positions, r / 2)")
    _i32(positions, T, "positions")
    _i32(seq_of_token, T, "seq_of_token")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    a = torch.empty((T, q_rank), dtype=down.dtype, device=down.device)
    _check(lib().gs_latent_prep(_p(down), _dt(down), ld, q_off, q_rank, kv_off, c, r, _p(q_weight), _p(kv_weight),
                                float(eps), _p(cos) if r else None, _p(sin) if r else None, _p(positions),
                                _p(seq_of_token), _p(block_table), block_table.shape[1], page_size, _p(cache), _p(a),
                                1 if write_kv else 0, T, _stream()))
    return a


def latent_q_rot(q, H, n, r, c, cos, sin, positions, qa) -> None:
    """The last ``r`` features of every head of ``q (T, H (n + r))``, rotated by the token's position, into
    ``qa (T, H (c + r))`` behind each head's first ``c`` columns."""
    _dev(q, positions, qa)
    T = q.shape[0]
    _need(q.shape == (T, H * (n + r)) and qa.shape == (T, H * (c + r)) and qa.dtype == q.dtype,
          "latent_q_rot: q is (T, H (n + r)), qa (T, H (c + r)) of one type")
    _i32(positions, T, "positions")
    if r == 0:
        return
    _dev(cos, sin)
    _need(cos.dtype == torch.float32 and sin.shape == cos.shape and cos.dim() == 2 and cos.shape[1] == r // 2,
          "latent_q_rot: cos and sin are float32 (positions, r / 2)")
    _check(lib().gs_latent_q_rot(_p(q), _dt(q), q.stride(0), H, n, r, c, _p(cos), _p(sin), _p(positions), _p(qa), T,
                                 _stream()))


def heads_product(x, hx: int, w, y, hy: int, K: int, gate=None, gate_each: bool = False) -> torch.Tensor:
    """``y[t, h hy : h hy + N] = w[h] @ x[t, h hx : h hx + K]`` for every head ``h`` of ``w (H, N, K)``, float32 sums in
    a fixed order; with ``gate (T, >= H)`` the result of head ``h`` is multiplied by ``sigmoid(gate[t, h])``, with
    ``gate_each`` and ``gate (T, >= H N)`` output ``n`` of head ``h`` by ``sigmoid(gate[t, h N + n])``."""
    _need(x.is_cuda and y.is_cuda and w.is_cuda and w.is_contiguous() and x.dim() == 2 and y.dim() == 2
          and x.stride(1) == 1 and y.stride(1) == 1, "heads_product: rows with unit column stride, on the GPU")
    H, N, Kw = w.shape
    _need(Kw == K and x.shape[0] == y.shape[0] and y.dtype == x.dtype, "heads_product: shapes or types differ")
    M = x.shape[0]
    ldg = 0
    if gate is not None:
        _need(gate.is_cuda and gate.dim() == 2 and gate.stride(1) == 1 and gate.shape[0] == M
              and gate.shape[1] >= (H * N if gate_each else H) and gate.dtype == x.dtype,
              "heads_product: the gate is (T, >= H), or (T, >= H N) with a gate each, of the rows' type")
        ldg = gate.stride(0) if M > 1 else gate.shape[1]
    _check(lib().gs_heads_product(_p(x), _dt(x), x.stride(0) if M > 1 else x.shape[1], hx, _p(w), _dt(w), _p(y),
                                  y.stride(0) if M > 1 else y.shape[1], hy, _p(gate), ldg, 1 if gate_each else 0, M, N, K,
                                  H, _stream()))
    return y


def attention_latent(qa, cache, positions, seq_of_token, block_table, page_size, window, scale, H, c, r, ntok,
                     out: torch.Tensor = None) -> torch.Tensor:
    """Attention of ``qa (T, H (c + r))`` over cached rows ``[c | r]``: scores over all ``c + r`` columns, the output
    ``(T, H c)`` a softmax-weighted sum of the rows' first ``c`` columns.  Any sizes, float32 arithmetic."""
    _dev(qa, cache, positions, seq_of_token, block_table, out)
    _need(qa.shape == (ntok, H * (c + r)) and cache.dtype == qa.dtype, "attention_latent: qa is (T, H (c + r)) in the cache's type")
    _need(cache.dim() == 4 and cache.shape[1:] == (1, page_size, c + r), "attention_latent: the cache is (pages, 1, page_size, c + r)")
    _i32(positions, ntok, "positions")
    _i32(seq_of_token, ntok, "seq_of_token")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if out is None:
        out = torch.empty((ntok, H * c), dtype=qa.dtype, device=qa.device)
    _need(out.shape == (ntok, H * c) and out.dtype == qa.dtype, "attention_latent: out has the wrong shape or type")
    _check(lib().gs_attention_latent(_p(qa), _p(cache), _dt(qa), _p(positions), _p(seq_of_token), _p(block_table),
                                     block_table.shape[1], page_size, window or 0, float(scale), _p(out), ntok, H, c, r,
                                     _stream()))
    return out


# ---------------------------------------------------------------------- feed-forwards routed by a table

def relu_squared(x: torch.Tensor, F: int) -> torch.Tensor:
    """``relu(x[:, :F])^2`` as contiguous rows ``(T, F)``."""
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.shape[1] >= F, "relu_squared: rows (T, >= F) on the GPU")
    T = x.shape[0]
    out = torch.empty((T, F), dtype=x.dtype, device=x.device)
    _check(lib().gs_relu_squared(_p(x), _dt(x), x.stride(0) if T > 1 else x.shape[1], _p(out), T, F, _stream()))
    return out


def moe_table(x, ids, table, up, down, shared=None, gate=None) -> torch.Tensor:
    """``y[t] = (1 / top) sum_k down[e_k] relu(up[e_k] x[t])^2`` with ``e_k = table[ids[t], k]``; ``up (E, F, H)``,
    ``down (E, H, F)``, ``table (vocab, top)`` int32.  With ``shared (T, H)`` and ``gate`` (one number a token, the
    first column of its rows): ``+ sigmoid(gate[t]) * shared[t]``.  Token by token: only the chosen experts' weights
    are read."""
    _dev(ids, table, up, down, shared)
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1, "moe_table: rows (T, H) on the GPU")
    T, H = x.shape
    E, F, Hw = up.shape
    _need(Hw == H and down.shape == (E, H, F) and up.dtype == down.dtype, "moe_table: up is (E, F, H), down (E, H, F)")
    _need(table.dtype == torch.int32 and table.dim() == 2, "moe_table: the table is int32 (vocab, top)")
    top = table.shape[1]
    _i32(ids, T, "token ids")
    ldg = 0
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == x.dtype and gate is not None and gate.is_cuda and gate.dim() == 2
              and gate.shape[0] == T and gate.dtype == x.dtype and gate.stride(1) == 1,
              "moe_table: shared rows (T, H) come with a gate (T, >= 1) of the rows' type")
        ldg = gate.stride(0) if T > 1 else gate.shape[1]
    a = torch.empty((T, top, F), dtype=x.dtype, device=x.device)
    y = torch.empty((T, H), dtype=x.dtype, device=x.device)
    _check(lib().gs_moe_table_up(_p(x), _dt(x), x.stride(0) if T > 1 else H, _p(ids), _p(table), top, _p(up), _dt(up), F,
                                 H, _p(a), T, _stream()))
    _check(lib().gs_moe_table_down(_p(a), _dt(a), _p(ids), _p(table), top, _p(down), _dt(down), F, H, _p(shared),
                                   _p(gate) if shared is not None else None, ldg, _p(y), T, _stream()))
    return y


def attention_latent_mfma_supports(H: int, c: int, r: int) -> bool:
    """Whether the matrix-core kernel over latent rows takes these sizes (bfloat16; value columns in tiles of 16 up to
    512, rows of whole 16-byte pieces)."""
    return bool(lib().gs_attention_latent_mfma_supports(H, c, r))


def attention_latent_mfma_tokens(H: int) -> int:
    """How many consecutive tokens of a sequence one block of :func:`attention_latent_mfma` takes."""
    return int(lib().gs_attention_latent_mfma_tokens(H))


_latent_parts = {}


def _latent_workspace(device, rows: int, c: int, nsplit: int):
    """Room for the shares of blocks that walk a row's keys in parts: kept per device and made anew when more is asked."""
    need = nsplit * rows * (c + 2)
    held = _latent_parts.get(device)
    if held is None or held.numel() < need:
        held = _latent_parts[device] = torch.empty(need, dtype=torch.float32, device=device)
    return held[:nsplit * rows * c], held[nsplit * rows * c:need]


def attention_latent_mfma(qa, cache, positions, tiles, block_table, page_size, window, scale, H, c, r, ntok,
                          out: torch.Tensor = None, nsplit: int = 1) -> torch.Tensor:
    """:func:`attention_latent` on the matrix cores (bfloat16).  ``tiles``: int32 ``(3, n)``, the sequence, first row
    and token count (at most :func:`attention_latent_mfma_tokens`) of every tile of consecutive tokens of one
    sequence; None: sequence ``i`` brings the single token ``i``.  ``nsplit`` > 1: as many blocks share a tile's keys out
    between them in runs of whole steps, and a second kernel adds their shares."""
    _dev(qa, cache, positions, block_table, out, tiles)
    _need(1 <= nsplit <= 64, "attention_latent_mfma: 1 to 64 parts")
    _need(qa.dtype == torch.bfloat16 and cache.dtype == torch.bfloat16, "attention_latent_mfma takes bfloat16")
    _need(qa.shape == (ntok, H * (c + r)), "attention_latent_mfma: qa is (T, H (c + r))")
    _need(cache.dim() == 4 and cache.shape[1:] == (1, page_size, c + r), "attention_latent_mfma: the cache is (pages, 1, page_size, c + r)")
    _need(qa.data_ptr() % 16 == 0 and cache.data_ptr() % 16 == 0, "attention_latent_mfma: operands are 16-byte aligned")
    _i32(positions, ntok, "positions")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 (nseq, max_blocks)")
    if tiles is None:
        _need(block_table.shape[0] >= ntok, "attention_latent_mfma: single tokens need a block table row each")
        n, rows = ntok, (None, None, None)
    else:
        _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[0] == 3, "tiles must be int32 (3, n)")
        n, rows = tiles.shape[1], (tiles[0], tiles[1], tiles[2])
    if out is None:
        out = torch.empty((ntok, H * c), dtype=qa.dtype, device=qa.device)
    _need(out.shape == (ntok, H * c) and out.dtype == qa.dtype and out.data_ptr() % 16 == 0,
          "attention_latent_mfma: out has the wrong shape or type")
    part_o, part_ml = _latent_workspace(qa.device, ntok * H, c, nsplit) if nsplit > 1 else (None, None)
    _check(lib().gs_attention_latent_mfma(_p(qa), _p(cache), _p(positions), _p(rows[0]), _p(rows[1]), _p(rows[2]), n,
                                          _p(block_table), block_table.shape[1], page_size, window or 0, float(scale),
                                          _p(out), H, c, r, nsplit, _p(part_o), _p(part_ml), ntok, _stream()))
    return out


def moe_grouped_ok(x, up, down) -> bool:
    """Whether :func:`moe_table_grouped` takes these operands: bfloat16 throughout, widths in whole 16-byte pieces."""
    bf = torch.bfloat16
    return (x.dtype is bf and up.dtype is bf and down.dtype is bf and x.dim() == 2 and x.stride(1) == 1
            and x.shape[1] % 8 == 0 and up.shape[1] % 8 == 0 and (x.shape[0] <= 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0 and up.shape[0] <= 4096)


def moe_table_grouped(x, ids, table, up, down, shared=None, gate=None) -> torch.Tensor:
    """:func:`moe_table` for steps of many tokens (bfloat16): the (token, choice) pairs are sorted by expert on the
    device and every expert's weights are read once, by products on the matrix cores over its pairs' rows."""
    _dev(ids, table, up, down, shared)
    _need(moe_grouped_ok(x, up, down), "moe_table_grouped: bfloat16 rows and weights, widths multiples of 8")
    T, H = x.shape
    E, F, Hw = up.shape
    _need(Hw == H and down.shape == (E, H, F), "moe_table_grouped: up is (E, F, H), down (E, H, F)")
    _need(table.dtype == torch.int32 and table.dim() == 2, "moe_table_grouped: the table is int32 (vocab, top)")
    top = table.shape[1]
    _i32(ids, T, "token ids")
    ldg = 0
    if shared is not None:
        _need(shared.shape == (T, H) and shared.dtype == x.dtype and gate is not None and gate.is_cuda and gate.dim() == 2
              and gate.shape[0] == T and gate.dtype == x.dtype and gate.stride(1) == 1,
              "moe_table_grouped: shared rows (T, H) come with a gate (T, >= 1) of the rows' type")
        ldg = gate.stride(0) if T > 1 else gate.shape[1]
    P = T * top
    dev = x.device
    max_tiles = -(-P // lib().gs_moe_group_rows()) + E
    index = torch.empty(2 * P + 3 * max_tiles + 1, dtype=torch.int32, device=dev)
    perm, place_of, tiles, n_tiles = index[:P], index[P:2 * P], index[2 * P:2 * P + 3 * max_tiles], index[2 * P + 3 * max_tiles:]
    inner = torch.empty((P, F), dtype=torch.bfloat16, device=dev)
    ys = torch.empty((P, H), dtype=torch.float32, device=dev)
    y = torch.empty((T, H), dtype=x.dtype, device=dev)
    s = _stream()
    L = lib()
    _check(L.gs_moe_route(_p(ids), _p(table), T, top, E, _p(perm), _p(place_of), _p(tiles), max_tiles, _p(n_tiles), s))
    _check(L.gs_moe_group_gemm(_p(x), x.stride(0) if T > 1 else H, _p(perm), _p(up), _p(inner), BF16, F, _p(tiles), max_tiles,
                               _p(n_tiles), F, H, 2, s))
    _check(L.gs_moe_group_gemm(_p(inner), F, None, _p(down), _p(ys), F32, H, _p(tiles), max_tiles, _p(n_tiles), H, F, 0, s))
    _check(L.gs_moe_combine(_p(ys), _p(place_of), top, _p(shared), _p(gate) if shared is not None else None, ldg, _p(y),
                            _dt(y), T, H, s))
    return y


# ---------------------------------------------------------------------- norms in parts, convolutions over time

def _cols(x, what: str):
    """Row stride of ``x (T, C)``, which may be a range of columns of wider rows."""
    _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1, f"{what}: rows (T, C) with unit column stride, on the GPU")
    return x.stride(0) if x.shape[0] > 1 else max(x.shape[1], x.stride(0))


def add_group_rmsnorm(res, d1, d2, weight, eps: float, groups: int, out_dtype, rows=None) -> torch.Tensor:
    """``res += d1 + d2`` (each where given; not written back when ``rows`` are gathered), then every row cut into
    ``groups`` equal parts, each divided by its own root mean square, times ``weight``.  ``rows``: int32 indices of the
    rows to norm (None: all)."""
    _dev(res, d1, d2, weight, rows)
    _need(res.dtype == torch.float32 and res.dim() == 2, "add_group_rmsnorm: the residual stream is float32 (T, H)")
    T, H = res.shape
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "add_group_rmsnorm: the weight must be float32 (H,)")
    _need(groups >= 1 and H % groups == 0, f"add_group_rmsnorm: {groups} parts do not divide rows of {H}")
    ds = [d for d in (d1, d2) if d is not None]
    for d in ds:
        _need(d.shape == res.shape and d.dtype == ds[0].dtype, "add_group_rmsnorm: deltas have the stream's shape and one type")
    n_out = T
    if rows is not None:
        _i32(rows, what="rows")
        n_out = rows.numel()
    out = torch.empty((n_out, H), dtype=out_dtype, device=res.device)
    _check(lib().gs_add_group_rmsnorm(_p(res), _p(ds[0]) if ds else None, _p(ds[1]) if len(ds) > 1 else None,
                                      _dt(ds[0]) if ds else _dt(out), _p(weight), float(eps), groups, _p(out), _dt(out),
                                      _p(rows), n_out, H, _stream()))
    return out


def gated_group_norm(y, z, weight, eps: float, groups: int, out_dtype) -> torch.Tensor:
    """``y (T, H)`` float32 times ``silu(z)`` (``z (T, H)``, possibly a range of columns of wider rows), then the norm in
    ``groups`` equal parts, times ``weight``.  float32 arithmetic; the result in ``out_dtype`` (the type of ``z``)."""
    _dev(y, weight)
    T, H = y.shape
    _need(y.dtype == torch.float32 and z.shape == (T, H) and z.dtype == out_dtype, "gated_group_norm: y is float32 (T, H), z (T, H) in the result's type")
    _need(weight.dtype == torch.float32 and weight.shape == (H,), "gated_group_norm: the weight must be float32 (H,)")
    _need(groups >= 1 and H % groups == 0, f"gated_group_norm: {groups} parts do not divide rows of {H}")
    ldz = _cols(z, "gated_group_norm")
    out = torch.empty((T, H), dtype=out_dtype, device=y.device)
    _check(lib().gs_gated_group_norm(_p(y), _p(z), _dt(z), ldz, _p(weight), float(eps), groups, _p(out), _dt(out), T, H,
                                     _stream()))
    return out


def channel_conv(x, taps, bias, state, seq_of_token, q_start, slots, nseq: int, all_single: bool, out_dtype,
                 activation=None, residual: bool = False) -> torch.Tensor:
    """A causal convolution over time per channel, ``y_t = act(bias + sum_j taps[:, j] x_(t - K + 1 + j)) (+ x_t)``, over
    the step's sequence portions.  ``x (T, C)`` may be a range of columns of wider rows; ``taps (C, K)`` and ``bias (C,)``
    float32; ``state (slots, K - 1, C)`` float32 holds each request's last ``K - 1`` inputs and is moved on."""
    _dev(taps, bias, state, seq_of_token, q_start, slots)
    ldx = _cols(x, "channel_conv")
    T, C = x.shape
    K = taps.shape[1]
    _need(taps.dtype == torch.float32 and taps.shape == (C, K), "channel_conv: taps must be float32 (C, K)")
    _need(bias is None or (bias.dtype == torch.float32 and bias.shape == (C,)), "channel_conv: the bias must be float32 (C,)")
    _need(state.dtype == torch.float32 and state.dim() == 3 and (state.shape[1:] == (K - 1, C) or K == 1),
          "channel_conv: the state must be float32 (slots, K - 1, C)")
    _need(activation in _ACTS, f"channel_conv: activation is None or 'silu', not {activation!r}")
    _i32(seq_of_token, T, "seq_of_token")
    _i32(q_start, nseq + 1, "q_start")
    _i32(slots, nseq, "slots")
    out = torch.empty((T, C), dtype=out_dtype, device=x.device)
    _check(lib().gs_channel_conv(_p(x), _dt(x), ldx, _p(taps), _p(bias), _p(state), _p(seq_of_token), _p(q_start),
                                 _p(slots), _p(out), _dt(out), C, T, nseq, C, K, _ACTS[activation], 1 if residual else 0,
                                 1 if all_single else 0, _stream()))
    return out


# ---------------------------------------------------------------------- a state-space recurrence

def ssd_max_state(P: int) -> int:
    """The most state rows :func:`ssd_scan` holds for heads of ``P`` value columns."""
    return int(lib().gs_ssd_max_state(int(P)))


def ssd_scan(xbc, rows, odt: int, dt_bias, a_log, d_skip, state, q_start, slots, nseq: int, H: int, P: int, N: int,
             G: int, segments=None) -> torch.Tensor:
    """Per sequence and head ``h`` (group ``h // (H / G)``): ``dt = softplus(d + dt_bias[h])``,
    ``S <- exp(-exp(a_log[h]) dt) S + dt B x^T``, ``y = S^T C + d_skip[h] x``.  ``xbc (T, H P + 2 G N)`` float32 holds
    x, B and C side by side; ``d`` stands in ``rows (T, ld)`` from column ``odt`` on; ``state (slots, H, N, P)`` float32
    is read and advanced.  Token by token, float32; returns ``(T, H P)`` float32.  ``segments``: ``(table, count)`` as
    ``BatchContext.state_segments`` makes them: the portions are then walked segment by segment side by side (three
    launches: what each segment adds to a state, every segment's first state, the segments with their outputs)."""
    _dev(xbc, rows, dt_bias, a_log, d_skip, state, q_start, slots)
    T = xbc.shape[0]
    _need(xbc.dtype == torch.float32 and xbc.shape == (T, H * P + 2 * G * N), "ssd_scan: x | B | C rows must be float32 (T, H P + 2 G N)")
    _need(rows.dim() == 2 and rows.shape[0] == T and odt + H <= rows.shape[1], "ssd_scan: the step sizes do not fit their rows")
    for v in (dt_bias, a_log, d_skip):
        _need(v.dtype == torch.float32 and v.shape == (H,), "ssd_scan: dt_bias, a_log and d_skip must be float32 (H,)")
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.shape[1:] == (H, N, P), "ssd_scan: the state must be float32 (slots, H, N, P)")
    _i32(q_start, nseq + 1, "q_start")
    _i32(slots, nseq, "slots")
    out = torch.empty((T, H * P), dtype=torch.float32, device=xbc.device)
    if segments is not None:
        table, nsegs = segments
        _i32(table, nseq + 1 + 4 * nsegs, "segments")
        ws = torch.empty((nsegs * H * N * P + nsegs * H,), dtype=torch.float32, device=xbc.device)
        _check(lib().gs_ssd_scan_segments(_p(xbc), xbc.shape[1], H * P, H * P + G * N, _p(rows), _dt(rows), rows.shape[1],
                                          odt, _p(dt_bias), _p(a_log), _p(d_skip), _p(state), _p(q_start), _p(slots),
                                          _p(out), nseq, H, P, N, G, table.data_ptr(), table.data_ptr() + 4 * (nseq + 1),
                                          nsegs, ws.data_ptr(), ws.data_ptr() + 4 * nsegs * H * N * P, _stream()))
        return out
    _check(lib().gs_ssd_scan(_p(xbc), xbc.shape[1], H * P, H * P + G * N, _p(rows), _dt(rows), rows.shape[1], odt,
                             _p(dt_bias), _p(a_log), _p(d_skip), _p(state), _p(q_start), _p(slots), _p(out), nseq, H, P, N,
                             G, _stream()))
    return out


# ---------------------------------------------------------------------- feed-forwards chosen by a router

ROUTER_SCORES = {"softmax": 0, "sigmoid": 1}


def moe_router(x, router, correction, top: int, score: str = "softmax", renormalize: bool = True, scale: float = 1.0):
    """Scores = softmax (or, with ``score="sigmoid"``, each output's sigmoid) of ``router (EA, H) @ x[t]`` in float32; the
    ``top`` outputs with the largest score + ``correction`` are chosen (of equal ones the lowest index), their weights
    are their scores divided by the chosen scores' sum (+ 1e-20) (as they are without ``renormalize``), times ``scale``.
    Returns ``(choice int32 (T, top), weight float32 (T, top))``."""
    _need(score in ROUTER_SCORES, f"moe_router: scores are one of {sorted(ROUTER_SCORES)}, not {score!r}")
    _dev(router, correction)
    ldx = _cols(x, "moe_router")
    T, H = x.shape
    EA = router.shape[0]
    _need(router.shape == (EA, H) and 1 <= top <= EA, "moe_router: the router is (outputs, H), top within its outputs")
    _need(correction is None or (correction.dtype == torch.float32 and correction.shape == (EA,)), "moe_router: the correction must be float32 (outputs,)")
    choice = torch.empty((T, top), dtype=torch.int32, device=x.device)
    weight = torch.empty((T, top), dtype=torch.float32, device=x.device)
    _check(lib().gs_moe_router(_p(x), _dt(x), ldx, _p(router), _dt(router), _p(correction), top, EA, H, _p(choice),
                               _p(weight), T, ROUTER_SCORES[score], 1 if renormalize else 0, float(scale), _stream()))
    return choice, weight


def clamped_glu(gu, limit: float, alpha: float, out_dtype) -> torch.Tensor:
    """``gu (rows, 2F)`` = gate | up  ->  ``g sigmoid(alpha g) (u + 1)`` with ``g = min(gate, limit)``,
    ``u = clamp(up, -limit, limit)``: ``(rows, F)`` in ``out_dtype``, float32 arithmetic."""
    _dev(gu)
    _need(gu.dim() == 2 and gu.shape[1] % 2 == 0, "clamped_glu: rows hold gate and up side by side")
    R, F2 = gu.shape
    out = torch.empty((R, F2 // 2), dtype=out_dtype, device=gu.device)
    _check(lib().gs_clamped_glu(_p(gu), _dt(gu), _p(out), _dt(out), R, F2 // 2, float(limit), float(alpha), _stream()))
    return out


def _routed_operands(x, choice, weight, gate_up, down, shared, what):
    _dev(choice, weight, gate_up, down, shared)
    ldx = _cols(x, what)
    T, H = x.shape
    _need(down.dim() == 3 and gate_up.dim() == 3, f"{what}: gate_up is (E, 2F, H), down (E, H, F)")
    E, Hd, F = down.shape
    _need(Hd == H and gate_up.shape == (E, 2 * F, H) and gate_up.dtype == down.dtype, f"{what}: gate_up is (E, 2F, H), down (E, H, F)")
    _need(choice.dtype == torch.int32 and choice.dim() == 2 and choice.shape[0] == T and weight.dtype == torch.float32
          and weight.shape == choice.shape, f"{what}: choices int32 (T, top) with float32 weights")
    _need(shared is None or (shared.shape == (T, H) and shared.dtype == x.dtype), f"{what}: the shared expert's rows are (T, H) of the rows' type")
    return ldx, T, H, E, F, choice.shape[1]


def moe_routed(x, choice, weight, gate_up, down, limit: float, alpha: float, shared=None) -> torch.Tensor:
    """``y[t] = sum_k weight[t, k] * expert(choice[t, k])(x[t]) (+ shared[t])``, token by token: only the chosen experts'
    weights are read.  A choice ``>= E`` names no weights: that expert gives back ``x[t]``.  ``gate_up (E, 2F, H)`` holds
    each expert's gate rows, then its up rows; ``down (E, H, F)``."""
    ldx, T, H, E, F, top = _routed_operands(x, choice, weight, gate_up, down, shared, "moe_routed")
    a = torch.empty((T, top, max(F, 1)), dtype=x.dtype, device=x.device)
    y = torch.empty((T, H), dtype=x.dtype, device=x.device)
    _check(lib().gs_moe_routed_up(_p(x), _dt(x), ldx, _p(choice), top, E, _p(gate_up), _dt(gate_up), F, H, float(limit),
                                  float(alpha), _p(a), T, _stream()))
    _check(lib().gs_moe_routed_down(_p(a), _dt(a), _p(x), ldx, _p(choice), _p(weight), top, E, _p(down), _dt(down), F, H,
                                    _p(shared), _p(y), T, _stream()))
    return y


def moe_routed_grouped_ok(x, gate_up, down) -> bool:
    """Whether :func:`moe_routed_grouped` takes these operands: bfloat16 throughout, widths in whole 16-byte pieces."""
    bf = torch.bfloat16
    return (x.dtype is bf and gate_up.dtype is bf and down.dtype is bf and x.dim() == 2 and x.stride(1) == 1
            and x.shape[1] % 8 == 0 and down.shape[2] % 8 == 0 and (x.shape[0] <= 1 or x.stride(0) % 8 == 0)
            and x.data_ptr() % 16 == 0 and 0 < down.shape[0] <= 4096)


def moe_routed_grouped(x, choice, weight, gate_up, down, limit: float, alpha: float, shared=None) -> torch.Tensor:
    """:func:`moe_routed` for steps of many tokens (bfloat16): the (token, choice) pairs are sorted by expert on the
    device and every expert's weights are read once, by products on the matrix cores over its pairs' rows."""
    _need(moe_routed_grouped_ok(x, gate_up, down), "moe_routed_grouped: bfloat16 rows and weights, widths multiples of 8")
    ldx, T, H, E, F, top = _routed_operands(x, choice, weight, gate_up, down, shared, "moe_routed_grouped")
    P = T * top
    dev = x.device
    max_tiles = -(-P // lib().gs_moe_group_rows()) + E
    index = torch.empty(2 * P + 3 * max_tiles + 1, dtype=torch.int32, device=dev)
    perm, place_of, tiles, n_tiles = index[:P], index[P:2 * P], index[2 * P:2 * P + 3 * max_tiles], index[2 * P + 3 * max_tiles:]
    gu = torch.empty((P, 2 * F), dtype=torch.bfloat16, device=dev)
    ys = torch.empty((P, H), dtype=torch.float32, device=dev)
    y = torch.empty((T, H), dtype=x.dtype, device=dev)
    s = _stream()
    L = lib()
    _check(L.gs_moe_route(None, _p(choice), T, top, E, _p(perm), _p(place_of), _p(tiles), max_tiles, _p(n_tiles), s))
    _check(L.gs_moe_group_gemm(_p(x), ldx, _p(perm), _p(gate_up), _p(gu), BF16, 2 * F, _p(tiles), max_tiles, _p(n_tiles),
                               2 * F, H, 1, s))
    inner = clamped_glu(gu, limit, alpha, torch.bfloat16)
    _check(L.gs_moe_group_gemm(_p(inner), F, None, _p(down), _p(ys), F32, H, _p(tiles), max_tiles, _p(n_tiles), H, F, 0, s))
    _check(L.gs_moe_routed_combine(_p(ys), _p(place_of), _p(weight), top, _p(x), ldx, _p(shared), _p(y), _dt(y), T, H, s))
    return y


# ---------------------------------------------------------------------- layer norm, the sum of two normed branches, a gate on rows

def add_layernorm(res: torch.Tensor, delta, weight: torch.Tensor, bias, eps: float, out_dtype, rows=None,
                  out: torch.Tensor = None) -> torch.Tensor:
    """``res += delta`` (when given and no ``rows``), then ``out = (res - mean) / sqrt(var + eps) * weight + bias`` with
    the variance the mean of the squared deviations.  ``rows`` (int32) picks source rows; then ``res`` is not written."""
    _dev(res, delta, weight, bias, rows, out)
    _need(res.dtype == torch.float32 and res.dim() == 2, "add_layernorm: the residual stream is float32 (T, H)")
    T, H = res.shape
    for v in (weight, bias):
        _need(v is None or (v.dtype == torch.float32 and v.shape == (H,)), "add_layernorm: weight and bias must be float32 (H,)")
    _need(weight is not None, "add_layernorm: a weight")
    _need(delta is None or delta.shape == res.shape, "add_layernorm: delta must have the stream's shape")
    n_out = T
    if rows is not None:
        _i32(rows, what="rows")
        n_out = rows.numel()
    if out is None:
        out = torch.empty((n_out, H), dtype=out_dtype, device=res.device)
    _need(out.shape == (n_out, H) and out.dtype == out_dtype, "add_layernorm: out has the wrong shape or type")
    _check(lib().gs_add_layernorm(_p(res), _p(delta), _dt(delta) if delta is not None else _dt(out), _p(weight), _p(bias),
                                  float(eps), _p(out), _dt(out), _p(rows), n_out, H, _stream()))
    return out


def normed_pair_sum(a, wa, sa: float, b, wb, sb: float, eps: float, out_dtype) -> torch.Tensor:
    """``sa * rms(a) * wa + sb * rms(b) * wb`` row by row, ``rms(x) = x / sqrt(mean(x^2) + eps)``: ``a``, ``b`` float32
    ``(T, W)`` (two branches' last products), ``wa``, ``wb`` float32 ``(W,)``; one rounding, to ``out_dtype``."""
    _dev(a, b, wa, wb)
    _need(a.dtype == torch.float32 and b.dtype == torch.float32 and a.dim() == 2 and a.shape == b.shape,
          "normed_pair_sum: the branches' rows are float32 (T, W)")
    T, W = a.shape
    for w in (wa, wb):
        _need(w.dtype == torch.float32 and w.shape == (W,), "normed_pair_sum: weights must be float32 (W,)")
    out = torch.empty((T, W), dtype=out_dtype, device=a.device)
    _check(lib().gs_normed_pair_sum(_p(a), _p(b), _p(wa), _p(wb), float(eps), float(sa), float(sb), _p(out), _dt(out), T, W,
                                    _stream()))
    return out


def gated_rows(o, gate_rows, og: int, gate: str = "sigmoid") -> torch.Tensor:
    """``o (T, W)`` times ``sigmoid`` or ``silu`` of the gate, which stands in ``gate_rows (T, ldg)`` from column ``og``
    on; float32 arithmetic, the result in the rows' type."""
    _dev(o, gate_rows)
    _need(o.dim() == 2 and gate_rows.dim() == 2 and gate_rows.shape[0] == o.shape[0] and gate_rows.dtype == o.dtype,
          "gated_rows: rows (T, W) and gate rows (T, ldg) of one type")
    _need(gate in _GATES, f"gated_rows: the gate is 'sigmoid' or 'silu', not {gate!r}")
    T, W = o.shape
    out = torch.empty_like(o)
    _check(lib().gs_gated_rows(_p(o), _p(gate_rows), _dt(o), gate_rows.shape[1], og, _GATES[gate], _p(out), T, W, _stream()))
    return out


# ---------------------------------------------------------------------- recurrences with token-dependent decay

GATED_STATE_MAX_KEY = 256


def gated_state_scan(x, oq: int, ok: int, ov: int, H: int, qk_heads: int, n: int, m: int, decay, oa: int,
                     per_channel: bool, state, q_start, slots, nseq: int, q_scale: float = 1.0, beta=None, ob: int = 0,
                     out: torch.Tensor = None, want_out: bool = True) -> torch.Tensor:
    """Per sequence and head ``S <- diag(a_t) S; u = beta_t (v_t - S^T k_t)`` (``u = v_t`` without ``beta``);
    ``S <- S + k_t u^T; o_t = S^T (q_scale q_t)``.

    ``x (T, ld)`` float32 or bfloat16 holds q of head ``h`` at ``[oq + (h // (H / qk_heads)) n, ...)``, k likewise from
    ``ok``, v at ``[ov + h m, ...)`` (``ov`` < 0: every value is zero).  ``decay`` float32 rows: ``a_t`` of head ``h`` at
    ``[oa + h]``, or with ``per_channel`` one a key channel at ``[oa + h n, ...)``.  ``beta`` float32 rows with head ``h``
    at ``[ob + h]``.  ``state (slots, H, n, m)`` float32 is read and advanced.  Returns ``(T, H m)`` float32, or None
    without ``want_out`` (the states alone are wanted)."""
    _dev(x, decay, beta, state, q_start, slots, out)
    _need(x.dim() == 2 and decay.dim() == 2 and decay.dtype == torch.float32 and decay.shape[0] == x.shape[0],
          "gated_state_scan: rows (T, ld) and float32 decay rows (T, lda)")
    _need(beta is None or (beta.dim() == 2 and beta.dtype == torch.float32 and beta.shape[0] == x.shape[0]),
          "gated_state_scan: the write strengths are float32 rows (T, ldb)")
    T, ld = x.shape
    _need(n <= GATED_STATE_MAX_KEY, f"gated_state_scan: keys of {n} features, the kernel holds up to {GATED_STATE_MAX_KEY}")
    _need(state.dtype == torch.float32 and state.dim() == 4 and state.shape[1:] == (H, n, m),
          "gated_state_scan: state must be float32 (slots, H, n, m)")
    _i32(q_start, nseq + 1, "q_start")
    _i32(slots, nseq, "slots")
    if want_out:
        if out is None:
            out = torch.empty((T, H * m), dtype=torch.float32, device=x.device)
        _need(out.shape == (T, H * m) and out.dtype == torch.float32, "gated_state_scan: out must be float32 (T, H m)")
    else:
        out = None
    _check(lib().gs_gated_state_scan(_p(x), _dt(x), ld, oq, ok, ov, qk_heads, float(q_scale), _p(decay), decay.shape[1], oa,
                                     1 if per_channel else 0, _p(beta), beta.shape[1] if beta is not None else 0, ob,
                                     _p(state), _p(q_start), _p(slots), _p(out), nseq, H, n, m, _stream()))
    return out


def state_segment_tables(q_lens, seg_len: int, device):
    """A step's portions cut into segments of at most ``seg_len`` tokens: int32 on the device, ``(where each segment's
    tokens begin among the step's rows (segments + 1), where each sequence's segments begin (sequences + 1), the
    segments' numbers (segments))``, and the number of segments."""
    starts, first, at = [0], [0], 0
    for L in q_lens:
        for a in range(0, L, seg_len):
            starts.append(at + min(a + seg_len, L))
        at += L
        first.append(len(starts) - 1)
    nseg = len(starts) - 1
    t = torch.tensor(starts + first + list(range(nseg)), dtype=torch.int32).pin_memory().to(device, non_blocking=True)
    return t[:nseg + 1], t[nseg + 1:nseg + 1 + len(first)], t[nseg + 1 + len(first):], nseg


def gated_state_scan_segments(x, oq: int, ok: int, ov: int, H: int, qk_heads: int, n: int, m: int, decay, oa: int,
                              per_channel: bool, state, q_lens, slots, seg_len: int, q_scale: float = 1.0, beta=None,
                              ob: int = 0) -> torch.Tensor:
    """:func:`gated_state_scan` with the portions (``q_lens``: tokens of each sequence, on the host) cut into segments of
    ``seg_len`` tokens that run side by side.  Over a segment the state goes ``S -> M S + B``: the kernel gives every
    segment's ``B`` (from a state of zeros) and ``M`` (from the identity, every value zero); ``gated_state_chain`` walks
    each sequence's segments in order, leaves every segment's first state and the request's new state; the kernel then
    runs from those states for the outputs.  The same arithmetic in another association (float32 rounding apart)."""
    _dev(state, slots)
    nseq = len(q_lens)
    seg_start, seq_seg, ids, nseg = state_segment_tables(q_lens, seg_len, x.device)
    dev, f32 = x.device, torch.float32
    B = torch.zeros((nseg, H, n, m), dtype=f32, device=dev)
    M = torch.eye(n, dtype=f32, device=dev).expand(nseg, H, n, n).contiguous()
    first = torch.empty((nseg, H, n, m), dtype=f32, device=dev)
    args = (H, qk_heads, n)
    kw = dict(q_scale=q_scale, beta=beta, ob=ob)
    gated_state_scan(x, oq, ok, ov, *args, m, decay, oa, per_channel, B, seg_start, ids, nseg, want_out=False, **kw)
    gated_state_scan(x, oq, ok, -1, *args, n, decay, oa, per_channel, M, seg_start, ids, nseg, want_out=False, **kw)
    _i32(slots, nseq, "slots")
    _need(state.dtype == f32 and state.dim() == 4 and state.shape[1:] == (H, n, m), "gated_state_scan: state must be float32 (slots, H, n, m)")
    _check(lib().gs_gated_state_chain(_p(M), _p(B), _p(first), _p(state), _p(seq_seg), _p(slots), nseq, H, n, m, _stream()))
    return gated_state_scan(x, oq, ok, ov, *args, m, decay, oa, per_channel, first, seg_start, ids, nseg, **kw)


def delta_rule_prep(c, G: int, n: int, q_scale: float, unit_eps: float, rows, oa: int, ob: int, a_log, dt_bias, H: int):
    """In place on ``c (T, >= 2 G n)`` float32: each of the ``G`` q heads (first) and ``G`` k heads (behind them) becomes
    ``x / sqrt(sum(x^2) + unit_eps)``, q also times ``q_scale``.  Returns float32 ``(T, 2 H)``:
    ``exp(-exp(a_log) softplus(rows[:, oa + h] + dt_bias))`` in the first ``H`` columns, ``sigmoid(rows[:, ob + h])`` in
    the others."""
    _dev(c, rows, a_log, dt_bias)
    T = c.shape[0]
    _need(c.dtype == torch.float32 and c.dim() == 2 and c.shape[1] >= 2 * G * n, "delta_rule_prep: float32 rows that hold q and k")
    _need(rows.dim() == 2 and rows.shape[0] == T, "delta_rule_prep: the gates' products are rows (T, ld)")
    for v in (a_log, dt_bias):
        _need(v.dtype == torch.float32 and v.shape == (H,), "delta_rule_prep: a_log and dt_bias must be float32 (H,)")
    gates = torch.empty((T, 2 * H), dtype=torch.float32, device=c.device)
    _check(lib().gs_delta_rule_prep(_p(c), c.shape[1], G, n, float(q_scale), float(unit_eps), _p(rows), _dt(rows),
                                    rows.shape[1], oa, ob, _p(a_log), _p(dt_bias), _p(gates), T, H, _stream()))
    return gates


def channel_decay(z, tau: float) -> torch.Tensor:
    """In place on float32 ``z``: ``sigmoid(z)^(1/tau)``."""
    _dev(z)
    _need(z.dtype == torch.float32, "channel_decay: float32 values")
    _check(lib().gs_channel_decay(_p(z), z.numel(), float(tau), _stream()))
    return z
