"""Python face of the HIP kernels.

Every function checks on the host that the operands are what the kernel and
its launch grid assume (device, dtype, contiguity, shapes) and raises
before anything is launched otherwise.  A missing or unloadable library is an
error, never a reason to compute some other way.
"""
from __future__ import annotations

import ctypes
import math
from typing import Optional

import torch

from . import build as _build
from .build import KernelBuildError, load_lib

F32, BF16 = 0, 1
# The 16-bit types.  A library that handles 16-bit values exists once for each (kernels.build.HALF_LIBS); BF16 is the
# code of "the library's 16-bit type" in the entry points' dtype arguments, whichever build is called.
LOWP = (torch.bfloat16, torch.float16)
_CODES = {torch.float32: F32, torch.bfloat16: BF16, torch.float16: BF16}


class KernelError(RuntimeError):
    pass


def _code(t: torch.Tensor) -> int:
    try:
        return _CODES[t.dtype]
    except KeyError:
        raise KernelError(f"dtype {t.dtype} is not handled by the kernels (float32, bfloat16 and float16 are)") from None


def _half(*ts) -> bool:
    """Which build of a library a call needs: True if the 16-bit tensors among `ts` are float16.  The two 16-bit
    types do not meet in one call."""
    kinds = {t.dtype for t in ts if t is not None and t.dtype in LOWP}
    if len(kinds) > 1:
        raise KernelError("bfloat16 and float16 tensors in one call")
    return torch.float16 in kinds


def _any_build(name: str, head_dim: Optional[int] = None):
    """A library for a question whose answer is the same in both of its builds (launch shapes, sizes of scratch
    memory): the build that is loaded already, so that a float16 model does not compile the bfloat16 one for it."""
    for half in (False, True):
        lib = _build._loaded.get(_build.lib_spec(name, head_dim, half)[0])
        if lib is not None:
            return lib
    return load_lib(name, head_dim)


def _lowp(t: torch.Tensor, name: str) -> torch.dtype:
    """The 16-bit type of a call's leading tensor."""
    if t.dtype not in LOWP:
        raise KernelError(f"{name}: dtype {t.dtype}, expected bfloat16 or float16")
    return t.dtype


def _chk(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not t.is_cuda:
        raise KernelError(f"{name}: tensor is on {t.device}, the kernels run on the GPU only")
    if not t.is_contiguous():
        raise KernelError(f"{name}: tensor is not contiguous")
    if dtype is not None and t.dtype != dtype:
        raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")


def _ptr(t: Optional[torch.Tensor]):
    return ctypes.c_void_p(t.data_ptr() if t is not None else 0)


def _stream():
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _run(lib, fn: str, *args) -> None:
    rc = getattr(lib, fn)(*args)
    if rc != 0:
        raise KernelError(lib.vt_last_error().decode("utf-8", "replace"))


def _i(v) -> ctypes.c_int:
    return ctypes.c_int(int(v))


def _f(v) -> ctypes.c_float:
    return ctypes.c_float(float(v))


# ---------------------------------------------------------------------------
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
    """out[t] = table[ids[t]] * scale, the product in float32."""
    n = ids.numel()
    vocab, hidden = table.shape
    _chk(table, "embed.table")
    _chk(ids, "embed.ids", torch.int32)
    _chk(out, "embed.out", torch.float32, (n, hidden))
    _run(load_lib("vt_elementwise", half=_half(table)), "vt_embed", _ptr(table), _i(_code(table)), _ptr(ids), _ptr(out), _i(n), _i(hidden),
         _i(vocab), _f(scale), _stream())
    return out


def rmsnorm(h: torch.Tensor, delta: Optional[torch.Tensor], gain: torch.Tensor, out: torch.Tensor, eps: float,
            rows: Optional[torch.Tensor] = None, update_h: bool = True) -> torch.Tensor:
    """out[r] = gain * x / sqrt(mean(x^2) + eps), x = h[row] + delta[row]; with update_h the sum is written back to h."""
    hidden = h.shape[-1]
    _chk(h, "rmsnorm.h", torch.float32)
    _chk(gain, "rmsnorm.gain", torch.float32, (hidden,))
    if delta is not None:
        _chk(delta, "rmsnorm.delta", None, h.shape)
    if rows is not None:
        _chk(rows, "rmsnorm.rows", torch.int32)
        n_out = rows.numel()
        update_h = False
    else:
        n_out = h.shape[0]
    _chk(out, "rmsnorm.out", None, (n_out, hidden))
    _run(load_lib("vt_elementwise", half=_half(delta, out)), "vt_rmsnorm", _ptr(h), _ptr(delta), _i(_code(delta) if delta is not None else -1),
         _ptr(gain), _ptr(out), _i(_code(out)), _ptr(rows), _i(n_out), _i(hidden), _f(eps),
         _i(1 if (update_h and delta is not None) else 0), _stream())
    return out


def residual_add(h: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    _chk(h, "residual_add.h", torch.float32)
    _chk(delta, "residual_add.delta", None, h.shape)
    _run(load_lib("vt_elementwise", half=_half(delta)), "vt_residual_add", _ptr(h), _ptr(delta), _i(_code(delta)),
         ctypes.c_longlong(h.numel()), _stream())
    return h


def add_row(h: torch.Tensor, delta: Optional[torch.Tensor], row: torch.Tensor) -> torch.Tensor:
    """h[t] += delta[t] (if given) + row, for every token t: one vector added to the whole stream."""
    n, hidden = h.shape
    _chk(h, "add_row.h", torch.float32)
    _chk(row, "add_row.row", torch.float32, (hidden,))
    if delta is not None:
        _chk(delta, "add_row.delta", None, h.shape)
    _run(load_lib("vt_elementwise", half=_half(delta)), "vt_add_row", _ptr(h), _ptr(delta),
         _i(_code(delta) if delta is not None else F32), _ptr(row), ctypes.c_longlong(n), _i(hidden), _stream())
    return h


def layernorm(h: torch.Tensor, delta: Optional[torch.Tensor], gain: torch.Tensor, bias: Optional[torch.Tensor],
              out: torch.Tensor, eps: float, rows: Optional[torch.Tensor] = None, update_h: bool = True,
              delta2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = (x - mean(x)) / sqrt(mean((x - mean(x))^2) + eps) * gain + bias with x = h[row] + (delta[row] +
    delta2[row]), everything in float32; with update_h the sum is written back to h."""
    hidden = h.shape[-1]
    _chk(h, "layernorm.h", torch.float32)
    _chk(gain, "layernorm.gain", torch.float32, (hidden,))
    if bias is not None:
        _chk(bias, "layernorm.bias", torch.float32, (hidden,))
    if delta is not None:
        _chk(delta, "layernorm.delta", None, h.shape)
    if delta2 is not None:
        if delta is None:
            raise KernelError("layernorm: a second addend without a first")
        _chk(delta2, "layernorm.delta2", delta.dtype, h.shape)
    if rows is not None:
        _chk(rows, "layernorm.rows", torch.int32)
        n_out = rows.numel()
        update_h = False
    else:
        n_out = h.shape[0]
    _chk(out, "layernorm.out", None, (n_out, hidden))
    _run(load_lib("vt_elementwise", half=_half(delta, out)), "vt_layernorm", _ptr(h), _ptr(delta), _ptr(delta2),
         _i(_code(delta) if delta is not None else F32), _ptr(gain), _ptr(bias), _ptr(out), _i(_code(out)), _ptr(rows),
         _i(n_out), _i(hidden), _f(eps), _i(1 if (update_h and delta is not None) else 0), _stream())
    return out


def residual_add2(h: torch.Tensor, a: torch.Tensor, b: torch.Tensor) -> torch.Tensor:
    """h += (a + b): two results joined first, then added to the float32 stream."""
    _chk(h, "residual_add2.h", torch.float32)
    _chk(a, "residual_add2.a", None, h.shape)
    _chk(b, "residual_add2.b", a.dtype, h.shape)
    _run(load_lib("vt_elementwise", half=_half(a)), "vt_residual_add2", _ptr(h), _ptr(a), _ptr(b), _i(_code(a)),
         ctypes.c_longlong(h.numel()), _stream())
    return h


def scaled_sum(a: torch.Tensor, sa: float, b: torch.Tensor, sb: float, out: torch.Tensor) -> torch.Tensor:
    """out = sa * a + sb * b, float32."""
    _chk(a, "scaled_sum.a")
    _chk(b, "scaled_sum.b", None, a.shape)
    _chk(out, "scaled_sum.out", torch.float32, a.shape)
    _run(load_lib("vt_elementwise", half=_half(a, b)), "vt_scaled_sum", _ptr(a), _i(_code(a)), _f(sa), _ptr(b), _i(_code(b)),
         _f(sb), _ptr(out), ctypes.c_longlong(a.numel()), _stream())
    return out


def concat_cast(a: torch.Tensor, b: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = [a[t] | b[t]] in out's dtype, from two float32 tensors with the same rows."""
    n = a.shape[0]
    _chk(a, "concat_cast.a", torch.float32)
    _chk(b, "concat_cast.b", torch.float32)
    if a.dim() != 2 or b.dim() != 2 or b.shape[0] != n:
        raise KernelError(f"concat_cast: shapes {tuple(a.shape)} and {tuple(b.shape)}")
    _chk(out, "concat_cast.out", None, (n, a.shape[1] + b.shape[1]))
    _run(load_lib("vt_elementwise", half=_half(out)), "vt_concat_cast", _ptr(a), _ptr(b), _ptr(out), _i(_code(out)),
         ctypes.c_longlong(n), _i(a.shape[1]), _i(b.shape[1]), _stream())
    return out


def set_plus_row(h: torch.Tensor, y: torch.Tensor, row: Optional[torch.Tensor]) -> torch.Tensor:
    """h[t] = y[t] + row (row None: h = y), for every token t: the float32 stream replaced."""
    n, hidden = h.shape
    _chk(h, "set_plus_row.h", torch.float32)
    _chk(y, "set_plus_row.y", None, h.shape)
    if row is not None:
        _chk(row, "set_plus_row.row", torch.float32, (hidden,))
    _run(load_lib("vt_elementwise", half=_half(y)), "vt_set_plus_row", _ptr(h), _ptr(y), _i(_code(y)), _ptr(row),
         ctypes.c_longlong(n), _i(hidden), _stream())
    return h


def silu_mul(gu: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    n, two_i = gu.shape
    _chk(gu, "silu_mul.gu")
    _chk(out, "silu_mul.out", None, (n, two_i // 2))
    if two_i % 2:
        raise KernelError(f"silu_mul: input width {two_i} is odd")
    _run(load_lib("vt_elementwise", half=_half(gu, out)), "vt_silu_mul", _ptr(gu), _i(_code(gu)), _ptr(out), _i(_code(out)), _i(n),
         _i(two_i // 2), _stream())
    return out


def gated_act(gu: torch.Tensor, out: torch.Tensor, alpha: float = 1.0, limit: float = 0.0, shift: float = 0.0,
              cubic: float = 0.0) -> torch.Tensor:
    """gu [n, 2 I] (gate columns, then up columns) -> out [n, I] = g sigmoid(alpha g (1 + cubic g^2)) (u + shift) with
    g = min(gate, limit) and u = clamp(up, -limit, limit); limit 0: no bounds."""
    n, two_i = gu.shape
    _chk(gu, "gated_act.gu")
    _chk(out, "gated_act.out", None, (n, two_i // 2))
    if two_i % 2:
        raise KernelError(f"gated_act: input width {two_i} is odd")
    if out.dtype == torch.float32 and gu.dtype != torch.float32:
        raise KernelError("gated_act: float32 results need float32 inputs")
    _run(load_lib("vt_elementwise", half=_half(gu, out)), "vt_gated_act", _ptr(gu), _i(_code(gu)), _ptr(out), _i(_code(out)),
         _i(n), _i(two_i // 2), _f(alpha), _f(limit), _f(shift), _f(cubic), _stream())
    return out


def tanh_cap(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap), in place; float32."""
    _chk(x, "tanh_cap.x", torch.float32)
    if not cap > 0:
        raise KernelError(f"tanh_cap: cap {cap} must be positive")
    _run(_any_build("vt_elementwise"), "vt_tanh_cap", _ptr(x), ctypes.c_longlong(x.numel()), _f(cap), _stream())
    return x


def gather_rows(x: torch.Tensor, rows: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    _chk(x, "gather_rows.x")
    n = rows.numel() if rows is not None else x.shape[0]
    if rows is not None:
        _chk(rows, "gather_rows.rows", torch.int32)
    _chk(out, "gather_rows.out", None, (n, x.shape[1]))
    _run(load_lib("vt_elementwise", half=_half(x, out)), "vt_gather_rows", _ptr(x), _i(_code(x)), _ptr(rows), _ptr(out), _i(_code(out)),
         _i(n), _i(x.shape[1]), _stream())
    return out


def stream_read(buf: torch.Tensor, sums: torch.Tensor, blocks: int = 256) -> torch.Tensor:
    """Read `buf` once with a kernel that does nothing else (the measured ceiling of weight streaming).
    sums: int32 [blocks * 16]; the XOR of its words is the XOR of the buffer's 32-bit words."""
    _chk(buf, "stream_read.buf")
    _chk(sums, "stream_read.sums", torch.int32, (blocks * 16,))
    nbytes = buf.numel() * buf.element_size()
    if nbytes % 16:
        raise KernelError(f"stream_read: {nbytes} bytes are not whole 16-byte pieces")
    _run(load_lib("vt_elementwise"), "vt_stream_read", _ptr(buf), ctypes.c_longlong(nbytes), _ptr(sums), _i(blocks), _stream())
    return sums


def random_normal(out: torch.Tensor, key: int, scale: float, mean: float, first: int = 0) -> torch.Tensor:
    """out.flat[i] = mean + scale * (twelve 16-bit integers of element first + i, summed and centred): close to
    N(mean, (65536 scale)^2), and the same bits as weights.random_init.counter_normal makes on the host."""
    _chk(out, "random_normal.out")
    _run(load_lib("vt_elementwise", half=_half(out)), "vt_random_normal", _ptr(out), _i(_code(out)), ctypes.c_longlong(out.numel()),
         ctypes.c_longlong(int(first)), ctypes.c_ulonglong(int(key) & 0xFFFFFFFFFFFFFFFF), _f(scale), _f(mean), _stream())
    return out


def rope_store(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
               tok_entry: torch.Tensor, block_table: Optional[torch.Tensor], q_out: torch.Tensor,
               k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], n_heads: int, n_kv: int, head_dim: int,
               write_kv: bool = True) -> None:
    """Rotate queries and keys by the tables' angles at `positions`, write the queries to q_out and, with
    write_kv, keys and values into their pages ([page][kv][slot][D] and [page][kv][D][slot])."""
    n = qkv.shape[0]
    width = (n_heads + (2 * n_kv if write_kv else 0)) * head_dim
    _chk(qkv, "rope_store.qkv")
    if qkv.shape[1] < width:
        raise KernelError(f"rope_store.qkv: {qkv.shape[1]} columns, need {width}")
    _chk(positions, "rope_store.positions", torch.int32, (n,))
    _chk(tok_entry, "rope_store.tok_entry", torch.int32, (n,))
    _chk(q_out, "rope_store.q_out", None, (n, n_heads * head_dim))
    rot = 0
    max_pos = 0
    if cos is not None:
        _chk(cos, "rope_store.cos", torch.float32)
        _chk(sin, "rope_store.sin", torch.float32, cos.shape)
        max_pos, half = cos.shape
        rot = 2 * half
    page_size = num_pages = max_blocks = 0
    if write_kv:
        num_pages, kvh, page_size, d = k_pages.shape
        if (kvh, d) != (n_kv, head_dim):
            raise KernelError(f"rope_store.k_pages: shape {tuple(k_pages.shape)} does not fit kv heads {n_kv} x {head_dim}")
        _chk(k_pages, "rope_store.k_pages", q_out.dtype)
        _chk(v_pages, "rope_store.v_pages", q_out.dtype, (num_pages, n_kv, head_dim, page_size))
        _chk(block_table, "rope_store.block_table", torch.int32)
        max_blocks = block_table.shape[1]
    _run(load_lib("vt_elementwise", half=_half(qkv, q_out, k_pages)), "vt_rope_store", _ptr(qkv), _i(_code(qkv)), ctypes.c_longlong(qkv.stride(0)),
         _ptr(cos), _ptr(sin), _i(rot), _i(max_pos), _ptr(positions), _ptr(tok_entry), _ptr(block_table),
         _i(max_blocks), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _i(_code(q_out)), _i(page_size), _i(num_pages),
         _i(n), _i(n_heads), _i(n_kv), _i(head_dim), _i(1 if write_kv else 0), _stream())


# ---------------------------------------------------------------------------
def linear_f32(x: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
    n, k = x.shape
    m = w.shape[0]
    _chk(x, "linear_f32.x", torch.float32)
    _chk(w, "linear_f32.w", torch.float32, (m, k))
    _chk(out, "linear_f32.out", torch.float32, (n, m))
    if bias is not None:
        _chk(bias, "linear_f32.bias", torch.float32, (m,))
    _run(load_lib("vt_gemm_f32"), "vt_linear_f32", _ptr(x), _ptr(w), _ptr(bias), _ptr(out), _i(n), _i(m), _i(k), _stream())
    return out


class PackedMatrix:
    """W [rows, cols] in bfloat16 in the order the matrix instruction reads it (vt_gemm_bf16.hip): tiles of
    16 rows x 32 columns, each stored as the 64 lanes' fragments; rows padded to 16 and columns to 128 by zeros.
    `halves` = 2: two matrices of `rows` rows each, packed one after the other (gate, then up)."""

    __slots__ = ("data", "rows", "cols", "halves")

    def __init__(self, data: torch.Tensor, rows: int, cols: int, halves: int = 1):
        self.data, self.rows, self.cols, self.halves = data, int(rows), int(cols), int(halves)

    def first_rows(self, n: int) -> "PackedMatrix":
        """The matrix of the first n rows (a multiple of 16): the packed rows of tiles are contiguous."""
        if self.halves != 1 or n % 16 or not 0 < n <= self.rows:
            raise KernelError(f"cannot take the first {n} rows of a packed matrix of {self.rows}")
        per_tile_row = self.data.numel() // ((self.rows + 15) // 16)
        return PackedMatrix(self.data[:(n // 16) * per_tile_row], n, self.cols)


def pack_matrix_bf16(w: torch.Tensor, halves: int = 1) -> PackedMatrix:
    """Pack W [rows, cols] (halves = 2: [2 * rows, cols], the two matrices stacked) for linear_bf16 /
    gated_linear_bf16."""
    lp = _lowp(w, "pack_matrix_bf16.w")
    _chk(w, "pack_matrix_bf16.w", lp)
    if w.dim() != 2 or w.shape[0] % halves:
        raise KernelError(f"pack_matrix_bf16: shape {tuple(w.shape)} is not {halves} stacked matrices")
    rows, cols = w.shape[0] // halves, w.shape[1]
    lib = load_lib("vt_gemm_bf16", half=_half(w))
    lib.vt_packed_elems.restype = ctypes.c_longlong
    per = int(lib.vt_packed_elems(_i(rows), _i(cols)))
    data = torch.empty(halves * per, dtype=lp, device=w.device)
    for h in range(halves):
        _run(lib, "vt_pack_matrix_bf16", _ptr(w[h * rows:(h + 1) * rows]), _ptr(data[h * per:(h + 1) * per]), _i(rows),
             _i(cols), _stream())
    return PackedMatrix(data, rows, cols, halves)


def unpack_matrix_bf16(packed: PackedMatrix, out: torch.Tensor) -> torch.Tensor:
    """The row-major matrix [halves * rows, cols] back from its packed form, into `out`."""
    lp = _lowp(packed.data, "unpack_matrix_bf16.packed")
    _chk(out, "unpack_matrix_bf16.out", lp, (packed.halves * packed.rows, packed.cols))
    lib = load_lib("vt_gemm_bf16", half=_half(packed.data))
    per = packed.data.numel() // packed.halves
    for h in range(packed.halves):
        _run(lib, "vt_unpack_matrix_bf16", _ptr(packed.data[h * per:(h + 1) * per]),
             _ptr(out[h * packed.rows:(h + 1) * packed.rows]), _i(packed.rows), _i(packed.cols), _stream())
    return out


def linear_bf16_workspace(n: int, m: int, k: int) -> int:
    """Floats of scratch memory that linear_bf16 needs for x [n, k], W [m, k] (0: none)."""
    lib = _any_build("vt_gemm_bf16")
    lib.vt_linear_bf16_workspace.restype = ctypes.c_longlong
    return int(lib.vt_linear_bf16_workspace(_i(n), _i(m), _i(k), _i(0)))


NORM_MAX_ROWS = 16         # rows up to which the few-row product applies an RMSNorm in front
LINK_MAX_ROWS = 64         # rows up to which a product takes a norm that the product in front has prepared
_adds_residual = {}


def linear_bf16_adds_residual(n: int, m: int, k: int) -> bool:
    """Whether linear_bf16 takes `residual` for x [n, k] and W [m, k]: up to 16 rows always (k a multiple of 8); 17
    to 64 rows where the kernel that keeps all of k inside a block is the faster one for this W, and where k is split
    over blocks (the launch that adds the partial sums then adds the residual too)."""
    key = (n, m, k)
    if key not in _adds_residual:
        _adds_residual[key] = bool(_any_build("vt_gemm_bf16").vt_linear_bf16_adds_residual(_i(n), _i(m), _i(k)))
    return _adds_residual[key]


def linear_bf16(x: torch.Tensor, w, bias: Optional[torch.Tensor], out: torch.Tensor,
                workspace: Optional[torch.Tensor] = None, norm_gain: Optional[torch.Tensor] = None,
                norm_eps: float = 0.0, residual: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Few rows (decoding, short portions): W is read once per 64 rows.  w: a PackedMatrix (a plain [m, k] tensor
    is packed on the spot, which costs more than the product).  Shapes whose k range is split over blocks need
    `workspace` (float32, at least linear_bf16_workspace(n, m, k) elements).
    float32 output: with norm_gain (up to 16 rows), x is the float32 residual stream and rmsnorm(x; gain, eps) is
    what gets multiplied; with residual (where linear_bf16_adds_residual says so; float32 [n, m], may be `out`), out =
    residual + the product (17 to 64 rows of a shape whose k range is split: by the launch that adds the partial sums,
    which needs the workspace)."""
    n, k = x.shape
    lp = _lowp((w.data if isinstance(w, PackedMatrix) else w), "linear_bf16.w")
    if not isinstance(w, PackedMatrix):
        _chk(w, "linear_bf16.w", lp, (w.shape[0], k))
        w = pack_matrix_bf16(w)
    m = w.rows
    if w.cols != k or w.halves != 1:
        raise KernelError(f"linear_bf16: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    fused = norm_gain is not None or residual is not None
    _chk(x, "linear_bf16.x", torch.float32 if norm_gain is not None else lp)
    _chk(w.data, "linear_bf16.w", lp)
    _chk(out, "linear_bf16.out", torch.float32 if fused else None, (n, m))
    if bias is not None:
        _chk(bias, "linear_bf16.bias", torch.float32, (m,))
    if fused:
        if k % 8 or (norm_gain is not None and n > NORM_MAX_ROWS):
            raise KernelError(f"linear_bf16: the fused norm takes at most {NORM_MAX_ROWS} rows and k a multiple of 8 "
                              f"(n={n}, k={k})")
        if residual is not None and not linear_bf16_adds_residual(n, m, k):
            raise KernelError(f"linear_bf16: {n} rows of [{m}, {k}] do not take a residual (linear_bf16_adds_residual)")
        if norm_gain is not None:
            _chk(norm_gain, "linear_bf16.norm_gain", torch.float32, (k,))
        if residual is not None:
            _chk(residual, "linear_bf16.residual", torch.float32, (n, m))
        need = linear_bf16_workspace(n, m, k) if n > 16 else 0
        if need and (workspace is None or workspace.numel() < need):
            raise KernelError(f"linear_bf16: x [{n}, {k}] with W [{m}, {k}] needs a workspace of {need} floats")
        if need:
            _chk(workspace, "linear_bf16.workspace", torch.float32)
        _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_linear_bf16_fused", _ptr(x), _ptr(norm_gain), _f(norm_eps), _ptr(w.data), _ptr(bias),
             _ptr(residual), _ptr(out), _ptr(workspace if need else None), _i(n), _i(m), _i(k), _stream())
        return out
    need = linear_bf16_workspace(n, m, k) if n > 16 else 0
    if need:
        if workspace is None:
            raise KernelError(f"linear_bf16: x [{n}, {k}] with W [{m}, {k}] needs a workspace of {need} floats")
        _chk(workspace, "linear_bf16.workspace", torch.float32)
        if workspace.numel() < need:
            raise KernelError(f"linear_bf16: workspace of {workspace.numel()} floats, need {need}")
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_linear_bf16", _ptr(x), _ptr(w.data), _ptr(bias), _ptr(out), _i(_code(out)),
         _ptr(workspace if need else None), _i(n), _i(m), _i(k), _stream())
    return out


_link_shares = {}


def linear_bf16_link_shares(n: int, m: int, k: int) -> int:
    """Blocks' shares of the rows' sums of squares that a product of this shape writes when it hands an RMSNorm on to
    the product behind it (linear_bf16_link with xn_out); 0: this shape cannot."""
    key = (n, m, k)
    if key not in _link_shares:
        _link_shares[key] = int(_any_build("vt_gemm_bf16").vt_linear_bf16_link_shares(_i(n), _i(m), _i(k)))
    return _link_shares[key]


def link_stride(n: int) -> int:
    """Floats between the shares of the rows' sums of squares that products of n rows write and read."""
    return 16 if n <= 16 else 64


def linear_bf16_link(x: torch.Tensor, w: PackedMatrix, bias: Optional[torch.Tensor], out: torch.Tensor,
                     residual: Optional[torch.Tensor] = None, ssq_in: Optional[torch.Tensor] = None, eps_in: float = 0.0,
                     xn_out: Optional[torch.Tensor] = None, gain_next: Optional[torch.Tensor] = None,
                     ssq_out: Optional[torch.Tensor] = None, workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The few-row product between RMSNorms that are no kernels of their own (up to 64 rows).
    ssq_in (float32 [shares, link_stride(n)]): x is bf16(h * gain) as the product in front left it, and the result
    is divided by the norm's root, which the shares of the rows' sums of squares give (eps_in: the norm's eps).
    xn_out (bfloat16 [n, m]; needs residual): beside out = residual + product, xn_out = bf16(out * gain_next) and this
    product's own shares ssq_out (float32 [linear_bf16_link_shares(n, m, k), link_stride(n)]) for the product behind
    the next norm.  workspace: as for linear_bf16."""
    n, k = x.shape
    lp = _lowp(w.data, "linear_bf16_link.w")
    m = w.rows
    if w.cols != k or w.halves != 1:
        raise KernelError(f"linear_bf16_link: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    _chk(x, "linear_bf16_link.x", lp)
    _chk(w.data, "linear_bf16_link.w", lp)
    _chk(out, "linear_bf16_link.out", torch.float32, (n, m))
    if bias is not None:
        _chk(bias, "linear_bf16_link.bias", torch.float32, (m,))
    if residual is not None:
        _chk(residual, "linear_bf16_link.residual", torch.float32, (n, m))
        if not linear_bf16_adds_residual(n, m, k):
            raise KernelError(f"linear_bf16_link: {n} rows of [{m}, {k}] do not take a residual (linear_bf16_adds_residual)")
    n_ssq = 0
    if ssq_in is not None:
        _chk(ssq_in, "linear_bf16_link.ssq_in", torch.float32)
        if ssq_in.dim() != 2 or ssq_in.shape[1] != link_stride(n):
            raise KernelError(f"linear_bf16_link.ssq_in: shape {tuple(ssq_in.shape)}, expected [shares, {link_stride(n)}]")
        n_ssq = ssq_in.shape[0]
    if xn_out is not None:
        shares = linear_bf16_link_shares(n, m, k)
        if residual is None or shares == 0:
            raise KernelError(f"linear_bf16_link: {n} rows of [{m}, {k}] cannot hand a norm on (linear_bf16_link_shares)")
        _chk(xn_out, "linear_bf16_link.xn_out", lp, (n, m))
        _chk(gain_next, "linear_bf16_link.gain_next", torch.float32, (m,))
        _chk(ssq_out, "linear_bf16_link.ssq_out", torch.float32, (shares, link_stride(n)))
    need = linear_bf16_workspace(n, m, k) if n > 16 else 0
    if need:
        if workspace is None or workspace.numel() < need:
            raise KernelError(f"linear_bf16_link: x [{n}, {k}] with W [{m}, {k}] needs a workspace of {need} floats")
        _chk(workspace, "linear_bf16_link.workspace", torch.float32)
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_linear_bf16_link", _ptr(x), _ptr(w.data), _ptr(bias), _ptr(residual), _ptr(out),
         _ptr(workspace if need else None), _i(n), _i(m), _i(k), _ptr(ssq_in), _i(n_ssq), _f(eps_in), _ptr(xn_out),
         _ptr(gain_next), _ptr(ssq_out), _stream())
    return out


def gated_linear_bf16_link(x: torch.Tensor, w: PackedMatrix, out: torch.Tensor, ssq_in: torch.Tensor,
                           eps_in: float) -> torch.Tensor:
    """gated_linear_bf16 behind an RMSNorm that the product in front has prepared: x = bf16(h * gain), ssq_in its
    shares of the rows' sums of squares (up to 64 rows)."""
    n, k = x.shape
    lp = _lowp(w.data, "gated_linear_bf16_link.w")
    if w.cols != k or w.halves != 2:
        raise KernelError(f"gated_linear_bf16_link: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    _chk(x, "gated_linear_bf16_link.x", lp)
    _chk(w.data, "gated_linear_bf16_link.w", lp)
    _chk(out, "gated_linear_bf16_link.out", None, (n, w.rows))
    _chk(ssq_in, "gated_linear_bf16_link.ssq_in", torch.float32)
    if n > 64 or ssq_in.dim() != 2 or ssq_in.shape[1] != link_stride(n):
        raise KernelError(f"gated_linear_bf16_link: {n} rows, ssq_in of shape {tuple(ssq_in.shape)}: up to 64 rows and "
                          f"[shares, {link_stride(n)}]")
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_gated_linear_bf16_link", _ptr(x), _ptr(w.data), _ptr(out), _i(_code(out)), _i(n),
         _i(w.rows), _i(k), _ptr(ssq_in), _i(ssq_in.shape[0]), _f(eps_in), _stream())
    return out


def gated_linear_bf16(x: torch.Tensor, w_gate_up, out: torch.Tensor, norm_gain: Optional[torch.Tensor] = None,
                      norm_eps: float = 0.0) -> torch.Tensor:
    """out = silu(x Wg^T) * (x Wu^T).  w_gate_up: a PackedMatrix of two halves (pack_matrix_bf16(w, halves=2)), or
    the stacked [2 I, k] tensor, which is packed on the spot.  With norm_gain (up to 16 rows), x is the float32
    residual stream and rmsnorm(x; gain, eps) is what gets multiplied."""
    n, k = x.shape
    lp = _lowp((w_gate_up.data if isinstance(w_gate_up, PackedMatrix) else w_gate_up), "gated_linear_bf16.w")
    if not isinstance(w_gate_up, PackedMatrix):
        _chk(w_gate_up, "gated_linear_bf16.w", lp, (w_gate_up.shape[0], k))
        w_gate_up = pack_matrix_bf16(w_gate_up, halves=2)
    w = w_gate_up
    if w.cols != k or w.halves != 2:
        raise KernelError(f"gated_linear_bf16: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    _chk(x, "gated_linear_bf16.x", torch.float32 if norm_gain is not None else lp)
    _chk(w.data, "gated_linear_bf16.w", lp)
    _chk(out, "gated_linear_bf16.out", None, (n, w.rows))
    if norm_gain is not None:
        if n > 16 or k % 8:
            raise KernelError(f"gated_linear_bf16: the fused norm takes at most 16 rows and k a multiple of 8 (n={n}, k={k})")
        _chk(norm_gain, "gated_linear_bf16.norm_gain", torch.float32, (k,))
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_gated_linear_bf16", _ptr(x), _ptr(w.data), _ptr(out), _i(_code(out)), _i(n),
         _i(w.rows), _i(k), _ptr(norm_gain), _f(norm_eps), _stream())
    return out


def gated_linear_bf16_form(x: torch.Tensor, w: PackedMatrix, bias: Optional[torch.Tensor], out: torch.Tensor,
                           alpha: float, limit: float, shift: float, norm_gain: Optional[torch.Tensor] = None,
                           norm_eps: float = 0.0, ssq_in: Optional[torch.Tensor] = None, cubic: float = 0.0) -> torch.Tensor:
    """out = gate(x Wg^T + bias[:I], x Wu^T + bias[I:]) with gate(g, u) = g' sigmoid(alpha g' (1 + cubic g'^2)) (u' + shift),
    g' = min(g, limit), u' = clamp(u, -limit, limit) (limit 0: no bounds); w: two packed halves.  x: 16-bit tokens;
    or with norm_gain the float32 residual stream whose RMSNorm is what gets multiplied (up to 16 rows); or with
    ssq_in a norm that the product in front has prepared (gated_linear_bf16_link's x and ssq_in, eps in norm_eps)."""
    n, k = x.shape
    lp = _lowp(w.data, "gated_linear_bf16_form.w")
    if w.cols != k or w.halves != 2:
        raise KernelError(f"gated_linear_bf16_form: x [{n}, {k}] does not fit a packed matrix [{w.rows}, {w.cols}] x {w.halves}")
    if norm_gain is not None and ssq_in is not None:
        raise KernelError("gated_linear_bf16_form: a norm in front is applied here or was prepared, not both")
    _chk(x, "gated_linear_bf16_form.x", torch.float32 if norm_gain is not None else lp)
    _chk(w.data, "gated_linear_bf16_form.w", lp)
    _chk(out, "gated_linear_bf16_form.out", None, (n, w.rows))
    if bias is not None:
        _chk(bias, "gated_linear_bf16_form.bias", torch.float32, (2 * w.rows,))
    if norm_gain is not None:
        if n > 16 or k % 8:
            raise KernelError(f"gated_linear_bf16_form: the fused norm takes at most 16 rows and k a multiple of 8 (n={n}, k={k})")
        _chk(norm_gain, "gated_linear_bf16_form.norm_gain", torch.float32, (k,))
    n_ssq = 0
    if ssq_in is not None:
        _chk(ssq_in, "gated_linear_bf16_form.ssq_in", torch.float32)
        if n > 64 or ssq_in.dim() != 2 or ssq_in.shape[1] != link_stride(n):
            raise KernelError(f"gated_linear_bf16_form: {n} rows, ssq_in of shape {tuple(ssq_in.shape)}: up to 64 rows and "
                              f"[shares, {link_stride(n)}]")
        n_ssq = ssq_in.shape[0]
    if not alpha > 0 or limit < 0:
        raise KernelError(f"gated_linear_bf16_form: gate with alpha {alpha} and limit {limit}")
    _run(load_lib("vt_gemm_bf16", half=_half(w.data, x, out)), "vt_gated_linear_bf16_form", _ptr(x), _ptr(w.data), _ptr(bias),
         _ptr(out), _i(_code(out)), _i(n), _i(w.rows), _i(k), _ptr(norm_gain), _f(norm_eps), _ptr(ssq_in), _i(n_ssq),
         _f(alpha), _f(limit), _f(shift), _f(cubic), _stream())
    return out


# ---------------------------------------------------------------------------
def attention_f32(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, positions: torch.Tensor,
                  tok_entry: torch.Tensor, block_table: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv: int,
                  head_dim: int, window: int, scale: float) -> torch.Tensor:
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    _chk(q, "attention_f32.q", torch.float32, (n, n_heads * head_dim))
    _chk(k_pages, "attention_f32.k_pages", torch.float32, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_f32.v_pages", torch.float32, (num_pages, n_kv, head_dim, page_size))
    _chk(positions, "attention_f32.positions", torch.int32, (n,))
    _chk(tok_entry, "attention_f32.tok_entry", torch.int32, (n,))
    _chk(block_table, "attention_f32.block_table", torch.int32)
    _chk(out, "attention_f32.out", torch.float32, (n, n_heads * head_dim))
    _run(load_lib("vt_attn_f32"), "vt_attn_f32", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(positions), _ptr(tok_entry),
         _ptr(block_table), _ptr(out), _i(n), _i(n_heads), _i(n_kv), _i(head_dim), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


ATTN_F32_MAX_HEAD_DIM = 256     # the float32 attention kernel keeps a head's dims in a block's registers: up to this many
ATTN_ITEM_INTS = 8
ATTN_CITEM_INTS = 6


def attention_bf16(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                   items: torch.Tensor, n_items: int, citems: Optional[torch.Tensor], n_citems: int, out: torch.Tensor,
                   part_o: Optional[torch.Tensor], part_ml: Optional[torch.Tensor], n_heads: int, n_kv: int,
                   head_dim: int, window: int, scale: float, max_part: int = 0, rt: int = 1) -> torch.Tensor:
    """`items` [>=n_items, 8] int32: entry, q_tok0, q_len, pos0, first row, key_lo, key_hi, partial index (-1 = final);
    an item covers 16 * rt rows.  `citems` [>=n_citems, 6] int32: q_tok0, q_len, first row of a 16-row tile, first
    partial index, number of items, tile index within the item.  The planner (engine) makes them; `max_part` is the
    number of partial indices it used, checked against the workspace here."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16: head size {head_dim} is not a multiple of 16 in 16..256")
    if rt not in (1, 2, 3):
        raise KernelError(f"attention_bf16: {rt} row tiles per item (1 or 2)")
    _chk(q, "attention_bf16.q", lp, (n, n_heads * head_dim))
    _chk(k_pages, "attention_bf16.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16.block_table", torch.int32)
    _chk(items, "attention_bf16.items", torch.int32)
    _chk(out, "attention_bf16.out", lp, (n, n_heads * head_dim))
    if items.numel() < n_items * ATTN_ITEM_INTS:
        raise KernelError("attention_bf16: item list shorter than n_items")
    if n_citems:
        _chk(citems, "attention_bf16.citems", torch.int32)
        _chk(part_o, "attention_bf16.part_o", torch.float32)
        _chk(part_ml, "attention_bf16.part_ml", torch.float32)
        if citems.numel() < n_citems * ATTN_CITEM_INTS:
            raise KernelError("attention_bf16: combine list shorter than n_citems")
        if part_o.numel() < max_part * rt * n_kv * 16 * head_dim or part_ml.numel() < max_part * rt * n_kv * 16 * 2:
            raise KernelError("attention_bf16: workspace for split keys is too small")
    lib = load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out))
    _run(lib, "vt_attn_bf16", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), _ptr(items), _i(n_items), _i(rt),
         _ptr(citems), _i(n_citems), _ptr(out), _ptr(part_o), _ptr(part_ml), _i(n_heads), _i(n_kv), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


def attention_bf16_direct(head_dim: int) -> bool:
    """Whether the bfloat16 attention kernels of this head size load their key/value blocks straight into LDS; the
    host cuts their work differently then (parts.attention_plan)."""
    return bool(_any_build("vt_attn_bf16", head_dim).vt_attn_bf16_direct())


def attention_bf16_tiles(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                         items: torch.Tensor, n_items: int, out: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                         window: int, scale: float, rt: int = 1, citems: Optional[torch.Tensor] = None, n_citems: int = 0,
                         part_o: Optional[torch.Tensor] = None, part_ml: Optional[torch.Tensor] = None,
                         n_parts: int = 0) -> torch.Tensor:
    """Long portions: `items` as for attention_bf16, each 64 * rt rows of one entry against all the keys they may
    see, or (partial index >= 0) against one of several ranges of them; key and value blocks go through LDS once per
    block of four waves.  `citems` [>=n_citems, 6] as for attention_bf16, one per 16-row tile of every item whose keys
    were split (4 * rt tiles per item); part_o / part_ml: float32 workspaces of at least n_parts * 4 * rt * n_kv *
    16 * head_dim and n_parts * 4 * rt * n_kv * 32 elements."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16_tiles.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16_tiles: head size {head_dim} is not a multiple of 16 in 16..256")
    if rt not in (1, 2):
        raise KernelError(f"attention_bf16_tiles: {rt} row tiles per wave (1 or 2)")
    _chk(q, "attention_bf16_tiles.q", lp, (n, n_heads * head_dim))
    _chk(k_pages, "attention_bf16_tiles.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16_tiles.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16_tiles.block_table", torch.int32)
    _chk(items, "attention_bf16_tiles.items", torch.int32)
    _chk(out, "attention_bf16_tiles.out", lp, (n, n_heads * head_dim))
    if items.numel() < n_items * ATTN_ITEM_INTS:
        raise KernelError("attention_bf16_tiles: item list shorter than n_items")
    if n_citems or n_parts:
        if citems is None or part_o is None or part_ml is None:
            raise KernelError("attention_bf16_tiles: split keys need citems and the two workspaces")
        _chk(citems, "attention_bf16_tiles.citems", torch.int32)
        _chk(part_o, "attention_bf16_tiles.part_o", torch.float32)
        _chk(part_ml, "attention_bf16_tiles.part_ml", torch.float32)
        if citems.numel() < n_citems * ATTN_CITEM_INTS:
            raise KernelError("attention_bf16_tiles: combine list shorter than n_citems")
        if part_o.numel() < n_parts * 4 * rt * n_kv * 16 * head_dim or part_ml.numel() < n_parts * 4 * rt * n_kv * 32:
            raise KernelError(f"attention_bf16_tiles: workspaces too small for {n_parts} partial results")
    _run(load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out)), "vt_attn_bf16_tiles", _ptr(q), _ptr(k_pages), _ptr(v_pages), _ptr(block_table),
         _ptr(items), _i(n_items), _i(rt), _ptr(citems if n_citems else None), _i(n_citems), _ptr(out),
         _ptr(part_o if n_citems else None), _ptr(part_ml if n_citems else None), _i(n_heads), _i(n_kv), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


def attention_bf16_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                          entry_pos0: torch.Tensor, dec_params: torch.Tensor, p_max: int, out: torch.Tensor,
                          part_o: torch.Tensor, part_ml: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                          window: int, scale: float) -> torch.Tensor:
    """One token per entry (token i is entry i at position entry_pos0[i]); every entry's keys are cut into at most
    p_max items of dec_params[0] keys.  All that changes from step to step is read from device memory."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16_decode.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16_decode: head size {head_dim} is not a multiple of 16 in 16..256")
    _chk(q, "attention_bf16_decode.q", lp, (n, n_heads * head_dim))
    _chk(k_pages, "attention_bf16_decode.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16_decode.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16_decode.block_table", torch.int32)
    if block_table.shape[0] < n:
        raise KernelError("attention_bf16_decode: fewer block table rows than entries")
    _chk(entry_pos0, "attention_bf16_decode.entry_pos0", torch.int32, (n,))
    _chk(dec_params, "attention_bf16_decode.dec_params", torch.int32)
    _chk(out, "attention_bf16_decode.out", lp, (n, n_heads * head_dim))
    _chk(part_o, "attention_bf16_decode.part_o", torch.float32)
    _chk(part_ml, "attention_bf16_decode.part_ml", torch.float32)
    if part_o.numel() < n * p_max * n_kv * 16 * head_dim or part_ml.numel() < n * p_max * n_kv * 32:
        raise KernelError("attention_bf16_decode: workspace too small")
    _run(load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out)), "vt_attn_bf16_decode", _ptr(q), _ptr(k_pages), _ptr(v_pages),
         _ptr(block_table), _ptr(entry_pos0), _ptr(dec_params), _i(n), _i(p_max), _ptr(out), _ptr(part_o), _ptr(part_ml),
         _i(n_heads), _i(n_kv), _i(page_size), _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


def attention_bf16_decode_fused(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                                k_pages: torch.Tensor, v_pages: torch.Tensor, block_table: torch.Tensor,
                                entry_pos0: torch.Tensor, dec_params: torch.Tensor, p_max: int, out: torch.Tensor,
                                part_o: torch.Tensor, part_ml: torch.Tensor, n_heads: int, n_kv: int, head_dim: int,
                                window: int, scale: float) -> torch.Tensor:
    """attention_bf16_decode from the projections' fp32 output (queries, keys, values of token i = entry i in row i):
    the attention kernel rotates queries and the new key and writes key and value into the token's page itself."""
    n = qkv.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    lp = _lowp(k_pages, "attention_bf16_decode_fused.k_pages")
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention_bf16_decode_fused: head size {head_dim} is not a multiple of 16 in 16..256")
    _chk(qkv, "attention_bf16_decode_fused.qkv", torch.float32)
    if qkv.dim() != 2 or qkv.shape[1] < (n_heads + 2 * n_kv) * head_dim or qkv.stride(1) != 1:
        raise KernelError(f"attention_bf16_decode_fused.qkv: shape {tuple(qkv.shape)} does not hold {n_heads}+2x{n_kv} heads of {head_dim}")
    rot = max_pos = 0
    if cos is not None:
        _chk(cos, "attention_bf16_decode_fused.cos", torch.float32)
        _chk(sin, "attention_bf16_decode_fused.sin", torch.float32, cos.shape)
        max_pos, half = cos.shape
        rot = 2 * half
        if rot % 16 or rot > head_dim:
            raise KernelError(f"attention_bf16_decode_fused: {rot} rotated dims (a multiple of 16 up to {head_dim})")
    _chk(k_pages, "attention_bf16_decode_fused.k_pages", lp, (num_pages, n_kv, page_size, head_dim))
    _chk(v_pages, "attention_bf16_decode_fused.v_pages", lp, (num_pages, n_kv, head_dim, page_size))
    _chk(block_table, "attention_bf16_decode_fused.block_table", torch.int32)
    if block_table.shape[0] < n:
        raise KernelError("attention_bf16_decode_fused: fewer block table rows than entries")
    _chk(entry_pos0, "attention_bf16_decode_fused.entry_pos0", torch.int32, (n,))
    _chk(dec_params, "attention_bf16_decode_fused.dec_params", torch.int32)
    _chk(out, "attention_bf16_decode_fused.out", lp, (n, n_heads * head_dim))
    _chk(part_o, "attention_bf16_decode_fused.part_o", torch.float32)
    _chk(part_ml, "attention_bf16_decode_fused.part_ml", torch.float32)
    if part_o.numel() < n * p_max * n_kv * 16 * head_dim or part_ml.numel() < n * p_max * n_kv * 32:
        raise KernelError("attention_bf16_decode_fused: workspace too small")
    _run(load_lib("vt_attn_bf16", head_dim, half=_half(k_pages, v_pages, out)), "vt_attn_bf16_decode_fused", _ptr(qkv), ctypes.c_longlong(qkv.stride(0)),
         _ptr(cos), _ptr(sin), _i(rot), _i(max_pos), _ptr(k_pages), _ptr(v_pages), _ptr(block_table), _ptr(entry_pos0),
         _ptr(dec_params), _i(n), _i(p_max), _ptr(out), _ptr(part_o), _ptr(part_ml), _i(n_heads), _i(n_kv),
         _i(page_size), _i(block_table.shape[1]), _i(num_pages), _i(window), _f(scale), _stream())
    return out


# ---------------------------------------------------------------------------
# attention with separate key and value sizes, capped scores, chunk or window masks and head gates (vt_attn_masked.hip)
MASKED_MAX_KEY_DIM = 256        # what vt_qk_prepare takes
MASKED_MAX_VALUE_DIM = 1024     # what vt_attn_masked takes (its keys: up to ATTN_MASKED_MAX_KEY_DIM); the matrix-core kernels 256
ATTN_MASKED_MAX_KEY_DIM = 8192


def qk_prepare(x: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
               tok_entry: torch.Tensor, block_table: Optional[torch.Tensor], q_out: torch.Tensor,
               k_pages: Optional[torch.Tensor], v_pages: Optional[torch.Tensor], n_heads: int, n_kv: int, key_dim: int,
               value_dim: int, unit_rms_eps: Optional[float], write_kv: bool = True,
               q_temp: Optional[tuple] = None, v_first: Optional[torch.Tensor] = None,
               v_lambda: Optional[torch.Tensor] = None, q_gain: Optional[torch.Tensor] = None,
               k_gain: Optional[torch.Tensor] = None) -> None:
    """x [n, >= (H + G) D + G Dv]: query heads, key heads, value heads.  Rotates the leading 2 * cos.shape[1] elements
    of every query and key head by the tables' angles at `positions`, divides each head by its root mean square
    (eps inside the root) unless unit_rms_eps is None, writes queries to q_out [n, H * D] and, with write_kv, keys and
    values into their pages ([page][kv][slot][D] and, transposed, [page][kv][Dv][slot]).
    q_temp (coef, every): the queries of position p times 1 + coef ln(floor((p + 1) / every) + 1).
    v_first (float32 [n, G * Dv]): without v_lambda the tokens' values are left there as well; with v_lambda (one
    float32 on the device) the pages get (1 - lambda) v + lambda v_first instead of v.
    q_gain / k_gain (float32 [D], shared by the heads): a gain per element on the scaled queries / keys."""
    n = x.shape[0]
    _chk(x, "qk_prepare.x")
    for g, name in ((q_gain, "q_gain"), (k_gain, "k_gain")):
        if g is not None:
            _chk(g, "qk_prepare." + name, torch.float32, (key_dim,))
    need = (n_heads + (n_kv if write_kv else 0)) * key_dim + (n_kv * value_dim if write_kv else 0)
    if x.dim() != 2 or x.shape[1] < need:
        raise KernelError(f"qk_prepare.x: shape {tuple(x.shape)}, need {need} columns")
    _chk(positions, "qk_prepare.positions", torch.int32, (n,))
    _chk(tok_entry, "qk_prepare.tok_entry", torch.int32, (n,))
    _chk(q_out, "qk_prepare.q_out", None, (n, n_heads * key_dim))
    if q_out.dtype != torch.float32 and x.dtype not in (torch.float32, q_out.dtype):
        raise KernelError(f"qk_prepare: {x.dtype} inputs and {q_out.dtype} queries")
    if q_out.dtype == torch.float32 and x.dtype != torch.float32:
        raise KernelError("qk_prepare: float32 queries need float32 inputs")
    rot = max_pos = 0
    if cos is not None:
        _chk(cos, "qk_prepare.cos", torch.float32)
        _chk(sin, "qk_prepare.sin", torch.float32, cos.shape)
        max_pos, half = cos.shape
        rot = 2 * half
        if rot > key_dim:
            raise KernelError(f"qk_prepare: {rot} rotated elements in heads of {key_dim}")
    page_size = num_pages = max_blocks = 0
    if write_kv:
        _chk(k_pages, "qk_prepare.k_pages", q_out.dtype)
        num_pages, kvh, page_size, d = k_pages.shape
        if (kvh, d) != (n_kv, key_dim):
            raise KernelError(f"qk_prepare.k_pages: shape {tuple(k_pages.shape)} does not fit kv heads {n_kv} x {key_dim}")
        _chk(v_pages, "qk_prepare.v_pages", q_out.dtype, (num_pages, n_kv, value_dim, page_size))
        _chk(block_table, "qk_prepare.block_table", torch.int32)
        max_blocks = block_table.shape[1]
    coef, every = (float(q_temp[0]), int(q_temp[1])) if q_temp else (0.0, 0)
    if q_temp and every <= 0:
        raise KernelError(f"qk_prepare: a query factor every {every} positions")
    vmix = 0
    if v_first is not None:
        if not write_kv:
            raise KernelError("qk_prepare: values are mixed on their way into the pages")
        _chk(v_first, "qk_prepare.v_first", torch.float32, (n, n_kv * value_dim))
        vmix = 1
        if v_lambda is not None:
            _chk(v_lambda, "qk_prepare.v_lambda", torch.float32)
            if v_lambda.numel() != 1:
                raise KernelError("qk_prepare.v_lambda: one number")
            vmix = 2
    _run(load_lib("vt_attn_masked", half=_half(x, q_out)), "vt_qk_prepare", _ptr(x), _i(_code(x)),
         ctypes.c_longlong(x.stride(0)), _ptr(cos), _ptr(sin), _i(rot), _i(max_pos), _ptr(positions), _ptr(tok_entry),
         _ptr(block_table), _i(max_blocks), _ptr(q_out), _ptr(k_pages), _ptr(v_pages), _i(_code(q_out)), _i(page_size),
         _i(num_pages), _i(n), _i(n_heads), _i(n_kv), _i(key_dim), _i(value_dim), _i(1 if write_kv else 0),
         _i(0 if unit_rms_eps is None else 1), _f(unit_rms_eps or 0.0), _f(coef), _i(every), _i(vmix), _ptr(v_first),
         _ptr(v_lambda if vmix == 2 else None), _ptr(q_gain), _ptr(k_gain), _stream())


def attention_masked(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, positions: torch.Tensor,
                     tok_entry: torch.Tensor, block_table: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv: int,
                     key_dim: int, value_dim: int, scale: float, cap: float = 0.0, window: int = 0, chunk: int = 0,
                     gate: Optional[torch.Tensor] = None, gate_column: int = 0, sink: Optional[torch.Tensor] = None,
                     slopes: Optional[torch.Tensor] = None, dist_log: Optional[tuple] = None,
                     score_shift: Optional[torch.Tensor] = None, sigmoid_weights: bool = False,
                     gate_wide: bool = False) -> torch.Tensor:
    """out [n, H * Dv] = softmax over the seen keys of cap * tanh(scale q.k / cap) (cap 0: scale q.k), times V, times
    sigmoid(gate[:, gate_column + head]) if `gate` (a 2-d tensor whose rows are the tokens') is given.  Key j is seen
    from position i if j <= i, i - j < window (0: unbounded) and j is in i's chunk of `chunk` positions (0: unbounded).
    slopes (float32 [H]): slopes[h] * (i - j) is taken off the score; sink (float32 [H]): exp(sink[h]) is added to the
    softmax's denominator.  dist_log (r1, r2), float32 [H] each: r1[h] ln(1 + r2[h] (i - j)) is taken off the score;
    score_shift (float32 [H]): a number per head added to every score; sigmoid_weights: the weight of a seen key is
    sigmoid(score), nothing is normalized; gate_wide: the gate is one logit per output element, gate[:, gate_column +
    head * Dv + d]."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    dt = q.dtype
    _chk(q, "attention_masked.q", None, (n, n_heads * key_dim))
    _chk(k_pages, "attention_masked.k_pages", dt, (num_pages, n_kv, page_size, key_dim))
    _chk(v_pages, "attention_masked.v_pages", dt, (num_pages, n_kv, value_dim, page_size))
    _chk(out, "attention_masked.out", dt, (n, n_heads * value_dim))
    _chk(positions, "attention_masked.positions", torch.int32, (n,))
    _chk(tok_entry, "attention_masked.tok_entry", torch.int32, (n,))
    _chk(block_table, "attention_masked.block_table", torch.int32)
    if value_dim > MASKED_MAX_VALUE_DIM:
        raise KernelError(f"attention_masked: value heads of {value_dim} (up to {MASKED_MAX_VALUE_DIM})")
    gptr, gcode, ldg = ctypes.c_void_p(0), F32, 0
    if gate is not None:
        _chk(gate, "attention_masked.gate")
        g_cols = n_heads * value_dim if gate_wide else n_heads
        if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < gate_column + g_cols:
            raise KernelError(f"attention_masked.gate: shape {tuple(gate.shape)} has no {g_cols} columns from {gate_column}")
        if dt == torch.float32 and gate.dtype != torch.float32:
            raise KernelError("attention_masked: float32 attention takes float32 gates")
        gptr = ctypes.c_void_p(gate.data_ptr() + gate_column * gate.element_size())
        gcode, ldg = _code(gate), gate.stride(0)
    _per_head(sink, "attention_masked.sink", n_heads)
    _per_head(slopes, "attention_masked.slopes", n_heads)
    r1, r2 = _score_forms("attention_masked", n_heads, dist_log, score_shift, sigmoid_weights, sink)
    _run(load_lib("vt_attn_masked", half=_half(q, gate)), "vt_attn_masked", _ptr(q), _ptr(k_pages), _ptr(v_pages), _i(_code(q)),
         _ptr(positions), _ptr(tok_entry), _ptr(block_table), gptr, _i(gcode), ctypes.c_longlong(ldg), _ptr(out), _i(n),
         _i(n_heads), _i(n_kv), _i(key_dim), _i(value_dim), _i(page_size), _i(block_table.shape[1]), _i(num_pages),
         _i(window), _i(chunk), _f(scale), _f(cap), _ptr(sink), _ptr(slopes), _ptr(r1), _ptr(r2), _ptr(score_shift),
         _i(1 if sigmoid_weights else 0), _i(1 if (gate_wide and gate is not None) else 0), _stream())
    return out


def _score_forms(who: str, n_heads: int, dist_log, score_shift, sigmoid_weights: bool, sink):
    """Checks of the score's optional forms that the three masked attention kernels share; returns (r1, r2)."""
    r1 = r2 = None
    if dist_log is not None:
        r1, r2 = dist_log
        _per_head(r1, who + ".dist_log[0]", n_heads)
        _per_head(r2, who + ".dist_log[1]", n_heads)
        if r1 is None or r2 is None:
            raise KernelError(who + ": the distance bias takes both of its numbers per head")
    _per_head(score_shift, who + ".score_shift", n_heads)
    if sigmoid_weights and sink is not None:
        raise KernelError(who + ": sigmoid weights have no denominator for a sink to join")
    return r1, r2


def _per_head(t: Optional[torch.Tensor], name: str, n_heads: int) -> None:
    if t is not None:
        _chk(t, name, torch.float32, (n_heads,))


def attention_masked_mfma_takes(key_dim: int, value_dim: int, page_size: int) -> bool:
    """Whether the matrix-core kernel takes heads and pages of these sizes."""
    return (key_dim % 16 == 0 and value_dim % 16 == 0 and 16 <= key_dim <= 256 and 16 <= value_dim <= 256
            and page_size % 16 == 0)


def attention_masked_mfma(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, positions: torch.Tensor,
                          tok_entry: torch.Tensor, block_table: torch.Tensor, tiles: torch.Tensor, out: torch.Tensor,
                          n_heads: int, n_kv: int, key_dim: int, value_dim: int, scale: float, cap: float = 0.0,
                          window: int = 0, chunk: int = 0, gate: Optional[torch.Tensor] = None,
                          gate_column: int = 0, sink: Optional[torch.Tensor] = None,
                          slopes: Optional[torch.Tensor] = None, dist_log: Optional[tuple] = None,
                          score_shift: Optional[torch.Tensor] = None, sigmoid_weights: bool = False,
                          gate_wide: bool = False) -> torch.Tensor:
    """attention_masked for the 16-bit types on the matrix cores.  tiles: int32 [n_tiles, 2], (first row, rows) of
    runs of up to 16 consecutive tokens of one request that together cover every token of the step once."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    dt = _lowp(q, "attention_masked_mfma.q")
    if not attention_masked_mfma_takes(key_dim, value_dim, page_size):
        raise KernelError(f"attention_masked_mfma: heads of {key_dim}/{value_dim} and pages of {page_size} "
                          f"(multiples of 16 up to 256)")
    _chk(q, "attention_masked_mfma.q", dt, (n, n_heads * key_dim))
    _chk(k_pages, "attention_masked_mfma.k_pages", dt, (num_pages, n_kv, page_size, key_dim))
    _chk(v_pages, "attention_masked_mfma.v_pages", dt, (num_pages, n_kv, value_dim, page_size))
    _chk(out, "attention_masked_mfma.out", dt, (n, n_heads * value_dim))
    _chk(positions, "attention_masked_mfma.positions", torch.int32, (n,))
    _chk(tok_entry, "attention_masked_mfma.tok_entry", torch.int32, (n,))
    _chk(block_table, "attention_masked_mfma.block_table", torch.int32)
    _chk(tiles, "attention_masked_mfma.tiles", torch.int32)
    if tiles.numel() % 2:
        raise KernelError("attention_masked_mfma.tiles: pairs of (first row, rows)")
    gptr, gcode, ldg = ctypes.c_void_p(0), F32, 0
    if gate is not None:
        _chk(gate, "attention_masked_mfma.gate")
        g_cols = n_heads * value_dim if gate_wide else n_heads
        if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < gate_column + g_cols:
            raise KernelError(f"attention_masked_mfma.gate: shape {tuple(gate.shape)} has no {g_cols} columns from {gate_column}")
        gptr = ctypes.c_void_p(gate.data_ptr() + gate_column * gate.element_size())
        gcode, ldg = _code(gate), gate.stride(0)
    _per_head(sink, "attention_masked_mfma.sink", n_heads)
    _per_head(slopes, "attention_masked_mfma.slopes", n_heads)
    r1, r2 = _score_forms("attention_masked_mfma", n_heads, dist_log, score_shift, sigmoid_weights, sink)
    _run(load_lib("vt_attn_masked_mfma", (key_dim, value_dim), half=_half(q, gate)), "vt_attn_masked_mfma", _ptr(q), _ptr(k_pages),
         _ptr(v_pages), _ptr(positions), _ptr(tok_entry), _ptr(block_table), _ptr(tiles), _i(tiles.numel() // 2), gptr,
         _i(gcode), ctypes.c_longlong(ldg), _ptr(out), _i(n_heads), _i(n_kv), _i(key_dim), _i(value_dim), _i(page_size),
         _i(block_table.shape[1]), _i(num_pages), _i(window), _i(chunk), _f(scale), _f(cap), _ptr(sink), _ptr(slopes),
         _ptr(r1), _ptr(r2), _ptr(score_shift), _i(1 if sigmoid_weights else 0),
         _i(1 if (gate_wide and gate is not None) else 0), _stream())
    return out


def attention_masked_decode_splits(n: int, n_heads: int, n_kv: int, max_len: int) -> int:
    """Into how many blocks of four waves a decoding step's keys are dealt per (token, group of heads): enough to give
    every compute unit a few waves, no more than there are turns of 32 keys in the longest sequence.  It depends on
    the number of tokens and the engine's limits alone, so that a recorded step can be replayed."""
    tiles = max(1, n) * n_kv * (-(-(n_heads // n_kv) // 16))
    return int(max(1, min(-(-512 // tiles), max(1, max_len // 128), 16)))


def attention_masked_decode(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, positions: torch.Tensor,
                            tok_entry: torch.Tensor, block_table: torch.Tensor, out: torch.Tensor, part: torch.Tensor,
                            splits: int, n_heads: int, n_kv: int, key_dim: int, value_dim: int, scale: float,
                            cap: float = 0.0, window: int = 0, chunk: int = 0, gate: Optional[torch.Tensor] = None,
                            gate_column: int = 0, sink: Optional[torch.Tensor] = None,
                            slopes: Optional[torch.Tensor] = None, dist_log: Optional[tuple] = None,
                            score_shift: Optional[torch.Tensor] = None, sigmoid_weights: bool = False,
                            gate_wide: bool = False) -> torch.Tensor:
    """attention_masked for steps of single tokens in the 16-bit types on the matrix cores: the rows of a product are
    the query heads that share a key/value head.  part: float32 scratch of attention_masked_decode_scratch floats."""
    n = q.shape[0]
    num_pages, kvh, page_size, d = k_pages.shape
    dt = _lowp(q, "attention_masked_decode.q")
    if not attention_masked_mfma_takes(key_dim, value_dim, page_size):
        raise KernelError(f"attention_masked_decode: heads of {key_dim}/{value_dim} and pages of {page_size} "
                          f"(multiples of 16 up to 256)")
    _chk(q, "attention_masked_decode.q", dt, (n, n_heads * key_dim))
    _chk(k_pages, "attention_masked_decode.k_pages", dt, (num_pages, n_kv, page_size, key_dim))
    _chk(v_pages, "attention_masked_decode.v_pages", dt, (num_pages, n_kv, value_dim, page_size))
    _chk(out, "attention_masked_decode.out", dt, (n, n_heads * value_dim))
    _chk(positions, "attention_masked_decode.positions", torch.int32, (n,))
    _chk(tok_entry, "attention_masked_decode.tok_entry", torch.int32, (n,))
    _chk(block_table, "attention_masked_decode.block_table", torch.int32)
    _chk(part, "attention_masked_decode.part", torch.float32)
    gptr, gcode, ldg = ctypes.c_void_p(0), F32, 0
    if gate is not None:
        _chk(gate, "attention_masked_decode.gate")
        g_cols = n_heads * value_dim if gate_wide else n_heads
        if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < gate_column + g_cols:
            raise KernelError(f"attention_masked_decode.gate: shape {tuple(gate.shape)} has no {g_cols} columns from {gate_column}")
        gptr = ctypes.c_void_p(gate.data_ptr() + gate_column * gate.element_size())
        gcode, ldg = _code(gate), gate.stride(0)
    _per_head(sink, "attention_masked_decode.sink", n_heads)
    _per_head(slopes, "attention_masked_decode.slopes", n_heads)
    r1, r2 = _score_forms("attention_masked_decode", n_heads, dist_log, score_shift, sigmoid_weights, sink)
    _run(load_lib("vt_attn_masked_mfma", (key_dim, value_dim), half=_half(q, gate)), "vt_attn_masked_decode", _ptr(q),
         _ptr(k_pages), _ptr(v_pages), _ptr(positions), _ptr(tok_entry), _ptr(block_table), gptr, _i(gcode),
         ctypes.c_longlong(ldg), _ptr(out), _ptr(part), ctypes.c_longlong(part.numel()), _i(splits), _i(n), _i(n_heads),
         _i(n_kv), _i(key_dim), _i(value_dim), _i(page_size), _i(block_table.shape[1]), _i(num_pages), _i(window), _i(chunk),
         _f(scale), _f(cap), _ptr(sink), _ptr(slopes), _ptr(r1), _ptr(r2), _ptr(score_shift), _i(1 if sigmoid_weights else 0),
         _i(1 if (gate_wide and gate is not None) else 0), _stream())
    return out


def attention_masked_decode_scratch(n: int, n_heads: int, n_kv: int, value_dim: int, splits: int) -> int:
    """Floats of scratch memory that attention_masked_decode needs."""
    return n * n_kv * (-(-(n_heads // n_kv) // 16)) * 4 * splits * 16 * (value_dim + 4)


# ---------------------------------------------------------------------------
# attention over a low-rank cache (vt_latent.hip): what stands around the masked attention kernels
HEAD_LINEAR_MAX_IN = 8192


def latent_prepare(x: torch.Tensor, q_column: int, c_column: int, norm_w: torch.Tensor, eps: float,
                   cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], positions: torch.Tensor,
                   tok_entry: torch.Tensor, block_table: torch.Tensor, q_out: torch.Tensor, k_pages: torch.Tensor,
                   v_pages: torch.Tensor, n_heads: int, plain_dim: int, rot_dim: int, rank: int) -> None:
    """x [n, ...]: from column q_column the heads' queries, each [plain_dim | rot_dim]; from column c_column the
    low-rank part [rank | rot_dim].  c = the first `rank` over their root mean square (eps inside the root) times
    norm_w goes into the key page's leading `rank` elements and, transposed, into the value page; the `rot_dim`
    behind it, its leading 2 * cos.shape[1] elements rotated by the tables' angles at `positions`, into the key page
    behind c; every head's rot_dim query elements, rotated alike, into q_out[:, head, rank:].
    q_out [n, H * (rank + rot_dim)], k_pages [pages, 1, page_size, rank + rot_dim], v_pages [pages, 1, rank, page_size]."""
    n = x.shape[0]
    dk = rank + rot_dim
    _chk(x, "latent_prepare.x")
    if x.dim() != 2 or x.shape[1] < max(q_column + n_heads * (plain_dim + rot_dim), c_column + dk) or min(q_column, c_column) < 0:
        raise KernelError(f"latent_prepare.x: shape {tuple(x.shape)} does not hold the queries and the low-rank part")
    _chk(positions, "latent_prepare.positions", torch.int32, (n,))
    _chk(tok_entry, "latent_prepare.tok_entry", torch.int32, (n,))
    _chk(block_table, "latent_prepare.block_table", torch.int32)
    _chk(norm_w, "latent_prepare.norm_w", torch.float32, (rank,))
    _chk(q_out, "latent_prepare.q_out", None, (n, n_heads * dk))
    if q_out.dtype != torch.float32 and x.dtype not in (torch.float32, q_out.dtype):
        raise KernelError(f"latent_prepare: {x.dtype} inputs and {q_out.dtype} queries")
    if q_out.dtype == torch.float32 and x.dtype != torch.float32:
        raise KernelError("latent_prepare: float32 queries need float32 inputs")
    rot = max_pos = 0
    if cos is not None:
        _chk(cos, "latent_prepare.cos", torch.float32)
        _chk(sin, "latent_prepare.sin", torch.float32, cos.shape)
        max_pos, half = cos.shape
        rot = 2 * half
        if rot > rot_dim:
            raise KernelError(f"latent_prepare: {rot} rotated elements in a part of {rot_dim}")
    _chk(k_pages, "latent_prepare.k_pages", q_out.dtype)
    if k_pages.dim() != 4 or k_pages.shape[1] != 1 or k_pages.shape[3] != dk:
        raise KernelError(f"latent_prepare.k_pages: shape {tuple(k_pages.shape)}, expected [pages, 1, page_size, {dk}]")
    num_pages, _, page_size, _ = k_pages.shape
    _chk(v_pages, "latent_prepare.v_pages", q_out.dtype, (num_pages, 1, rank, page_size))
    _run(load_lib("vt_latent", half=_half(x, q_out)), "vt_latent_prepare", _ptr(x), _i(_code(x)),
         ctypes.c_longlong(x.stride(0)), _i(q_column), _i(c_column), _ptr(norm_w), _f(eps), _ptr(cos), _ptr(sin), _i(rot),
         _i(max_pos), _ptr(positions), _ptr(tok_entry), _ptr(block_table), _i(block_table.shape[1]), _ptr(q_out),
         _ptr(k_pages), _ptr(v_pages), _i(_code(q_out)), _i(page_size), _i(num_pages), _i(n), _i(n_heads), _i(plain_dim),
         _i(rot_dim), _i(rank), _stream())


def head_linear(x: torch.Tensor, x_column: int, x_head: int, w: torch.Tensor, transposed: bool, y: torch.Tensor,
                y_column: int, y_head: int, n_heads: int, n_in: int, n_out: int, gate: Optional[torch.Tensor] = None,
                gate_column: int = 0) -> torch.Tensor:
    """One small matrix per head: y[t, y_column + h * y_head + o] = sum_i W_h[o, i] x[t, x_column + h * x_head + i]
    (w [H * n_out, n_in]), or with `transposed` sum_i W_h[i, o] x[...] (w [H * n_in, n_out]); times
    sigmoid(gate[t, gate_column + h * n_out + o]) if `gate` is given.  x and y are 2-d tensors whose rows are the
    tokens'; float32 sums.  16-bit results come from the matrix cores (float32 inputs are rounded on their way in)."""
    n = x.shape[0]
    _chk(x, "head_linear.x")
    _chk(y, "head_linear.y")
    _chk(w, "head_linear.w", y.dtype, (n_heads * (n_in if transposed else n_out), n_out if transposed else n_in))
    if x.dim() != 2 or y.dim() != 2 or y.shape[0] != n:
        raise KernelError("head_linear: x and y are [tokens, columns]")
    if x_column < 0 or x.shape[1] < x_column + (n_heads - 1) * x_head + n_in or x_head < 0:
        raise KernelError(f"head_linear.x: shape {tuple(x.shape)} has no {n_heads} heads of {n_in} from column {x_column}")
    if y_column < 0 or y.shape[1] < y_column + (n_heads - 1) * y_head + n_out or y_head < n_out:
        raise KernelError(f"head_linear.y: shape {tuple(y.shape)} has no {n_heads} heads of {n_out} from column {y_column}")
    if n_in > HEAD_LINEAR_MAX_IN:
        raise KernelError(f"head_linear: {n_in} inputs per head (up to {HEAD_LINEAR_MAX_IN})")
    if y.dtype == torch.float32 and x.dtype != torch.float32:
        raise KernelError("head_linear: float32 results need float32 inputs")
    gptr, gcode, ldg = ctypes.c_void_p(0), F32, 0
    if gate is not None:
        _chk(gate, "head_linear.gate")
        if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < gate_column + n_heads * n_out:
            raise KernelError(f"head_linear.gate: shape {tuple(gate.shape)} has no {n_heads * n_out} columns from {gate_column}")
        if y.dtype == torch.float32 and gate.dtype != torch.float32:
            raise KernelError("head_linear: float32 results take float32 gates")
        gptr = ctypes.c_void_p(gate.data_ptr() + gate_column * gate.element_size())
        gcode, ldg = _code(gate), gate.stride(0)
    xptr = ctypes.c_void_p(x.data_ptr() + x_column * x.element_size())
    yptr = ctypes.c_void_p(y.data_ptr() + y_column * y.element_size())
    cores = (y.dtype in LOWP and n_in % 4 == 0 and x_head % 4 == 0 and x.stride(0) % 4 == 0 and x_column % 4 == 0)
    _run(load_lib("vt_latent", half=_half(x, y, gate)), "vt_head_linear", xptr, _i(_code(x)), ctypes.c_longlong(x.stride(0)),
         _i(x_head), _ptr(w), gptr, _i(gcode), ctypes.c_longlong(ldg), yptr, _i(_code(y)), ctypes.c_longlong(y.stride(0)),
         _i(y_head), _i(n), _i(n_heads), _i(n_in), _i(n_out), _i(1 if transposed else 0), _i(1 if cores else 0), _stream())
    return y


# ---------------------------------------------------------------------------
# the gated delta rule and what stands around it (vt_delta.hip)
DELTA_MAX_KEY_DIM = 256
CONV_MAX_TAPS = 16


def _state_rows(state: torch.Tensor, name: str, need: int):
    """state [slots, per_slot] float32 (a view whose rows may lie apart): (pointer, stride in floats)."""
    if not state.is_cuda or state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1:
        raise KernelError(f"{name}: state must be a float32 [slots, n] tensor on the GPU with unit stride in a slot")
    if state.shape[1] < need:
        raise KernelError(f"{name}: state slots of {state.shape[1]} floats, need {need}")
    return ctypes.c_void_p(state.data_ptr()), ctypes.c_longlong(state.stride(0))


def short_conv(x: torch.Tensor, channels: int, taps: torch.Tensor, state: torch.Tensor, tok_entry: torch.Tensor,
               entry_start: torch.Tensor, slots: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """y[t, c] = silu(sum_j taps[c, j] * x[t - (K-1) + j, c]) for the first `channels` columns of x, causal within
    each entry of the step; inputs from before the entry's first token are read from state[slot] ([K-1, channels],
    the oldest first).  The state is not changed (short_conv_carry does that, afterwards)."""
    n = x.shape[0]
    _chk(x, "short_conv.x")
    if x.dim() != 2 or x.shape[1] < channels:
        raise KernelError(f"short_conv.x: shape {tuple(x.shape)} has no {channels} channels")
    k = taps.shape[1]
    _chk(taps, "short_conv.taps", torch.float32, (channels, k))
    if not 1 <= k <= CONV_MAX_TAPS:
        raise KernelError(f"short_conv: {k} taps (1 to {CONV_MAX_TAPS})")
    _chk(y, "short_conv.y", None, (n, channels))
    _chk(tok_entry, "short_conv.tok_entry", torch.int32, (n,))
    _chk(entry_start, "short_conv.entry_start", torch.int32)
    _chk(slots, "short_conv.slots", torch.int32)
    n_entries = entry_start.numel() - 1
    sp, ss = _state_rows(state, "short_conv", (k - 1) * channels)
    _run(load_lib("vt_delta", half=_half(x, y)), "vt_short_conv", _ptr(x), _i(_code(x)), ctypes.c_longlong(x.stride(0)),
         _ptr(taps), sp, ss, _ptr(tok_entry), _ptr(entry_start), _ptr(slots), _ptr(y), _i(_code(y)), _i(n), _i(n_entries),
         _i(channels), _i(k), _stream())
    return y


def short_conv_carry(x: torch.Tensor, channels: int, k: int, state: torch.Tensor, entry_start: torch.Tensor,
                     slots: torch.Tensor) -> None:
    """state[slot] <- the last k - 1 inputs of every entry (older ones move up where an entry brought fewer)."""
    _chk(x, "short_conv_carry.x")
    _chk(entry_start, "short_conv_carry.entry_start", torch.int32)
    _chk(slots, "short_conv_carry.slots", torch.int32)
    if x.dim() != 2 or x.shape[1] < channels or not 1 <= k <= CONV_MAX_TAPS:
        raise KernelError(f"short_conv_carry: x of shape {tuple(x.shape)}, {channels} channels, {k} taps")
    sp, ss = _state_rows(state, "short_conv_carry", (k - 1) * channels)
    _run(load_lib("vt_delta", half=_half(x)), "vt_short_conv_carry", _ptr(x), _i(_code(x)), ctypes.c_longlong(x.stride(0)),
         sp, ss, _ptr(entry_start), _ptr(slots), _i(entry_start.numel() - 1), _i(channels), _i(k), _stream())


def delta_rule(qkv: torch.Tensor, ba: torch.Tensor, ba_column: int, a_log: torch.Tensor, dt_bias: torch.Tensor,
               state: torch.Tensor, entry_start: torch.Tensor, slots: torch.Tensor, out: torch.Tensor, n_heads: int,
               n_kv: int, key_dim: int, value_dim: int) -> torch.Tensor:
    """The gated delta rule over the tokens of every entry, from and into state[slot] ([H, Dv, D] float32).
    qkv [n, 2 G D + H Dv]: queries, keys (G heads of D), values (H heads of Dv); ba: a 2-d tensor whose rows are the
    tokens', with the H logits of the write strength from column ba_column and the H logits of the decay behind them
    (float32, or the 16-bit type of qkv).  out [n, H * Dv] float32."""
    n = qkv.shape[0]
    c = 2 * n_kv * key_dim + n_heads * value_dim
    _chk(qkv, "delta_rule.qkv", None, (n, c))
    _chk(ba, "delta_rule.ba")
    if ba.dim() != 2 or ba.shape[0] != n or ba.shape[1] < ba_column + 2 * n_heads:
        raise KernelError(f"delta_rule.ba: shape {tuple(ba.shape)} has no {2 * n_heads} columns from {ba_column}")
    if ba.dtype != torch.float32 and ba.dtype != qkv.dtype:
        raise KernelError(f"delta_rule: logits of dtype {ba.dtype} beside inputs of {qkv.dtype}")
    _chk(a_log, "delta_rule.a_log", torch.float32, (n_heads,))
    _chk(dt_bias, "delta_rule.dt_bias", torch.float32, (n_heads,))
    _chk(out, "delta_rule.out", torch.float32, (n, n_heads * value_dim))
    _chk(entry_start, "delta_rule.entry_start", torch.int32)
    _chk(slots, "delta_rule.slots", torch.int32)
    if key_dim > DELTA_MAX_KEY_DIM or n_heads % n_kv:
        raise KernelError(f"delta_rule: heads {n_heads}/{n_kv} of {key_dim}")
    sp, ss = _state_rows(state, "delta_rule", n_heads * key_dim * value_dim)
    bptr = ctypes.c_void_p(ba.data_ptr() + ba_column * ba.element_size())
    _run(load_lib("vt_delta", half=_half(qkv, ba)), "vt_delta_rule", _ptr(qkv), _i(_code(qkv)), bptr, _i(_code(ba)),
         ctypes.c_longlong(ba.stride(0)), _ptr(a_log), _ptr(dt_bias), sp, ss, _ptr(entry_start), _ptr(slots), _ptr(out),
         _i(entry_start.numel() - 1), _i(n_heads), _i(n_kv), _i(key_dim), _i(value_dim), _stream())
    return out


def gated_rmsnorm(o: torch.Tensor, weight: torch.Tensor, gate: torch.Tensor, gate_column: int, out: torch.Tensor,
                  n_heads: int, value_dim: int, eps: float, gate_kind: str = "silu") -> torch.Tensor:
    """out[t, h] = o[t, h] / sqrt(mean(o[t, h]^2) + eps) * weight * act(gate[t, gate_column + h * Dv ...]), per head;
    weight [Dv] (shared by the heads) or [H * Dv] (one per head); gate_kind "silu" or "sigmoid"."""
    n = o.shape[0]
    _chk(o, "gated_rmsnorm.o", torch.float32, (n, n_heads * value_dim))
    _chk(weight, "gated_rmsnorm.weight", torch.float32)
    if tuple(weight.shape) not in ((value_dim,), (n_heads * value_dim,)):
        raise KernelError(f"gated_rmsnorm.weight: shape {tuple(weight.shape)}, expected ({value_dim},) or ({n_heads * value_dim},)")
    per_head = tuple(weight.shape) == (n_heads * value_dim,) and n_heads > 1
    if gate_kind not in ("silu", "sigmoid"):
        raise KernelError(f"gated_rmsnorm: gate kind {gate_kind!r} ('silu' and 'sigmoid' are known)")
    _chk(gate, "gated_rmsnorm.gate")
    _chk(out, "gated_rmsnorm.out", None, (n, n_heads * value_dim))
    if gate.dim() != 2 or gate.shape[0] != n or gate.shape[1] < gate_column + n_heads * value_dim:
        raise KernelError(f"gated_rmsnorm.gate: shape {tuple(gate.shape)} has no {n_heads * value_dim} columns from {gate_column}")
    gptr = ctypes.c_void_p(gate.data_ptr() + gate_column * gate.element_size())
    _run(load_lib("vt_delta", half=_half(gate, out)), "vt_gated_rmsnorm", _ptr(o), _ptr(weight), gptr, _i(_code(gate)),
         ctypes.c_longlong(gate.stride(0)), _ptr(out), _i(_code(out)), _i(n), _i(n_heads), _i(value_dim), _f(eps),
         _i(1 if per_head else 0), _i(1 if gate_kind == "sigmoid" else 0), _stream())
    return out


def lowrank_tanh(x: torch.Tensor, x_column: int, w2: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                 tanh: bool = True, decay: Optional[tuple] = None) -> torch.Tensor:
    """out[t, j] = bias[j] + sum_l w2[j, l] * tanh(x[t, x_column + l]): float32 sums in the order of l, float32 results.
    x: a 2-d tensor whose rows are the tokens'; w2 [M, L] in float32 or the 16-bit type.  tanh False: the low-rank part
    enters as it is (the second half of a linear low-rank projection, kept in float32).  decay (a_log, per_head): the
    sums leave as decays, out = exp(-exp(a_log[j // per_head]) * softplus(sum)), a_log float32 [M / per_head]."""
    n = x.shape[0]
    m, low = w2.shape
    _chk(x, "lowrank_tanh.x")
    _chk(w2, "lowrank_tanh.w2")
    if x.dim() != 2 or x_column < 0 or x.shape[1] < x_column + low:
        raise KernelError(f"lowrank_tanh.x: shape {tuple(x.shape)} has no {low} columns from {x_column}")
    if x.dtype != torch.float32 and w2.dtype != x.dtype:
        raise KernelError(f"lowrank_tanh: inputs of {x.dtype} beside a matrix of {w2.dtype}")
    if bias is not None:
        _chk(bias, "lowrank_tanh.bias", torch.float32, (m,))
    _chk(out, "lowrank_tanh.out", torch.float32, (n, m))
    a_log, per_head = decay if decay is not None else (None, 0)
    if a_log is not None:
        if per_head <= 0 or m % per_head:
            raise KernelError(f"lowrank_tanh: {m} outputs in heads of {per_head}")
        _chk(a_log, "lowrank_tanh.a_log", torch.float32, (m // per_head,))
    xptr = ctypes.c_void_p(x.data_ptr() + x_column * x.element_size())
    _run(load_lib("vt_delta", half=_half(x, w2)), "vt_lowrank_tanh", xptr, _i(_code(x)), ctypes.c_longlong(x.stride(0)),
         _ptr(w2), _i(_code(w2)), _ptr(bias), _ptr(out), _i(n), _i(low), _i(m), _i(1 if tanh else 0), _ptr(a_log),
         _i(per_head), _stream())
    return out


def general_delta(x: torch.Tensor, r_column: int, k_column: int, v_column: int, a_column: int, decay_logits: torch.Tensor,
                  a_bias: Optional[torch.Tensor], state: torch.Tensor, entry_start: torch.Tensor, slots: torch.Tensor,
                  out: torch.Tensor, n_heads: int, key_dim: int, value_dim: int, decay_scale: float, key_eps: float) -> torch.Tensor:
    """The generalized delta rule over the tokens of every entry, from and into state[slot] ([H, Dv, D] float32):
    S <- diag(w) S - (a u)(u^T S) + k v^T, o = S^T r, with u = k / sqrt(|k|^2 + key_eps), w = exp(-decay_scale *
    sigmoid(decay_logits)) and a = sigmoid(removal logits + a_bias).  x: a 2-d tensor whose rows are the tokens', with
    H heads of D read-out elements from r_column, of D keys from k_column, of Dv values from v_column and of D removal
    logits from a_column; decay_logits [n, H * D] float32; out [n, H * Dv] float32."""
    n = x.shape[0]
    hd = n_heads * key_dim
    _chk(x, "general_delta.x")
    if x.dim() != 2 or min(r_column, k_column, v_column, a_column) < 0 or \
            x.shape[1] < max(max(r_column, k_column, a_column) + hd, v_column + n_heads * value_dim):
        raise KernelError(f"general_delta.x: shape {tuple(x.shape)} does not hold its columns")
    _chk(decay_logits, "general_delta.decay_logits", torch.float32, (n, hd))
    if a_bias is not None:
        _chk(a_bias, "general_delta.a_bias", torch.float32, (hd,))
    _chk(out, "general_delta.out", torch.float32, (n, n_heads * value_dim))
    _chk(entry_start, "general_delta.entry_start", torch.int32)
    _chk(slots, "general_delta.slots", torch.int32)
    if not 1 <= key_dim <= DELTA_MAX_KEY_DIM:
        raise KernelError(f"general_delta: keys of {key_dim} (up to {DELTA_MAX_KEY_DIM})")
    sp, ss = _state_rows(state, "general_delta", n_heads * key_dim * value_dim)
    _run(load_lib("vt_delta", half=_half(x)), "vt_general_delta", _ptr(x), _i(_code(x)), ctypes.c_longlong(x.stride(0)),
         _i(r_column), _i(k_column), _i(v_column), _i(a_column), _ptr(decay_logits), _ptr(a_bias), sp, ss, _ptr(entry_start),
         _ptr(slots), _ptr(out), _i(entry_start.numel() - 1), _i(n_heads), _i(key_dim), _i(value_dim), _f(decay_scale),
         _f(key_eps), _stream())
    return out


def delta_rule_channel(qkv: torch.Tensor, beta: torch.Tensor, beta_column: int, decays: torch.Tensor,
                       state: torch.Tensor, entry_start: torch.Tensor, slots: torch.Tensor,
                       out: torch.Tensor, n_heads: int, n_kv: int, key_dim: int, value_dim: int) -> torch.Tensor:
    """The gated delta rule with a decay per key channel, S <- diag(g) S, over the tokens of every entry, from and
    into state[slot] ([H, Dv, D] float32).  qkv as for delta_rule; beta: a 2-d tensor whose rows are the tokens', with
    the H logits of the write strength from column beta_column; decays g [n, H * D] float32 (lowrank_tanh with
    `decay` makes them); out [n, H * Dv] float32."""
    n = qkv.shape[0]
    c = 2 * n_kv * key_dim + n_heads * value_dim
    _chk(qkv, "delta_rule_channel.qkv", None, (n, c))
    _chk(beta, "delta_rule_channel.beta")
    if beta.dim() != 2 or beta.shape[0] != n or beta.shape[1] < beta_column + n_heads:
        raise KernelError(f"delta_rule_channel.beta: shape {tuple(beta.shape)} has no {n_heads} columns from {beta_column}")
    if beta.dtype != torch.float32 and beta.dtype != qkv.dtype:
        raise KernelError(f"delta_rule_channel: logits of dtype {beta.dtype} beside inputs of {qkv.dtype}")
    _chk(decays, "delta_rule_channel.decays", torch.float32, (n, n_heads * key_dim))
    _chk(out, "delta_rule_channel.out", torch.float32, (n, n_heads * value_dim))
    _chk(entry_start, "delta_rule_channel.entry_start", torch.int32)
    _chk(slots, "delta_rule_channel.slots", torch.int32)
    if not 1 <= key_dim <= DELTA_MAX_KEY_DIM or n_heads % n_kv:
        raise KernelError(f"delta_rule_channel: heads {n_heads}/{n_kv} of {key_dim}")
    sp, ss = _state_rows(state, "delta_rule_channel", n_heads * key_dim * value_dim)
    bptr = ctypes.c_void_p(beta.data_ptr() + beta_column * beta.element_size())
    _run(load_lib("vt_delta", half=_half(qkv, beta)), "vt_delta_rule_channel", _ptr(qkv), _i(_code(qkv)), bptr, _i(_code(beta)),
         ctypes.c_longlong(beta.stride(0)), _ptr(decays), sp, ss, _ptr(entry_start), _ptr(slots),
         _ptr(out), _i(entry_start.numel() - 1), _i(n_heads), _i(n_kv), _i(key_dim), _i(value_dim), _stream())
    return out


def matrix_memory_state_floats(n_heads: int, key_dim: int, value_dim: int) -> int:
    """Floats of a request's state for matrix_memory: the heads' matrices [H, Dv, D], then per head and block of 16
    value columns a normalizer [D], then per head and block the running maximum."""
    zb = -(-value_dim // 16)
    return n_heads * value_dim * key_dim + n_heads * zb * key_dim + n_heads * zb


def matrix_memory(x: torch.Tensor, q_column: int, k_column: int, v_column: int, i_column: int, f_column: int,
                  i_bias: Optional[torch.Tensor], f_bias: Optional[torch.Tensor], state: torch.Tensor,
                  entry_start: torch.Tensor, slots: torch.Tensor, out: torch.Tensor, n_heads: int, key_dim: int,
                  value_dim: int, gate_cap: float, q_scale: float) -> torch.Tensor:
    """The matrix memory of xLSTM over the tokens of every entry, from and into state[slot] (float32,
    matrix_memory_state_floats long, zero at the start of a sequence).  With i = cap tanh((a_i + i_bias) / cap) and
    f = logsigmoid(cap tanh((a_f + f_bias) / cap)) (cap 0: no cap):
        m' = max(f + m, i);  S <- e^(f + m - m') S + e^(i - m') k v^T;  n <- e^(f + m - m') n + e^(i - m') k;
        o = S^T (q_scale q) / (max(|n . q_scale q|, e^(-m')) + 1e-6).
    x: a 2-d tensor whose rows are the tokens', with H heads of D queries from q_column, of D keys from k_column, of
    Dv values from v_column, and the H logits a_i from i_column and a_f from f_column; out [n, H * Dv] float32."""
    n = x.shape[0]
    hd = n_heads * key_dim
    _chk(x, "matrix_memory.x")
    if x.dim() != 2 or min(q_column, k_column, v_column, i_column, f_column) < 0 or \
            x.shape[1] < max(max(q_column, k_column) + hd, v_column + n_heads * value_dim, max(i_column, f_column) + n_heads):
        raise KernelError(f"matrix_memory.x: shape {tuple(x.shape)} does not hold its columns")
    for b, name in ((i_bias, "i_bias"), (f_bias, "f_bias")):
        if b is not None:
            _chk(b, "matrix_memory." + name, torch.float32, (n_heads,))
    _chk(out, "matrix_memory.out", torch.float32, (n, n_heads * value_dim))
    _chk(entry_start, "matrix_memory.entry_start", torch.int32)
    _chk(slots, "matrix_memory.slots", torch.int32)
    if not 1 <= key_dim <= DELTA_MAX_KEY_DIM or gate_cap < 0:
        raise KernelError(f"matrix_memory: keys of {key_dim} (up to {DELTA_MAX_KEY_DIM}), cap {gate_cap}")
    sp, ss = _state_rows(state, "matrix_memory", matrix_memory_state_floats(n_heads, key_dim, value_dim))
    _run(load_lib("vt_delta", half=_half(x)), "vt_matrix_memory", _ptr(x), _i(_code(x)), ctypes.c_longlong(x.stride(0)),
         _i(q_column), _i(k_column), _i(v_column), _i(i_column), _i(f_column), _ptr(i_bias), _ptr(f_bias), sp, ss,
         _ptr(entry_start), _ptr(slots), _ptr(out), _i(entry_start.numel() - 1), _i(n_heads), _i(key_dim), _i(value_dim),
         _f(gate_cap), _f(q_scale), _stream())
    return out


# ---------------------------------------------------------------------------
# several residual streams and the token shift (vt_streams.hip)
STREAMS_MAX = 8


def streams_fill(h: torch.Tensor, x: torch.Tensor) -> torch.Tensor:
    """x [n, S, W] float32: every stream of a token starts as h[token] (h [n, W] float32)."""
    n, s, w = x.shape
    _chk(h, "streams_fill.h", torch.float32, (n, w))
    _chk(x, "streams_fill.x", torch.float32)
    _run(load_lib("vt_streams"), "vt_streams_fill", _ptr(h), _ptr(x), _i(n), _i(s), _i(w), _stream())
    return x


def streams_read(x: torch.Tensor, w_in: torch.Tensor, gain: torch.Tensor, out: torch.Tensor, eps: float,
                 rows: Optional[torch.Tensor] = None) -> torch.Tensor:
    """out[r] = RMSNorm(sum_s w_in[s] x[t, s]; gain, eps) with t = rows[r] (or r); x [n, S, W] float32, out [R, W] in
    float32 or a 16-bit type."""
    n, s, w = x.shape
    _chk(x, "streams_read.x", torch.float32)
    _chk(w_in, "streams_read.w_in", torch.float32, (s,))
    _chk(gain, "streams_read.gain", torch.float32, (w,))
    if not 1 <= s <= STREAMS_MAX:
        raise KernelError(f"streams_read: {s} streams (1 to {STREAMS_MAX})")
    r = n
    if rows is not None:
        _chk(rows, "streams_read.rows", torch.int32)
        r = rows.numel()
    _chk(out, "streams_read.out", None, (r, w))
    _run(load_lib("vt_streams", half=_half(out)), "vt_streams_read", _ptr(x), _ptr(w_in), _ptr(gain), _ptr(rows), _ptr(out),
         _i(_code(out)), _i(r), _i(s), _i(w), _f(eps), _stream())
    return out


def streams_write(x: torch.Tensor, mix: torch.Tensor, w_out: torch.Tensor, y: torch.Tensor,
                  gate: Optional[torch.Tensor] = None) -> torch.Tensor:
    """x[t, to] <- sum_s mix[s, to] x[t, s] + w_out[to] * y[t] * sigmoid(gate[t]) (no gate: without the factor), all
    streams at once from the old ones; x [n, S, W] float32 in place, y and gate [n, W]."""
    n, s, w = x.shape
    _chk(x, "streams_write.x", torch.float32)
    _chk(mix, "streams_write.mix", torch.float32, (s, s))
    _chk(w_out, "streams_write.w_out", torch.float32, (s,))
    _chk(y, "streams_write.y", None, (n, w))
    if gate is not None:
        _chk(gate, "streams_write.gate", None, (n, w))
    if not 1 <= s <= STREAMS_MAX:
        raise KernelError(f"streams_write: {s} streams (1 to {STREAMS_MAX})")
    _run(load_lib("vt_streams", half=_half(y, gate)), "vt_streams_write", _ptr(x), _ptr(mix), _ptr(w_out), _ptr(y),
         _i(_code(y)), _ptr(gate), _i(_code(gate) if gate is not None else F32), _i(n), _i(s), _i(w), _stream())
    return x


def token_shift(h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, tok_entry: torch.Tensor, entry_start: torch.Tensor,
                slots: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """out[t] = h[t] + (h[t - 1] - h[t]) * mu, where the token before an entry's first comes from state[slot] ([W]
    float32: zeros at the start of a sequence); state[slot] then takes the entry's last h.  out must not be h."""
    n, w = h.shape
    _chk(h, "token_shift.h")
    _chk(out, "token_shift.out", h.dtype, (n, w))
    if out.data_ptr() == h.data_ptr():
        raise KernelError("token_shift: the result needs a buffer of its own")
    _chk(mu, "token_shift.mu", torch.float32, (w,))
    _chk(tok_entry, "token_shift.tok_entry", torch.int32, (n,))
    _chk(entry_start, "token_shift.entry_start", torch.int32)
    _chk(slots, "token_shift.slots", torch.int32)
    sp, ss = _state_rows(state, "token_shift", w)
    _run(load_lib("vt_streams", half=_half(h)), "vt_token_shift", _ptr(h), _i(_code(h)), _ptr(mu), sp, ss, _ptr(tok_entry),
         _ptr(entry_start), _ptr(slots), _ptr(out), _i(n), _i(w), _stream())
    return out


# ---------------------------------------------------------------------------
# a feed-forward of many experts (vt_moe.hip)
def moe_route(x: torch.Tensor, router: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, score: str = "sigmoid",
              renormalize: bool = False) -> None:
    """ids[t], weights[t] <- the `top` experts with the largest scores of token t and those scores (the largest
    first, the lower index among equals); scores are sigmoid or softmax of router x, in float32; renormalize: the
    chosen scores are divided by their sum.  x [n, W], router [E, W] float32, ids [n, top] int32, weights [n, top]."""
    n, w = x.shape
    e = router.shape[0]
    _chk(x, "moe_route.x")
    _chk(router, "moe_route.router", torch.float32, (e, w))
    top = ids.shape[1] if ids.dim() == 2 else 0
    _chk(ids, "moe_route.ids", torch.int32, (n, top))
    _chk(weights, "moe_route.weights", torch.float32, (n, top))
    if score not in ("sigmoid", "softmax") or not 1 <= top <= e:
        raise KernelError(f"moe_route: score {score!r}, {top} of {e} experts")
    _run(load_lib("vt_moe", half=_half(x)), "vt_moe_route", _ptr(x), _i(_code(x)), _ptr(router), _ptr(ids), _ptr(weights),
         _i(n), _i(e), _i(w), _i(top), _i(1 if score == "softmax" else 0), _i(1 if renormalize else 0), _stream())


def moe_gate_up(x: torch.Tensor, w_gu: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, act: torch.Tensor,
                scale_input: bool, alpha: float = 1.0, cubic: float = 0.0) -> torch.Tensor:
    """act[t * top + k] = f(W_gate,e xe) * (W_up,e xe) for e = ids[t, k], xe = x[t] (times weights[t, k] if
    scale_input, rounded to x's type), f(g) = g sigmoid(alpha g (1 + cubic g^2)); w_gu [E, 2 F, W] (gate rows, then up
    rows); act [n * top, F] in x's type.  An expert's matrices are read once per token that chose it."""
    n, w = x.shape
    e, two_f, _ = w_gu.shape
    top = ids.shape[1]
    _chk(x, "moe_gate_up.x")
    _chk(w_gu, "moe_gate_up.w_gu", x.dtype, (e, two_f, w))
    _chk(ids, "moe_gate_up.ids", torch.int32, (n, top))
    _chk(weights, "moe_gate_up.weights", torch.float32, (n, top))
    _chk(act, "moe_gate_up.act", x.dtype, (n * top, two_f // 2))
    _run(load_lib("vt_moe", half=_half(x)), "vt_moe_gate_up", _ptr(x), _i(_code(x)), _ptr(w_gu), _i(_code(w_gu)), _ptr(ids),
         _ptr(weights), _ptr(act), _i(n), _i(e), _i(w), _i(two_f // 2), _i(top), _i(1 if scale_input else 0), _f(alpha),
         _f(cubic), _stream())
    return act


def moe_down(act: torch.Tensor, w_down: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor, out: torch.Tensor,
             scale_output: bool) -> torch.Tensor:
    """out[t] = sum_k (weights[t, k] if scale_output) * W_down,e act[t * top + k], e = ids[t, k], in the order of k;
    w_down [E, W, F]; out [n, W] float32."""
    e, w, f = w_down.shape
    n, top = ids.shape
    _chk(act, "moe_down.act", None, (n * top, f))
    _chk(w_down, "moe_down.w_down", act.dtype)
    _chk(ids, "moe_down.ids", torch.int32)
    _chk(weights, "moe_down.weights", torch.float32, (n, top))
    _chk(out, "moe_down.out", torch.float32, (n, w))
    _run(load_lib("vt_moe", half=_half(act)), "vt_moe_down", _ptr(act), _i(_code(act)), _ptr(w_down), _i(_code(w_down)),
         _ptr(ids), _ptr(weights), _ptr(out), _i(n), _i(e), _i(w), _i(f), _i(top), _i(1 if scale_output else 0), _stream())
    return out


MOE_GROUPED_MAX_EXPERTS = 1024
MOE_TILE_PAIRS = 128        # pairs of one expert that a block of the grouped products takes


def moe_plan_size(pairs: int, experts: int) -> int:
    """int32 elements of the plan that moe_sort writes for `pairs` (token, choice) pairs."""
    tiles = -(-int(pairs) // MOE_TILE_PAIRS) + int(experts)         # what vt_moe_plan_tiles says
    return 1 + int(pairs) + 3 * tiles


def moe_grouped_ok(x: torch.Tensor, experts: int, width: int, inter: int) -> bool:
    """Whether the grouped products take this feed-forward: a 16-bit type, sizes that are multiples of 8."""
    return x.dtype in LOWP and width % 8 == 0 and inter % 8 == 0 and experts <= MOE_GROUPED_MAX_EXPERTS


def moe_sort(ids: torch.Tensor, plan: torch.Tensor, experts: int) -> torch.Tensor:
    """plan <- the pairs in the order of their experts, cut into tiles of pairs of one expert (what the grouped
    products read).  ids [n, top] int32 with values below `experts`; plan: moe_plan_size(n * top, experts) int32."""
    _chk(ids, "moe_sort.ids", torch.int32)
    pairs = ids.numel()
    _chk(plan, "moe_sort.plan", torch.int32, (moe_plan_size(pairs, experts),))
    _run(load_lib("vt_moe"), "vt_moe_sort", _ptr(ids), _ptr(plan), _i(pairs), _i(experts), _stream())
    return plan


def moe_gate_up_grouped(x: torch.Tensor, w_gu: torch.Tensor, plan: torch.Tensor, weights: torch.Tensor, act: torch.Tensor,
                        top: int, scale_input: bool, alpha: float = 1.0, cubic: float = 0.0) -> torch.Tensor:
    """moe_gate_up on the matrix cores for many tokens: act [n * top, F] in the plan's order (pairs sorted by expert),
    an expert's matrices read once per tile of pairs.  x [n, W] and w_gu [E, 2 F, W] of one 16-bit type."""
    n, w = x.shape
    e, two_f, _ = w_gu.shape
    _chk(x, "moe_gate_up_grouped.x")
    if x.dtype not in LOWP:
        raise KernelError("moe_gate_up_grouped: a 16-bit type is needed")
    _chk(w_gu, "moe_gate_up_grouped.w_gu", x.dtype, (e, two_f, w))
    _chk(plan, "moe_gate_up_grouped.plan", torch.int32, (moe_plan_size(n * top, e),))
    _chk(weights, "moe_gate_up_grouped.weights", torch.float32, (n, top))
    _chk(act, "moe_gate_up_grouped.act", x.dtype, (n * top, two_f // 2))
    _run(load_lib("vt_moe", half=_half(x)), "vt_moe_gate_up_grouped", _ptr(x), _ptr(w_gu), _ptr(plan), _ptr(weights), _ptr(act),
         _i(n), _i(e), _i(w), _i(two_f // 2), _i(top), _i(1 if scale_input else 0), _f(alpha), _f(cubic), _stream())
    return act


def moe_down_grouped(act: torch.Tensor, w_down: torch.Tensor, plan: torch.Tensor, weights: torch.Tensor, out: torch.Tensor,
                     scratch: Optional[torch.Tensor], scale_output: bool) -> torch.Tensor:
    """moe_down on the matrix cores from activations in the plan's order; scratch [n * top, W] float32 where a token
    has more than one choice (the choices' results, added in their order afterwards)."""
    e, w, f = w_down.shape
    n, top = weights.shape
    _chk(act, "moe_down_grouped.act", None, (n * top, f))
    if act.dtype not in LOWP:
        raise KernelError("moe_down_grouped: a 16-bit type is needed")
    _chk(w_down, "moe_down_grouped.w_down", act.dtype)
    _chk(plan, "moe_down_grouped.plan", torch.int32, (moe_plan_size(n * top, e),))
    _chk(weights, "moe_down_grouped.weights", torch.float32)
    _chk(out, "moe_down_grouped.out", torch.float32, (n, w))
    if top > 1:
        if scratch is None:
            raise KernelError("moe_down_grouped: several choices per token need scratch")
        _chk(scratch, "moe_down_grouped.scratch", torch.float32, (n * top, w))
    _run(load_lib("vt_moe", half=_half(act)), "vt_moe_down_grouped", _ptr(act), _ptr(w_down), _ptr(plan), _ptr(weights), _ptr(out),
         _ptr(scratch if top > 1 else None), _i(n), _i(e), _i(w), _i(f), _i(top), _i(1 if scale_output else 0), _stream())
    return out


# ---------------------------------------------------------------------------
def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, work: torch.Tensor, out: torch.Tensor,
           partials: Optional[torch.Tensor] = None) -> torch.Tensor:
    """partials: scratch of sample_partials_size(rows) floats (made here if not given)."""
    rows, vocab = logits.shape
    _chk(logits, "sample.logits", torch.float32)
    _chk(temperature, "sample.temperature", torch.float32, (rows,))
    _chk(top_k, "sample.top_k", torch.int32, (rows,))
    _chk(top_p, "sample.top_p", torch.float32, (rows,))
    _chk(uniform, "sample.uniform", torch.float32, (rows,))
    _chk(work, "sample.work", torch.float32)
    if work.numel() < rows * vocab:
        raise KernelError("sample: workspace smaller than the logits")
    _chk(out, "sample.out", torch.int32, (rows,))
    if partials is None:
        partials = torch.empty(sample_partials_size(rows), dtype=torch.float32, device=logits.device)
    _chk(partials, "sample.partials", torch.float32)
    if partials.numel() < sample_partials_size(rows):
        raise KernelError("sample: scratch for the slices' maxima is too small")
    _run(load_lib("vt_sampling"), "vt_sample", _ptr(logits), _i(rows), _i(vocab), _ptr(temperature), _ptr(top_k),
         _ptr(top_p), _ptr(uniform), _ptr(work), _ptr(partials), _ptr(out), _stream())
    return out


def sample_partials_size(rows: int) -> int:
    return 2 * max(1, rows) * int(load_lib("vt_sampling").vt_sample_slices())


def require_gpu() -> torch.device:
    if not torch.cuda.is_available():
        raise KernelError("no GPU is visible: this engine has no CPU path")
    return torch.device("cuda", torch.cuda.current_device())
