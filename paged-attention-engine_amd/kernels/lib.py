"""ctypes bindings of the gfx950 kernel library and thin, checked wrappers.

Every wrapper takes torch tensors that already live on the GPU, checks on the
host that shapes and dtypes match what the kernel and its grid assume, launches
on torch's current stream and raises `KernelError` with the library's message
on refusal.  There is no fallback: without the library or without a GPU these
functions raise.
"""

from __future__ import annotations

import ctypes
import os
from ctypes import c_char_p, c_float, c_int, c_int64, c_void_p
from typing import Optional

import torch

from .build import ensure_built

F32, BF16 = 0, 1
_CODE = {torch.float32: F32, torch.bfloat16: BF16}


class KernelError(RuntimeError):
    pass


_lib = None


def library():
    """The loaded kernel library (built at the first call if necessary)."""
    global _lib
    if _lib is None:
        # PAE_KERNEL_LIBRARY: a library built by hand from the same sources (a variant under measurement)
        path = os.environ.get("PAE_KERNEL_LIBRARY") or ensure_built()
        try:
            lib = ctypes.CDLL(path)
        except OSError as err:
            raise KernelError(f"cannot load the kernel library {path}: {err}") from err
        _declare(lib)
        _lib = lib
    return _lib


def loaded_library_path() -> Optional[str]:
    return getattr(_lib, "_name", None) if _lib is not None else None


def _declare(lib) -> None:
    lib.pae_last_error.restype = c_char_p
    P, I, L, F = c_void_p, c_int, c_int64, c_float
    sig = {
        "pae_device_arch": [c_char_p, I],
        "pae_embedding": [I, P, P, P, I, I, I, F, P],
        "pae_logits_finish": [P, L, F, F, P],
        "pae_add_rmsnorm": [I, P, P, I, L, P, I, F, P, P, I, I, I, P],
        "pae_residual_add": [I, P, P, L, P],
        "pae_scatter_i32": [P, P, P, P, I, P],
        "pae_copy_i32": [P, P, I, P],
        "pae_rope_table": [P, P, P, I, I, P],
        "pae_rope_kv_write": [I, P, L, I, I, I, I, I, P, I, P, P, P, P, I, I, P, P, I, P],
        "pae_swiglu": [I, P, P, I, I, I, P],
        "pae_gemm_skinny": [I, P, L, P, L, P, P, I, I, I, I, I, L, P, P, P, I, F, P, L, P, I, P, P],
        "pae_gemm_skinny_rope": [P, L, P, L, P, P, I, I, I, I, I, I, I, P, P, P, P, I, I, P, P, I, P, P, P, I, F, P],
        "pae_embedding_rows": [I, P, P, P, I, I, I, F, P, P, I, P, P],
        "pae_scaled_rows": [P, P, P, I, F, I, I, P],
        "pae_skinny_ticket_slots": [I, I],
        "pae_gemm_plain": [I, I, P, L, P, L, P, P, I, I, I, I, P],
        "pae_paged_attention_generic": [I, P, L, P, L, P, P, P, P, P, I, I, I, I, I, I, F, I, P],
        "pae_sample": [P, P, L, P, P, I, I, P, P, P, P],
        "pae_sample_chunks": [I],
        "pae_sample_static": [P, P, L, P, P, I, I, P],
        "pae_sample_static_slots": [],
        "pae_sample_static_prepare": [],
        "pae_attn_decode_bf16": [P, L, P, L, P, P, P, I, P, I, I, I, I, I, F, I, P, P, P],
        "pae_attn_decode_split": [],
        "pae_attn_prefill_bf16": [P, L, P, L, P, P, P, I, P, P, I, I, I, I, I, F, I, P],
        "pae_program_phase_bytes": [],
        "pae_program_barrier_bytes": [],
        "pae_program_max_rows": [],
        "pae_program_max_groups": [],
        "pae_program_put_product": [P, I, I, P, L, P, L, P, P, I, I, I, I, I, P, P, P, I, F, P, L, P, I, P, P],
        "pae_program_put_product_rope": [P, I, P, L, P, L, P, P, I, I, I, I, I, I, I, P, P, P, P, I, I, P, P, I, P, P, P,
                                         I, F],
        "pae_program_put_attention": [P, I, P, L, P, L, P, P, P, I, P, I, I, I, I, I, F, I, P, P],
        "pae_program_run": [P, I, P, P, I, I, I, I, P, P],
        "pae_program_activation_bytes": [I, I, I],
        "pae_program_lds_limit": [],
    }
    for name, args in sig.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = c_int
    lib.pae_skinny_ticket_floats.argtypes = [I, I, I]
    lib.pae_skinny_ticket_floats.restype = c_int64


def _check(code: int) -> None:
    if code != 0:
        raise KernelError(library().pae_last_error().decode("utf-8", "replace"))


def _stream() -> int:
    # the raw handle of torch's current stream (also the capture stream while a graph records)
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


def code_of(dtype: torch.dtype) -> int:
    try:
        return _CODE[dtype]
    except KeyError:
        raise KernelError(f"dtype {dtype} is not one the kernels take (float32, bfloat16)") from None


def _gpu(*tensors) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise KernelError("kernel operands must live on the GPU; there is no CPU path")


def _ptr(t: Optional[torch.Tensor]) -> Optional[int]:
    return None if t is None else t.data_ptr()


def _param(t: Optional[torch.Tensor]):
    """(pointer, is_f32) of a vector parameter stored in float32 or bfloat16."""
    if t is None:
        return None, 0
    if t.dtype not in _CODE:
        raise KernelError(f"parameter dtype {t.dtype} not supported")
    return t.data_ptr(), 1 if t.dtype == torch.float32 else 0


def _check_pools(k_cache, v_cache, nkv: int, bs: int, hd: int) -> None:
    """Keys [block][kv head][bs][hd]; values transposed within the page, [block][kv head][hd][bs]."""
    assert tuple(k_cache.shape[1:]) == (nkv, bs, hd) and k_cache.is_contiguous()
    assert tuple(v_cache.shape) == (k_cache.shape[0], nkv, hd, bs) and v_cache.is_contiguous()
    assert k_cache.dtype == v_cache.dtype


def device_arch() -> str:
    buf = ctypes.create_string_buffer(64)
    _check(library().pae_device_arch(buf, 64))
    return buf.value.decode().split(":")[0]


def embedding(out: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float = 1.0) -> None:
    """out[t] = scale * table[ids[t]] as float32; ids int32 (checked against the table by the caller)."""
    _not_while_recording("embedding")
    _gpu(out, table, ids)
    T, H = out.shape
    assert out.dtype == torch.float32 and out.is_contiguous() and table.is_contiguous()
    assert ids.dtype == torch.int32 and ids.numel() == T and table.shape[1] == H
    _check(library().pae_embedding(code_of(table.dtype), out.data_ptr(), table.data_ptr(), ids.data_ptr(),
                                   T, H, table.shape[0], float(scale), _stream()))


def logits_finish(logits: torch.Tensor, scale: float = 1.0, softcap: float = 0.0) -> None:
    """In place: logits = scale * logits, then with a soft cap c > 0, c * tanh(logits / c)."""
    _not_while_recording("logits_finish")
    _gpu(logits)
    assert logits.dtype == torch.float32 and logits.is_contiguous()
    _check(library().pae_logits_finish(logits.data_ptr(), logits.numel(), float(scale), float(softcap), _stream()))


def add_rmsnorm(residual: torch.Tensor, delta: Optional[torch.Tensor], weight: torch.Tensor, eps: float,
                out: torch.Tensor, rows: Optional[torch.Tensor] = None, write_residual: bool = True) -> None:
    """residual (+= delta); out = weight * round(residual * rsqrt(mean(residual^2) + eps)).

    `delta` is the pending branch output: [T, H] in out's dtype, or float32 partial sums
    [P, T, H] that are added in order.  With `rows` (int32), out[b] comes from source row
    rows[b] and nothing is written back."""
    _not_while_recording("add_rmsnorm")
    _gpu(residual, delta, weight, out, rows)
    H = residual.shape[-1]
    n = out.shape[0]
    assert residual.dtype == torch.float32 and residual.is_contiguous() and out.is_contiguous()
    assert out.shape[-1] == H and weight.numel() == H
    parts, part_stride = 0, 0
    if delta is not None:
        assert delta.is_contiguous()
        if delta.dim() == 3:
            assert delta.dtype == torch.float32 and delta.shape[1:] == residual.shape
            parts, part_stride = delta.shape[0], residual.numel()
        else:
            assert delta.dtype == out.dtype and delta.shape == residual.shape
    if rows is None:
        assert residual.shape[0] == n
    else:
        assert rows.dtype == torch.int32 and rows.numel() == n
        write_residual = False
    wp, wf = _param(weight)
    _check(library().pae_add_rmsnorm(code_of(out.dtype), residual.data_ptr(), _ptr(delta), parts, part_stride,
                                     wp, wf, float(eps),
                                     _ptr(rows), out.data_ptr(), n, H, 1 if write_residual else 0, _stream()))


def residual_add(residual: torch.Tensor, delta: torch.Tensor) -> None:
    _not_while_recording("residual_add")
    _gpu(residual, delta)
    assert residual.dtype == torch.float32 and residual.shape == delta.shape
    assert residual.is_contiguous() and delta.is_contiguous()
    _check(library().pae_residual_add(code_of(delta.dtype), residual.data_ptr(), delta.data_ptr(),
                                      residual.numel(), _stream()))


def copy_int32_from_pinned(dst: torch.Tensor, src: torch.Tensor, n: int) -> None:
    """dst[:n] = src[:n] by a kernel on the current stream; `src` is pinned host memory (which the
    GPU reads in place) and must stay as it is until the kernel has run."""
    _not_while_recording("copy_int32_from_pinned")
    _gpu(dst)
    assert dst.dtype == torch.int32 == src.dtype and dst.is_contiguous() and src.is_contiguous()
    assert src.is_pinned() and 0 <= n <= min(dst.numel(), src.numel())
    _check(library().pae_copy_i32(dst.data_ptr(), src.data_ptr(), n, _stream()))


def scatter_int32(dst: torch.Tensor, dst_idx: torch.Tensor, src: torch.Tensor, src_idx: torch.Tensor, n: int) -> None:
    """dst[dst_idx[i]] = src[src_idx[i]] for i < n (int32 everywhere; the index lists may be longer than n).
    The caller vouches for the indices: they are not checked on the device."""
    _not_while_recording("scatter_int32")
    _gpu(dst, dst_idx, src, src_idx)
    for t in (dst, dst_idx, src, src_idx):
        assert t.dtype == torch.int32 and t.is_contiguous()
    assert 0 <= n <= min(dst_idx.numel(), src_idx.numel())
    _check(library().pae_scatter_i32(dst.data_ptr(), dst_idx.data_ptr(), src.data_ptr(), src_idx.data_ptr(), n,
                                     _stream()))


def rope_table(positions: torch.Tensor, inv_freq: torch.Tensor) -> torch.Tensor:
    """[T, len(inv_freq), 2] float32: cosine and sine of positions[t] * inv_freq[i]."""
    _gpu(positions, inv_freq)
    assert positions.dtype == torch.int32 and inv_freq.dtype == torch.float32 and inv_freq.is_contiguous()
    T, half = positions.numel(), inv_freq.numel()
    out = torch.empty((T, half, 2), dtype=torch.float32, device=positions.device)
    _check(library().pae_rope_table(out.data_ptr(), positions.data_ptr(), inv_freq.data_ptr(), T, half, _stream()))
    return out


def _check_cos_sin(cos_sin: Optional[torch.Tensor], rot: int, T: int) -> None:
    if rot:
        assert cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.is_contiguous()
        assert tuple(cos_sin.shape) == (T, rot // 2, 2)


def rope_kv_write(qkv: torch.Tensor, nh: int, nkv: int, hd: int, rot: int, cos_sin: Optional[torch.Tensor],
                  positions: torch.Tensor, tok_seq: Optional[torch.Tensor], block_tables: Optional[torch.Tensor],
                  block_size: int, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  bias: Optional[torch.Tensor] = None) -> None:
    """Rotate the query heads of `qkv` in place by the angles whose cosines and sines `cos_sin`
    holds ([T, rot / 2, 2], see `rope_table`); rotate the key heads and copy the value heads
    into their cache slots (skipped when `k_cache` is None: then the row holds query heads only
    and nkv must be 0).  With `bias` (one value per feature of the row) the row stands for the
    projection without its bias, which is added here first."""
    _not_while_recording("rope_kv_write")
    _gpu(qkv, cos_sin, positions, tok_seq, block_tables, k_cache, v_cache, bias)
    if bias is not None:
        assert bias.numel() == (nh + 2 * nkv) * hd
    T = qkv.shape[0]
    assert qkv.dim() == 2 and qkv.stride(1) == 1 and positions.dtype == torch.int32 and positions.numel() == T
    write = k_cache is not None
    _check_cos_sin(cos_sin, rot, T)
    max_blocks = 0
    if write:
        assert v_cache is not None and k_cache.dtype == qkv.dtype == v_cache.dtype
        assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
        assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
        _check_pools(k_cache, v_cache, nkv, block_size, hd)
        max_blocks = block_tables.shape[1]
    bp, bf = _param(bias)
    _check(library().pae_rope_kv_write(code_of(qkv.dtype), qkv.data_ptr(), qkv.stride(0), T, nh, nkv, hd, rot,
                                       bp, bf, _ptr(cos_sin) if rot else None, positions.data_ptr(), _ptr(tok_seq),
                                       _ptr(block_tables), max_blocks, block_size, _ptr(k_cache), _ptr(v_cache),
                                       1 if write else 0, _stream()))


def rotate_heads(x: torch.Tensor, num_heads: int, hd: int, rot: int, cos_sin: torch.Tensor,
                 positions: torch.Tensor) -> None:
    """Rotate the first `num_heads` heads (each `hd` wide) of every row of `x` in place; nothing is stored."""
    rope_kv_write(x, num_heads, 0, hd, rot, cos_sin, positions, None, None, 1, None, None)


def kv_store(qkv: torch.Tensor, nh: int, nkv: int, hd: int, positions: torch.Tensor, tok_seq: torch.Tensor,
             block_tables: torch.Tensor, block_size: int, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
    """Copy the key and value heads of rows [q heads | k heads | v heads] into their cache slots, as they are."""
    rope_kv_write(qkv, nh, nkv, hd, 0, None, positions, tok_seq, block_tables, block_size, k_cache, v_cache)


def swiglu(out: torch.Tensor, x: torch.Tensor, block: int = 0) -> None:
    """out[t, j] = silu(gate_j) * up_j for x of width 2 I: gate = x[:, :I], up = x[:, I:], or,
    with `block` > 0, blocks of `block` gate features each followed by their up features."""
    _not_while_recording("swiglu")
    _gpu(out, x)
    T, I = out.shape
    assert x.shape == (T, 2 * I) and x.dtype == out.dtype and x.is_contiguous() and out.is_contiguous()
    _check(library().pae_swiglu(code_of(x.dtype), out.data_ptr(), x.data_ptr(), T, I, block, _stream()))


# ---------------------------------------------------------------------------------- decode programs
# A decode step's products and attention as one resident kernel (csrc/decode_program.hip).  While a
# program is recording, `gemm_skinny`, `gemm_skinny_rope` and `attn_decode` append a phase to it
# instead of launching; `rope_table`, which reads the step's positions only, runs at once; every other
# wrapper refuses.  `launch()` then runs the phases in the order they were recorded, each after the
# one before it has finished everywhere, as the separate launches would.
_RECORDING = None
PROGRAM_SPIN_LIMIT = 2_000_000  # polls of a barrier before a workgroup gives up (about two seconds)


def _not_while_recording(name: str) -> None:
    if _RECORDING is not None:
        raise KernelError(f"{name} cannot be a phase of a decode program; a part that calls it must not say it is fusable")


def program_max_rows() -> int:
    return library().pae_program_max_rows()


def program_takes_product(rows: int, K: int, splits: int, quad_bytes: int = 27 * 1024) -> bool:
    """Whether a decode program has the LDS for a product of `rows` rows over k ranges of K / splits
    (a workgroup keeps one range's activations there, beside its quads' own `quad_bytes` each)."""
    lib = library()
    return 2 * quad_bytes + lib.pae_program_activation_bytes(rows, K, splits) <= lib.pae_program_lds_limit()


_PROGRAM_BARRIERS: dict = {}  # (device index, workgroups) -> zeroed barrier block


class DecodeProgram:
    """Room for a list of phases (in pinned host memory, where it is written, and on the device, where
    the kernel reads it) and what running them needs.  A program recorded into a HIP graph keeps its
    list for as long as the graph lives: every replay copies it to the device again."""

    def __init__(self, device, max_phases: int, groups: Optional[int] = None) -> None:
        lib = library()
        self.device = torch.device(device)
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("a decode program's buffers must exist before a graph is recorded")
        with torch.cuda.device(self.device):
            most = lib.pae_program_max_groups()
        if most < 1:
            _check(most)
        self.groups = most if groups is None else int(groups)
        if not 1 <= self.groups <= most:
            raise KernelError(f"{self.groups} workgroups cannot all be resident (at most {most})")
        self.phase_bytes = lib.pae_program_phase_bytes()
        self.max_phases = max_phases
        ints = self.phase_bytes * max_phases // 4
        self.host = torch.zeros(ints, dtype=torch.int32, pin_memory=True)
        self.on_device = torch.zeros(ints, dtype=torch.int32, device=self.device)
        self.error = torch.zeros(1, dtype=torch.int32, pin_memory=True)
        key = (self.device.index or 0, self.groups)
        if key not in _PROGRAM_BARRIERS:
            _PROGRAM_BARRIERS[key] = torch.zeros(lib.pae_program_barrier_bytes() // 4, dtype=torch.int32, device=self.device)
        self.barrier = _PROGRAM_BARRIERS[key]
        skinny_tickets(self.device)
        self.host_ptr = self.host.data_ptr()
        self.count = 0
        self.quad_lds = 0        # bytes of LDS a quad needs: the most any phase asked for
        self.activation_lds = 0  # bytes of LDS for a product's activations: likewise
        self.keep: list = []
        self._read: Optional[torch.cuda.Event] = None
        self.trace: Optional[torch.Tensor] = None  # int64 [phases, workgroups, 2] clock readings of the next launches, if set

    def begin(self) -> None:
        if self._read is not None:
            self._read.synchronize()  # the launch before has copied the list to the device
        self.count, self.quad_lds, self.activation_lds, self.keep = 0, 0, 0, []

    def room(self, phases: int) -> None:
        """Raise unless `phases` more fit the list (asked before a pae_program_put_* call writes them)."""
        if self.count + phases > self.max_phases:
            raise KernelError(f"a decode program of more than {self.max_phases} phases")

    def add(self, code: int, *tensors, activation_bytes: int = 0) -> None:
        """`code`: what a pae_program_put_* call returned (the bytes of LDS a quad needs, or an error);
        `activation_bytes`: the LDS a product's activations take (pae_program_activation_bytes)."""
        if code < 0:
            _check(code)
        self.room(1)
        self.count += 1
        self.quad_lds = max(self.quad_lds, code)
        self.activation_lds = max(self.activation_lds, activation_bytes)
        self.keep.append(tensors)  # what the phase reads and writes stays alive until the program has run

    def launch(self) -> None:
        if self.count == 0:
            return
        global _RECORDING
        assert _RECORDING is None, "a program is launched after its recording has ended"
        copy_int32_from_pinned(self.on_device, self.host, self.count * self.phase_bytes // 4)
        _check(library().pae_program_run(self.on_device.data_ptr(), self.count, self.barrier.data_ptr(),
                                         self.error.data_ptr(), self.groups, self.quad_lds, self.activation_lds,
                                         PROGRAM_SPIN_LIMIT, _ptr(self.trace), _stream()))
        if not torch.cuda.is_current_stream_capturing():
            self._read = self._read or torch.cuda.Event()
            self._read.record()

    def trace_phases(self) -> torch.Tensor:
        """From now on every launch leaves, per phase and workgroup, eight numbers: clock readings (100 MHz)
        [0] when it began the phase's work, [1] when it ended it (the difference to the next phase's
        beginning is its wait at the barrier), [2..5] marks of the phase's own (see pae_program_run; zero
        where a phase leaves none), and [7] the die that the workgroup ran on."""
        self.trace = torch.zeros((self.max_phases, self.groups, 8), dtype=torch.int64, device=self.device)
        return self.trace

    def check(self) -> None:
        """Raise if a launch of this program gave up at a barrier (call after the device has been waited for)."""
        code = int(self.error[0])
        if code:
            self.error[0] = 0
            self.barrier.zero_()
            skinny_tickets(self.device).zero_()
            raise KernelError(f"the decode program's workgroups did not all arrive at the barrier after phase {code - 1}: "
                              "the program was abandoned and its results are invalid")


class recording:
    """`with recording(program):` the product and decode-attention wrappers append phases to `program`."""

    def __init__(self, program: DecodeProgram) -> None:
        self.program = program

    def __enter__(self):
        global _RECORDING
        if _RECORDING is not None:
            raise KernelError("a decode program is already recording")
        self.program.begin()
        _RECORDING = self.program
        return self.program

    def __exit__(self, *exc):
        global _RECORDING
        _RECORDING = None
        return False


SKINNY_MAX_ROWS = 64
# Up to this many rows a norm may be folded into the products around it (see parts.OwedRows): as many as
# the few-rows products take (PAE_FOLD_MAX_ROWS: fewer, for a measurement).  Above 16 rows only while
# rows x width stays within FOLD_MAX_ELEMENTS.  Measured with the step itself: folding gains 2 to 6 % at 24
# to 64 rows of the 0.5B, 1.5B and 3B shapes (widths 896 to 2,048), 1.3 / 0.6 % at 24 / 32 rows of the 7B
# shape (3,584) and 2.6 % at 24 rows of the 14B shape (5,120), is even at 40 rows of the 7B shape and loses
# 1.7 / 1.2 % at its 48 / 64 rows, where the norm kernel is cheaper than the products' epilogues that stand
# in for it.
FOLD_MAX_ROWS = int(os.environ.get("PAE_FOLD_MAX_ROWS", "64"))
FOLD_MAX_ELEMENTS = 64 * 2048


def folds(rows: int, width: int) -> bool:
    """Whether a norm of `width` columns is folded into the products around it in a step of `rows` rows."""
    if not 0 < rows <= FOLD_MAX_ROWS:
        return False
    return rows <= SAME_ORDER_MAX_ROWS or rows * width <= FOLD_MAX_ELEMENTS


SAME_ORDER_MAX_ROWS = 16  # up to this many rows a product's k ranges depend on its sizes alone
EPI_BF16, EPI_F32, EPI_SWIGLU, EPI_RESIDUAL = 0, 1, 2, 4


def stat_tiles(width: int) -> int:
    """Shares a row's sum of squares is kept in: one per 16 columns."""
    return -(-width // 16)


def _row_scale(row_scale, M: int, K: int):
    """(pointer, tiles, eps) of the shares of the rows' sums of squares, for a product whose rows
    are still to be divided by their root mean square; (None, 0, 0) for plain rows."""
    if row_scale is None:
        return None, 0, 0.0
    stats, eps = row_scale
    assert stats.is_cuda and stats.dtype == torch.float32 and stats.is_contiguous()
    assert stats.dim() == 2 and stats.shape[0] >= M and stats.shape[1] == stat_tiles(K)
    return stats.data_ptr(), stats.shape[1], float(eps)


def embedding_rows(residual: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, scale: float,
                   next_rows: torch.Tensor, next_w: torch.Tensor, next_stats: torch.Tensor) -> None:
    """`embedding` for a step whose first norm is folded into the products: beside residual[t] =
    scale * table[ids[t]], next_rows[t] = bfloat16(residual[t] * next_w) and next_stats[t][j] = the sum
    of squares of residual[t] over columns 16 j .. 16 j + 15."""
    _not_while_recording("embedding_rows")
    _gpu(residual, table, ids, next_rows, next_w, next_stats)
    T, H = residual.shape
    assert residual.dtype == torch.float32 and residual.is_contiguous() and table.is_contiguous()
    assert ids.dtype == torch.int32 and ids.numel() == T and table.shape[1] == H
    assert next_rows.dtype == torch.bfloat16 and next_rows.shape == (T, H) and next_rows.is_contiguous()
    assert next_stats.dtype == torch.float32 and next_stats.shape == (T, stat_tiles(H)) and next_stats.is_contiguous()
    assert next_w.numel() == H
    wp, wf = _param(next_w)
    _check(library().pae_embedding_rows(code_of(table.dtype), residual.data_ptr(), table.data_ptr(), ids.data_ptr(),
                                        T, H, table.shape[0], float(scale), next_rows.data_ptr(), wp, wf,
                                        next_stats.data_ptr(), _stream()))


def scaled_rows(rows: torch.Tensor, stats: torch.Tensor, eps: float) -> torch.Tensor:
    """rows[m] * rsqrt(sum(stats[m]) / width + eps) as bfloat16: rows whose scale was owed, paid."""
    _not_while_recording("scaled_rows")
    _gpu(rows, stats)
    M, H = rows.shape
    assert rows.dtype == torch.bfloat16 and rows.is_contiguous()
    assert stats.dtype == torch.float32 and stats.shape == (M, stat_tiles(H)) and stats.is_contiguous()
    out = torch.empty_like(rows)
    _check(library().pae_scaled_rows(out.data_ptr(), rows.data_ptr(), stats.data_ptr(), stats.shape[1], float(eps),
                                     M, H, _stream()))
    return out


def skinny_supported(a: torch.Tensor, w: torch.Tensor) -> bool:
    """The weight-streaming product takes bfloat16, at most 64 rows and rows of 16-byte multiples."""
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.shape[0] <= SKINNY_MAX_ROWS
            and a.shape[1] % 8 == 0 and a.stride(0) % 8 == 0 and a.stride(1) == 1)


def skinny_splits(N: int, K: int, M: int = 1) -> int:
    """k ranges for a product whose consumer adds float32 partials: enough workgroups to fill the
    chip (a workgroup takes 16 weight rows, or 32 and more with more than 8 rows of activations)."""
    rows = 32 if M > 8 else 16
    tiles = -(-N // rows)
    # (ranges of at least 1,024 of k: the 0.5B sizes at 8 rows, O 5.3 us in three ranges and 3.9 in one, down
    # 8.0 us in eight and 7.4 in four)
    wanted = max(1, min(512 // tiles, K // 1024, 8))
    if M <= 8 and tiles >= 200 and tiles * wanted < 640 and K >= 4096:
        # one or two workgroups per compute unit, each with a long way to go (14B down at 8 rows:
        # 320 workgroups over 13,824 of k take 48 us with the norm, three ranges 35 us)
        wanted = min(8, -(-960 // tiles))
    if M > 8:
        # every range costs its partial sums a trip to memory and back in the norm that adds them, so a
        # workgroup wants about 128 KB of weights before another range pays (with the norm, at 64 rows:
        # 1.5B O one range 9.8 us, six 11.5; 1.5B down four 21.0, eight 22.9; 7B O two 18.2, four 19.8)
        wanted = max(1, min(8, round(rows * K * 2 / 131072)))
        # enough ranges of at least 1024 for the many-weight-rows kernel (128 rows a workgroup) to fill
        # the chip twice, where that many exist (72B down at 64 rows: 2 ranges 177 us, 8 ranges 115 us)
        groups = -(-N // 128)
        many = min(12, -(-512 // groups))
        while many > 1 and K // many < 1024:
            many -= 1
        if groups * many >= 256:
            wanted = max(wanted, many)
        # or fewer, longer ranges for that kernel's 64-row workgroups, where those fill the chip and the
        # 128-row ones do not (7B down at 48 rows: 12 ranges 47 us, 8 ranges of 64-row workgroups 42 us)
        # (ranges down to 768 of k: 14B/32B O, 5,120 x 5,120, at 24 / 64 rows from HBM with the norm: two ranges
        # 28.2 / 38.0 us, six 22.7 / 27.6)
        fewer = -(-448 // -(-N // 64))
        if fewer <= 8 and K // fewer >= 768 and groups * fewer < 256:
            wanted = fewer
        # or, with few weight rows, as many ranges as make one round of 32-row workgroups over the chip (3B
        # down, 64 x 4: 19.9 / 23.7 us with the norm against 23.1 / 29.0 with five ranges; 1.5B down, 48 x 5)
        one_round = _compute_units() // -(-N // 32)
        if M > SAME_ORDER_MAX_ROWS and 4 <= one_round <= 8 and K // one_round >= 1024:
            wanted = one_round
    k_per = -(-(-(-K // wanted)) // 128) * 128
    return -(-K // k_per)


_UNITS = 0


def _compute_units() -> int:
    global _UNITS
    if not _UNITS:
        _UNITS = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count if torch.cuda.is_available() else 256
    return _UNITS


def residual_splits(N: int, K: int, M: int = 1) -> int:
    """k ranges for a product that adds itself into the residual (EPI_RESIDUAL).  Up to 16 rows from
    the product's sizes alone: a row's sums are the same bits whatever it is batched with, launched by
    itself or as a phase of a decode program.  Four ranges run side by side in one workgroup of sixteen
    wavefronts, with no tickets and no trip to memory for partial sums, and are ahead wherever the 16-row
    workgroups fill the chip or have little to read (1.5B O at 8 rows 7.2 -> 5.9 us, 7B down 38.3 -> 36.1
    us, 72B down 111 -> 107.5 us); a few workgroups with much to read each want ticketed ranges (1.5B
    down: 96 workgroups of 287 KB, 17.4 us in one workgroup each, 12.5 in five ranges)."""
    if M > SAME_ORDER_MAX_ROWS:
        # Where norms are folded beyond that many rows (all from HBM, at 24 and 64 rows):
        groups32 = -(-N // 32)
        if groups32 <= 96 and K <= 6144:
            # few and short weight rows: one range, no tickets, the rows of A shared out over the workgroups
            # (0.5B down: 10.7 / 11.2 us against 15.5 / 19.6 in two ticketed ranges and 11.0 / 12.6 in seven)
            return 1
        # else the ranges of the partial-sum rule, which suit the residual epilogue as well (1.5B down, 48 x 5
        # workgroups: 15.6 / 17.9 us against 16.8 / 19.9 with four ranges; 3B down, 64 x 4: 18.5 / 22.9 against
        # 21.8 / 28.4 with five; 7B down: eight, 35 / 47 us; 14B: six, 33 / 44; 14B O: six, 19 / 27 against 27 / 37
        # with two)
        return skinny_splits(N, K, M)
    tiles = -(-N // 16)
    # one such workgroup fills a compute unit, so the tiles should fill the chip's units a whole number of
    # times, or nearly (14B/32B down: 320 tiles are a full round and a quarter of one; 32B at 8 rows 86.7 us
    # side by side, ticketed ranges are ahead)
    units = _compute_units()
    rounds_full = tiles <= units or tiles % units == 0 or tiles % units >= 3 * units // 4
    if K >= 1024 and (tiles >= 192 or 32 * K <= 65536) and rounds_full:
        return -(-K // (-(-(-(-K // 4)) // 128) * 128))  # four, as the rounding to 128 leaves them
    splits = skinny_splits(N, K, 1)
    if splits == 4 and K >= 1024 and (tiles >= 192 or 32 * K <= 65536):
        # four would be taken side by side (the same sums, slower here)
        return 5 if K // 5 >= 256 else 3
    return splits  # (four ticketed ranges where the launcher keeps them apart: 3B down at 8 rows 14.7 us, five 16.5)


def gemm_skinny(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                epilogue: int = EPI_BF16, splits: int = 1, row_scale=None, following=None) -> None:
    """out = a @ w^T for at most 64 rows of `a`, reading `w` once.

    EPI_BF16: out [M, N] bfloat16 (+bias).  EPI_F32: out [M, N] float32, or [splits, M, N]
    partial sums over k ranges.  EPI_SWIGLU: w holds blocks of 8 gate rows followed by their 8
    up rows; out [M, N / 2] = silu(gate) * up.  With several k ranges the other epilogues'
    partial sums are added up inside the kernel (see `skinny_tickets`).

    `row_scale = (stats, eps)`: the rows of `a` are bfloat16(x * w_norm) of rows x that are still
    to be divided by their root mean square; `stats[m]` holds shares that add up to sum(x[m]^2),
    and row m's sums are multiplied by rsqrt(that / K + eps) before the epilogue.
    EPI_RESIDUAL: `out` is the float32 residual [M, N], to which the product is added in place;
    `following = (next_rows, next_w, next_stats)` receives bfloat16(out * next_w) [M, N] and the
    shares [M, stat_tiles(N)] of the new rows' sums of squares, for the product after the next norm."""
    _gpu(out, a, w, bias)
    M, K_ = a.shape
    N = w.shape[0]
    assert skinny_supported(a, w) and w.shape == (N, K_) and w.is_contiguous() and out.is_contiguous()
    nr = nw = ns = None
    nwf, ld_next = 0, 0
    if epilogue == EPI_SWIGLU:
        assert out.shape == (M, N // 2) and out.dtype == torch.bfloat16 and bias is None
    elif epilogue == EPI_F32:
        assert out.dtype == torch.float32
        assert tuple(out.shape) == ((M, N) if splits == 1 and out.dim() == 2 else (splits, M, N))
    elif epilogue == EPI_RESIDUAL:
        assert out.shape == (M, N) and out.dtype == torch.float32 and bias is None and following is not None
        next_rows, next_w, next_stats = following
        _gpu(next_rows, next_w, next_stats)
        assert next_rows.dtype == torch.bfloat16 and next_rows.shape == (M, N) and next_rows.stride(1) == 1
        assert next_stats.dtype == torch.float32 and next_stats.shape == (M, stat_tiles(N)) and next_stats.is_contiguous()
        assert next_w.numel() == N
        nr, ns, ld_next = next_rows.data_ptr(), next_stats.data_ptr(), next_rows.stride(0)
        nw, nwf = _param(next_w)
    else:
        assert out.shape == (M, N) and out.dtype == torch.bfloat16
    bp, bf = _param(bias)
    sp, st, se = _row_scale(row_scale, M, K_)
    parts, counters = _ticket_scratch(a.device, M, N, splits if epilogue != EPI_F32 else 1)
    if _RECORDING is not None:
        _RECORDING.add(library().pae_program_put_product(
            _RECORDING.host_ptr, _RECORDING.count, epilogue, out.data_ptr(), out.stride(-2), a.data_ptr(), a.stride(0),
            w.data_ptr(), bp, bf, M, N, K_, splits, _ptr(parts), _ptr(counters), sp, st, se, nr, ld_next, nw, nwf, ns,
            None), out, a, w, bias, parts, row_scale, following,
            activation_bytes=library().pae_program_activation_bytes(M, K_, splits))
        return
    checking = (parts is not None and CHECK_TICKET_SUMS and not torch.cuda.is_current_stream_capturing())
    before = out.clone() if checking and epilogue == EPI_RESIDUAL else None
    _launch_ticketed(counters, lambda: library().pae_gemm_skinny(
        epilogue, out.data_ptr(), out.stride(-2), a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, N, K_, splits,
        M * N, _ptr(parts), _ptr(counters), sp, st, se, nr, ld_next, nw, nwf, ns, _stream()))
    if checking:
        _check_ticket_sums(out, before, a, w, bias, epilogue, splits, row_scale, following)


# PAE_CHECK_TICKETS=sums: every product whose k ranges are added up inside the kernel is computed a
# second time in one k range (no tickets, no partial sums in memory) and the two results are compared.
# A partial sum read stale (from an earlier launch, or before it had arrived) is a whole k range's worth
# of error and shows far above the difference that the other order of adding leaves.
CHECK_TICKET_SUMS = os.environ.get("PAE_CHECK_TICKETS", "") == "sums"


def _check_ticket_sums(out, before, a, w, bias, epilogue, splits, row_scale, following) -> None:
    again = before if before is not None else torch.empty_like(out)
    follow = None
    if following is not None:
        follow = (torch.empty_like(following[0]), following[1], torch.empty_like(following[2]))
    pairs = [(out, again)] + ([(following[0], follow[0])] if follow is not None else [])
    gemm_skinny(again, a, w, bias, epilogue, 1, row_scale, follow)
    for got, want in pairs:
        got, want = got.float(), want.float()
        bound = 2.0 ** -6 * float(want.abs().max()) + 1e-30
        worst = float((got - want).abs().max())
        if not worst <= bound:
            raise KernelError(f"a product of {tuple(a.shape)} by {tuple(w.shape)} added up over {splits} k ranges inside "
                              f"the kernel differs from the same product in one range by {worst:.3e} (bound {bound:.3e}): "
                              "a partial sum was read before it had arrived, or left over from another launch")


TICKET_ARCHS = ("gfx950",)  # chips on which the fence-free ticket scheme has been validated
_TICKETS: dict = {}        # device index -> counters
_TICKET_STREAM: dict = {}  # device index -> the stream whose launches use them


def skinny_tickets(device) -> torch.Tensor:
    """The zeroed counters of products whose k ranges are added up inside the kernel.  Every launch
    leaves them zero, and launches share them, so they must run one after the other: the counters
    belong to the stream that is current when they are made (a model asks when it is bound, before
    any step is recorded as a graph), and `_ticket_scratch` refuses launches from another stream.
    Recording a graph on torch's capture stream is not a launch; its replays are, on the stream
    they are replayed on."""
    index = torch.device(device).index or 0
    if index not in _TICKETS:
        if torch.cuda.is_current_stream_capturing():
            raise KernelError("the ticket counters must exist before a graph is recorded")
        if device_arch() not in TICKET_ARCHS:
            # the scheme leans on how this chip's device-scope stores and loads reach the memory side
            # (see SkinnyTickets in csrc/gemm_skinny.hip); it has been validated on these chips only
            raise KernelError(f"k ranges added up inside a kernel are validated on {', '.join(TICKET_ARCHS)} only, "
                              f"not on {device_arch()}")
        _TICKETS[index] = torch.zeros(1 << 16, dtype=torch.int32, device=device)
        _TICKET_STREAM[index] = torch.cuda.current_stream(device).cuda_stream
    return _TICKETS[index]


def check_tickets_zero(device) -> None:
    """Raise unless every ticket counter is zero (it waits for the device: a check for tests and
    for runs with PAE_CHECK_TICKETS set, after each step)."""
    index = torch.device(device).index or 0
    counters = _TICKETS.get(index)
    if counters is not None and bool(counters.any()):
        where = counters.nonzero().flatten()[:8].tolist()
        raise KernelError(f"ticket counters {where} are not zero between launches: a product with k ranges "
                          "was cut short, or launches from two streams overlapped")


def _ticket_scratch(device, M: int, N: int, splits: int):
    """(partial sums, counters) for a product whose k ranges are added up inside the kernel."""
    if splits <= 1:
        return None, None
    lib, counters = library(), skinny_tickets(device)
    index = torch.device(device).index or 0
    if (not torch.cuda.is_current_stream_capturing()
            and torch.cuda.current_stream(device).cuda_stream != _TICKET_STREAM[index]):
        raise KernelError("products with k ranges share their ticket counters and must all be launched on the "
                          "stream the counters were made on; this launch comes from another stream")
    if lib.pae_skinny_ticket_slots(M, N) > counters.numel():
        raise KernelError(f"{N} weight rows by {M} rows need more ticket counters than there are")
    return torch.empty(lib.pae_skinny_ticket_floats(M, N, splits), dtype=torch.float32, device=device), counters


def _launch_ticketed(counters, call) -> None:
    """Run a launch that uses the ticket counters; if it is refused or fails, the counters are put
    back to zero before the error goes up (a later product would otherwise add up the wrong ranges)."""
    try:
        _check(call())
    except KernelError:
        if counters is not None and not torch.cuda.is_current_stream_capturing():
            counters.zero_()
        raise


def whole_sum_splits(N: int, K: int, M: int) -> int:
    """k ranges for a product whose epilogue needs whole sums (gate, rotation, bias), which the
    kernel then adds up itself.  That costs a trip to memory, and pays with more than 8 rows of
    activations where workgroups are few (measured at the 1.5B to 72B layer sizes):
    * the many-weight-rows kernel with little more than one workgroup per compute unit (7B gate/up
      at 64 rows: 85 -> 72 us; with more weight rows, or somewhat fewer, one range is as fast or faster);
    * few weight rows (the QKV products): ranges of about 1,280 (7B at 64 rows 26 -> 22 us in three,
      14B 37 -> 31 us in four, 72B 87 -> 54 us in six);
    * not with very few weight rows, where the rows of activations are shared out instead."""
    tiles, groups = -(-N // 32), -(-N // 128)
    if M <= SAME_ORDER_MAX_ROWS:
        # from the sizes alone, so that a row's sums do not depend on the batch (as `residual_splits`): one
        # range at every size (QKV from HBM at 1 / 8 / 16 rows, one range against the best of two to six: 72B
        # 37.2 / 43.7 / 52.0 us against 36.4 / 42.8 / 59.6; 14B 18.7 / 23.3 / 29.4 against 20.7 / 24.1 / 30.3; 7B 13.1 /
        # 15.2 / 20.4 against 13.1 / 14.1 / 20.9; gate/up likewise at all seven widths)
        return 1
    waves = -(-(-(-N // 16)) // 256)  # wavefronts of 16 weight rows a workgroup for at most 256 workgroups
    if 5 <= waves <= 8 and -(-(-(-N // 16)) // waves) >= 216:
        # one workgroup per compute unit, nearly all units busy: one range (the launcher then takes the
        # kernel of `waves` wavefronts; 1.5B gate/up at 32 rows 19.1 -> 16.7 us, at 64 rows 23.4 -> 22.2)
        return 1
    if 128 <= groups < 256:
        # a couple of workgroups of 32 weight rows per compute unit: three ranges from 32
        # rows on (1.5B gate/up at 64 rows 27.2 -> 23.3 us, at 32 rows 20.2 -> 19.0 us; below, one range is ahead)
        return 3 if M >= 32 and K >= 1536 else 1
    if tiles <= 96 or groups >= 384:
        return 1
    if groups >= 256:
        wanted = -(-(768 if M > 48 else 512) // groups)
        if K // wanted < 512:
            return 1
    else:
        # (and no more than make about a thousand 32-row workgroups: 72B QKV at 32 / 64 rows, 320 tiles, six
        # ranges 44.6 / 56.8 us, three 40.3 / 52.9)
        wanted = min(8, max(1, (K + 640) // 1280), max(1, round(1000 / tiles)))
    k_per = -(-(-(-K // wanted)) // 128) * 128
    return -(-K // k_per)


def skinny_rope_supported(a: torch.Tensor, w: torch.Tensor, hd: int, rot: int) -> bool:
    """Whether `gemm_skinny_rope` takes this product: a skinny product whose head size and
    rotated width are multiples of 16."""
    return skinny_supported(a, w) and hd % 16 == 0 and rot % 16 == 0 and 0 <= rot <= hd


def gemm_skinny_rope(q_out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor], nh: int,
                     nkv: int, hd: int, rot: int, cos_sin: Optional[torch.Tensor], positions: torch.Tensor,
                     tok_seq: Optional[torch.Tensor], block_tables: Optional[torch.Tensor], block_size: int,
                     k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                     splits: Optional[int] = None, row_scale=None) -> None:
    """Query/key/value projection of at most 64 rows with the rotation and the cache write in its
    epilogue: q_out[M, nh * hd] = rotated queries; rotated keys and raw values go to their slots
    (nkv == 0: `w` holds the query rows only and nothing is stored).  `cos_sin`: see `rope_table`."""
    _gpu(q_out, a, w, bias, cos_sin, positions, tok_seq, block_tables, k_cache, v_cache)
    M, K_ = a.shape
    assert skinny_rope_supported(a, w, hd, rot) and w.shape == ((nh + 2 * nkv) * hd, K_) and w.is_contiguous()
    assert q_out.shape == (M, nh * hd) and q_out.dtype == torch.bfloat16 and q_out.stride(1) == 1
    assert positions.dtype == torch.int32 and positions.numel() == M
    _check_cos_sin(cos_sin, rot, M)
    max_blocks = 0
    if nkv:
        assert k_cache.dtype == torch.bfloat16 == v_cache.dtype
        assert tok_seq.dtype == torch.int32 and tok_seq.numel() == M
        assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
        _check_pools(k_cache, v_cache, nkv, block_size, hd)
        max_blocks = block_tables.shape[1]
    bp, bf = _param(bias)
    lib, N = library(), w.shape[0]
    splits = 1 if splits is None else splits
    parts, counters = _ticket_scratch(a.device, M, N, splits)
    sp, st, se = _row_scale(row_scale, M, K_)
    if _RECORDING is not None:
        _RECORDING.add(lib.pae_program_put_product_rope(
            _RECORDING.host_ptr, _RECORDING.count, q_out.data_ptr(), q_out.stride(0), a.data_ptr(), a.stride(0),
            w.data_ptr(), bp, bf, M, K_, nh, nkv, hd, rot, _ptr(cos_sin) if rot else None, positions.data_ptr(),
            _ptr(tok_seq), _ptr(block_tables), max_blocks, block_size, _ptr(k_cache), _ptr(v_cache), splits, _ptr(parts),
            _ptr(counters), sp, st, se), q_out, a, w, bias, cos_sin, parts, row_scale,
            activation_bytes=lib.pae_program_activation_bytes(M, K_, splits))
        return
    _launch_ticketed(counters, lambda: lib.pae_gemm_skinny_rope(
        q_out.data_ptr(), q_out.stride(0), a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, K_, nh, nkv, hd, rot,
        _ptr(cos_sin) if rot else None, positions.data_ptr(), _ptr(tok_seq), _ptr(block_tables), max_blocks,
        block_size, _ptr(k_cache), _ptr(v_cache), splits, _ptr(parts), _ptr(counters), sp, st, se, _stream()))


def gemm_plain(out: torch.Tensor, a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None) -> None:
    """out[M, N] = a[M, K] @ w[N, K]^T (+ bias), float32 accumulation in k order."""
    _not_while_recording("gemm_plain")
    _gpu(out, a, w, bias)
    M, K = a.shape
    N = w.shape[0]
    assert w.shape == (N, K) and w.is_contiguous() and w.dtype == a.dtype
    assert out.shape == (M, N) and a.stride(1) == 1 and out.stride(1) == 1
    if bias is not None:
        assert bias.numel() == N
    bp, bf = _param(bias)
    _check(library().pae_gemm_plain(code_of(a.dtype), code_of(out.dtype), out.data_ptr(), out.stride(0),
                                    a.data_ptr(), a.stride(0), w.data_ptr(), bp, bf, M, N, K, _stream()))


def paged_attention_generic(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            positions: torch.Tensor, tok_seq: torch.Tensor, block_tables: torch.Tensor,
                            nh: int, nkv: int, hd: int, scale: float, window: int) -> None:
    """out[t, h*hd:(h+1)*hd] = attention of query head h of token t over the cached
    keys start..positions[t] of sequence tok_seq[t]."""
    _not_while_recording("paged_attention_generic")
    _gpu(out, q, k_cache, v_cache, positions, tok_seq, block_tables)
    T = q.shape[0]
    bs = k_cache.shape[2]
    assert q.dim() == 2 and q.stride(1) == 1 and q.shape[1] >= nh * hd and q.dtype == k_cache.dtype == out.dtype
    assert out.shape[0] == T and out.stride(1) == 1 and out.shape[1] >= nh * hd
    _check_pools(k_cache, v_cache, nkv, bs, hd)
    assert positions.dtype == torch.int32 and positions.numel() == T
    assert tok_seq.dtype == torch.int32 and tok_seq.numel() == T
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    _check(library().pae_paged_attention_generic(
        code_of(q.dtype), out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(),
        v_cache.data_ptr(), positions.data_ptr(), tok_seq.data_ptr(), block_tables.data_ptr(),
        block_tables.shape[1], bs, T, nh, nkv, hd, float(scale), int(window), _stream()))


def mfma_attention_supported(dtype: torch.dtype, nh: int, nkv: int, hd: int, bs: int) -> bool:
    """Shapes the matrix-core attention kernels take; others go through the generic kernel."""
    return dtype == torch.bfloat16 and hd % 32 == 0 and 32 <= hd <= 256 and bs % 16 == 0 and nh // nkv <= 16


def attn_decode(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                dec_work: torch.Tensor, block_tables: torch.Tensor, nh: int, nkv: int, hd: int, scale: float,
                window: int) -> None:
    """Attention of the single new token of each sequence listed in `dec_work` over that sequence's
    cached keys: split over the keys, then merged.  dec_work[i] = (flat row of the token, its
    position, row of its sequence in `block_tables`, 0)."""
    _gpu(out, q, k_cache, v_cache, dec_work, block_tables)
    bs = k_cache.shape[2]
    assert q.dtype == torch.bfloat16 == out.dtype == k_cache.dtype and q.stride(1) == 1 and out.stride(1) == 1
    assert q.shape[1] >= nh * hd and out.shape[1] >= nh * hd and out.shape[0] == q.shape[0]
    _check_pools(k_cache, v_cache, nkv, bs, hd)
    assert dec_work.dtype == torch.int32 and dec_work.dim() == 2 and dec_work.shape[1] == 4 and dec_work.is_contiguous()
    assert dec_work.data_ptr() % 16 == 0, "the decode work list must start on a 16-byte boundary"
    n = dec_work.shape[0]
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    # (the kernel looks at row i of the tables before it knows token i's own row: the rows must be there)
    assert n <= block_tables.shape[0], "more single tokens than sequences in the tables"
    max_splits = -(-block_tables.shape[1] * bs // library().pae_attn_decode_split())
    part_acc = torch.empty((n * nh * max_splits, hd), dtype=torch.float32, device=q.device)
    part_ml = torch.empty((n * nh * max_splits, 2), dtype=torch.float32, device=q.device)
    if _RECORDING is not None:
        _RECORDING.room(2)  # the splits' partial results, then their merge
        code = library().pae_program_put_attention(
            _RECORDING.host_ptr, _RECORDING.count, out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0),
            k_cache.data_ptr(), v_cache.data_ptr(), dec_work.data_ptr(), n, block_tables.data_ptr(),
            block_tables.shape[1], bs, nh, nkv, hd, float(scale), int(window), part_acc.data_ptr(), part_ml.data_ptr())
        _RECORDING.add(code, out, q, part_acc, part_ml)
        _RECORDING.add(code)
        return
    _check(library().pae_attn_decode_bf16(
        out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        dec_work.data_ptr(), n, block_tables.data_ptr(), block_tables.shape[1], bs, nh, nkv, hd, float(scale),
        int(window), part_acc.data_ptr(), part_ml.data_ptr(), _stream()))


PREFILL_TILE = 64  # tokens per run of the prefill attention kernel (one workgroup each)


def attn_prefill(out: torch.Tensor, q: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                 tiles: torch.Tensor, positions: torch.Tensor, block_tables: torch.Tensor,
                 nh: int, nkv: int, hd: int, scale: float, window: int) -> None:
    """Attention of runs of consecutive tokens; tiles[t] = (table row of the sequence, first
    flat token, number of tokens <= PREFILL_TILE).  One workgroup per run and head, whose
    wavefronts share out the keys; workgroups start in the order of `tiles`, so the runs with
    the most keys should come first."""
    _not_while_recording("attn_prefill")
    _gpu(out, q, k_cache, v_cache, tiles, positions, block_tables)
    bs = k_cache.shape[2]
    assert q.dtype == torch.bfloat16 == out.dtype == k_cache.dtype and q.stride(1) == 1 and out.stride(1) == 1
    assert q.shape[1] >= nh * hd and out.shape[1] >= nh * hd and out.shape[0] == q.shape[0]
    _check_pools(k_cache, v_cache, nkv, bs, hd)
    assert tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 3 and tiles.is_contiguous()
    assert positions.dtype == torch.int32 and positions.numel() == q.shape[0]
    assert block_tables.dtype == torch.int32 and block_tables.dim() == 2 and block_tables.is_contiguous()
    _check(library().pae_attn_prefill_bf16(
        out.data_ptr(), out.stride(0), q.data_ptr(), q.stride(0), k_cache.data_ptr(), v_cache.data_ptr(),
        tiles.data_ptr(), tiles.shape[0], positions.data_ptr(), block_tables.data_ptr(), block_tables.shape[1],
        bs, nh, nkv, hd, float(scale), int(window), _stream()))


def sample(tokens: torch.Tensor, logits: torch.Tensor, temperature: Optional[torch.Tensor],
           uniform: Optional[torch.Tensor]) -> None:
    """tokens[r] = argmax(logits[r]) where temperature[r] == 0 (or no temperatures
    are given), else the inverse-CDF sample of softmax(logits[r] / temperature[r]) at uniform[r]."""
    _not_while_recording("sample")
    _gpu(tokens, logits, temperature, uniform)
    R, V = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    assert tokens.dtype == torch.int32 and tokens.numel() == R
    for t in (temperature, uniform):
        if t is not None:
            assert t.dtype == torch.float32 and t.numel() == R
    chunks = library().pae_sample_chunks(V)
    chunk_max = torch.empty(R * chunks, dtype=torch.float32, device=logits.device)
    chunk_arg = torch.empty(R * chunks, dtype=torch.int32, device=logits.device)
    chunk_sum = (torch.empty(R * chunks, dtype=torch.float64, device=logits.device)
                 if temperature is not None else None)
    _check(library().pae_sample(tokens.data_ptr(), logits.data_ptr(), logits.stride(0), _ptr(temperature),
                                _ptr(uniform), R, V, chunk_max.data_ptr(), chunk_arg.data_ptr(),
                                _ptr(chunk_sum), _stream()))


def sample_static(tokens: torch.Tensor, logits: torch.Tensor, temperature: Optional[torch.Tensor],
                  uniform: Optional[torch.Tensor]) -> None:
    """`sample` without a workspace: the chunk results go to a buffer inside the library's image on
    the GPU, so nothing is allocated here or there.  Rows times chunks beyond that buffer's slots
    are refused; calls that overlap on one GPU race (they share the buffer)."""
    _not_while_recording("sample_static")
    _gpu(tokens, logits, temperature, uniform)
    R, V = logits.shape
    assert logits.dtype == torch.float32 and logits.stride(1) == 1
    assert tokens.dtype == torch.int32 and tokens.numel() == R
    for t in (temperature, uniform):
        if t is not None:
            assert t.dtype == torch.float32 and t.numel() == R
    _check(library().pae_sample_static(tokens.data_ptr(), logits.data_ptr(), logits.stride(0), _ptr(temperature),
                                       _ptr(uniform), R, V, _stream()))
