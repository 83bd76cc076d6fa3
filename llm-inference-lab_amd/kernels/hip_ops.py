"""The kernel set of the engine: thin, checked ctypes calls into the HIP
libraries.  There is no other implementation on the product path: without a
GPU, or if a library cannot be built or loaded, constructing ``HipOps`` raises.

Every call checks on the host that dtypes, shapes, strides and devices are what
the kernel and its grid assume before it launches anything; a size that the
kernels do not take is refused with ``UnsupportedSizeError``.  Kernels run on
the current PyTorch stream, so they can be captured into a HIP graph.
"""
from __future__ import annotations

import ctypes
import dataclasses
from typing import Dict, Optional

import torch

from ..config.errors import UnsupportedSizeError
from ..parts.base import PendingSums
from . import build
from .debug import DispatchRules, KernelDebug

DT_F32, DT_BF16 = 0, 1
EPI_STORE, EPI_RESID, EPI_F32, EPI_SWIGLU, EPI_QKV, EPI_PART = 0, 1, 2, 3, 4, 5
EPI_RELU2 = 6        # STORE through max(z, 0)^2, taken on the float32 sum
EPI_GEGLU = 7        # the paired product with gelu (tanh form) on the gate instead of silu
GATE_EPILOGUES = {"silu": EPI_SWIGLU, "gelu_tanh": EPI_GEGLU}

_c_int, _c_long, _c_float, _c_size, _c_ptr = (ctypes.c_int, ctypes.c_long, ctypes.c_float,
                                              ctypes.c_size_t, ctypes.c_void_p)


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return DT_F32
    if t.dtype == torch.bfloat16:
        return DT_BF16
    raise TypeError(f"kernels take float32 or bfloat16 tensors, got {t.dtype}")


class KernelError(RuntimeError):
    pass


_NO_HEADS = (None, None, None, None, 0, 0, None, None, 0, 0, 0)     # a few-row product without the q/k/v epilogue


class PackedWeight:
    """A bfloat16 matrix [n, k] in the order the matrix cores read it: strips of 16
    rows, a strip a run of 1 KB tiles (16 rows x 32 columns, one MFMA B operand,
    lane l owning 16 bytes), zero-padded to whole tiles.  Made by
    ``HipOps.prepare_weight``; the product kernels take nothing else in bfloat16."""

    __slots__ = ("data", "shape", "dtype", "device")

    def __init__(self, data: torch.Tensor, n: int, k: int):
        self.data = data
        self.shape = (n, k)
        self.dtype = data.dtype
        self.device = data.device

    def data_ptr(self) -> int:
        return self.data.data_ptr()

    def is_contiguous(self) -> bool:
        return True

    def numel(self) -> int:
        return self.shape[0] * self.shape[1]

    def element_size(self) -> int:
        return self.data.element_size()


class StackedWeight:
    """Several matrices of equal shape ``[n, k]`` kept as one operand (``HipOps.prepare_stacked``):
    ``data`` is the float32 tensor ``[members * n, k]`` or the packed bfloat16 matrix of ``members *
    padded`` rows; a grouped product addresses member ``e`` by its first strip of rows."""

    def __init__(self, data, members: int, n: int, padded: int, k: int):
        self.data, self.members, self.n, self.padded, self.k = data, int(members), int(n), int(padded), int(k)
        self.dtype = data.dtype

    def numel(self) -> int:
        return self.members * self.n * self.k

    def element_size(self) -> int:
        return self.data.element_size()


class MoePlan:
    """The rows of a step sorted by expert (``HipOps.moe_plan``): ``capacity`` places in tiles of
    ``bm``; ``place_of [rows, top]``, ``place_row [capacity]``, ``tile_member [capacity / bm]``."""

    __slots__ = ("bm", "capacity", "place_of", "place_row", "tile_member")

    def __init__(self, bm, capacity, place_of, place_row, tile_member):
        self.bm, self.capacity = int(bm), int(capacity)
        self.place_of, self.place_row, self.tile_member = place_of, place_row, tile_member


class LaunchRecord:
    """The calls into the kernel libraries that a part made while it was recorded, so that
    the same part under the same conditions can make them again without its Python code:
    ``calls[i]`` is ``(function, argument list, library)``, or ``(None, callable, None)``
    for a call that depends on the step's data and is made anew through its closure
    (``HipOps.live``).  ``dry``: nothing is launched while recording (a recorded sequence is
    only compared with one kept from before)."""

    __slots__ = ("calls", "dry")

    def __init__(self, dry: bool = False):
        self.calls = []
        self.dry = dry

    def same_as(self, other: "LaunchRecord") -> bool:
        if len(self.calls) != len(other.calls):
            return False
        for (fa, aa, _), (fb, ab, _) in zip(self.calls, other.calls):
            if (fa is None) != (fb is None):
                return False
            if fa is not None and (fa is not fb or list(aa[:-1]) != list(ab[:-1])):     # (the last is the stream)
                return False
        return True


class AttentionCall:
    """An attention call with its unchanging arguments checked and laid out
    (``HipOps.prepare_attention``)."""

    __slots__ = ("ops", "lib", "args", "most_requests", "most_context", "row_req", "heads", "dtype")
    N_REQS, MAX_Q, MAX_CTX, ROW_REQ, SHORT_LEN, N_SHORT, SHORT_CTX, STREAM = 12, 13, 14, 23, 24, 25, 26, 29

    def __init__(self, ops, lib, args, most_requests, most_context, row_req, heads, dtype):
        self.ops, self.lib, self.args = ops, lib, args
        self.most_requests, self.most_context, self.row_req = most_requests, most_context, row_req
        self.heads, self.dtype = heads, dtype

    def launch(self, n_reqs: int, max_q_len: int, max_ctx_len: int, short=None) -> None:
        if n_reqs > self.most_requests:
            raise ValueError("attention: request arrays are shorter than the number of requests")
        if max_ctx_len > self.most_context:
            raise ValueError("attention: the block table is too narrow for the longest context")
        a = self.args
        a[self.N_REQS], a[self.MAX_Q], a[self.MAX_CTX] = n_reqs, max_q_len, max_ctx_len
        if short is not None:
            _, short_len, n_short, short_ctx = short
            if (short_len != self.ops.attention_short_limit(self.heads[0], self.heads[1], self.dtype, max_q_len)
                    or not 0 < n_short < n_reqs or short_ctx > max_ctx_len or self.row_req is None):
                raise ValueError("attention: the description of the step's short requests does not fit")
            a[self.ROW_REQ], a[self.SHORT_LEN], a[self.N_SHORT], a[self.SHORT_CTX] = self.row_req, short_len, n_short, short_ctx
        else:
            a[self.ROW_REQ], a[self.SHORT_LEN], a[self.N_SHORT], a[self.SHORT_CTX] = None, 0, 0, 0
        a[self.STREAM] = self.ops._stream()
        self.ops._call(self.lib.llmlab_paged_attention, *a, lib=self.lib)


class HipOps:
    WORKSPACE_FLOATS = 16 * 1024 * 1024      # 64 MiB of float32 scratch (split partial sums)
    ARRIVED_INTS = 64 * 1024                 # arrival counters: one per (request, kv head) of a step

    def __init__(self, device="cuda:0"):
        if not torch.cuda.is_available():
            raise RuntimeError(
                "no GPU is visible: the engine runs on hand-written HIP kernels for gfx950 "
                "and has no CPU path")
        self.device = torch.device(device)
        if self.device.type != "cuda":
            raise RuntimeError(f"the kernels need a GPU device, got '{device}'")
        torch.cuda.set_device(self.device)
        if self.device.index is None:
            self.device = torch.device("cuda", torch.cuda.current_device())
        self._core = self._load(build.core_library())
        self._declare_core()
        if self._core.llmlab_abi_version() != 8:
            raise RuntimeError("kernel library and Python bindings disagree on the interface")
        self._attn: Dict[int, ctypes.CDLL] = {}
        self._mixer_libs: Dict[str, ctypes.CDLL] = {}
        self._shared: Dict[int, tuple] = {}
        self.num_cus = int(torch.cuda.get_device_properties(self.device).multi_processor_count)
        self.workspace = torch.empty(self.WORKSPACE_FLOATS, dtype=torch.float32, device=self.device)
        # Counters by which blocks of one kernel find out which of them is the last to arrive
        # (the key splits of decode attention, the pieces of the argmax).  Zero between
        # launches: the block that reads the full count sets its counter back.
        self.arrived = torch.zeros(self.ARRIVED_INTS, dtype=torch.int32, device=self.device)
        self.loaded_libraries = [self._core._name]
        self.calls_made = 0          # calls into the kernel libraries so far
        self._record: Optional[LaunchRecord] = None
        self.debug_epoch = 0         # counts the changes of forced kernel choices (kernels/debug.py)
        self.rules = DispatchRules()         # the measured thresholds of the dispatch, in one place
        self.debug = KernelDebug(self)       # forcing kernel choices from outside (tests, measurements)

    # ---------------------------------------------------------------- loading
    @staticmethod
    def _load(path: str) -> ctypes.CDLL:
        try:
            return ctypes.CDLL(path)
        except OSError as e:
            raise RuntimeError(f"cannot load the kernel library {path}: {e}") from None

    def _declare_core(self) -> None:
        c = self._core
        c.llmlab_last_error.restype = ctypes.c_char_p
        c.llmlab_abi_version.restype = _c_int
        c.llmlab_embed.argtypes = [_c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_rmsnorm.argtypes = [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_ptr, _c_int,
                                     _c_int, _c_ptr, _c_int, _c_size, _c_ptr]
        c.llmlab_rope_kv_write.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
                                           _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr,
                                           _c_ptr, _c_ptr]
        c.llmlab_rope_inplace.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_long, _c_long,
                                          _c_ptr, _c_ptr, _c_ptr]
        c.llmlab_linear.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_int,
                                    _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_sample.argtypes = [_c_ptr, _c_long, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr]
        c.llmlab_gather_tokens.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]
        c.llmlab_gather_tokens.restype = _c_int
        c.llmlab_packed_elements.argtypes = [_c_int, _c_int]
        c.llmlab_packed_elements.restype = _c_long
        c.llmlab_pack_weight.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]
        c.llmlab_pack_weight.restype = _c_int
        c.llmlab_argmax.argtypes = [_c_ptr, _c_long, _c_int, _c_int, _c_ptr, _c_ptr, _c_size, _c_ptr, _c_size,
                                    _c_ptr]
        c.llmlab_argmax.restype = _c_int
        c.llmlab_linear_qkv.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                                        _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr,
                                        _c_int, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_linear_tile.argtypes = [_c_int, _c_int, _c_int, _c_int]
        c.llmlab_linear_tile.restype = _c_int
        c.llmlab_linear_partials.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
                                             _c_int, _c_int, _c_size, _c_int, _c_ptr]
        c.llmlab_qkv_from_pieces.argtypes = [_c_ptr, _c_int, _c_size, _c_int, _c_ptr, _c_int, _c_int, _c_int,
                                             _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                                             _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]
        c.llmlab_qkv_from_pieces.restype = _c_int
        c.llmlab_linear_plan.argtypes = [_c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_linear_plan.restype = None
        c.llmlab_skinny_linear.argtypes = [
            _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr,
            _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
            _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int,
            _c_ptr, _c_int, _c_int, _c_size, _c_int, _c_size, _c_ptr]
        c.llmlab_add_pending.argtypes = [_c_ptr, _c_ptr, _c_int, _c_size, _c_int, _c_int, _c_ptr]
        c.llmlab_add_pending.restype = _c_int
        c.llmlab_layernorm.argtypes = [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr]
        c.llmlab_layernorm.restype = _c_int
        c.llmlab_layernorm_add.argtypes = [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                                           _c_ptr]
        c.llmlab_layernorm_add.restype = _c_int
        c.llmlab_activation.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_long, _c_ptr]
        c.llmlab_activation.restype = _c_int
        c.llmlab_gate_heads.argtypes = [_c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]
        c.llmlab_gate_heads.restype = _c_int
        c.llmlab_add_row_vector.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]
        c.llmlab_add_row_vector.restype = _c_int
        c.llmlab_linear_grouped.argtypes = [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
                                            _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr]
        c.llmlab_linear_grouped.restype = _c_int
        for fn in (c.llmlab_embed, c.llmlab_rmsnorm, c.llmlab_rope_kv_write, c.llmlab_rope_inplace,
                   c.llmlab_linear, c.llmlab_sample, c.llmlab_skinny_linear,
                   c.llmlab_linear_partials, c.llmlab_linear_qkv):
            fn.restype = _c_int

    def _attention_lib(self, head_dim: int) -> ctypes.CDLL:
        lib = self._attn.get(head_dim)
        if lib is None:
            lib = self._load(build.attention_library(head_dim))
            lib.llmlab_last_error.restype = ctypes.c_char_p
            lib.llmlab_attention_head_dim.restype = _c_int
            if lib.llmlab_attention_head_dim() != head_dim:
                raise RuntimeError(f"attention library for head size {head_dim} reports "
                                   f"{lib.llmlab_attention_head_dim()}")
            lib.llmlab_paged_attention.argtypes = [
                _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr,
                _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr, _c_int, _c_ptr, _c_size,
                _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_size, _c_ptr]
            lib.llmlab_paged_attention.restype = _c_int
            self._attn[head_dim] = lib
            self.loaded_libraries.append(lib._name)
        return lib

    def check_attention_sizes(self, num_heads: int, num_kv_heads: int, head_dim: int, dtype) -> None:
        if head_dim % 16 != 0 or not 16 <= head_dim <= 256:
            raise UnsupportedSizeError(
                f"attention kernels take head sizes that are multiples of 16 from 16 to 256, "
                f"got {head_dim} (in float32 too: the pages of keys and values are laid out in "
                f"blocks of 16 numbers of a head for both dtypes, and the kernels are compiled "
                f"per head size)")
        if num_heads % num_kv_heads != 0:
            raise UnsupportedSizeError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        self._attention_lib(head_dim)

    def check_product_sizes(self, inner: int, dtype, what: str) -> None:
        """Refuse at load time what the matrix product kernels do not take."""
        if dtype == torch.bfloat16 and inner % 8 != 0:
            raise UnsupportedSizeError(
                f"{what}: bfloat16 matrix products need an inner size that is a multiple of 8, "
                f"got {inner} (the float32 path takes any size)")

    def prepare_weight(self, w: torch.Tensor, shared: bool = False):
        """What the product kernels take for the matrix ``w`` [n, k]: float32 as it is,
        bfloat16 packed in fragment order (a copy; ``w`` itself is not kept).

        ``shared``: parts that may be bound to one and the same tensor (an embedding
        and an output head with tied weights) get one packed copy between them;
        the model calls ``release_shared()`` when all its parts are bound."""
        if shared and id(w) in self._shared:
            return self._shared[id(w)][1]
        packed = self._prepare(w)
        if shared:
            self._shared[id(w)] = (w, packed)       # w is held so that its id stays its own
        return packed

    def release_shared(self) -> None:
        self._shared.clear()

    def _prepare(self, w: torch.Tensor):
        self._need(w, "weight")
        if w.dim() != 2:
            raise ValueError(f"a weight matrix has two dimensions, got {tuple(w.shape)}")
        if w.dtype == torch.float32:
            return w
        if w.dtype != torch.bfloat16:
            raise TypeError(f"weights are float32 or bfloat16, got {w.dtype}")
        n, k = w.shape
        self.check_product_sizes(k, w.dtype, "weight matrix")
        data = torch.empty(self._core.llmlab_packed_elements(n, k), dtype=torch.bfloat16, device=self.device)
        self._call(self._core.llmlab_pack_weight, self._ptr(w), self._ptr(data), n, k, self._stream())
        return PackedWeight(data, n, k)

    def _weight(self, w, name: str):
        """The weight operand of a product: packed if bfloat16."""
        if isinstance(w, PackedWeight):
            if w.device != self.device:
                raise ValueError(f"{name} is on {w.device}, the kernels run on {self.device}")
            return w
        self._need(w, name)
        if w.dtype == torch.bfloat16:
            raise TypeError(f"{name}: bfloat16 weights go through prepare_weight() once, when the "
                            f"part is bound; the product kernels read the packed order only")
        return w

    # ---------------------------------------------------------------- helpers
    def _stream(self):
        # the raw handle of the current stream (under graph capture: the capturing one);
        # asked for at every launch, so by the short way where torch has one
        raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)
        if raw is not None:
            return raw(self.device.index)
        return torch.cuda.current_stream(self.device).cuda_stream

    def _call(self, fn, *args, lib=None) -> None:
        """One call into the kernel libraries; a failure raises with the library's message."""
        self.calls_made += 1
        if self._record is not None:
            self._record.calls.append((fn, list(args), lib))
            if self._record.dry:
                return
        code = fn(*args)
        if code != 0:
            self._check(code, lib)

    # ------------------------------------------------- recorded launch sequences
    def begin_recording(self, dry: bool = False) -> LaunchRecord:
        """From now until ``end_recording`` every call into the kernel libraries is also
        written down (``engine/model.py`` keeps the sequences of its blocks and replays
        them for steps of the same shape)."""
        if self._record is not None:
            raise RuntimeError("a recording is already under way")
        self._record = LaunchRecord(dry)
        return self._record

    def end_recording(self) -> Optional[LaunchRecord]:
        record, self._record = self._record, None
        return record

    def live(self, launch) -> None:
        """``launch()`` makes calls whose arguments depend on the step's data (how many
        requests, how long their histories): while a sequence is recorded it is written
        down as a closure, to be called anew at every replay, and its own calls are not."""
        record = self._record
        if record is None:
            launch()
            return
        record.calls.append((None, launch, None))
        if record.dry:
            return
        self._record = None
        try:
            launch()
        finally:
            self._record = record

    def replay(self, record: LaunchRecord) -> None:
        """Make a recorded sequence of calls again, on the current stream."""
        stream = self._stream()
        for fn, args, lib in record.calls:
            if fn is None:
                args()
                continue
            args[-1] = stream
            self.calls_made += 1
            code = fn(*args)
            if code != 0:
                self._check(code, lib)

    def fingerprint(self):
        """What the host-side choices of the kernel set depend on beside the shapes."""
        return (self.num_cus, self.debug_epoch, dataclasses.astuple(self.rules))

    def _check(self, code: int, lib=None) -> None:
        if code != 0:
            msg = (lib or self._core).llmlab_last_error()
            raise KernelError(msg.decode() if msg else f"kernel call failed with code {code}")

    def _need(self, t: torch.Tensor, name: str, dtype=None, contiguous=True) -> torch.Tensor:
        if t.device != self.device:
            raise ValueError(f"{name} is on {t.device}, the kernels run on {self.device}")
        if dtype is not None and t.dtype != dtype:
            raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
        if contiguous and not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
        return t

    @staticmethod
    def _ptr(t: Optional[torch.Tensor]):
        # (a plain integer: ctypes makes the pointer argument of it, None is the null pointer)
        return t.data_ptr() if t is not None else None

    def synchronize(self) -> None:
        torch.cuda.synchronize(self.device)

    # ------------------------------------------------------------ elementwise
    def embed(self, table, ids, out) -> None:
        """Rows of ``table`` (float32, bfloat16, or bfloat16 packed by prepare_weight)."""
        packed = isinstance(table, PackedWeight)
        if not packed:
            self._need(table, "embedding table")
        self._need(ids, "token ids", torch.int32)
        self._need(out, "embedding output", torch.float32)
        rows, hidden = out.shape
        if ids.numel() != rows or table.shape[1] != hidden:
            raise ValueError(f"embed: ids {tuple(ids.shape)}, table {tuple(table.shape)}, "
                             f"out {tuple(out.shape)} do not fit")
        self._call(self._core.llmlab_embed, self._ptr(table), _dt(table), 1 if packed else 0,
                                            self._ptr(ids), self._ptr(out), rows, hidden, table.shape[0],
                                            self._stream())

    def gather_tokens(self, dst, dst_index, src, src_index, n) -> None:
        """dst[dst_index[i]] = src[src_index[i]] for i < n (all int32 on the GPU)."""
        for t, name in ((dst, "dst"), (dst_index, "dst_index"), (src, "src"), (src_index, "src_index")):
            self._need(t, f"gather_tokens {name}", torch.int32)
        if dst_index.numel() < n or src_index.numel() < n:
            raise ValueError("gather_tokens: index arrays are shorter than the count")
        self._call(self._core.llmlab_gather_tokens, self._ptr(dst), self._ptr(dst_index), self._ptr(src),
                                                    self._ptr(src_index), int(n), self._stream())

    def rmsnorm(self, x, weight, eps, out, rows=None, pending=None) -> None:
        """``out[i] = norm(x[rows[i]])``.  ``pending`` (all rows in order only): the pieces are
        folded into ``x`` on the way, ``x += sum_s parts[s]``, and the whole rows are normed."""
        self._need(x, "norm input", torch.float32)
        self._need(weight, "norm weight")
        self._need(out, "norm output")
        hidden = x.shape[1]
        n_out = out.shape[0]
        if weight.numel() != hidden or out.shape[1] != hidden:
            raise ValueError(f"rmsnorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, "
                             f"out {tuple(out.shape)} do not fit")
        if rows is None:
            if n_out != x.shape[0]:
                raise ValueError("rmsnorm: output rows differ from input rows")
        else:
            self._need(rows, "norm row indices", torch.int32)
            if rows.numel() != n_out:
                raise ValueError("rmsnorm: one row index per output row")
        pend = (None, 0, 0)
        if pending is not None:
            p = pending.parts
            if rows is not None or p.shape[1] != n_out or p.shape[2] != hidden or not p[0].is_contiguous():
                raise ValueError("rmsnorm: pending sums go with all rows in order and the same shape")
            pend = (self._ptr(p), pending.splits, p.stride(0))
        self._call(self._core.llmlab_rmsnorm, self._ptr(x), self._ptr(weight), _dt(weight), float(eps),
                                              self._ptr(out), _dt(out), self._ptr(rows), n_out, hidden,
                                              pend[0], pend[1], pend[2], self._stream())

    # ----------------------------------------------------------------- linear
    def _linear(self, x, w, out, bias, epilogue, n_out, pending: Optional[PendingSums] = None) -> None:
        self._need(x, "linear input")
        w = self._weight(w, "linear weight")
        if x.dtype != w.dtype:
            raise TypeError(f"linear: input is {x.dtype} but the weight is {w.dtype}")
        if out.device != self.device or out.stride(-1) != 1:
            raise ValueError("linear: output must be on the GPU with unit column stride")
        m, k = x.shape
        n = w.shape[0]
        if w.shape[1] != k or out.shape[0] != m or out.shape[1] != n_out:
            raise ValueError(f"linear: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} "
                             f"do not fit")
        if x.dtype == torch.bfloat16 and k % 8 != 0:
            raise UnsupportedSizeError(
                f"bfloat16 matrix products need an inner size that is a multiple of 8, got {k}")
        want_out = x.dtype if epilogue in (EPI_STORE, EPI_SWIGLU, EPI_RELU2, EPI_GEGLU) else torch.float32
        if out.dtype != want_out:
            raise TypeError(f"linear: output must be {want_out}, got {out.dtype}")
        if bias is not None:
            self._need(bias, "linear bias")
            if bias.numel() != n:
                raise ValueError("linear: bias length differs from the output width")
        ldo = out.stride(0) if m > 1 else max(out.stride(0), n_out)
        # few rows: the block kernel that splits K inside a block; from 17 rows on only
        # for narrow outputs (the tiled kernel has too few tiles there), measured
        if x.dtype == torch.bfloat16 and (m <= 16 or (n < 8192 and self.few_rows_take(m, n, k))):
            self._skinny(x, False, None, None, 0.0, w, bias, epilogue, out, m, n, k, ldo, n_out,
                         pending=pending)
            return
        if pending is not None:
            self.add_pending(out, pending)
        self._call(self._core.llmlab_linear,
            self._ptr(x), self._ptr(w), _dt(x), epilogue, self._ptr(out), self._ptr(bias),
            _dt(bias) if bias is not None else 0, m, n, k, ldo, n_out, self.num_cus, self._stream())

    def linear(self, x, w, out, bias=None) -> None:
        self._linear(x, w, out, bias, EPI_STORE, w.shape[0])

    def linear_relu2(self, x, w, out) -> None:
        """``out = max(x w^T, 0) ** 2`` in the compute dtype: the activation is taken on the float32
        sums and rounded once."""
        self._linear(x, w, out, None, EPI_RELU2, w.shape[0])

    def linear_residual(self, x, w, resid, bias=None, pending: Optional[PendingSums] = None) -> None:
        """``resid += x w^T (+ bias)``, and the pending pieces of ``resid`` with it."""
        self._linear(x, w, resid, bias, EPI_RESID, w.shape[0], pending)

    def linear_logits(self, x, w, out) -> None:
        self._linear(x, w, out, None, EPI_F32, w.shape[0])

    def linear_swiglu(self, x, w_gate_up, out, activation: str = "silu") -> None:
        """``out = act(x Wg^T) * (x Wu^T)`` with the rows of gate and up interleaved in runs of 16;
        ``activation``: ``silu`` or ``gelu_tanh``, taken on the float32 sums."""
        inter = out.shape[1]
        if w_gate_up.shape[0] != 2 * ((inter + 15) // 16 * 16):
            raise ValueError(f"linear_swiglu: {w_gate_up.shape[0]} interleaved rows do not belong "
                             f"to {inter} outputs")
        if activation not in GATE_EPILOGUES:
            raise ValueError(f"linear_swiglu: the gate's activation is one of {sorted(GATE_EPILOGUES)}, got {activation!r}")
        self._linear(x, w_gate_up, out, None, GATE_EPILOGUES[activation], inter)

    # ----------------------------------------------- few rows: fused kernels
    FUSED_MAX_ROWS = 1024         # most rows the few-row kernels take at all
    FEW_ROWS = 64                 # up to here a product may take them whatever its matrix
    FUSE_TILE_ROWS = 16           # the few-row kernels cut the rows into tiles of so many

    def few_rows_take(self, rows: int, outer: int, inner: int) -> bool:
        """Whether a plain product of ``rows`` rows with an ``[outer, inner]`` matrix goes to the
        few-row kernels: always up to 64 rows; beyond, up to ``rules.few_rows_max`` rows while
        the matrix, read once per tile of 16 rows, stays below ``rules.few_rows_read_bytes``."""
        if rows <= self.FEW_ROWS:
            return True
        tiles = (rows + self.FUSE_TILE_ROWS - 1) // self.FUSE_TILE_ROWS
        return (rows <= min(self.rules.few_rows_max, self.FUSED_MAX_ROWS)
                and 2.0 * outer * inner * tiles < self.rules.few_rows_read_bytes)
    STAGE_BYTES = 118 * 1024      # most LDS the staged rows of a fused kernel may take

    def can_fuse(self, rows: int, dtype, inner: int, outer: Optional[int] = None) -> bool:
        """Whether the fused few-row kernels take this step: bfloat16, few rows, a tile
        of rows (``inner`` wide) fits the staging buffer in LDS, and beyond one tile the
        matrix (``outer`` rows) is a small one."""
        if dtype != torch.bfloat16 or not 0 < rows <= min(max(self.FEW_ROWS, self.rules.few_rows_max), self.FUSED_MAX_ROWS):
            return False
        tiles = (rows + self.FUSE_TILE_ROWS - 1) // self.FUSE_TILE_ROWS
        limit = self.rules.fuse_read_bytes if rows <= self.FEW_ROWS else self.rules.few_rows_read_bytes
        if tiles > 1 and (outer is None or 2.0 * outer * inner * tiles >= limit):
            return False
        return min(rows, self.FUSE_TILE_ROWS) * ((inner + 31) // 32 * 32 + 8) * 2 <= self.STAGE_BYTES

    def _skinny(self, x, norm, x_rows, norm_w, eps, w, bias, epilogue, out, m, n, k, ldo, n_out,
                qkv=None, pending: Optional[PendingSums] = None, ksplit: int = 1,
                part_stride: int = 0) -> None:
        if pending is not None:
            p = pending.parts
            if (p.dtype != torch.float32 or p.dim() != 3 or p.stride(2) != 1 or p.device != self.device
                    or pending.splits > p.shape[0]):
                raise ValueError("pending sums: float32 [splits, rows, width] on the GPU expected")
            width = x.shape[1] if norm else n
            if p.shape[2] != width:
                raise ValueError(f"pending sums are {p.shape[2]} wide, the rows they belong to {width}")
            pend = (self._ptr(p), pending.splits, p.stride(1), p.stride(0))
        else:
            pend = (None, 0, 0, 0)
        if qkv is None:
            heads = _NO_HEADS
        else:
            table, ptr = qkv["table"], self._ptr
            heads = (ptr(qkv["inv_freq"]), ptr(qkv["positions"]), ptr(qkv["row_req"]), ptr(table),
                     table.stride(0) if table is not None else 0, qkv["page_size"], ptr(qkv["k_cache"]),
                     ptr(qkv["v_cache"]), qkv["nq"], qkv["nkv"], qkv["d"])
        self._call(self._core.llmlab_skinny_linear,
            x.data_ptr(), 1 if norm else 0, self._ptr(x_rows), self._ptr(norm_w),
            _dt(norm_w) if norm_w is not None else 0, float(eps), w.data_ptr(), self._ptr(bias),
            _dt(bias) if bias is not None else 0, epilogue, out.data_ptr(), m, n, k, ldo, n_out,
            *heads, self.num_cus, pend[0], pend[1], pend[2], pend[3], int(ksplit),
            int(part_stride), self._stream())

    # --------------------------------------------- sums left in pieces (deferred)
    MAX_SPLITS = 8
    split_max_rows = 32           # most rows of a few-row product that is left in pieces

    def pieces_too_large_to_read_per_block(self, pending: Optional[PendingSums]) -> bool:
        """A fused kernel that takes pieces on adds them as it reads the rows, in every one
        of its blocks; beyond this size the norm kernel should fold them once instead
        (32 rows of width 3584 in 7 pieces, 3.2 MB: 12 us a layer more in the fused kernels)."""
        if pending is None:
            return False
        p = pending.parts
        return pending.splits * p.shape[1] * p.shape[2] * 4 > self.rules.pieces_per_block_bytes

    def pieces_by_tiles(self, rows: int, n: int, k: int) -> bool:
        """Whether a product left in pieces is cut by the tiled kernel (else by the few-row one)."""
        return rows > self.FEW_ROWS or (rows > self.FUSE_TILE_ROWS and 2.0 * n * k >= self.rules.tiled_pieces_bytes)

    def split_count(self, rows: int, dtype, n: int, k: int) -> int:
        """Into how many pieces along the inner size a few-row product ``[rows, k] x
        [n, k]^T`` should be cut so that it spreads over the chip: a narrow output
        gives too few blocks otherwise, and a compute unit draws only so much from
        memory.  1: do not cut."""
        if dtype != torch.bfloat16 or rows <= 0:
            return 1
        if self.pieces_by_tiles(rows, n, k):
            # many rows, tiled kernel: its own estimate (rounds of blocks over the chip times
            # the K tiles of a block, plus a write and a read of the result for every piece)
            if k % 8:
                return 1
            if self.rules.forced_tiled_pieces:
                return max(1, min(self.rules.forced_tiled_pieces, (k + 63) // 64, self.MAX_SPLITS))
            return self._linear_plan(rows, n, k)[0]
        if rows > self.split_max_rows:
            return 1
        strips, steps = (n + 15) // 16, (k + 31) // 32
        most = min(steps // self.rules.min_steps_per_split, self.MAX_SPLITS)
        if strips > self.num_cus and rows <= self.FUSE_TILE_ROWS:
            # a wide output whose strips do not go evenly over the units (320 strips on 256
            # units: the busiest unit streams two, the chip waits for it): cut so that the
            # blocks fill whole rounds (5120 x 27648 at 8 rows: 70 us whole, 53 in 4 pieces)
            def waste(p):
                rounds = strips * p / self.num_cus
                return -(-strips * p // self.num_cus) / rounds
            if waste(1) < self.rules.uneven_rounds_waste:
                return 1
            for p in range(2, max(most, 1) + 1):
                if waste(p) <= 1.07:       # (3 pieces, 3.75 rounds, do as well as 4 and cost the next reader less)
                    return p
            return 1
        want = self.num_cus // max(strips, 1)
        return max(1, min(want, most))

    def _linear_plan(self, rows: int, n: int, k: int):
        """(pieces, tile) for a many-row product that adds into float32 rows."""
        out = (_c_int * 2)()
        self._core.llmlab_linear_plan(rows, n, k, self.num_cus, self.MAX_SPLITS, self.rules.min_tiles_per_split, out)
        return out[0], out[1]

    def linear_partials(self, x, w, parts: torch.Tensor, splits: int, bias=None) -> PendingSums:
        """``parts[s] = x[:, K_s] w[:, K_s]^T`` for the ``splits`` pieces ``K_s`` of the inner
        size (bias in piece 0): the product without the final sum."""
        self._need(x, "linear input", torch.bfloat16)
        w = self._weight(w, "linear weight")
        m, k = x.shape
        n = w.shape[0]
        if (w.shape[1] != k or parts.dtype != torch.float32 or parts.dim() != 3 or parts.shape[0] < splits
                or parts.shape[1] != m or parts.shape[2] != n or parts.stride(2) != 1
                or parts.device != self.device):
            raise ValueError(f"linear_partials: x {tuple(x.shape)}, w {tuple(w.shape)}, "
                             f"parts {tuple(parts.shape)} for {splits} pieces do not fit")
        if not 1 <= splits <= self.MAX_SPLITS:
            raise ValueError(f"linear_partials: {splits} pieces")
        if not self.pieces_by_tiles(m, n, k):
            self._skinny(x, False, None, None, 0.0, w, bias, EPI_PART, parts, m, n, k, parts.stride(1), n,
                         ksplit=splits, part_stride=parts.stride(0))
        else:
            if bias is not None:
                self._need(bias, "bias")
            self._call(self._core.llmlab_linear_partials,
                self._ptr(x), self._ptr(w), self._ptr(parts), self._ptr(bias),
                _dt(bias) if bias is not None else 0, m, n, k, parts.stride(1), splits, parts.stride(0),
                self._linear_plan(m, n, k)[1], self._stream())
        return PendingSums(parts, splits)

    def add_pending(self, x: torch.Tensor, pending: PendingSums) -> None:
        """``x += sum_s parts[s]``: fold the pieces into the float32 stream."""
        self._need(x, "residual stream", torch.float32)
        p = pending.parts
        rows, width = x.shape
        if p.shape[1] != rows or p.shape[2] != width or not p[0].is_contiguous():
            raise ValueError("add_pending: pieces and stream differ in shape")
        self._call(self._core.llmlab_add_pending, self._ptr(x), self._ptr(p), pending.splits, p.stride(0),
                                                  rows, width, self._stream())

    def _fused_common(self, x, norm_w, w, rows):
        self._need(x, "residual stream", torch.float32)
        self._need(norm_w, "norm weight")
        w = self._weight(w, "weight")
        if w.dtype != torch.bfloat16:
            raise TypeError("the fused few-row kernels are bfloat16 kernels")
        k = x.shape[1]
        if norm_w.numel() != k or w.shape[1] != k:
            raise ValueError(f"fused norm + product: x {tuple(x.shape)}, norm weight "
                             f"{tuple(norm_w.shape)}, w {tuple(w.shape)} do not fit")
        if k % 8 != 0:
            raise UnsupportedSizeError(
                f"bfloat16 matrix products need an inner size that is a multiple of 8, got {k}")
        if not 0 < rows <= self.FUSED_MAX_ROWS:
            raise ValueError(f"the fused kernels take 1..{self.FUSED_MAX_ROWS} rows, got {rows}")
        return w, k

    def _qkv_checks(self, what, rows, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions,
                    row_req, block_table, page_size, k_cache, v_cache, q_out) -> int:
        n = (num_heads + 2 * num_kv_heads) * head_dim
        if w_qkv.shape[0] != n or tuple(q_out.shape) != (rows, num_heads * head_dim):
            raise ValueError(f"{what}: weight or output shape does not fit the heads")
        self._need(q_out, "q output", torch.bfloat16)
        self._need(positions, "positions", torch.int32)
        if positions.numel() < rows:
            raise ValueError(f"{what}: one position per row")
        if b_qkv is not None and b_qkv.numel() != n:
            raise ValueError(f"{what}: bias length")
        if inv_freq is not None and (inv_freq.dtype != torch.float32 or inv_freq.numel() != head_dim // 2):
            raise ValueError(f"{what}: the frequency table must hold head_dim/2 float32 entries")
        if k_cache is not None:
            self._need(row_req, "row -> request map", torch.int32)
            self._need(block_table, "block table", torch.int32)
            pages = k_cache.shape[0]
            if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, head_dim)
                    or tuple(v_cache.shape) != (pages, num_kv_heads, head_dim, page_size)
                    or not k_cache.is_contiguous() or not v_cache.is_contiguous()
                    or k_cache.dtype != torch.bfloat16 or v_cache.dtype != torch.bfloat16
                    or row_req.numel() < rows):
                raise ValueError(f"{what}: cache tensors do not have the paged layout")
        return n

    def fused_norm_qkv(self, x, norm_w, eps, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq,
                       positions, row_req, block_table, page_size, k_cache, v_cache, q_out,
                       pending: Optional[PendingSums] = None) -> None:
        """q_out = rotate(norm(x) Wq^T + bq); rotated k and v of the new positions go to
        their pages (skipped when no cache is given).  ``pending``: pieces still owed to
        the rows of x, added while they are read (x itself is left as it is)."""
        rows = x.shape[0]
        w_qkv, k = self._fused_common(x, norm_w, w_qkv, rows)
        n = self._qkv_checks("fused_norm_qkv", rows, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim,
                             inv_freq, positions, row_req, block_table, page_size, k_cache, v_cache, q_out)
        self._skinny(x, True, None, norm_w, eps, w_qkv, b_qkv, EPI_QKV, q_out, rows, n, k,
                     q_out.shape[1], n,
                     dict(inv_freq=inv_freq, positions=positions, row_req=row_req, table=block_table,
                          page_size=page_size, k_cache=k_cache, v_cache=v_cache, nq=num_heads,
                          nkv=num_kv_heads, d=head_dim), pending=pending)

    QKV_ROPE_MAX_ROWS = 64        # up to here the few-row kernel, beyond it the tiled one
    QKV_PIECES_MAX_ROWS = 384     # up to here a large matrix may go through pieces along its inner size

    def can_fuse_qkv_rope(self, rows: int, dtype, head_dim: int, n: Optional[int] = None,
                          k: Optional[int] = None) -> bool:
        """Whether ``qkv_rope_cache`` takes this step: bfloat16, and a head that one block
        holds (few rows: the few-row kernel's block; more: the tile that a product ``[rows, k]
        x [n, k]^T`` gets, which a head must divide)."""
        if dtype != torch.bfloat16 or rows <= 0 or head_dim % 16 or head_dim < 16:
            return False
        if rows <= self.QKV_ROPE_MAX_ROWS:
            return head_dim <= (128 if rows > 32 else 256)
        if n is not None and k is not None and (self.few_rows_take(rows, n, k)
                                                or self._qkv_pieces_plan(rows, n, k) is not None):
            return True
        return (n is not None and k is not None
                and self._core.llmlab_linear_tile(rows, n, k, self.num_cus) % head_dim == 0)

    def _qkv_pieces_plan(self, rows: int, n: int, k: int):
        """``(pieces, tile)`` if q/k/v of these sizes goes through pieces along the inner size
        (then any head size does: the second kernel rotates whole rows), else None."""
        if not (self.rules.qkv_pieces_min_rows <= rows <= self.QKV_PIECES_MAX_ROWS and self.pieces_by_tiles(rows, n, k)):
            return None
        if rows > self.FEW_ROWS and self.few_rows_take(rows, n, k):
            return None
        pieces, tile = self._linear_plan(rows, n, k)
        if rows > self.FEW_ROWS and k >= 2 * 64 * self.rules.min_tiles_per_split:
            # (65 to 384 rows: two pieces at least.  4608 x 3584 at 192 / 256 rows: 24 / 31 us
            # against 33 / 39 whole; 2560 x 2048: 15 / 18.5 against 20.5; the estimate of
            # the plan, made for products that add into the stream, says one)
            pieces = max(pieces, 2)
        if self.rules.forced_tiled_pieces:
            pieces = max(1, min(self.rules.forced_tiled_pieces, (k + 63) // 64, self.MAX_SPLITS))
        if pieces > 1 and pieces * rows * n <= self.workspace.numel():
            return pieces, tile
        return None

    def qkv_rope_cache(self, h, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions,
                       row_req, block_table, page_size, k_cache, v_cache, q_out) -> None:
        """The same for activations ``h`` (bfloat16, already normed): product, bias, rotation
        and cache write in one kernel."""
        rows, k = h.shape
        self._need(h, "activations", torch.bfloat16)
        w_qkv = self._weight(w_qkv, "weight")
        n = w_qkv.shape[0]
        if w_qkv.shape[1] != k or k % 8 != 0 or not self.can_fuse_qkv_rope(rows, h.dtype, head_dim, n, k):
            raise ValueError(f"qkv_rope_cache: {rows} rows of {k}, heads of {head_dim} do not fit")
        self._qkv_checks("qkv_rope_cache", rows, w_qkv, b_qkv, num_heads, num_kv_heads, head_dim,
                         inv_freq, positions, row_req, block_table, page_size, k_cache, v_cache, q_out)
        plan = self._qkv_pieces_plan(rows, n, k)
        if plan is not None:
            # some rows of a large matrix: a head per block leaves most of the chip idle, so
            # the product is cut along K by the tiled kernel and a second kernel sums the
            # pieces, rotates and writes the cache (64 rows of 7168 x 5120: 26 us against 52
            # in one kernel, of 4608 x 3584: 19 against 24; the same at 24 rows, slower below)
            pieces, tile = plan
            if b_qkv is not None:
                self._need(b_qkv, "bias")
            parts = self.workspace[:pieces * rows * n].view(pieces, rows, n)
            self._call(self._core.llmlab_linear_partials,
                self._ptr(h), self._ptr(w_qkv), self._ptr(parts), None, 0, rows, n, k, n, pieces,
                rows * n, tile, self._stream())
            self._call(self._core.llmlab_qkv_from_pieces,
                self._ptr(parts), pieces, rows * n, n, self._ptr(b_qkv),
                _dt(b_qkv) if b_qkv is not None else 0, rows, num_heads, num_kv_heads, head_dim,
                self._ptr(inv_freq), self._ptr(positions), self._ptr(row_req), self._ptr(block_table),
                block_table.stride(0) if block_table is not None else 0, int(page_size),
                self._ptr(k_cache), self._ptr(v_cache), self._ptr(q_out), q_out.stride(0), self._stream())
            return
        if rows <= self.QKV_ROPE_MAX_ROWS or self.few_rows_take(rows, n, k):
            self._skinny(h, False, None, None, 0.0, w_qkv, b_qkv, EPI_QKV, q_out, rows, n, k,
                         q_out.shape[1], n,
                         dict(inv_freq=inv_freq, positions=positions, row_req=row_req, table=block_table,
                              page_size=page_size, k_cache=k_cache, v_cache=v_cache, nq=num_heads,
                              nkv=num_kv_heads, d=head_dim))
            return
        if b_qkv is not None:
            self._need(b_qkv, "bias")
        self._call(self._core.llmlab_linear_qkv,
            self._ptr(h), self._ptr(w_qkv), self._ptr(b_qkv), _dt(b_qkv) if b_qkv is not None else 0,
            self._ptr(q_out), rows, n, k, q_out.stride(0), self._ptr(inv_freq), self._ptr(positions),
            self._ptr(row_req), self._ptr(block_table), block_table.stride(0) if block_table is not None else 0,
            int(page_size), self._ptr(k_cache), self._ptr(v_cache), num_heads, num_kv_heads, head_dim,
            self.num_cus, self._stream())

    def fused_norm_swiglu(self, x, norm_w, eps, w_gate_up, out, pending: Optional[PendingSums] = None,
                          activation: str = "silu") -> None:
        rows, inter = out.shape
        w_gate_up, k = self._fused_common(x, norm_w, w_gate_up, rows)
        self._need(out, "SwiGLU output", torch.bfloat16)
        if x.shape[0] != rows or w_gate_up.shape[0] != 2 * ((inter + 15) // 16 * 16):
            raise ValueError("fused_norm_swiglu: shapes do not fit")
        self._skinny(x, True, None, norm_w, eps, w_gate_up, None, GATE_EPILOGUES[activation], out, rows,
                     w_gate_up.shape[0], k, out.shape[1], inter, pending=pending)

    def fused_norm_logits(self, x, rows_index, norm_w, eps, w, out, pending: Optional[PendingSums] = None) -> None:
        """out[i] = norm(x[rows_index[i]]) W^T in float32."""
        rows, vocab = out.shape
        w, k = self._fused_common(x, norm_w, w, rows)
        self._need(out, "logits", torch.float32)
        if w.shape[0] != vocab:
            raise ValueError("fused_norm_logits: weight rows differ from the vocabulary")
        if rows_index is not None:
            self._need(rows_index, "row indices", torch.int32)
            if rows_index.numel() < rows:
                raise ValueError("fused_norm_logits: one row index per output row")
        elif x.shape[0] != rows:
            raise ValueError("fused_norm_logits: rows differ")
        self._skinny(x, True, rows_index, norm_w, eps, w, None, EPI_F32, out, rows, vocab, k,
                     out.shape[1], vocab, pending=pending)

    # ------------------------------------------------------------------- rope
    def rope_inplace(self, x, positions, inv_freq) -> None:
        rows, heads, d = x.shape
        if x.stride(2) != 1:
            raise ValueError("rope: the head dimension must be contiguous")
        self._need(positions, "positions", torch.int32)
        self._need(inv_freq, "rotary frequencies", torch.float32)
        if inv_freq.numel() != d // 2 or positions.numel() < rows:
            raise ValueError("rope: frequency table or positions do not fit")
        self._call(self._core.llmlab_rope_inplace,
            self._ptr(x), _dt(x), rows, heads, d, x.stride(0), x.stride(1), self._ptr(inv_freq),
            self._ptr(positions), self._stream())

    def rope_kv_write(self, qkv, num_heads, num_kv_heads, head_dim, inv_freq, positions, row_req,
                      block_table, page_size, k_cache, v_cache) -> None:
        self._need(qkv, "qkv", contiguous=False)
        rows = qkv.shape[0]
        if qkv.stride(1) != 1 or qkv.shape[1] != (num_heads + 2 * num_kv_heads) * head_dim:
            raise ValueError(f"rope_kv_write: qkv {tuple(qkv.shape)} does not hold {num_heads}+2*"
                             f"{num_kv_heads} heads of {head_dim}")
        self._need(positions, "positions", torch.int32)
        if positions.numel() < rows:
            raise ValueError("rope_kv_write: one position per row")
        if inv_freq is not None:
            self._need(inv_freq, "rotary frequencies", torch.float32)
            if inv_freq.numel() != head_dim // 2:
                raise ValueError("rope_kv_write: the frequency table must hold head_dim/2 entries")
        table_stride = 0
        if k_cache is not None:
            self._need(row_req, "row -> request map", torch.int32)
            self._need(block_table, "block table", torch.int32)
            if row_req.numel() < rows:
                raise ValueError("rope_kv_write: one request index per row")
            pages = k_cache.shape[0]
            if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, head_dim)
                    or tuple(v_cache.shape) != (pages, num_kv_heads, head_dim, page_size)
                    or not k_cache.is_contiguous() or not v_cache.is_contiguous()
                    or k_cache.dtype != qkv.dtype or v_cache.dtype != qkv.dtype):
                raise ValueError("rope_kv_write: cache tensors do not have the paged layout")
            table_stride = block_table.stride(0)
        self._call(self._core.llmlab_rope_kv_write,
            self._ptr(qkv), _dt(qkv), rows, qkv.stride(0) if rows > 1 else qkv.shape[1], num_heads,
            num_kv_heads, head_dim, self._ptr(inv_freq), self._ptr(positions), self._ptr(row_req),
            self._ptr(block_table), table_stride, page_size, self._ptr(k_cache), self._ptr(v_cache),
            self._stream())

    # -------------------------------------------------------------- attention
    def attention_short_limit(self, num_heads: int, num_kv_heads: int, dtype, max_q_len: int) -> int:
        """A mixed step (portions of prompts beside decoding requests) is served by two
        launches: its requests of a few tokens go to the one that splits their keys over
        the chip, the portions to the tiled one.  Returns the most tokens a request may
        bring to count as short in such a step, or 0 if the step is not divided."""
        group = num_heads // num_kv_heads
        if group <= 16 < max_q_len * group:
            return 16 // group
        return 0

    def paged_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table,
                        page_size, q_start, start_pos, n_reqs, max_q_len, max_ctx_len, window, scale,
                        out, short=None) -> None:
        """``short``: ``(row_req, limit, count, longest)`` for a step in which ``count`` of the
        requests (not all) bring at most ``limit = attention_short_limit(...)`` tokens, the
        longest context among those being ``longest``."""
        self.prepare_attention(qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table, page_size,
                               q_start, start_pos, window, scale, out,
                               short[0] if short is not None else None).launch(n_reqs, max_q_len, max_ctx_len, short)

    def prepare_attention(self, qkv, num_heads, num_kv_heads, head_dim, k_cache, v_cache, block_table,
                          page_size, q_start, start_pos, window, scale, out, row_req=None) -> "AttentionCall":
        """Everything of an attention call that does not change while the same buffers serve
        the same number of rows, checked and laid out once; ``launch`` then takes what a step
        brings (how many requests, their longest portion and context, its short requests).
        ``q_start`` and ``start_pos`` may be longer than a step's requests; ``row_req`` is
        needed only if a step will name short requests."""
        lib = self._attention_lib(head_dim)
        rows = qkv.shape[0]
        self._need(qkv, "queries", contiguous=False)
        self._need(out, "attention output")
        self._need(block_table, "block table", torch.int32)
        self._need(q_start, "request row starts", torch.int32)
        self._need(start_pos, "request start positions", torch.int32)
        pages = k_cache.shape[0]
        if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, head_dim)
                or tuple(v_cache.shape) != (pages, num_kv_heads, head_dim, page_size)
                or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
            raise ValueError("attention: cache tensors do not have the paged layout")
        if not (qkv.dtype == out.dtype == k_cache.dtype == v_cache.dtype):
            raise TypeError("attention: queries, cache and output must share one dtype")
        if qkv.stride(1) != 1 or qkv.shape[1] < num_heads * head_dim:
            raise ValueError("attention: the query rows are too narrow")
        if tuple(out.shape) != (rows, num_heads * head_dim):
            raise ValueError(f"attention: output {tuple(out.shape)} != ({rows}, {num_heads * head_dim})")
        if page_size < 16 or page_size & (page_size - 1):
            raise UnsupportedSizeError(f"page size {page_size} is not a power of two >= 16")
        if row_req is not None:
            self._need(row_req, "row -> request map", torch.int32)
            if row_req.numel() < rows:
                raise ValueError("attention: one request index per row")
        q_stride = qkv.stride(0) if rows > 1 else qkv.shape[1]
        args = [self._ptr(qkv), _dt(qkv), q_stride, num_heads, num_kv_heads, self._ptr(k_cache),
                self._ptr(v_cache), self._ptr(block_table), block_table.stride(0), page_size,
                self._ptr(q_start), self._ptr(start_pos), 0, 0, 0,
                int(window) if window else 0, float(scale), self._ptr(out), out.stride(0) if rows > 1 else
                out.shape[1], self._ptr(self.workspace), self.workspace.numel(), rows, self.num_cus,
                None, 0, 0, 0, self._ptr(self.arrived), self.arrived.numel(), None]
        return AttentionCall(self, lib, args, most_requests=min(q_start.numel() - 1, start_pos.numel(), block_table.shape[0]),
                             most_context=block_table.shape[1] * page_size, row_req=self._ptr(row_req),
                             heads=(num_heads, num_kv_heads), dtype=qkv.dtype)

    # ------------------------------------------- layer norm, plain activations
    def layernorm(self, x, weight, eps, out, rows=None) -> None:
        """``out[i] = (x[r] - mean) / sqrt(var + eps) * weight`` for ``r = rows[i]`` (all rows in
        order when ``rows`` is None); ``x`` float32, ``out`` the compute dtype."""
        self._need(x, "norm input", torch.float32)
        self._need(weight, "norm weight")
        self._need(out, "norm output")
        hidden, n_out = x.shape[1], out.shape[0]
        if weight.numel() != hidden or out.shape[1] != hidden:
            raise ValueError(f"layernorm: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)} do not fit")
        if rows is None:
            if n_out != x.shape[0]:
                raise ValueError("layernorm: output rows differ from input rows")
        else:
            self._need(rows, "norm row indices", torch.int32)
            if rows.numel() != n_out:
                raise ValueError("layernorm: one row index per output row")
        self._call(self._core.llmlab_layernorm, self._ptr(x), self._ptr(weight), _dt(weight), float(eps),
                   self._ptr(out), _dt(out), self._ptr(rows), n_out, hidden, self._stream())

    def layernorm_add(self, y, weight, eps, resid, copy=None) -> None:
        """``resid += layernorm(y)`` on the float32 stream; ``copy`` (compute dtype, same shape)
        receives the stream's new rows for the product that reads them next."""
        self._need(y, "sublayer output", torch.float32)
        self._need(resid, "residual stream", torch.float32)
        self._need(weight, "norm weight")
        rows, hidden = resid.shape
        if tuple(y.shape) != (rows, hidden) or weight.numel() != hidden or y.data_ptr() == resid.data_ptr():
            raise ValueError(f"layernorm_add: y {tuple(y.shape)}, weight {tuple(weight.shape)}, stream "
                             f"{tuple(resid.shape)} do not fit (and are two buffers)")
        if copy is not None:
            self._need(copy, "copy of the stream")
            if tuple(copy.shape) != (rows, hidden):
                raise ValueError("layernorm_add: the copy has the stream's shape")
        self._call(self._core.llmlab_layernorm_add, self._ptr(y), self._ptr(weight), _dt(weight), float(eps),
                   self._ptr(resid), self._ptr(copy), _dt(copy) if copy is not None else DT_F32, rows, hidden,
                   self._stream())

    ACTIVATIONS = {"cast": 0, "relu2": 1, "zero": 2}

    def activation(self, x, out, kind: str) -> None:
        """``out = act(x)`` element by element, ``x`` float32, ``out`` any kernel dtype of the same
        shape (``cast``: the value itself; ``relu2``: ``max(x, 0) ** 2``; ``zero``: 0 whatever ``x``)."""
        self._need(x, "activation input", torch.float32)
        self._need(out, "activation output")
        if kind not in self.ACTIVATIONS:
            raise ValueError(f"unknown activation '{kind}'; known: {', '.join(sorted(self.ACTIVATIONS))}")
        if tuple(x.shape) != tuple(out.shape):
            raise ValueError(f"activation: {tuple(x.shape)} -> {tuple(out.shape)}")
        self._call(self._core.llmlab_activation, self._ptr(x), self._ptr(out), _dt(out), self.ACTIVATIONS[kind],
                   x.numel(), self._stream())

    def gate_heads(self, out, gate, num_heads: int, head_dim: int, kind: str = "sigmoid") -> None:
        """``out[r, h, :] *= sigmoid(gate[r, h])`` in place: ``out [rows, heads * head_dim]`` of a kernel
        dtype, ``gate [rows, heads]`` float32; sigmoid and product in float32, one rounding."""
        if kind != "sigmoid":
            raise ValueError(f"gate_heads: unknown gate '{kind}'")
        self._need(out, "mixer output")
        self._need(gate, "head gates", torch.float32)
        rows = out.shape[0]
        if tuple(out.shape) != (rows, num_heads * head_dim) or tuple(gate.shape) != (rows, num_heads):
            raise ValueError(f"gate_heads: output {tuple(out.shape)}, gates {tuple(gate.shape)} do not fit "
                             f"{num_heads} heads of {head_dim}")
        self._call(self._core.llmlab_gate_heads, self._ptr(out), _dt(out), self._ptr(gate), rows, int(num_heads),
                   int(head_dim), self._stream())

    def add_row_vector(self, x, table, row: int) -> None:
        """``x[r, :] += table[row, :]`` for every row ``r`` of the float32 stream."""
        self._need(x, "residual stream", torch.float32)
        self._need(table, "offset table", torch.float32)
        if table.dim() != 2 or table.shape[1] != x.shape[1] or not 0 <= row < table.shape[0]:
            raise ValueError(f"add_row_vector: row {row} of a table {tuple(table.shape)} onto {tuple(x.shape)}")
        self._call(self._core.llmlab_add_row_vector, self._ptr(x), table.data_ptr() + row * table.shape[1] * 4,
                   x.shape[0], x.shape[1], self._stream())

    # --------------------------------- parts with run-time sizes (own libraries)
    def _mixer_lib(self, kind: str) -> ctypes.CDLL:
        lib = self._mixer_libs.get(kind)
        if lib is None:
            lib = self._load(build.mixer_library(kind))
            lib.llmlab_last_error.restype = ctypes.c_char_p
            if kind == "windowed_attention":
                lib.llmlab_project_norm_write.argtypes = [
                    _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr, _c_ptr,
                    _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]
                lib.llmlab_project_norm_write.restype = _c_int
                lib.llmlab_sink_window_attention.argtypes = [
                    _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                    _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_float, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr,
                    _c_size, _c_int, _c_int, _c_ptr]
                lib.llmlab_sink_window_attention.restype = _c_int
                lib.llmlab_project_rotate_write.argtypes = [
                    _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_int, _c_float, _c_int,
                    _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                    _c_int, _c_ptr]
                lib.llmlab_project_rotate_write.restype = _c_int
                lib.llmlab_sink_window_attention_has_mfma.argtypes = [_c_int, _c_int, _c_int, _c_int]
                lib.llmlab_sink_window_attention_has_mfma.restype = _c_int
                lib.llmlab_debug_windowed_attention_plain.argtypes = [_c_int]
                lib.llmlab_debug_windowed_attention_plain.restype = None
                lib.llmlab_debug_windowed_attention_private_tiles.argtypes = [_c_int]
                lib.llmlab_debug_windowed_attention_private_tiles.restype = None
                lib.llmlab_latent_norm_write.argtypes = [
                    _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float, _c_ptr, _c_ptr, _c_ptr,
                    _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr]
                lib.llmlab_latent_norm_write.restype = _c_int
                lib.llmlab_head_products.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
                                                     _c_ptr, _c_ptr]
                lib.llmlab_head_products.restype = _c_int
            elif kind == "stream_ops":
                lib.llmlab_embed_pairs.argtypes = [
                    _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_float, _c_int, _c_int,
                    ctypes.c_longlong, ctypes.c_longlong, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_int, _c_ptr]
                lib.llmlab_embed_pairs.restype = _c_int
                lib.llmlab_causal_conv.argtypes = [_c_ptr, _c_int, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr,
                                                   _c_ptr, _c_int, _c_int, _c_ptr]
                lib.llmlab_causal_conv.restype = _c_int
                lib.llmlab_norm_conv.argtypes = [_c_ptr, _c_ptr, _c_int, _c_float, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr,
                                                 _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr]
                lib.llmlab_norm_conv.restype = _c_int
                lib.llmlab_gated_add.argtypes = [_c_ptr, _c_ptr, _c_int, _c_size, _c_ptr, _c_int, _c_ptr, _c_int, _c_int,
                                                 _c_ptr]
                lib.llmlab_gated_add.restype = _c_int
                lib.llmlab_softcap.argtypes = [_c_ptr, _c_float, _c_size, _c_ptr]
                lib.llmlab_softcap.restype = _c_int
                lib.llmlab_rmsnorm_add.argtypes = [_c_ptr, _c_ptr, _c_int, _c_size, _c_ptr, _c_float, _c_int, _c_int,
                                                   _c_ptr, _c_float, _c_ptr, _c_int, _c_ptr]
                lib.llmlab_rmsnorm_add.restype = _c_int
                lib.llmlab_scaled_sum.argtypes = [_c_ptr, _c_ptr, _c_float, _c_ptr, _c_float, _c_size, _c_ptr]
                lib.llmlab_scaled_sum.restype = _c_int
            elif kind == "linear_attention":
                lib.llmlab_gla_decay.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_float, _c_ptr,
                                                 _c_int, _c_ptr]
                lib.llmlab_gla_decay.restype = _c_int
                lib.llmlab_gla_slices.argtypes = [_c_int]
                lib.llmlab_gla_slices.restype = _c_int
                lib.llmlab_gla_scan.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_float, _c_int, _c_int,
                                                _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_ptr,
                                                _c_ptr, _c_int, _c_ptr]
                lib.llmlab_gla_scan.restype = _c_int
                lib.llmlab_gla_output.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_float, _c_ptr,
                                                  _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr]
                lib.llmlab_gla_output.restype = _c_int
                lib.llmlab_delta_gates.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr,
                                                   _c_ptr, _c_float, _c_float, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                                                   _c_ptr]
                lib.llmlab_delta_gates.restype = _c_int
                lib.llmlab_delta_scan.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int,
                                                  _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int,
                                                  _c_ptr, _c_ptr, _c_int, _c_ptr]
                lib.llmlab_delta_scan.restype = _c_int
            elif kind == "routed_experts":
                lib.llmlab_moe_select.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                                  _c_ptr, _c_ptr, _c_int, _c_ptr]
                lib.llmlab_moe_select.restype = _c_int
                lib.llmlab_moe_add_chosen.argtypes = [_c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
                                                      _c_int, _c_int, _c_ptr]
                lib.llmlab_moe_add_chosen.restype = _c_int
                lib.llmlab_moe_plan.argtypes = [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                                                _c_ptr]
                lib.llmlab_moe_plan.restype = _c_int
                lib.llmlab_moe_select_plan.argtypes = [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_float,
                                                       _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
                                                       _c_int, _c_ptr]
                lib.llmlab_moe_select_plan.restype = _c_int
                lib.llmlab_moe_combine.argtypes = [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int,
                                                   _c_int, _c_int, _c_ptr]
                lib.llmlab_moe_combine.restype = _c_int
            self._mixer_libs[kind] = lib
            self.loaded_libraries.append(lib._name)
        return lib

    # ------------------------------------------------------- routed experts
    def prepare_stacked(self, w: torch.Tensor, members: int) -> "StackedWeight":
        """``members`` matrices of equal shape ``[n, k]``, one below the other in ``w``, as the product
        kernels take them: float32 as they are; bfloat16 packed, every member padded to whole
        strips of 16 rows, so that a member is a run of whole strips of the packed order."""
        if w.dim() != 2 or members <= 0 or w.shape[0] % members:
            raise ValueError(f"prepare_stacked: {tuple(w.shape)} is not {members} matrices of equal height")
        n, k = w.shape[0] // members, w.shape[1]
        if w.dtype == torch.float32:
            return StackedWeight(self._need(w, "stacked weight"), members, n, n, k)
        padded = (n + 15) // 16 * 16
        if padded != n:
            grown = torch.zeros((members, padded, k), dtype=w.dtype, device=w.device)
            grown[:, :n] = w.view(members, n, k)
            w = grown.view(members * padded, k)
        return StackedWeight(self._prepare(w.contiguous()), members, n, padded, k)

    def stacked_member(self, stacked: "StackedWeight", e: int):
        """Member ``e`` as a weight operand of its own (a view, nothing is copied)."""
        if not 0 <= e < stacked.members:
            raise ValueError(f"a stack of {stacked.members} matrices has no member {e}")
        if isinstance(stacked.data, PackedWeight):
            per = self._core.llmlab_packed_elements(stacked.padded, stacked.k)
            return PackedWeight(stacked.data.data[e * per:(e + 1) * per], stacked.n, stacked.k)
        return stacked.data[e * stacked.n:(e + 1) * stacked.n]

    def moe_grouped(self, dtype) -> bool:
        """Whether the experts of this dtype run as grouped products over rows sorted by expert
        (bfloat16: the tiled matrix-core kernel in its grouped form; float32 runs every expert over
        all rows with the plain 32-bit products)."""
        return dtype == torch.bfloat16 and not self.rules.experts_one_by_one

    def _new_plan(self, rows: int, top: int, num_experts: int, scratch) -> "MoePlan":
        pairs = rows * top
        # tiles of 128 places once an expert's share of the rows fills several of them
        bm = 128 if pairs >= 512 * num_experts else 64
        capacity = (pairs + num_experts * (bm - 1) + bm - 1) // bm * bm
        return MoePlan(bm, capacity, scratch("experts.place_of", (rows, top), torch.int32),
                       scratch("experts.place_row", (capacity,), torch.int32),
                       scratch("experts.tile_member", (capacity // bm,), torch.int32))

    def moe_select_plan_takes(self, rows: int, outputs: int) -> bool:
        """Whether choice and sorting of a step of so many rows are one launch (``moe_select_plan``)."""
        return 0 < rows <= self.rules.select_plan_max_rows and outputs <= 64

    SCORINGS = {"softmax": 0, "sigmoid": 1}

    def moe_select_plan(self, logits, correction, groups: int, groups_keep: int, scale: float, chosen, weights,
                        num_experts: int, scratch, scoring: str = "softmax") -> "MoePlan":
        """``moe_select`` and ``moe_plan`` in one launch of one block, for steps of few rows."""
        lib = self._mixer_lib("routed_experts")
        for t, name, dt in ((logits, "router logits", torch.float32), (correction, "router correction", torch.float32),
                            (chosen, "chosen experts", torch.int32), (weights, "expert weights", torch.float32)):
            self._need(t, name, dt)
        rows, outputs = logits.shape
        top = chosen.shape[1]
        if (correction.numel() != outputs or tuple(chosen.shape) != (rows, top) or tuple(weights.shape) != (rows, top)
                or not self.moe_select_plan_takes(rows, outputs)):
            raise ValueError("moe_select_plan: shapes do not fit")
        plan = self._new_plan(rows, top, num_experts, scratch)
        self._call(lib.llmlab_moe_select_plan, self._ptr(logits), self._ptr(correction), rows, outputs, int(groups),
                   int(groups_keep), top, float(scale), self._ptr(chosen), self._ptr(weights), int(num_experts), plan.bm,
                   plan.capacity, self._ptr(plan.place_of), self._ptr(plan.place_row), self._ptr(plan.tile_member),
                   self.SCORINGS[scoring], self._stream(), lib=lib)
        return plan

    def moe_plan(self, chosen, num_experts: int, scratch) -> "MoePlan":
        """Sort the ``(row, choice)`` pairs of ``chosen [rows, top]`` by expert into tiles of places
        for the grouped products; choices at or beyond ``num_experts`` (outputs without tensors)
        get no place.  ``scratch(name, shape, dtype)`` hands out the plan's buffers."""
        lib = self._mixer_lib("routed_experts")
        self._need(chosen, "chosen experts", torch.int32)
        rows, top = chosen.shape
        plan = self._new_plan(rows, top, num_experts, scratch)
        bm, capacity = plan.bm, plan.capacity
        self._call(lib.llmlab_moe_plan, self._ptr(chosen), rows, top, int(num_experts), bm, capacity,
                   self._ptr(plan.place_of), self._ptr(plan.place_row), self._ptr(plan.tile_member), self._stream(),
                   lib=lib)
        return plan

    def _grouped(self, x, stacked: "StackedWeight", plan: "MoePlan", out, epilogue, n_out, rows_index) -> None:
        w = stacked.data
        if not isinstance(w, PackedWeight) or x.dtype != torch.bfloat16:
            raise TypeError("grouped products are bfloat16 products over a packed stack of matrices")
        self._need(x, "grouped product input", torch.bfloat16)
        self._need(out, "grouped product output")
        if x.shape[1] != stacked.k or out.shape[0] != plan.capacity or out.shape[1] != n_out:
            raise ValueError(f"grouped product: x {tuple(x.shape)}, members [{stacked.n}, {stacked.k}], "
                             f"out {tuple(out.shape)}, {plan.capacity} places")
        if rows_index is None and x.shape[0] != plan.capacity:
            raise ValueError("grouped product: one row of x per place")
        self._call(self._core.llmlab_linear_grouped, self._ptr(x), self._ptr(w), epilogue, self._ptr(out),
                   plan.capacity, stacked.padded, stacked.k, out.stride(0), int(n_out), self._ptr(plan.tile_member),
                   self._ptr(rows_index), plan.bm,
                   1 if plan.bm == 128 and stacked.padded >= self.rules.grouped_wide_min_columns else 0,
                   self._stream())

    def moe_gate_up(self, h, w_gate_up: "StackedWeight", plan: "MoePlan", act) -> None:
        """``act[place] = silu(h[row] Wg_e^T) * (h[row] Wu_e^T)`` for every place of the plan, ``e`` the
        expert of the place's tile and ``row`` the row of ``h`` at the place."""
        if act.dtype != torch.bfloat16 or 2 * ((act.shape[1] + 15) // 16 * 16) != w_gate_up.n:
            raise ValueError("moe_gate_up: the experts' gate and up rows do not interleave the outputs")
        self._grouped(h, w_gate_up, plan, act, EPI_SWIGLU, act.shape[1], plan.place_row)

    def moe_up_relu2(self, h, w_up: "StackedWeight", plan: "MoePlan", act) -> None:
        """``act[place] = max(h[row] Wu_e^T, 0) ** 2`` for every place of the plan (experts without a
        gate matrix); the square is taken on the float32 sums."""
        if act.dtype != torch.bfloat16 or act.shape[1] != w_up.padded:
            raise ValueError("moe_up_relu2: one output per (padded) row of an expert's up matrix")
        self._grouped(h, w_up, plan, act, EPI_RELU2, act.shape[1], plan.place_row)

    def moe_down(self, act, w_down: "StackedWeight", plan: "MoePlan", y) -> None:
        """``y[place] = act[place] Wd_e^T`` in float32."""
        if y.dtype != torch.float32 or y.shape[1] != w_down.n:
            raise ValueError("moe_down: the output is float32 [places, hidden]")
        self._grouped(act, w_down, plan, y, EPI_F32, w_down.n, None)

    def moe_combine(self, resid, y, plan: "MoePlan", chosen, weights, num_experts: int, h) -> None:
        """``resid[r] += sum_k weights[r, k] * y[place of (r, k)]``, the choices in their order; a
        choice at or beyond ``num_experts`` stands for ``h[r]`` itself."""
        lib = self._mixer_lib("routed_experts")
        self._need(resid, "residual stream", torch.float32)
        self._need(y, "expert outputs", torch.float32)
        self._need(h, "expert input")
        rows, hidden = resid.shape
        if (y.shape[1] != hidden or tuple(h.shape) != (rows, hidden) or chosen.shape[0] != rows
                or tuple(weights.shape) != tuple(chosen.shape) or tuple(plan.place_of.shape) != tuple(chosen.shape)):
            raise ValueError("moe_combine: shapes do not fit")
        self._call(lib.llmlab_moe_combine, self._ptr(resid), self._ptr(y), self._ptr(h), _dt(h),
                   self._ptr(plan.place_of), self._ptr(chosen), self._ptr(weights), rows, chosen.shape[1],
                   int(num_experts), hidden, self._stream(), lib=lib)

    def moe_select(self, logits, correction, groups: int, groups_keep: int, scale: float, chosen, weights,
                   scoring: str = "softmax") -> None:
        """Per row of the router's float32 ``logits [rows, outputs]``: scores ``softmax(logits)``
        (``scoring="sigmoid"``: the sigmoid of every logit by itself); choice
        values ``score + correction``; the outputs form ``groups`` equal groups of neighbours of which
        the ``groups_keep`` with the largest best choice value stay; ``chosen [rows, top]`` (int32) are
        the outputs with the largest choice values among those (ties: the smaller index), ``weights
        [rows, top]`` their scores times ``scale``."""
        lib = self._mixer_lib("routed_experts")
        self._need(logits, "router logits", torch.float32)
        self._need(correction, "router correction", torch.float32)
        self._need(chosen, "chosen experts", torch.int32)
        self._need(weights, "expert weights", torch.float32)
        rows, outputs = logits.shape
        top = chosen.shape[1]
        if correction.numel() != outputs or tuple(chosen.shape) != (rows, top) or tuple(weights.shape) != (rows, top):
            raise ValueError("moe_select: shapes do not fit")
        self._call(lib.llmlab_moe_select, self._ptr(logits), self._ptr(correction), rows, outputs, int(groups),
                   int(groups_keep), top, float(scale), self._ptr(chosen), self._ptr(weights), self.SCORINGS[scoring],
                   self._stream(), lib=lib)

    def moe_add_chosen(self, resid, src, chosen, weights, first: int, last: int) -> None:
        """``resid[r] += w_r * src[r]`` with ``w_r`` the sum of ``weights[r, k]`` over the ``k`` whose
        ``chosen[r, k]`` lies in ``[first, last)``; rows that chose none of them are left alone."""
        lib = self._mixer_lib("routed_experts")
        self._need(resid, "residual stream", torch.float32)
        self._need(src, "expert output")
        self._need(chosen, "chosen experts", torch.int32)
        self._need(weights, "expert weights", torch.float32)
        rows, hidden = resid.shape
        if tuple(src.shape) != (rows, hidden) or chosen.shape[0] != rows or tuple(weights.shape) != tuple(chosen.shape):
            raise ValueError("moe_add_chosen: shapes do not fit")
        self._call(lib.llmlab_moe_add_chosen, self._ptr(resid), self._ptr(src), _dt(src), self._ptr(chosen),
                   self._ptr(weights), rows, chosen.shape[1], int(first), int(last), hidden, self._stream(), lib=lib)

    def check_windowed_attention_sizes(self, num_heads, num_kv_heads, key_dim, value_dim, dtype) -> None:
        if num_heads % num_kv_heads:
            raise UnsupportedSizeError(f"{num_heads} heads are not a multiple of {num_kv_heads} kv heads")
        if not 0 < value_dim <= 1024 or not 0 < key_dim <= 4096:
            raise UnsupportedSizeError(f"windowed attention takes keys up to 4096 and values up to 1024 wide, "
                                       f"got {key_dim} and {value_dim}")
        self._mixer_lib("windowed_attention")

    def check_linear_attention_sizes(self, num_heads, key_dim, value_dim) -> None:
        if not 0 < key_dim <= 16 * 1024 or not 0 < value_dim <= 1024:
            raise UnsupportedSizeError(f"the linear attention scan takes up to 16384 key channels and 1024 value "
                                       f"channels per head, got {key_dim} and {value_dim}")
        self._mixer_lib("linear_attention")

    def check_delta_rule_sizes(self, num_heads, key_dim, value_dim) -> None:
        if not 0 < key_dim <= 256 or not 0 < value_dim <= 16384:
            raise UnsupportedSizeError(f"the delta rule scan keeps a column of the state in a thread's registers: "
                                       f"up to 256 key channels (and 16384 value channels) per head, got {key_dim} "
                                       f"and {value_dim}")
        self._mixer_lib("linear_attention")

    def _paged(self, k_cache, v_cache, num_kv_heads, page_size, key_dim, value_dim, dtype):
        pages = k_cache.shape[0]
        if (tuple(k_cache.shape) != (pages, num_kv_heads, page_size, key_dim)
                or tuple(v_cache.shape) != (pages, num_kv_heads, page_size, value_dim)
                or not k_cache.is_contiguous() or not v_cache.is_contiguous()):
            raise ValueError("windowed attention: cache tensors are pages [pages, kv heads, P, width]")
        if k_cache.dtype != dtype or v_cache.dtype != dtype:
            raise TypeError("windowed attention: queries and cache share one dtype")

    def project_norm_write(self, proj, num_heads, num_kv_heads, key_dim, value_dim, own_kv, q_norm, k_norm, eps,
                           q_out, k_cache, v_cache, page_size, positions, row_req, block_table) -> None:
        """From the float32 projections ``proj [rows, >= q (+ k + v)]``: the queries (divided by
        the root mean square over their whole width and multiplied by ``q_norm`` if that is
        given) into ``q_out``, and, if the layer has keys and values of its own, the keys
        (normed alike with ``k_norm``) and values into the rows' places in the pages."""
        lib = self._mixer_lib("windowed_attention")
        self._need(proj, "projections", torch.float32)
        self._need(q_out, "queries")
        rows = q_out.shape[0]
        q_size = num_heads * key_dim
        need = q_size + (num_kv_heads * (key_dim + value_dim) if own_kv else 0)
        if proj.shape[0] != rows or proj.shape[1] < need or tuple(q_out.shape) != (rows, q_size):
            raise ValueError(f"project_norm_write: projections {tuple(proj.shape)}, queries {tuple(q_out.shape)} "
                             f"do not fit {need} numbers a row")
        norm = q_norm is not None
        if norm:
            self._need(q_norm, "query norm weight", torch.float32)
            if q_norm.numel() != q_size:
                raise ValueError("project_norm_write: the query norm's weight spans all heads")
        if own_kv:
            self._paged(k_cache, v_cache, num_kv_heads, page_size, key_dim, value_dim, q_out.dtype)
            if norm:
                self._need(k_norm, "key norm weight", torch.float32)
                if k_norm.numel() != num_kv_heads * key_dim:
                    raise ValueError("project_norm_write: the key norm's weight spans all kv heads")
            for t, name in ((positions, "positions"), (row_req, "row -> request map"), (block_table, "block table")):
                self._need(t, name, torch.int32, contiguous=name != "block table")
            if positions.numel() < rows or row_req.numel() < rows or block_table.stride(1) != 1:
                raise ValueError("project_norm_write: one position and one request index per row")
        self._call(lib.llmlab_project_norm_write, self._ptr(proj), proj.stride(0), rows, num_heads, num_kv_heads,
                   key_dim, value_dim, 1 if own_kv else 0, 1 if norm else 0, float(eps), self._ptr(q_norm),
                   self._ptr(k_norm) if own_kv and norm else None, self._ptr(q_out),
                   self._ptr(k_cache) if own_kv else None, self._ptr(v_cache) if own_kv else None, _dt(q_out),
                   page_size, self._ptr(positions) if own_kv else None, self._ptr(row_req) if own_kv else None,
                   self._ptr(block_table) if own_kv else None, block_table.stride(0) if own_kv else 0,
                   self._stream(), lib=lib)

    def windowed_attention_long_rows(self, dtype, key_dim: int, value_dim: int, page_size: int) -> int:
        """From how many rows on a request's share of a step goes to the matrix-core kernel of the
        windowed attention (0: these sizes have none, every row goes to the plain kernel)."""
        lib = self._mixer_lib("windowed_attention")
        dt = DT_BF16 if dtype == torch.bfloat16 else DT_F32
        if not lib.llmlab_sink_window_attention_has_mfma(dt, int(key_dim), int(value_dim), int(page_size)):
            return 0
        return int(self.rules.windowed_attention_long_rows)

    def force_plain_windowed_attention(self, on: bool) -> None:
        """Tests and measurements: no matrix-core kernel for the windowed attention."""
        self._mixer_lib("windowed_attention").llmlab_debug_windowed_attention_plain(1 if on else 0)
        self.debug_epoch += 1

    def force_private_attention_tiles(self, on: bool) -> None:
        """Tests and measurements: prompts of heads that read the same keys and values go to the
        kernel whose waves fetch their own tiles, not to the one that stages them in LDS for a block."""
        self._mixer_lib("windowed_attention").llmlab_debug_windowed_attention_private_tiles(1 if on else 0)
        self.debug_epoch += 1

    def sink_window_attention(self, q, num_heads, num_kv_heads, key_dim, value_dim, k_cache, v_cache, block_table,
                              page_size, positions, row_req, window, keep_first, sink, scale, out,
                              q_start=None, long_from=0, launches=3, max_keys=0, weights: str = "softmax") -> None:
        """The query of row ``r`` at position ``i = positions[r]`` of request ``row_req[r]`` attends
        to the cached keys ``j <= i`` with ``i - j < window`` or ``j < keep_first`` (``window`` None:
        all); ``sink`` (float32 per head, or None) adds ``exp(sink)`` to the softmax's denominator.
        ``weights="sigmoid"``: no softmax; a visible key weighs ``sigmoid(score + sink[h])``
        (``sink``: then a bias per head on every score, None for none), not normalised over the keys.
        ``long_from > 0`` (``windowed_attention_long_rows``: sizes that the matrix cores take):
        requests that bring at least so many rows (by ``q_start``) are served in tiles of 16 rows
        of a head, the others a row and a group of heads at a time with the row's keys cut into
        shares; ``launches``: which of the two this step needs (bit 0 few rows, bit 1 many);
        ``max_keys``: the most keys a row of this step sees (sets the number of shares)."""
        lib = self._mixer_lib("windowed_attention")
        if long_from:
            self._need(q_start, "request row starts", torch.int32)
        self._need(q, "queries")
        self._need(out, "attention output")
        rows = q.shape[0]
        if tuple(q.shape) != (rows, num_heads * key_dim) or tuple(out.shape) != (rows, num_heads * value_dim):
            raise ValueError(f"windowed attention: queries {tuple(q.shape)}, output {tuple(out.shape)} do not fit "
                             f"{num_heads} heads of {key_dim} / {value_dim}")
        if q.dtype != out.dtype:
            raise TypeError("windowed attention: queries and output share one dtype")
        self._paged(k_cache, v_cache, num_kv_heads, page_size, key_dim, value_dim, q.dtype)
        for t, name in ((positions, "positions"), (row_req, "row -> request map")):
            self._need(t, name, torch.int32)
            if t.numel() < rows:
                raise ValueError(f"windowed attention: one entry of {name} per row")
        self._need(block_table, "block table", torch.int32, contiguous=False)
        if block_table.stride(1) != 1:
            raise ValueError("windowed attention: block table rows are contiguous")
        if sink is not None:
            self._need(sink, "sink", torch.float32)
            if sink.numel() != num_heads:
                raise ValueError("windowed attention: one sink per head")
        if value_dim > 1024:
            raise UnsupportedSizeError(f"windowed attention takes values up to 1024 wide, got {value_dim}")
        self._call(lib.llmlab_sink_window_attention, self._ptr(q), _dt(q), rows, num_heads, num_kv_heads, key_dim,
                   value_dim, self._ptr(k_cache), self._ptr(v_cache), self._ptr(block_table), block_table.stride(0),
                   page_size, self._ptr(positions), self._ptr(row_req), int(window) if window else 0,
                   int(keep_first or 0), self._ptr(sink), float(scale), self._ptr(out),
                   self._ptr(q_start) if long_from else None, int(long_from), int(launches), int(max_keys),
                   self._ptr(self.workspace), self.workspace.numel(), self.num_cus, self.ATTENTION_WEIGHTS[weights],
                   self._stream(), lib=lib)

    ATTENTION_WEIGHTS = {"softmax": 0, "sigmoid": 1}

    def project_rotate_write(self, proj, num_heads, num_kv_heads, key_dim, value_dim, bias, freq, rot_dims, magnitude,
                             mix, mix_weight, v_first, gate_out, q_out, k_cache, v_cache, page_size, positions,
                             row_req, block_table) -> None:
        """From the float32 projections ``proj [rows, q | k | v | gates]`` (``bias``, float32 in the same
        order, is added first): queries and keys with the first ``rot_dims`` channels of every head
        turned, channel ``2i`` together with ``2i + 1``, by ``positions[r] * freq[i]`` (sine and cosine
        times ``magnitude``); the queries go to ``q_out``, the keys and the values to the rows' places in
        the pages.  ``mix``: ``None`` the values as projected; ``"first"`` they are also left, unrounded,
        in ``v_first [rows, kv heads * value_dim]``; ``"mix"`` ``v <- (1 - mix_weight) v + mix_weight
        v_first`` before they are stored.  ``gate_out [rows, n]`` float32 (or None) receives the ``n``
        numbers behind the values."""
        lib = self._mixer_lib("windowed_attention")
        self._need(proj, "projections", torch.float32)
        self._need(q_out, "queries")
        rows = q_out.shape[0]
        q_size, k_size, v_size = num_heads * key_dim, num_kv_heads * key_dim, num_kv_heads * value_dim
        n_gate = 0 if gate_out is None else gate_out.shape[1]
        need = q_size + k_size + v_size + n_gate
        if proj.shape[0] != rows or proj.shape[1] < need or tuple(q_out.shape) != (rows, q_size):
            raise ValueError(f"project_rotate_write: projections {tuple(proj.shape)}, queries {tuple(q_out.shape)} "
                             f"do not fit {need} numbers a row")
        self._paged(k_cache, v_cache, num_kv_heads, page_size, key_dim, value_dim, q_out.dtype)
        if bias is not None:
            self._need(bias, "projection bias", torch.float32)
            if bias.numel() != need:
                raise ValueError(f"project_rotate_write: a bias of {bias.numel()} numbers for {need} projections")
        rot_dims = int(rot_dims or 0)
        if rot_dims:
            self._need(freq, "rotation frequencies", torch.float32)
            if rot_dims % 2 or rot_dims > key_dim or freq.numel() != rot_dims // 2:
                raise ValueError(f"project_rotate_write: {rot_dims} of {key_dim} channels with {freq.numel()} frequencies")
        code = {None: 0, "first": 1, "mix": 2}[mix]
        if code:
            self._need(v_first, "first values", torch.float32)
            if tuple(v_first.shape) != (rows, v_size):
                raise ValueError(f"project_rotate_write: first values {tuple(v_first.shape)}, not {(rows, v_size)}")
        if gate_out is not None:
            self._need(gate_out, "gates", torch.float32)
            if gate_out.shape[0] != rows:
                raise ValueError("project_rotate_write: one row of gates per row")
        for t, name in ((positions, "positions"), (row_req, "row -> request map"), (block_table, "block table")):
            self._need(t, name, torch.int32, contiguous=name != "block table")
        if positions.numel() < rows or row_req.numel() < rows or block_table.stride(1) != 1:
            raise ValueError("project_rotate_write: one position and one request index per row")
        self._call(lib.llmlab_project_rotate_write, self._ptr(proj), proj.stride(0), rows, num_heads, num_kv_heads,
                   key_dim, value_dim, self._ptr(bias), self._ptr(freq) if rot_dims else None, rot_dims,
                   float(magnitude), code, float(mix_weight or 0.0), self._ptr(v_first) if code else None, n_gate,
                   self._ptr(gate_out), self._ptr(q_out), self._ptr(k_cache), self._ptr(v_cache), _dt(q_out), page_size,
                   self._ptr(positions), self._ptr(row_req), self._ptr(block_table), block_table.stride(0),
                   self._stream(), lib=lib)

    def gla_slices(self, key_dim: int) -> int:
        """Into how many pieces the scan leaves each output (one per slice of key channels)."""
        return int(self._mixer_lib("linear_attention").llmlab_gla_slices(int(key_dim)))

    def gla_decay(self, low, rank, w2, bias, tau, decay) -> None:
        """``decay[r, c] = sigmoid(bias[c] + w2[c] . low[r, :rank]) ** (1 / tau)``, all float32."""
        lib = self._mixer_lib("linear_attention")
        for t, name in ((low, "low-rank projection"), (w2, "decay weight"), (decay, "decays")):
            self._need(t, name, torch.float32, contiguous=name != "low-rank projection")
        rows, channels = decay.shape
        if low.shape[0] != rows or low.shape[1] < rank or low.stride(1) != 1 or tuple(w2.shape) != (channels, rank):
            raise ValueError(f"gla_decay: low {tuple(low.shape)}, weight {tuple(w2.shape)}, decays "
                             f"{tuple(decay.shape)} do not fit rank {rank}")
        if bias is not None:
            self._need(bias, "decay bias", torch.float32)
            if bias.numel() != channels:
                raise ValueError("gla_decay: one bias per channel")
        self._call(lib.llmlab_gla_decay, self._ptr(low), low.stride(0), rows, int(rank), self._ptr(w2),
                   self._ptr(bias), float(tau), self._ptr(decay), channels, self._stream(), lib=lib)

    def gla_scan_chunk(self, rows: int, longest: int, num_heads: int, value_dim: int) -> int:
        """Into chunks of how many rows the scan cuts a step whose longest request brings
        ``longest`` rows (0: every request's rows in one run).  Chunks run side by side at the
        price of walking the rows twice, so short runs stay whole, and the chunks are as long
        as still gives every compute unit a few blocks."""
        if longest < 2 * self.rules.scan_min_chunk:
            return 0
        per_chunk = num_heads * ((value_dim + 63) // 64)
        chunk = self.rules.scan_max_chunk
        while chunk > self.rules.scan_min_chunk and (rows // chunk) * per_chunk < self.rules.scan_blocks_per_cu * self.num_cus:
            chunk //= 2
        return chunk

    def gla_scan(self, proj, off_q, off_k, off_v, decay, q_scale, num_heads, key_dim, value_dim, state, q_start,
                 req_rows, n_reqs, parts, chunk=0, chunk_state=None, chunk_decay=None) -> None:
        """The recurrence ``S = decay_t * S + k_t v_t^T; o_t = S^T (q_scale q_t)`` over the rows
        ``q_start[b] .. q_start[b + 1]`` of each of the step's ``n_reqs`` requests, on the float32
        state ``state[req_rows[b]]`` ``[heads, key_dim, value_dim]``, which is left updated;
        ``parts [rows, heads, gla_slices(key_dim), value_dim]`` receives each output in pieces.
        ``chunk > 0``: every request's rows in chunks of so many that run side by side, their
        states joined afterwards (``chunk_state [chunks, heads, key_dim, value_dim]`` and
        ``chunk_decay [chunks, heads, key_dim]`` float32 scratch, ``chunks >= rows // chunk +
        n_reqs``)."""
        lib = self._mixer_lib("linear_attention")
        for t, name in ((proj, "projections"), (decay, "decays"), (state, "recurrent state"), (parts, "output pieces")):
            self._need(t, name, torch.float32)
        self._need(q_start, "request row starts", torch.int32)
        self._need(req_rows, "state slots", torch.int32)
        rows = proj.shape[0]
        slices = self.gla_slices(key_dim)
        if (tuple(decay.shape) != (rows, num_heads * key_dim)
                or tuple(parts.shape) != (rows, num_heads, slices, value_dim)
                or tuple(state.shape[1:]) != (num_heads, key_dim, value_dim)
                or q_start.numel() < n_reqs + 1 or req_rows.numel() < n_reqs
                or min(off_q, off_k, off_v) < 0
                or max(off_q + num_heads * key_dim, off_k + num_heads * key_dim, off_v + num_heads * value_dim) > proj.shape[1]):
            raise ValueError("gla_scan: the operands do not fit each other")
        max_chunks = 0
        if chunk:
            self._need(chunk_state, "chunk states", torch.float32)
            self._need(chunk_decay, "chunk decays", torch.float32)
            max_chunks = chunk_state.shape[0]
            if (tuple(chunk_state.shape[1:]) != (num_heads, key_dim, value_dim)
                    or tuple(chunk_decay.shape) != (max_chunks, num_heads, key_dim)
                    or max_chunks < rows // chunk + n_reqs):
                raise ValueError(f"gla_scan: the scratch of the chunks does not fit {rows} rows of {n_reqs} requests "
                                 f"in chunks of {chunk}")
        self._call(lib.llmlab_gla_scan, self._ptr(proj), proj.stride(0), int(off_q), int(off_k), int(off_v),
                   self._ptr(decay), float(q_scale), num_heads, key_dim, value_dim, self._ptr(state),
                   self._ptr(q_start), self._ptr(req_rows), int(n_reqs), self._ptr(parts), rows, int(chunk),
                   self._ptr(chunk_state) if chunk else None, self._ptr(chunk_decay) if chunk else None, max_chunks,
                   self._stream(), lib=lib)

    OUTPUT_GATES = {"silu": 0, "sigmoid": 1}

    def gla_output(self, parts, num_heads, key_dim, value_dim, weight, eps, proj, off_gate, out, gate: str = "silu",
                   norm_count: int = 0) -> None:
        """``out[r, h] = rmsnorm(sum of parts[r, h]) * weight * silu(gate[r, h])`` with the gate at
        column ``off_gate`` of the float32 ``proj``; ``out`` in the compute dtype.  ``parts [rows, heads,
        pieces, value_dim]`` with any number of pieces; ``weight`` of ``value_dim`` numbers (the same for
        every head) or of ``heads * value_dim``; ``gate="sigmoid"``: ``... * sigmoid(gate[r, h])``; ``norm_count``:
        the mean of the squares is taken over so many channels of a head (the ones behind them are zeros)."""
        lib = self._mixer_lib("linear_attention")
        self._need(parts, "output pieces", torch.float32)
        self._need(proj, "projections", torch.float32)
        self._need(weight, "output norm weight", torch.float32)
        self._need(out, "mixer output")
        rows = parts.shape[0]
        if (parts.dim() != 4 or tuple(parts.shape) != (rows, num_heads, parts.shape[2], value_dim)
                or weight.numel() not in (value_dim, num_heads * value_dim)
                or tuple(out.shape) != (rows, num_heads * value_dim) or proj.shape[0] != rows
                or off_gate < 0 or off_gate + num_heads * value_dim > proj.shape[1] or gate not in self.OUTPUT_GATES):
            raise ValueError("gla_output: the operands do not fit each other")
        per_head = 1 if weight.numel() == num_heads * value_dim and num_heads > 1 else 0
        self._call(lib.llmlab_gla_output, self._ptr(parts), rows, num_heads, key_dim, value_dim, self._ptr(weight),
                   float(eps), self._ptr(proj), proj.stride(0), int(off_gate), self._ptr(out), _dt(out),
                   int(parts.shape[2]), per_head, self.OUTPUT_GATES[gate], int(norm_count or 0), self._stream(), lib=lib)

    def delta_gates(self, proj, off_low, rank, off_rate, off_k, w2, w0, rate_bias, decay_scale, key_eps, num_heads,
                    key_dim, decay, unit, removal) -> None:
        """What the delta rule's scan needs of every row, all float32 ``[rows, heads * key_dim]``:
        ``decay[r, c] = exp(-decay_scale * sigmoid(w0[c] + w2[c] . tanh(proj[r, off_low : off_low + rank])))``,
        the unit key ``unit = k / sqrt(|k|^2 + key_eps)`` head by head (``k`` at column ``off_k`` of
        ``proj``), and ``removal = sigmoid(proj[r, off_rate + c] + rate_bias[c]) * unit``."""
        lib = self._mixer_lib("linear_attention")
        for t, name in ((proj, "projections"), (w2, "decay weight"), (decay, "decays"), (unit, "unit keys"),
                        (removal, "removals")):
            self._need(t, name, torch.float32)
        rows, channels = decay.shape
        if (proj.shape[0] != rows or tuple(unit.shape) != (rows, channels) or tuple(removal.shape) != (rows, channels)
                or channels != num_heads * key_dim or tuple(w2.shape) != (channels, rank)
                or min(off_low, off_rate, off_k) < 0 or off_low + rank > proj.shape[1]
                or max(off_rate, off_k) + channels > proj.shape[1]):
            raise ValueError("delta_gates: the operands do not fit each other")
        for t, name in ((w0, "decay bias"), (rate_bias, "rate bias")):
            if t is not None:
                self._need(t, name, torch.float32)
                if t.numel() != channels:
                    raise ValueError(f"delta_gates: one {name} per channel")
        self._call(lib.llmlab_delta_gates, self._ptr(proj), proj.stride(0), rows, int(off_low), int(rank), int(off_rate),
                   int(off_k), self._ptr(w2), self._ptr(w0), self._ptr(rate_bias), float(decay_scale), float(key_eps),
                   self._ptr(decay), self._ptr(unit), self._ptr(removal), int(num_heads), int(key_dim), self._stream(),
                   lib=lib)

    DELTA_CHUNK_MAX_KEYS = 128      # wider states walk their rows in one run (a column no longer fits the registers)

    def delta_scan_chunk(self, rows: int, longest: int, num_heads: int, key_dim: int, value_dim: int) -> int:
        """Into chunks of how many rows the delta rule's scan cuts a step whose longest request brings
        ``longest`` rows (0: every request's rows in one run).  Chunks run side by side at the price of
        walking the rows twice, once more for the chunk's transition, and of joining the chunks one
        after the other; so short runs stay whole, and the chunks are as long as still gives every
        compute unit a block."""
        if longest < 2 * self.rules.scan_min_chunk or key_dim > self.DELTA_CHUNK_MAX_KEYS:
            return 0
        per_chunk = num_heads * ((value_dim + key_dim + 255) // 256)
        chunk = self.rules.delta_scan_max_chunk
        while chunk > self.rules.scan_min_chunk and (rows // chunk) * per_chunk < self.rules.scan_blocks_per_cu * self.num_cus:
            chunk //= 2
        return chunk

    def delta_scan(self, proj, off_r, off_k, off_v, decay, unit, removal, num_heads, key_dim, value_dim, state, q_start,
                   req_rows, n_reqs, out, chunk=0, chunk_state=None, chunk_trans=None) -> None:
        """The recurrence ``S = diag(decay_t) S - removal_t (unit_t^T S) + k_t v_t^T; o_t = S^T r_t`` over the
        rows ``q_start[b] .. q_start[b + 1]`` of each of the step's ``n_reqs`` requests, on the float32 state
        ``state[req_rows[b]]`` ``[heads, key_dim, value_dim]``, which is left updated; ``out [rows, heads, 1,
        value_dim]`` float32.  ``chunk > 0``: every request's rows in chunks of so many that run side by
        side, joined afterwards (``chunk_state [chunks, heads, key_dim, value_dim]`` and ``chunk_trans
        [chunks, heads, key_dim, key_dim]`` float32 scratch, ``chunks >= rows // chunk + n_reqs``)."""
        lib = self._mixer_lib("linear_attention")
        if key_dim > self.DELTA_CHUNK_MAX_KEYS:        # (the chunks' kernels take narrower states only)
            chunk = 0
        for t, name in ((proj, "projections"), (decay, "decays"), (unit, "unit keys"), (removal, "removals"),
                        (state, "recurrent state"), (out, "outputs")):
            self._need(t, name, torch.float32)
        self._need(q_start, "request row starts", torch.int32)
        self._need(req_rows, "state slots", torch.int32)
        rows = proj.shape[0]
        if (tuple(decay.shape) != (rows, num_heads * key_dim) or tuple(unit.shape) != tuple(decay.shape)
                or tuple(removal.shape) != tuple(decay.shape) or out.numel() != rows * num_heads * value_dim
                or tuple(state.shape[1:]) != (num_heads, key_dim, value_dim)
                or q_start.numel() < n_reqs + 1 or req_rows.numel() < n_reqs or min(off_r, off_k, off_v) < 0
                or max(off_r + num_heads * key_dim, off_k + num_heads * key_dim, off_v + num_heads * value_dim) > proj.shape[1]):
            raise ValueError("delta_scan: the operands do not fit each other")
        max_chunks = 0
        if chunk:
            self._need(chunk_state, "chunk states", torch.float32)
            self._need(chunk_trans, "chunk transitions", torch.float32)
            max_chunks = chunk_state.shape[0]
            if (tuple(chunk_state.shape[1:]) != (num_heads, key_dim, value_dim)
                    or tuple(chunk_trans.shape) != (max_chunks, num_heads, key_dim, key_dim)
                    or max_chunks < rows // chunk + n_reqs):
                raise ValueError(f"delta_scan: the scratch of the chunks does not fit {rows} rows of {n_reqs} requests "
                                 f"in chunks of {chunk}")
        self._call(lib.llmlab_delta_scan, self._ptr(proj), proj.stride(0), int(off_r), int(off_k), int(off_v),
                   self._ptr(decay), self._ptr(unit), self._ptr(removal), num_heads, key_dim, value_dim, self._ptr(state),
                   self._ptr(q_start), self._ptr(req_rows), int(n_reqs), self._ptr(out), rows, int(chunk),
                   self._ptr(chunk_state) if chunk else None, self._ptr(chunk_trans) if chunk else None, max_chunks,
                   self._stream(), lib=lib)

    # --------------------------------------------------------------- sampling
    # ------------------------------ the stream around sublayers; the latent form of attention
    def embed_pairs(self, table, pairs, ids, positions, row_req, q_start, req_rows, previous, scale: float,
                    buckets: int, mul_prev: int, mul_cur: int, norm_weight, eps: float, out) -> None:
        """``out[r] = norm(table[id_r] * scale + pairs[row_r])`` into the float32 stream.  ``row_r`` is
        ``buckets`` for a sequence's first token, else ``(previous id * mul_prev + id * mul_cur) mod
        buckets``; the id before a request's first row of the step comes from ``previous [slots, 1]``
        (int32), which then takes the request's last id of the step.  ``norm_weight``: the weight of an
        RMS norm over the sum (None: no norm).  ``buckets`` 0: no pairs."""
        lib = self._mixer_lib("stream_ops")
        self._need(table, "embedding table")
        self._need(out, "residual stream", torch.float32)
        self._need(ids, "token ids", torch.int32)
        rows, hidden = out.shape
        if table.dim() != 2 or table.shape[1] != hidden or ids.numel() < rows:
            raise ValueError(f"embed_pairs: table {tuple(table.shape)}, {ids.numel()} ids, stream {tuple(out.shape)}")
        if buckets:
            self._need(pairs, "pair table", table.dtype)
            self._need(previous, "previous-token slots", torch.int32)
            if tuple(pairs.shape) != (buckets + 1, hidden):
                raise ValueError(f"embed_pairs: a pair table of {buckets} buckets and one more row, got {tuple(pairs.shape)}")
            for t, name, least in ((positions, "positions", rows), (row_req, "row -> request map", rows),
                                   (q_start, "request row starts", 2), (req_rows, "request slots", 1)):
                self._need(t, name, torch.int32)
                if t.numel() < least:
                    raise ValueError(f"embed_pairs: {name} is too short")
        if norm_weight is not None:
            self._need(norm_weight, "norm weight")
            if norm_weight.numel() != hidden:
                raise ValueError("embed_pairs: the norm's weight spans the stream's width")
        self._call(lib.llmlab_embed_pairs, self._ptr(table), self._ptr(pairs) if buckets else None, _dt(table),
                   self._ptr(ids), self._ptr(positions) if buckets else None, self._ptr(row_req) if buckets else None,
                   self._ptr(q_start) if buckets else None, self._ptr(req_rows) if buckets else None,
                   self._ptr(previous) if buckets else None, float(scale), table.shape[0], int(buckets), int(mul_prev),
                   int(mul_cur), self._ptr(norm_weight), _dt(norm_weight) if norm_weight is not None else DT_F32,
                   float(eps), self._ptr(out), rows, hidden, self._stream(), lib=lib)

    def causal_conv(self, h, weight, state, positions, row_req, q_start, req_rows, out) -> None:
        """``out_t = h_t + sum_j weight[:, j] h_(t - taps + 1 + j)`` channel by channel over the positions
        of each request (``weight [width, taps]`` float32).  Inputs from before the step are read
        from ``state [slots, taps - 1, width]`` (the latest last; zeros before a sequence's start),
        which then takes each request's latest inputs.  ``h``, ``out``, ``state``: one kernel dtype."""
        lib = self._mixer_lib("stream_ops")
        self._need(h, "convolution input")
        self._need(out, "convolution output", h.dtype)
        self._need(weight, "convolution taps", torch.float32)
        rows, width = h.shape
        taps = weight.shape[1]
        if tuple(weight.shape) != (width, taps) or tuple(out.shape) != (rows, width):
            raise ValueError(f"causal_conv: input {tuple(h.shape)}, taps {tuple(weight.shape)}, output {tuple(out.shape)}")
        if state is not None:
            self._need(state, "convolution state", h.dtype)
            if tuple(state.shape[1:]) != (taps - 1, width):
                raise ValueError(f"causal_conv: state {tuple(state.shape)} does not hold {taps - 1} inputs of {width}")
        elif taps > 1:
            raise ValueError("causal_conv: more than one tap needs the slots of the requests")
        for t, name, least in ((row_req, "row -> request map", rows), (q_start, "request row starts", 2),
                               (req_rows, "request slots", 1)):
            self._need(t, name, torch.int32)
            if t.numel() < least:
                raise ValueError(f"causal_conv: {name} is too short")
        self._call(lib.llmlab_causal_conv, self._ptr(h), _dt(h), self._ptr(weight), taps, self._ptr(state),
                   self._ptr(row_req), self._ptr(q_start), self._ptr(req_rows), self._ptr(out), rows, width,
                   self._stream(), lib=lib)

    NORM_CONV_MAX_TAPS = 8

    def norm_conv(self, x, norm_weight, eps: float, weight, state, row_req, q_start, req_rows, h, out,
                  one_row_each: bool) -> None:
        """``h = rmsnorm(x) * norm_weight`` and ``out_t = h_t + sum_j weight[:, j] h_(t - taps + 1 + j)`` in
        one launch: the norm of the float32 stream's rows and ``causal_conv`` over them (up to
        ``NORM_CONV_MAX_TAPS`` taps).  ``one_row_each``: every request of the step brings exactly one
        row; then the slots are moved on in the same launch."""
        lib = self._mixer_lib("stream_ops")
        self._need(x, "residual stream", torch.float32)
        self._need(norm_weight, "norm weight")
        self._need(h, "normed rows")
        self._need(out, "convolution output", h.dtype)
        self._need(weight, "convolution taps", torch.float32)
        rows, width = x.shape
        taps = weight.shape[1]
        if tuple(weight.shape) != (width, taps) or tuple(out.shape) != (rows, width) or tuple(h.shape) != (rows, width) \
                or norm_weight.numel() != width:
            raise ValueError(f"norm_conv: stream {tuple(x.shape)}, norm weight {tuple(norm_weight.shape)}, taps "
                             f"{tuple(weight.shape)}, outputs {tuple(h.shape)} and {tuple(out.shape)}")
        if not 1 <= taps <= self.NORM_CONV_MAX_TAPS:
            raise ValueError(f"norm_conv: 1 to {self.NORM_CONV_MAX_TAPS} taps, got {taps}")
        if taps > 1:
            self._need(state, "convolution state", h.dtype)
            if tuple(state.shape[1:]) != (taps - 1, width):
                raise ValueError(f"norm_conv: state {tuple(state.shape)} does not hold {taps - 1} inputs of {width}")
        for t, name, least in ((row_req, "row -> request map", rows), (q_start, "request row starts", 2),
                               (req_rows, "request slots", 1)):
            self._need(t, name, torch.int32)
            if t.numel() < least:
                raise ValueError(f"norm_conv: {name} is too short")
        self._call(lib.llmlab_norm_conv, self._ptr(x), self._ptr(norm_weight), _dt(norm_weight), float(eps),
                   self._ptr(weight), taps, self._ptr(state) if taps > 1 else None, self._ptr(row_req), self._ptr(q_start),
                   self._ptr(req_rows), self._ptr(h), self._ptr(out), _dt(h), rows, width, 1 if one_row_each else 0,
                   self._stream(), lib=lib)

    GATED_ADD_MAX_PIECES = 8

    def gated_add(self, x, y, gate, bias) -> None:
        """``x += y * sigmoid(gate + bias)``, all float32: ``gate [rows, width]``, or ``[rows, 1]`` for
        one number a row; ``bias [width]`` or None; ``gate`` None: ``x += y``.  ``y``: a tensor
        ``[rows, width]``, or the ``PendingSums`` of a product left in up to ``GATED_ADD_MAX_PIECES``
        pieces, which are summed on the way."""
        lib = self._mixer_lib("stream_ops")
        self._need(x, "residual stream", torch.float32)
        rows, width = x.shape
        pieces, piece_stride = 1, 0
        if isinstance(y, PendingSums):
            p = y.parts
            if (p.dtype != torch.float32 or p.dim() != 3 or tuple(p.shape[1:]) != (rows, width) or not p[0].is_contiguous()
                    or not 1 <= y.splits <= min(p.shape[0], self.GATED_ADD_MAX_PIECES)):
                raise ValueError(f"gated_add: pieces {tuple(p.shape)} ({y.splits} used) onto {tuple(x.shape)}")
            pieces, piece_stride, y = y.splits, p.stride(0), p[0]
        self._need(y, "sublayer output", torch.float32)
        if tuple(y.shape) != (rows, width):
            raise ValueError(f"gated_add: {tuple(y.shape)} onto {tuple(x.shape)}")
        cols = 0
        if gate is not None:
            self._need(gate, "gate", torch.float32)
            cols = gate.shape[1]
            if gate.shape[0] != rows or cols not in (1, width):
                raise ValueError(f"gated_add: gates {tuple(gate.shape)} for {tuple(x.shape)}")
        if bias is not None:
            self._need(bias, "gate bias", torch.float32)
            if bias.numel() != width or gate is None:
                raise ValueError("gated_add: a bias per column of a gate")
        self._call(lib.llmlab_gated_add, self._ptr(x), self._ptr(y), pieces, piece_stride, self._ptr(gate), cols,
                   self._ptr(bias), rows, width, self._stream(), lib=lib)

    def rmsnorm_add(self, y, weight, eps: float, x, next_norm=None) -> None:
        """``x += y / sqrt(mean(y^2) + eps) * weight`` row by row, all float32: the norm of a sublayer's
        result on its way into the stream.  ``y [rows, width]``, or a product left in pieces
        (``PendingSums``), which are summed on the way.  ``next_norm = (weight, eps, out)``: the RMS norm
        that reads the stream next, in the same launch: ``out = norm(x)`` of the new rows (float32
        weight, ``out`` in a kernel dtype)."""
        lib = self._mixer_lib("stream_ops")
        self._need(x, "stream", torch.float32)
        self._need(weight, "norm weight", torch.float32)
        rows, width = x.shape
        if isinstance(y, PendingSums):
            parts, pieces = y.parts, y.splits
            if (parts.dtype != torch.float32 or parts.dim() != 3 or tuple(parts.shape[1:]) != (rows, width)
                    or not parts.is_contiguous() or pieces > parts.shape[0]):
                raise ValueError("rmsnorm_add: pieces are float32 [pieces, rows, width]")
            stride = parts.stride(0)
        else:
            self._need(y, "sublayer result", torch.float32)
            if tuple(y.shape) != (rows, width):
                raise ValueError(f"rmsnorm_add: result {tuple(y.shape)} onto a stream {tuple(x.shape)}")
            parts, pieces, stride = y, 1, 0
        if weight.numel() != width:
            raise ValueError("rmsnorm_add: one weight per column")
        next_w = next_out = None
        next_eps = 0.0
        if next_norm is not None:
            next_w, next_eps, next_out = next_norm
            self._need(next_w, "next norm's weight", torch.float32)
            self._need(next_out, "next norm's output")
            if next_w.numel() != width or tuple(next_out.shape) != (rows, width):
                raise ValueError("rmsnorm_add: the next norm's weight and output have the stream's shape")
        self._call(lib.llmlab_rmsnorm_add, self._ptr(x), self._ptr(parts), int(pieces), int(stride), self._ptr(weight),
                   float(eps), rows, width, self._ptr(next_w), float(next_eps), self._ptr(next_out),
                   _dt(next_out) if next_out is not None else 0, self._stream(), lib=lib)

    def scaled_sum(self, out, y1, a: float, y2, b: float) -> None:
        """``out = a * y1 + b * y2``, float32 tensors of one shape."""
        lib = self._mixer_lib("stream_ops")
        for t, name in ((out, "sum"), (y1, "first term"), (y2, "second term")):
            self._need(t, name, torch.float32)
        if tuple(out.shape) != tuple(y1.shape) or tuple(out.shape) != tuple(y2.shape):
            raise ValueError("scaled_sum: three tensors of one shape")
        self._call(lib.llmlab_scaled_sum, self._ptr(out), self._ptr(y1), float(a), self._ptr(y2), float(b), out.numel(),
                   self._stream(), lib=lib)

    def softcap(self, x, cap: float) -> None:
        """``x = cap * tanh(x / cap)`` in place, float32."""
        lib = self._mixer_lib("stream_ops")
        self._need(x, "logits", torch.float32)
        self._call(lib.llmlab_softcap, self._ptr(x), float(cap), x.numel(), self._stream(), lib=lib)

    def latent_norm_write(self, proj, q_rank: int, q_laid: int, kv_rank: int, latent: int, gates: int, q_norm, c_norm,
                          eps: float, cq_out, gate_out, k_cache, v_cache, page_size: int, positions, row_req,
                          block_table) -> None:
        """From the float32 projections ``proj [rows, q_laid + latent + gates]``: the query's latent (RMS
        norm over its first ``q_rank`` numbers, weight ``q_norm [q_laid]``) into ``cq_out [rows,
        q_laid]``; the cached latent (RMS norm over ``kv_rank`` numbers, weight ``c_norm [latent]``)
        into the row's place of both page tensors (``k``: row by row, ``v``: in quads of keys); the
        gates as they are into ``gate_out [rows, gates]``."""
        lib = self._mixer_lib("windowed_attention")
        self._need(proj, "projections", torch.float32)
        self._need(cq_out, "query latent")
        rows = cq_out.shape[0]
        if tuple(proj.shape) != (rows, q_laid + latent + gates) or tuple(cq_out.shape) != (rows, q_laid):
            raise ValueError(f"latent_norm_write: projections {tuple(proj.shape)}, query latent {tuple(cq_out.shape)}")
        self._need(q_norm, "query latent norm weight", torch.float32)
        self._need(c_norm, "cached latent norm weight", torch.float32)
        if q_norm.numel() != q_laid or c_norm.numel() != latent or not 0 < q_rank <= q_laid or not 0 < kv_rank <= latent:
            raise ValueError("latent_norm_write: the norms' weights span the laid-out latents")
        if gates:
            self._need(gate_out, "head gates", torch.float32)
            if tuple(gate_out.shape) != (rows, gates):
                raise ValueError("latent_norm_write: one gate per row and head")
        self._paged(k_cache, v_cache, 1, page_size, latent, latent, cq_out.dtype)
        for t, name in ((positions, "positions"), (row_req, "row -> request map"), (block_table, "block table")):
            self._need(t, name, torch.int32, contiguous=name != "block table")
        if positions.numel() < rows or row_req.numel() < rows or block_table.stride(1) != 1:
            raise ValueError("latent_norm_write: one position and one request index per row")
        self._call(lib.llmlab_latent_norm_write, self._ptr(proj), proj.stride(0), rows, int(q_rank), int(q_laid),
                   int(kv_rank), int(latent), int(gates), float(eps), self._ptr(q_norm), self._ptr(c_norm),
                   self._ptr(cq_out), self._ptr(gate_out) if gates else None, self._ptr(k_cache), self._ptr(v_cache),
                   _dt(cq_out), page_size, self._ptr(positions), self._ptr(row_req), self._ptr(block_table),
                   block_table.stride(0), self._stream(), lib=lib)

    def head_products(self, x, w, out, gate=None) -> None:
        """``out[r, a, :] = w[a] x[r, a, :]`` for a stack of matrices ``w [heads, n, k]``: ``x [rows, heads *
        k]``, ``out [rows, heads * n]``, all of one kernel dtype; sums in float32.  ``gate [rows, heads]``
        float32: head ``a`` of row ``r`` times ``sigmoid(gate[r, a])``, in float32 before the rounding."""
        lib = self._mixer_lib("windowed_attention")
        self._need(x, "head inputs")
        self._need(w, "head matrices", x.dtype)
        self._need(out, "head outputs", x.dtype)
        heads, n, k = w.shape
        rows = x.shape[0]
        if tuple(x.shape) != (rows, heads * k) or tuple(out.shape) != (rows, heads * n):
            raise ValueError(f"head_products: x {tuple(x.shape)}, matrices {tuple(w.shape)}, out {tuple(out.shape)}")
        if gate is not None:
            self._need(gate, "head gates", torch.float32)
            if tuple(gate.shape) != (rows, heads):
                raise ValueError(f"head_products: gates {tuple(gate.shape)} for {rows} rows of {heads} heads")
        self._call(lib.llmlab_head_products, self._ptr(x), self._ptr(w), self._ptr(out), _dt(x), rows, heads, n, k,
                   self._ptr(gate), self._stream(), lib=lib)

    def argmax(self, logits, out, one_pass: bool = True) -> None:
        """``out[r]`` = the largest logit's index (the smallest among equals; -1 for a row
        without a finite value).  ``one_pass=False``: in two kernels, without the counters."""
        self._need(logits, "logits", torch.float32, contiguous=False)
        self._need(out, "chosen tokens", torch.int32)
        rows, vocab = logits.shape
        if logits.stride(1) != 1 or out.numel() < rows:
            raise ValueError("argmax: logits rows must be contiguous and out must hold one token per row")
        self._call(self._core.llmlab_argmax,
            self._ptr(logits), logits.stride(0) if rows > 1 else vocab, rows, vocab, self._ptr(out),
            self._ptr(self.workspace), self.workspace.numel(),
            self._ptr(self.arrived) if one_pass else None, self.arrived.numel(), self._stream())

    def sample(self, logits, temperatures, uniforms, out) -> None:
        self._need(logits, "logits", torch.float32, contiguous=False)
        self._need(out, "chosen tokens", torch.int32)
        rows, vocab = logits.shape
        if logits.stride(1) != 1 or out.numel() < rows:
            raise ValueError("sample: logits rows must be contiguous and out must hold one token per row")
        if temperatures is not None:
            self._need(temperatures, "temperatures", torch.float32)
            self._need(uniforms, "uniform numbers", torch.float32)
            if temperatures.numel() < rows or uniforms.numel() < rows:
                raise ValueError("sample: one temperature and one uniform number per row")
        self._call(self._core.llmlab_sample,
            self._ptr(logits), logits.stride(0) if rows > 1 else vocab, rows, vocab,
            self._ptr(temperatures), self._ptr(uniforms), self._ptr(out), self._stream())
