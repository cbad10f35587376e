"""Bindings of the hand-written HIP kernels (loaded through ctypes).

There is no fallback: without a GPU and the built library `get_ops()` raises.
Every wrapper checks on the host that its operands have the shapes, dtypes and
layout its kernel and grid assume, and launches on torch's current stream.
"""
from __future__ import annotations

import contextlib
import ctypes
import math
import threading

import torch

from . import build as _build

_F32, _BF16 = 0, 1
_CODES = {torch.float32: _F32, torch.bfloat16: _BF16}


class KernelError(RuntimeError):
    pass


def _code(dtype: torch.dtype) -> int:
    try:
        return _CODES[dtype]
    except KeyError:
        raise KernelError(f"kernels take float32 or bfloat16, not {dtype}") from None


def _raw_stream(device_index: int) -> int:
    return torch._C._cuda_getCurrentRawStream(device_index)


class _Recording(threading.local):
    """What the thread that records a layer's calls is recording into (nothing, for every other thread)."""
    library = None        # the `_RecordingLibrary` that stands in for the loaded one
    keep: list | None = None      # every tensor whose address went into a recorded call


_RECORDING = _Recording()


def _ptr(tensor: torch.Tensor | None) -> ctypes.c_void_p:
    if tensor is None:
        return ctypes.c_void_p(0)
    keep = _RECORDING.keep
    if keep is not None:
        keep.append(tensor)
    return ctypes.c_void_p(tensor.data_ptr())


def _need(cond: bool, message: str) -> None:
    if not cond:
        raise KernelError(message)


def _dev(*tensors: torch.Tensor | None) -> None:
    for tensor in tensors:
        if tensor is not None:
            _need(tensor.is_cuda, "kernel operands must live on the GPU")
            _need(tensor.is_contiguous(), "kernel operands must be contiguous")


def _parts_of_k(k: int, splits: int, step: int) -> int:
    """Into how many parts K really falls when `splits` are asked for and a part is a multiple of `step`."""
    if splits <= 1:
        return 1
    chunk = -(-(-(-k // splits)) // step) * step
    return -(-k // chunk)


class PendingSum:
    """A product whose K was cut over workgroups, before its parts are added: float32 slabs [parts, M, N] and
    the bias that joins their sum.  `Ops.add_rmsnorm` takes it as the delta and adds the parts, the bias and the
    residual and normalises in one kernel; `resolve()` adds the parts on their own and gives the product."""

    def __init__(self, ops: "Ops", partial: torch.Tensor, bias: torch.Tensor | None, dtype: torch.dtype):
        self.ops, self.partial, self.bias, self.dtype = ops, partial, bias, dtype
        self.shape = tuple(partial.shape[1:])

    def resolve(self) -> torch.Tensor:
        parts, m, n = self.partial.shape
        out = torch.empty((m, n), dtype=self.dtype, device=self.partial.device)
        self.ops._check(self.ops.lib.ta_splitk_reduce(_ptr(self.partial), _ptr(self.bias), _ptr(out), m, n, n, parts,
                                                      _code(self.dtype), self.ops._stream()), "splitk_reduce")
        return out


class LaunchTape:
    """The library calls that one layer made, in order, each with its arguments and the status it returned.

    Layers of the same make (the same parts with the same sizes and constants) make the same calls on a step's
    batch; only the addresses of their own tensors differ.  `replay(put)` makes the calls again with every
    address found in `put` replaced: the Python between the calls (checks, choices of kernel and split, buffers)
    ran once, for the recorded layer.  The tape keeps every tensor whose address it holds, so the recorded
    layer's buffers are there for the layers that use them again (all on one stream, one after another).
    """

    def __init__(self):
        self.calls: list[tuple] = []          # (function, arguments, status, ((index, address), ...))
        self.keep: list[torch.Tensor] = []

    def replay(self, put: dict[int, int]) -> None:
        for function, args, status, addresses in self.calls:
            changed = None
            for index, address in addresses:
                to = put.get(address)
                if to is not None:
                    if changed is None:
                        changed = list(args)
                    changed[index] = ctypes.c_void_p(to)
            got = function(*args) if changed is None else function(*changed)
            if got != status:
                raise KernelError(f"a recorded call returned {got} where it had returned {status}")

    def addresses(self) -> set:
        """Every address that went into a recorded call."""
        return {address for _, _, _, addresses in self.calls for _, address in addresses}


class _RecordingLibrary:
    """Stands in for the loaded library while a tape is recorded: every call goes through and onto the tape."""

    def __init__(self, lib, tape: LaunchTape):
        self._lib, self._tape = lib, tape

    def __getattr__(self, name):
        function = getattr(self._lib, name)
        calls = self._tape.calls

        def call(*args):
            status = function(*args)
            calls.append((function, args, status,
                          tuple((i, a.value) for i, a in enumerate(args) if isinstance(a, ctypes.c_void_p) and a.value)))
            return status
        return call


class Ops:
    """The kernel library.  One instance per process; see `get_ops()`."""

    def __init__(self, path: str):
        self.path = path
        self._loaded = ctypes.CDLL(path)
        for name in ("ta_embedding", "ta_add_rmsnorm", "ta_silu_gate", "ta_rope_store",
                     "ta_paged_attention_generic", "ta_decode_attention_bf16", "ta_prefill_attention_bf16",
                     "ta_prefill_attention_shared_plan", "ta_prefill_attention_key_splits",
                     "ta_gemm_f32", "ta_gemm_bf16", "ta_gemm_bf16_splitk", "ta_gemm_skinny_bf16",
                     "ta_gemm_skinny_bf16_splitk", "ta_gemm_skinny_qkv_rope", "ta_fused_norm_qkv_rope",
                     "ta_fused_norm_gated", "ta_fused_linear_residual", "ta_fused_qkv_rope", "ta_fused_gated",
                     "ta_splitk_reduce", "ta_splitk_add_rmsnorm", "ta_argmax", "ta_argmax_next_step", "ta_sample",
                     "ta_sample_workspace_words", "ta_library_gemm_bf16", "ta_compute_units", "ta_read_stream",
                     "ta_embedding_streams", "ta_streams_step", "ta_token_shift", "ta_mlstm_scan", "ta_mlstm_chunked", "ta_head_norm_gate",
                     "ta_capped_gate", "ta_norm_add_rmsnorm", "ta_norm_rotate_store", "ta_differential_heads",
                     "ta_sigmoid_head_gate", "ta_route_top", "ta_expert_gate", "ta_side_gate", "ta_gelu_gate", "ta_norm_side_norm", "ta_route_rows", "ta_expert_slots", "ta_grouped_gemm_bf16", "ta_expert_combine",
                     "ta_add_pair_rmsnorm", "ta_latent_store", "ta_rotate_tails", "ta_head_linear", "ta_short_conv_silu",
                     "ta_delta_scan", "ta_route_sigmoid", "ta_route_rows_sigmoid", "ta_expert_act", "ta_relu2",
                     "ta_add_terms_rmsnorm", "ta_scale_cap", "ta_route_scores", "ta_selective_scan", "ta_route_rows_scores"):
            getattr(self.lib, name).restype = ctypes.c_int
        self.lib.ta_grouped_gemm_bf16.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int,
                                                  ctypes.c_int, ctypes.c_void_p, ctypes.c_long, ctypes.c_int, ctypes.c_void_p,
                                                  ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
        self.lib.ta_library_gemm_bf16.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 5 + [
            ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p]
        self._workspaces: dict[int, torch.Tensor] = {}
        self._filled: dict[int, tuple] = {}        # weights whose K was filled up to a multiple of eight, by address
        self.compute_units = int(self._loaded.ta_compute_units())     # what the splits below aim to fill

    @staticmethod
    def _stream() -> ctypes.c_void_p:
        """The current HIP stream of the current device (the raw handle, which costs far less to ask for
        than a stream object; every launch asks)."""
        return ctypes.c_void_p(_raw_stream(torch.cuda.current_device()))

    LIBRARY_WORKSPACE = 128 << 20      # bytes the vendor's matrix library may use per device (its first choice for
    #                                    the widest products of a 7B model wants some 60 MB)

    def _workspace(self, device: torch.device) -> torch.Tensor:
        index = device.index if device.index is not None else torch.cuda.current_device()
        space = self._workspaces.get(index)
        if space is None:
            space = self._workspaces[index] = torch.empty(self.LIBRARY_WORKSPACE, dtype=torch.uint8, device=device)
        return space

    @staticmethod
    def _check(status: int, what: str) -> None:
        if status != 0:
            raise KernelError(f"{what} failed with status {status}"
                              + (" (sizes the kernel does not take)" if status < 0 else " (HIP error)"))

    @property
    def lib(self):
        """The loaded library, or, on a thread that is recording a layer's calls, the recorder in front of it."""
        return _RECORDING.library or self._loaded

    @contextlib.contextmanager
    def record_launches(self):
        """Record every library call this thread makes inside the block on a `LaunchTape` (which the block
        receives).  Other threads' calls are not touched; a recording inside a recording takes over until it ends."""
        tape = LaunchTape()
        before = _RECORDING.library, _RECORDING.keep
        _RECORDING.library, _RECORDING.keep = _RecordingLibrary(self._loaded, tape), tape.keep
        try:
            yield tape
        finally:
            _RECORDING.library, _RECORDING.keep = before

    # ------------------------------------------------------------------ yardstick
    def read_stream(self, data: torch.Tensor, workgroups: int | None = None) -> torch.Tensor:
        """Read every byte of `data` once in the access pattern of the weight-streaming kernels; returns the xor
        of its 32-bit words per workgroup (uint32 as int32 [workgroups]).  A yardstick for what a kernel bound by
        HBM reaches on this device; no model code calls it."""
        _dev(data)
        nbytes = data.numel() * data.element_size()
        _need(nbytes % 16 == 0 and data.data_ptr() % 16 == 0, "the buffer must be whole 16-byte words")
        workgroups = workgroups or 8 * self.compute_units
        out = torch.empty(workgroups, dtype=torch.int32, device=data.device)
        self._check(self.lib.ta_read_stream(_ptr(data), ctypes.c_size_t(nbytes), _ptr(out), workgroups, self._stream()),
                    "read_stream")
        return out

    # ------------------------------------------------------------------ embedding
    def embedding(self, ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor, scale: float = 1.0) -> torch.Tensor:
        """out[t] = table[ids[t]] * scale as float32.  ids int32 [T]; table [V, H]; out float32 [T, H]."""
        _dev(ids, table, out)
        n, (vocab, hidden) = ids.numel(), table.shape
        _need(ids.dtype == torch.int32 and ids.dim() == 1, "ids must be int32 [T]")
        _need(out.dtype == torch.float32 and tuple(out.shape) == (n, hidden), "out must be float32 [T, H]")
        self._check(self.lib.ta_embedding(_ptr(ids), _ptr(table), _ptr(out), n, hidden, vocab,
                                          _code(table.dtype), ctypes.c_float(scale), self._stream()), "embedding")
        return out

    # ---------------------------------------------------------------------- norm
    def add_rmsnorm(self, residual: torch.Tensor, delta: torch.Tensor | None, weight: torch.Tensor,
                    eps: float, out: torch.Tensor, rows: torch.Tensor | None = None,
                    store_residual: bool = True) -> torch.Tensor:
        """x = residual[r] (+ delta[r]); optionally residual[r] = x; out[i] = rmsnorm(x) * weight.

        residual float32 [T, H]; delta [T, H] in out's dtype, None, or a `PendingSum` (the parts of a product
        still to be added: they are added here, in the same kernel); weight float32 [H];
        rows int32 [R] picks the rows (None: all, R = T); out [R, H].
        """
        if isinstance(delta, PendingSum):
            n_tokens, hidden = residual.shape
            if (rows is not None or not store_residual or hidden % 4 or hidden > 4096
                    or delta.shape != (n_tokens, hidden)):
                delta = delta.resolve()
            else:
                _dev(residual, weight, out)
                _need(residual.dtype == torch.float32, "the residual stream is float32")
                _need(weight.dtype == torch.float32 and weight.numel() == hidden, "norm weight must be float32 [H]")
                _need(tuple(out.shape) == (n_tokens, hidden) and out.dtype == delta.dtype, "norm output has the wrong shape")
                self._check(self.lib.ta_splitk_add_rmsnorm(
                    _ptr(residual), _ptr(delta.partial), delta.partial.shape[0], _ptr(delta.bias), _ptr(weight),
                    _ptr(out), n_tokens, hidden, ctypes.c_float(eps), _code(out.dtype), self._stream()),
                    "splitk_add_rmsnorm")
                return out
        _dev(residual, delta, weight, out, rows)
        n_tokens, hidden = residual.shape
        n_rows = n_tokens if rows is None else rows.numel()
        _need(residual.dtype == torch.float32, "the residual stream is float32")
        _need(weight.dtype == torch.float32 and weight.numel() == hidden, "norm weight must be float32 [H]")
        _need(tuple(out.shape) == (n_rows, hidden), "norm output has the wrong shape")
        if delta is not None:
            _need(delta.shape == residual.shape and delta.dtype == out.dtype, "delta must match residual and out")
        if rows is not None:
            _need(rows.dtype == torch.int32, "rows must be int32")
            _need(not store_residual, "a row subset never stores the residual")
        self._check(self.lib.ta_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(weight), _ptr(out), _ptr(rows),
                                            n_rows, hidden, ctypes.c_float(eps), int(store_residual),
                                            _code(out.dtype), self._stream()), "add_rmsnorm")
        return out

    def add_pair_rmsnorm(self, residual: torch.Tensor, first: torch.Tensor, second: torch.Tensor,
                         weight: torch.Tensor | None, eps: float, out: torch.Tensor, rows: torch.Tensor | None = None,
                         store_residual: bool = True) -> torch.Tensor:
        """x = residual[r] + (first[r] + second[r]) in float32; optionally residual[r] = x; out[i] = rmsnorm(x) * weight
        (weight None: out[i] = x).  residual float32 [T, H]; first, second [T, H] in out's dtype; weight float32 [H];
        rows int32 [R] picks the rows (None: all); out [R, H]."""
        _dev(residual, first, second, weight, out, rows)
        n_tokens, hidden = residual.shape
        n_rows = n_tokens if rows is None else rows.numel()
        _need(residual.dtype == torch.float32, "the residual stream is float32")
        _need(weight is None or (weight.dtype == torch.float32 and weight.numel() == hidden), "norm weight must be float32 [H]")
        _need(tuple(first.shape) == (n_tokens, hidden) == tuple(second.shape) and first.dtype == out.dtype == second.dtype,
              "the two terms are [T, H] in the output's dtype")
        _need(tuple(out.shape) == (n_rows, hidden), "norm output has the wrong shape")
        _need(rows is None or (rows.dtype == torch.int32 and not store_residual), "rows int32, and a subset stores nothing back")
        _need(hidden <= 8192, "rows of up to 8192 elements")
        self._check(self.lib.ta_add_pair_rmsnorm(_ptr(residual), _ptr(first), _ptr(second), _ptr(weight), _ptr(out), _ptr(rows),
                                                 n_rows, hidden, ctypes.c_float(eps), int(bool(store_residual)),
                                                 _code(out.dtype), self._stream()), "add_pair_rmsnorm")
        return out

    # ---------------------------------------------------- attention over a cached latent
    def latent_store(self, rows: torch.Tensor, q_offset: int, q_rank: int, q_norm: torch.Tensor, kv_offset: int, kv_rank: int,
                     kv_norm: torch.Tensor, rot_dim: int, rates: torch.Tensor | None, eps: float, positions: torch.Tensor,
                     slots: torch.Tensor | None, k_pages: torch.Tensor | None, v_pages: torch.Tensor | None,
                     latent_q: torch.Tensor) -> None:
        """latent_q[t] = rmsnorm(rows[t, q_offset : + q_rank]) * q_norm; the kept row of a token, [rmsnorm(rows[t,
        kv_offset : + kv_rank]) * kv_norm | the rot_dim coordinates behind them, coordinate i with i + rot_dim / 2 turned by
        positions[t] * rates[i]], goes into key pages [n_pages, 1, page_size, kv_rank + rot_dim] at slots[t] and,
        transposed within a page, into value pages [n_pages, 1, kv_rank + rot_dim, page_size] (slots None: nothing is
        stored).  Norms and angles are float32."""
        _dev(rows, q_norm, kv_norm, rates, positions, slots, k_pages, v_pages, latent_q)
        n_tokens = rows.shape[0]
        _need(rows.dim() == 2 and q_offset >= 0 and kv_offset >= 0 and q_offset + q_rank <= rows.shape[1]
              and kv_offset + kv_rank + rot_dim <= rows.shape[1] and q_rank > 0 and kv_rank > 0, "the latents do not fit the rows")
        _need(q_norm.dtype == torch.float32 and q_norm.numel() == q_rank and kv_norm.dtype == torch.float32
              and kv_norm.numel() == kv_rank, "the latents' norm weights are float32")
        _need(rot_dim >= 0 and rot_dim % 2 == 0 and (rot_dim == 0 or (rates is not None and rates.dtype == torch.float32
                                                                       and rates.numel() == rot_dim // 2)),
              "a rotation has an even number of coordinates and a float32 rate for each pair")
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        _need(tuple(latent_q.shape) == (n_tokens, q_rank) and latent_q.dtype == rows.dtype, "latent_q is [T, q_rank]")
        page_size = 0
        if slots is not None:
            _need(slots.dtype == torch.int32 and slots.numel() == n_tokens, "slots must be int32 [T]")
            _need(k_pages is not None and v_pages is not None and k_pages.dtype == rows.dtype == v_pages.dtype,
                  "pages must have the rows' dtype")
            page_size = self._page_size(k_pages, v_pages, 1, kv_rank + rot_dim)
        self._check(self.lib.ta_latent_store(_ptr(rows), rows.shape[1], q_offset, q_rank, _ptr(q_norm), kv_offset, kv_rank,
                                             _ptr(kv_norm), rot_dim, _ptr(rates), ctypes.c_float(eps), _ptr(positions),
                                             _ptr(slots), _ptr(k_pages if slots is not None else None),
                                             _ptr(v_pages if slots is not None else None), page_size, _ptr(latent_q),
                                             n_tokens, _code(rows.dtype), self._stream()), "latent_store")

    def head_linear(self, x: torch.Tensor, x_offset: int, x_head_stride: int, weight: torch.Tensor, out: torch.Tensor,
                    out_offset: int, out_head_stride: int) -> torch.Tensor:
        """Products head by head: out[t, h out_head_stride + out_offset + n] = sum_k x[t, h x_head_stride + x_offset + k]
        weight[h, n, k]; weight [heads, N, K]; float32 sums.  Other columns of `out` are left as they are."""
        _dev(x, weight, out)
        _need(weight.dim() == 3 and x.dim() == 2 and out.dim() == 2 and x.dtype == weight.dtype == out.dtype,
              "x [T, .], weight [heads, N, K], out [T, .] of one dtype")
        heads, n, k = weight.shape
        m = x.shape[0]
        _need(out.shape[0] == m and x_offset >= 0 and out_offset >= 0 and heads > 0
              and (heads - 1) * x_head_stride + x_offset + k <= x.shape[1]
              and (heads - 1) * out_head_stride + out_offset + n <= out.shape[1], "the heads do not fit the rows")
        self._check(self.lib.ta_head_linear(_ptr(x), x.shape[1], x_head_stride, x_offset, _ptr(weight), _ptr(out), out.shape[1],
                                            out_head_stride, out_offset, m, n, k, heads, _code(x.dtype), self._stream()),
                    "head_linear")
        return out

    def rotate_tails(self, q: torch.Tensor, heads: int, head_width: int, tail_offset: int, dims: int, rates: torch.Tensor,
                     positions: torch.Tensor, out: torch.Tensor, out_head_stride: int, out_offset: int) -> torch.Tensor:
        """out[t, h out_head_stride + out_offset + i], i < dims: coordinates tail_offset.. of head h of q [T, heads
        head_width], coordinate i with i + dims / 2 turned by positions[t] * rates[i] (float32 angles)."""
        _dev(q, rates, positions, out)
        n_tokens = q.shape[0]
        _need(q.shape[1] >= heads * head_width and tail_offset >= 0 and tail_offset + dims <= head_width and dims % 2 == 0,
              "the tails do not fit the heads")
        _need(rates.dtype == torch.float32 and rates.numel() == dims // 2, "a float32 rate for each pair")
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        _need(out.shape[0] == n_tokens and out.dtype == q.dtype and out_offset >= 0
              and (heads - 1) * out_head_stride + out_offset + dims <= out.shape[1], "the tails do not fit the output")
        self._check(self.lib.ta_rotate_tails(_ptr(q), q.shape[1], heads, head_width, tail_offset, dims, _ptr(rates),
                                             _ptr(positions), _ptr(out), out.shape[1], out_head_stride, out_offset, n_tokens,
                                             _code(q.dtype), self._stream()), "rotate_tails")
        return out

    # ---------------------------------------------------- delta rule with a decay per key channel
    def short_conv_silu(self, rows: torch.Tensor, offsets, widths, taps: torch.Tensor, state: torch.Tensor, state_offset: int,
                        cu_q: torch.Tensor, first_position: torch.Tensor, state_slots: torch.Tensor,
                        entry_of_token: torch.Tensor, out: torch.Tensor, bias: torch.Tensor | None = None) -> torch.Tensor:
        """A short causal convolution over time, channel by channel, (+ bias, float32 [channels],) then silu.  The channels are up to three runs of
        columns of `rows` (run i: widths[i] columns from offsets[i] on), side by side in `out` [T, channels]; taps float32
        [channels, n_taps], the last column the current token's.  Inputs before an entry's first row are its state row's
        [state_offset : + (n_taps - 1) channels] (oldest first; zeros if its first position is 0), which then takes the
        entry's last n_taps - 1 inputs."""
        _dev(rows, taps, state, cu_q, first_position, state_slots, entry_of_token, out, bias)
        offsets, widths = [int(o) for o in offsets], [int(w) for w in widths]
        _need(len(offsets) == len(widths) and 1 <= len(widths) <= 3, "one to three runs of channels")
        while len(widths) < 3:
            offsets.append(0)
            widths.append(0)
        channels, n_tokens = sum(widths), rows.shape[0]
        _need(all(w >= 0 and o >= 0 and o + w <= rows.shape[1] for o, w in zip(offsets, widths)), "the runs do not fit the rows")
        _need(taps.dtype == torch.float32 and taps.dim() == 2 and taps.shape[0] == channels and 1 <= taps.shape[1] <= 16,
              "taps float32 [channels, up to 16]")
        n_taps = taps.shape[1]
        _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= state_offset + (n_taps - 1) * channels,
              "state rows are too short")
        _need(tuple(out.shape) == (n_tokens, channels) and out.dtype == rows.dtype and entry_of_token.numel() == n_tokens,
              "out is [T, channels]")
        n_entries = cu_q.numel() - 1
        _need(first_position.numel() == n_entries == state_slots.numel(), "one first position and slot per entry")
        _need(bias is None or (bias.dtype == torch.float32 and bias.numel() == channels and bias.is_contiguous()),
              "the bias is float32 [channels]")
        self._check(self.lib.ta_short_conv_silu(_ptr(rows), rows.shape[1], offsets[0], widths[0], offsets[1], widths[1],
                                                offsets[2], widths[2], _ptr(taps), n_taps, _ptr(state),
                                                ctypes.c_long(state.shape[1]), state_offset, _ptr(cu_q), _ptr(first_position),
                                                _ptr(state_slots), _ptr(entry_of_token), _ptr(out), n_tokens, n_entries,
                                                _code(rows.dtype), _ptr(bias), self._stream()), "short_conv_silu")
        return out

    def selective_scan(self, x: torch.Tensor, pre: torch.Tensor, neg_rate: torch.Tensor, low: torch.Tensor, b_offset: int,
                       c_offset: int, skip: torch.Tensor, rows: torch.Tensor, z_offset: int, state: torch.Tensor,
                       cu_q: torch.Tensor, first_position: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor,
                       channels: int, n: int) -> torch.Tensor:
        """The selective scan over every entry's rows, from and into the entries' state rows (their first channels * n
        numbers; zeros if the entry's first position is 0).  Per channel c and state j, with d = softplus(pre[t, c]):
        S[c, j] <- exp(d neg_rate[c, j]) S[c, j] + d x[t, c] B[t, j]; y = sum_j S[c, j] C[t, j] + skip[c] x[t, c];
        out[t, c] = y * silu(z[t, c]).  x [T, channels]; pre float32 [T, channels]; neg_rate float32 [channels, n]; B and C
        are the columns b_offset.. and c_offset.. of `low`; z the columns z_offset.. of `rows`; out [T, channels]."""
        _dev(x, pre, neg_rate, low, skip, rows, state, cu_q, first_position, state_slots, out)
        n_tokens = x.shape[0]
        _need(x.dim() == 2 and x.shape[1] >= channels and x.stride(1) == 1, "x is [T, >= channels]")
        _need(pre.dtype == torch.float32 and tuple(pre.shape) == (n_tokens, channels) and pre.is_contiguous(),
              "the step sizes' pre-activations are float32 [T, channels]")
        _need(neg_rate.dtype == torch.float32 and tuple(neg_rate.shape) == (channels, n) and neg_rate.is_contiguous(),
              "the rates are float32 [channels, n]")
        _need(skip.dtype == torch.float32 and skip.numel() == channels, "the skip weights are float32 [channels]")
        _need(low.dtype == x.dtype and low.shape[0] == n_tokens and low.stride(1) == 1
              and 0 <= b_offset and b_offset + n <= low.shape[1] and 0 <= c_offset and c_offset + n <= low.shape[1],
              "B and C do not fit the narrow rows")
        _need(rows.dtype == x.dtype and rows.shape[0] == n_tokens and rows.stride(1) == 1 and 0 <= z_offset
              and z_offset + channels <= rows.shape[1], "z does not fit the rows")
        _need(tuple(out.shape) == (n_tokens, channels) and out.dtype == x.dtype and out.is_contiguous(), "out is [T, channels]")
        _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= channels * n and state.is_contiguous(),
              "state rows are too short")
        _need(0 < n <= 256, "up to 256 numbers of state a channel")
        n_entries = cu_q.numel() - 1
        _need(first_position.numel() == n_entries == state_slots.numel(), "one first position and slot per entry")
        # Steps with long portions cut them into chunks that run side by side (the choice depends on the step's counts
        # alone, so a captured step makes it as an eager one does).
        chunk = self.SCAN_CHUNK if n_tokens >= self.SCAN_CHUNKED_FROM else 0
        max_chunks, chunk_state, chunk_sum = 0, None, None
        if chunk:
            max_chunks = -(-n_tokens // chunk)
            slots = n_tokens // chunk + n_entries + 1
            chunk_state = torch.empty((slots, channels * n), dtype=torch.float32, device=x.device)
            chunk_sum = torch.empty((slots, channels), dtype=torch.float32, device=x.device)
        self._check(self.lib.ta_selective_scan(_ptr(x), x.stride(0), _ptr(pre), _ptr(neg_rate), _ptr(low), low.stride(0),
                                               int(b_offset), int(c_offset), _ptr(skip), _ptr(rows), rows.stride(0),
                                               int(z_offset), _ptr(state), ctypes.c_long(state.shape[1]), _ptr(cu_q),
                                               _ptr(first_position), _ptr(state_slots), _ptr(out), n_entries, channels, n,
                                               _code(x.dtype), chunk, max_chunks, _ptr(chunk_state), _ptr(chunk_sum),
                                               self._stream()), "selective_scan")
        return out

    SCAN_CHUNK = 64             # tokens a chunk of the selective scan's chunked form
    SCAN_CHUNKED_FROM = 192     # tokens in a step from which the chunked form runs

    def add_terms_rmsnorm(self, residual: torch.Tensor, terms, weight: torch.Tensor | None, eps: float, out: torch.Tensor,
                          rows: torch.Tensor | None = None, store_residual: bool = True, weight2: torch.Tensor | None = None,
                          eps2: float = 0.0, out2: torch.Tensor | None = None) -> torch.Tensor:
        """x = residual[r] + sum_k factor_k * scale_k * rows_k[r] in float32 (`terms`: up to four of (rows [T, H] in out's
        dtype, factor, scale float32 [H] or None)); optionally residual[r] = x; out[i] = rmsnorm(x) * weight (weight None:
        out[i] = x; out may be a view whose rows lie further apart than H); with out2, a second normalised copy under
        weight2 and eps2.  rows int32 [R] picks the rows (None: all)."""
        terms = tuple(terms)
        n_tokens, hidden = residual.shape
        n_rows = n_tokens if rows is None else rows.numel()
        _dev(residual, weight, rows, weight2, out2)
        _need(out.is_cuda, "kernel operands must live on the GPU")       # (its rows may lie apart: a half of wider rows)
        _need(len(terms) <= 4, "up to four terms")
        _need(residual.dtype == torch.float32 and residual.is_contiguous(), "the residual stream is float32")
        for term, _, scale in terms:
            _dev(term, scale)
            _need(tuple(term.shape) == (n_tokens, hidden) and term.dtype == out.dtype and term.is_contiguous(),
                  "a term is [T, H] in the output's dtype")
            _need(scale is None or (scale.dtype == torch.float32 and scale.numel() == hidden and scale.is_contiguous()),
                  "a term's scale is float32 [H]")
        for w in (weight, weight2):
            _need(w is None or (w.dtype == torch.float32 and w.numel() == hidden), "norm weight must be float32 [H]")
        _need(tuple(out.shape) == (n_rows, hidden) and out.stride(1) == 1 and out.stride(0) >= hidden, "norm output has the wrong shape")
        _need(out2 is None or (weight2 is not None and tuple(out2.shape) == (n_rows, hidden) and out2.dtype == out.dtype
                               and out2.is_contiguous()), "the second output is [R, H] with a weight of its own")
        _need(rows is None or (rows.dtype == torch.int32 and not store_residual), "rows int32, and a subset stores nothing back")
        _need(hidden <= 8192, "rows of up to 8192 elements")
        filled = list(terms) + [(None, 0.0, None)] * (4 - len(terms))
        self._check(self.lib.ta_add_terms_rmsnorm(
            _ptr(residual), len(terms), *[_ptr(t[0]) for t in filled], *[_ptr(t[2]) for t in filled],
            *[ctypes.c_float(float(t[1])) for t in filled], _ptr(weight), ctypes.c_float(eps), _ptr(out), out.stride(0),
            _ptr(weight2), ctypes.c_float(eps2), _ptr(out2), _ptr(rows), n_rows, hidden, int(bool(store_residual)),
            _code(out.dtype), self._stream()), "add_terms_rmsnorm")
        return out

    def scale_cap(self, x: torch.Tensor, scale: float, cap: float) -> torch.Tensor:
        """x <- cap * tanh(scale * x / cap) in place (cap 0: scale * x); x float32."""
        _dev(x)
        _need(x.dtype == torch.float32 and x.is_contiguous(), "float32 rows")
        self._check(self.lib.ta_scale_cap(_ptr(x), ctypes.c_size_t(x.numel()), ctypes.c_float(scale), ctypes.c_float(cap),
                                          self._stream()), "scale_cap")
        return x

    def route_scores(self, logits: torch.Tensor, correction: torch.Tensor | None, n_experts: int, n_groups: int,
                     keep_groups: int, chosen: torch.Tensor, weights: torch.Tensor, softmax: bool = False,
                     group_max: bool = False, gate: torch.Tensor | None = None) -> None:
        """As `route_sigmoid`, from scores of either kind: float32 `logits` [T, >= n_experts] (the experts' first);
        `softmax`: s = softmax over all experts (else sigmoid); `correction` may be None; `group_max`: a group is worth
        its largest choice score (else its two largest); `gate` (float32 [T]) gets sigmoid of the number behind the
        experts' logits in a row."""
        _dev(logits, correction, chosen, weights, gate)
        n_tokens, top = logits.shape[0], chosen.shape[1]
        _need(logits.dtype == torch.float32 and logits.is_contiguous() and logits.shape[1] >= n_experts + (gate is not None),
              "router logits are float32 [T, >= experts]")
        _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == n_experts), "the correction is float32")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32
              and tuple(chosen.shape) == (n_tokens, top) == tuple(weights.shape), "chosen int32 and weights float32 [T, top]")
        _need(gate is None or (gate.dtype == torch.float32 and gate.numel() == n_tokens), "the gate is float32 [T]")
        _need(0 < top <= min(n_experts, 64) and n_experts <= 1024, "between one and 64 of up to 1024 experts a token")
        _need(n_groups == 0 or (n_experts % n_groups == 0 and 0 < keep_groups <= n_groups
                                and keep_groups * (n_experts // n_groups) >= top), "the groups do not fit")
        self._check(self.lib.ta_route_scores(_ptr(logits), logits.shape[1], _ptr(correction), n_tokens, n_experts, int(n_groups),
                                             int(keep_groups), top, int(bool(softmax)), int(bool(group_max)), _ptr(chosen),
                                             _ptr(weights), _ptr(gate), self._stream()), "route_scores")

    def delta_scan(self, fresh: torch.Tensor, decay: torch.Tensor, neg_rate: torch.Tensor, rows: torch.Tensor, beta_offset: int,
                   state: torch.Tensor, cu_q: torch.Tensor, first_position: torch.Tensor, state_slots: torch.Tensor,
                   out: torch.Tensor, heads: int, groups: int, d: int, dv: int, unit_eps: float) -> torch.Tensor:
        """The gated delta rule over every entry's rows, from and into the entries' state rows.

        fresh [T, 2 groups d + heads dv]: q, k (groups of d; head h reads group h // (heads / groups)) and v (heads of
        dv); q and k become unit vectors, x / sqrt(sum x^2 + unit_eps), q times d^(-1/2).  decay float32 [T, heads d]:
        g = exp(neg_rate[h] * softplus(decay)); beta = sigmoid(rows[t, beta_offset + h]).  Per head and token:
        S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; out = S^T q.  state float32 [slots, >= heads d dv] (an
        entry whose first position is 0 starts from zeros); out float32 [T, heads dv].

        Steps with portions of many rows (more than `DELTA_PREPARE_ROWS` rows an entry on average) first make what does
        not depend on the state for all tokens side by side (unit vectors, q . k, beta and the decays, which then stand in
        `decay` in place of their pre-activations), so that the walk from token to token does nothing else."""
        _dev(fresh, decay, neg_rate, rows, state, cu_q, first_position, state_slots, out)
        n_tokens = fresh.shape[0]
        _need(heads > 0 and groups > 0 and heads % groups == 0 and 0 < d <= 256 and dv > 0, "heads of up to 256 key channels")
        _need(fresh.shape[1] == 2 * groups * d + heads * dv, "q, k, v do not fit the rows")
        _need(decay.dtype == torch.float32 and tuple(decay.shape) == (n_tokens, heads * d), "decay float32 [T, heads d]")
        _need(neg_rate.dtype == torch.float32 and neg_rate.numel() == heads, "neg_rate float32 [heads]")
        _need(rows.shape[0] == n_tokens and rows.dtype == fresh.dtype and 0 <= beta_offset and beta_offset + heads <= rows.shape[1],
              "beta does not fit the rows")
        _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= heads * d * dv, "state rows are too short")
        _need(out.dtype == torch.float32 and tuple(out.shape) == (n_tokens, heads * dv), "out float32 [T, heads dv]")
        n_entries = cu_q.numel() - 1
        _need(first_position.numel() == n_entries == state_slots.numel(), "one first position and slot per entry")
        prepared = None
        if n_tokens > self.DELTA_PREPARE_ROWS * n_entries:
            _need(decay.is_contiguous(), "the decays' rows are written in place")
            prepared = torch.empty((n_tokens, 2 * groups * d + heads + groups), dtype=torch.float32, device=fresh.device)
        self._check(self.lib.ta_delta_scan(_ptr(fresh), fresh.shape[1], _ptr(decay), _ptr(neg_rate), _ptr(rows), rows.shape[1],
                                           beta_offset, _ptr(state), ctypes.c_long(state.shape[1]), _ptr(cu_q),
                                           _ptr(first_position), _ptr(state_slots), _ptr(out), _ptr(prepared), n_tokens,
                                           n_entries, heads, groups, d, dv, ctypes.c_float(unit_eps), _code(fresh.dtype),
                                           self._stream()), "delta_scan")
        return out

    DELTA_PREPARE_ROWS = 4     # rows an entry (on average) above which the delta rule's inputs are prepared side by side

    # ---------------------------------------------------- sigmoid router with groups, ungated experts
    def route_sigmoid(self, logits: torch.Tensor, correction: torch.Tensor, n_groups: int, keep_groups: int,
                      chosen: torch.Tensor, weights: torch.Tensor) -> None:
        """For every row of float32 `logits` [T, E]: s = sigmoid(logit); choice scores s + correction; with n_groups > 0 only
        experts of the keep_groups best groups (a group is worth its two largest choice scores) can be chosen; the `top`
        largest choice scores (chosen int32 [T, top], falling, the lower index of equals first), weighted by their s over
        the chosen's sum + 1e-20 (weights float32 [T, top])."""
        _dev(logits, correction, chosen, weights)
        n_tokens, n_experts = logits.shape
        top = chosen.shape[1]
        _need(logits.dtype == torch.float32 and correction.dtype == torch.float32 and correction.numel() == n_experts,
              "router logits and the correction are float32")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32
              and tuple(chosen.shape) == (n_tokens, top) == tuple(weights.shape), "chosen int32 and weights float32 [T, top]")
        _need(0 < top <= min(n_experts, 64) and n_experts <= 1024, "between one and 64 of up to 1024 experts a token")
        _need(n_groups == 0 or (n_experts % n_groups == 0 and 0 < keep_groups <= n_groups
                                and keep_groups * (n_experts // n_groups) >= top), "the groups do not fit")
        self._check(self.lib.ta_route_sigmoid(_ptr(logits), _ptr(correction), n_tokens, n_experts, int(n_groups), int(keep_groups),
                                              top, _ptr(chosen), _ptr(weights), self._stream()), "route_sigmoid")

    def expert_act(self, up: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor, n_experts: int, inner: int,
                   out: torch.Tensor) -> torch.Tensor:
        """up [T, n_experts inner] -> out [T, >= n_experts inner]: weight * max(up, 0)^2 in the columns of the experts a
        token chose, zero everywhere else."""
        _dev(up, chosen, weights, out)
        n_tokens = up.shape[0]
        _need(up.shape[1] == n_experts * inner, "up width")
        _need(out.shape[0] == n_tokens and out.shape[1] >= n_experts * inner and out.dtype == up.dtype, "out is [T, >= E inner]")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32 and chosen.shape == weights.shape
              and chosen.shape[0] == n_tokens, "chosen and weights [T, top]")
        self._check(self.lib.ta_expert_act(_ptr(up), _ptr(chosen), _ptr(weights), n_tokens, chosen.shape[1], n_experts, inner,
                                           out.shape[1], _ptr(out), _code(out.dtype), self._stream()), "expert_act")
        return out

    def relu2(self, x: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
        """out = max(x, 0)^2, element by element."""
        _dev(x, out)
        _need(x.shape == out.shape and x.dtype == out.dtype, "relu2 shapes do not fit")
        self._check(self.lib.ta_relu2(_ptr(x), _ptr(out), ctypes.c_size_t(x.numel()), _code(x.dtype), self._stream()), "relu2")
        return out

    def norm_add_rmsnorm(self, residual: torch.Tensor, delta: torch.Tensor | None, post_weight: torch.Tensor | None,
                         post_eps: float, weight: torch.Tensor | None, eps: float, out: torch.Tensor,
                         rows: torch.Tensor | None = None, store_residual: bool = True) -> torch.Tensor:
        """The norm behind a sub-layer, the residual add and the norm before the next one in one kernel:
        x = residual + delta / sqrt(mean(delta^2) + post_eps) * post_weight (delta as it is without `post_weight`,
        nothing without `delta`), stored back into `residual` unless `rows` selects a subset or `store_residual` is
        off; out = x / sqrt(mean(x^2) + eps) * weight, or x itself without `weight`.

        residual float32 [T, H]; delta [T, H] float32 or bfloat16; weights float32 [H]; rows int32 or None; out
        [rows, H] in delta's dtype or float32."""
        _dev(residual, delta, post_weight, weight, out, rows)
        hidden = residual.shape[1]
        n_rows = residual.shape[0] if rows is None else rows.numel()
        _need(residual.dtype == torch.float32 and residual.is_contiguous(), "the residual stream is float32")
        _need(tuple(out.shape) == (n_rows, hidden) and out.is_contiguous(), "norm output shape")
        for vector in (post_weight, weight):
            _need(vector is None or (vector.dtype == torch.float32 and vector.numel() == hidden), "norm weights are float32 [H]")
        if delta is not None:
            _need(delta.shape == residual.shape and delta.is_contiguous(), "delta must match the residual's shape")
            _need(out.dtype in (delta.dtype, torch.float32), "out has delta's dtype or float32")
        if rows is not None:
            _need(rows.dtype == torch.int32 and not store_residual, "a row subset (int32) never stores the residual")
        delta_code = _code(delta.dtype) if delta is not None else _code(out.dtype)
        self._check(self.lib.ta_norm_add_rmsnorm(_ptr(residual), _ptr(delta), _ptr(post_weight), ctypes.c_float(post_eps),
                                                 _ptr(weight), ctypes.c_float(eps), _ptr(out), _ptr(rows), n_rows, hidden,
                                                 int(store_residual and delta is not None), delta_code, _code(out.dtype),
                                                 self._stream()), "norm_add_rmsnorm")
        return out

    def norm_side_norm(self, residual: torch.Tensor, delta: torch.Tensor, post_weight: torch.Tensor, post_eps: float,
                       gate: torch.Tensor, proj: torch.Tensor, side_norm: torch.Tensor, side_eps: float, table: torch.Tensor,
                       token_ids: torch.Tensor, offset: int, dim: int, weight: torch.Tensor | None, eps: float,
                       out: torch.Tensor, rows: torch.Tensor | None = None):
        """`norm_add_rmsnorm` with a token input between the add and the last norm, in one kernel: with x the stream
        after the add, g = gelu_tanh(gate[:dim] x) * table[token, offset : offset + dim], y = proj[:, :dim] g,
        x += y / sqrt(mean(y^2) + side_eps) * side_norm (stored back unless `rows` selects a subset), out = x /
        sqrt(mean(x^2) + eps) * weight.  gate [>= dim, H], proj [H, >= dim], table [V, W] and delta share out's dtype.
        Returns None for sizes the kernel does not take (rows of more than 4,096 elements, dim above 64)."""
        _dev(residual, delta, post_weight, gate, proj, side_norm, table, token_ids, weight, out, rows)
        hidden = residual.shape[1]
        if hidden > 4096 or dim > 64:
            return None
        n_rows = residual.shape[0] if rows is None else rows.numel()
        _need(residual.dtype == torch.float32 and residual.is_contiguous(), "the residual stream is float32")
        _need(delta.shape == residual.shape and delta.is_contiguous() and delta.dtype == out.dtype, "delta [T, H] of out's dtype")
        _need(tuple(out.shape) == (n_rows, hidden) and out.is_contiguous(), "norm output shape")
        for vector in (post_weight, side_norm, weight):
            _need(vector is None or (vector.dtype == torch.float32 and vector.numel() == hidden), "norm weights are float32 [H]")
        _need(gate.dtype == proj.dtype == table.dtype == out.dtype and gate.is_contiguous() and proj.is_contiguous()
              and table.is_contiguous(), "gate, proj and table are contiguous, of out's dtype")
        _need(gate.shape[0] >= dim and gate.shape[1] == hidden and proj.shape[0] == hidden and proj.shape[1] >= dim, "gate [dim, H], proj [H, dim]")
        _need(table.dim() == 2 and 0 <= offset and offset + dim <= table.shape[1], "the table's slice")
        _need(token_ids.dtype == torch.int32 and token_ids.numel() == residual.shape[0], "token ids are int32 [T]")
        _need(rows is None or rows.dtype == torch.int32, "rows are int32")
        self._check(self.lib.ta_norm_side_norm(
            _ptr(residual), _ptr(delta), _ptr(post_weight), ctypes.c_float(post_eps), _ptr(gate), _ptr(proj), proj.shape[1],
            _ptr(side_norm), ctypes.c_float(side_eps), _ptr(table), table.shape[1], _ptr(token_ids), offset, dim, _ptr(weight),
            ctypes.c_float(eps), _ptr(out), _ptr(rows), n_rows, hidden, int(rows is None), _code(out.dtype), self._stream()),
            "norm_side_norm")
        return out

    def norm_rotate_store(self, qkv: torch.Tensor, bias: torch.Tensor | None, positions: torch.Tensor,
                          rates: torch.Tensor | None, dims: int, slots: torch.Tensor | None,
                          k_pages: torch.Tensor | None, v_pages: torch.Tensor | None, n_q: int, n_k: int, n_v: int,
                          d: int, dv: int, q_norm: torch.Tensor | None = None, k_norm: torch.Tensor | None = None,
                          eps: float = 0.0) -> None:
        """In place on rows of `qkv` ([T, >= (n_q + n_k) d + n_v dv]: query heads, key heads, value heads): bias; an RMS
        norm with weight `q_norm` (float32 [n_q d]) over all query elements at once, `k_norm` likewise over the keys;
        rotation of coordinates i and i + dims / 2 (i < dims / 2) of every query and key head by position * rates[i]
        (float32 angles, accurate sine and cosine; the coordinates from `dims` on pass); keys and values written at
        `slots` into key pages [n_pages, n_k, page_size, d] and value pages [n_pages, n_v, dv, page_size]."""
        _dev(qkv, bias, positions, rates, slots, k_pages, v_pages, q_norm, k_norm)
        n_tokens, width = qkv.shape
        used = (n_q + n_k) * d + n_v * dv
        _need(width >= used and qkv.stride(1) == 1, "qkv is narrower than its heads")
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        _need(dims % 2 == 0 and 0 <= dims <= d and dims <= 256, "the rotation covers an even number of a head's coordinates")
        if dims:
            _need(rates is not None and rates.dtype == torch.float32 and rates.numel() == dims // 2, "rates are float32 [dims / 2]")
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() >= used, "bias must be float32 over the heads")
        _need(q_norm is None or (q_norm.dtype == torch.float32 and q_norm.numel() == n_q * d), "q_norm is float32 [n_q d]")
        _need(k_norm is None or (k_norm.dtype == torch.float32 and k_norm.numel() == n_k * d), "k_norm is float32 [n_k d]")
        page_size = 1
        if slots is not None:
            _need(slots.dtype == torch.int32 and slots.numel() == n_tokens, "slots must be int32 [T]")
            _need(k_pages is not None and v_pages is not None, "slots without pages")
            _need(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "pages must have the dtype of qkv")
            page_size = self._page_size(k_pages, v_pages, n_k, d, dv, n_v)
        self._check(self.lib.ta_norm_rotate_store(
            _ptr(qkv), qkv.stride(0), _ptr(bias), _ptr(positions), _ptr(rates if dims else None), dims, _ptr(slots),
            _ptr(k_pages), _ptr(v_pages), n_tokens, n_q, n_k, n_v, d, dv, page_size, _ptr(q_norm), _ptr(k_norm),
            ctypes.c_float(eps), _code(qkv.dtype), self._stream()), "norm_rotate_store")

    def differential_heads(self, mixed: torch.Tensor, lam: torch.Tensor, eps: float, out_scale: float, n_heads: int,
                           group: int, dv: int, out: torch.Tensor) -> torch.Tensor:
        """mixed [T, 2 n_heads dv], laid out (kv head, map, head within the group of `group`, dv); out [T, n_heads dv]:
        o = map 1 - lam[0] * map 2 per head, o / sqrt(mean(o^2) + eps) * out_scale.  lam float32 [1]."""
        _dev(mixed, lam, out)
        n_tokens = mixed.shape[0]
        _need(mixed.is_contiguous() and tuple(mixed.shape) == (n_tokens, 2 * n_heads * dv), "the maps' outputs are [T, 2 H dv]")
        _need(out.is_contiguous() and tuple(out.shape) == (n_tokens, n_heads * dv) and out.dtype == mixed.dtype, "out is [T, H dv]")
        _need(lam.dtype == torch.float32 and lam.numel() == 1 and 0 < dv <= 256 and n_heads % group == 0, "lam is float32 [1]")
        self._check(self.lib.ta_differential_heads(_ptr(mixed), _ptr(lam), ctypes.c_float(eps), ctypes.c_float(out_scale),
                                                   n_tokens, n_heads, group, dv, _ptr(out), _code(out.dtype), self._stream()),
                    "differential_heads")
        return out

    def sigmoid_head_gate(self, mixed: torch.Tensor, rows: torch.Tensor, offset: int, n_heads: int, dv: int) -> torch.Tensor:
        """mixed[t, h, :] *= sigmoid(rows[t, offset + h]) in place; mixed [T, n_heads dv], rows [T, >= offset + n_heads]."""
        _dev(mixed, rows)
        n_tokens = mixed.shape[0]
        _need(mixed.is_contiguous() and tuple(mixed.shape) == (n_tokens, n_heads * dv), "mixed is [T, H dv]")
        _need(rows.shape[0] == n_tokens and rows.stride(1) == 1 and rows.shape[1] >= offset + n_heads and rows.dtype == mixed.dtype,
              "the gates' rows do not fit")
        self._check(self.lib.ta_sigmoid_head_gate(_ptr(mixed), _ptr(rows), rows.stride(0), offset, n_tokens, n_heads, dv,
                                                  _code(mixed.dtype), self._stream()), "sigmoid_head_gate")
        return mixed

    def route_top(self, logits: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor) -> None:
        """For every row of float32 `logits` [T, E]: the indices of its `top` largest (chosen int32 [T, top], falling
        order, the lower index of equals first) and the softmax over those alone (weights float32 [T, top])."""
        _dev(logits, chosen, weights)
        n_tokens, n_experts = logits.shape
        top = chosen.shape[1]
        _need(logits.dtype == torch.float32 and logits.is_contiguous(), "router logits are float32")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32 and chosen.is_contiguous() and weights.is_contiguous()
              and tuple(chosen.shape) == (n_tokens, top) == tuple(weights.shape), "chosen int32 and weights float32 [T, top]")
        _need(0 < top <= min(n_experts, 64), "between one and 64 experts a token, no more than there are")
        self._check(self.lib.ta_route_top(_ptr(logits), n_tokens, n_experts, top, _ptr(chosen), _ptr(weights), self._stream()),
                    "route_top")

    def route_rows(self, x: torch.Tensor, router: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor) -> bool:
        """`route_top` of the float32 logits x @ router.T without leaving them in memory: product and choice in one
        kernel.  x [T, H], router [E, H] of one dtype.  Returns False for sizes the kernel does not take (more than 256
        experts, rows that are not whole pieces of sixteen bytes or longer than 4,096 bfloat16 / 2,048 float32
        elements): the caller then forms the logits with `linear` and calls `route_top`."""
        _dev(x, router, chosen, weights)
        n_tokens, hidden = x.shape
        n_experts, top = router.shape[0], chosen.shape[1]
        _need(x.dtype == router.dtype and x.stride(1) == 1 and router.is_contiguous() and router.shape[1] == hidden, "router [E, H]")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32 and chosen.is_contiguous() and weights.is_contiguous()
              and tuple(chosen.shape) == (n_tokens, top) == tuple(weights.shape), "chosen int32 and weights float32 [T, top]")
        _need(0 < top <= min(n_experts, 64), "between one and 64 experts a token, no more than there are")
        status = self.lib.ta_route_rows(_ptr(x), x.stride(0) if n_tokens > 1 else hidden, _ptr(router), n_tokens, hidden,
                                        n_experts, top, _ptr(chosen), _ptr(weights), _code(x.dtype), self._stream())
        if status == -2:
            return False
        self._check(status, "route_rows")
        return True

    def route_rows_scores(self, x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor | None, n_experts: int,
                          n_groups: int, keep_groups: int, chosen: torch.Tensor, weights: torch.Tensor, softmax: bool = False,
                          group_max: bool = False, gate: torch.Tensor | None = None) -> bool:
        """`route_scores` of the float32 logits x @ router.T without leaving them in memory (router [n_experts, H], or with
        a gate [n_experts + 1, H], the gate's row last): product and choice in one kernel, a token a workgroup (for the few
        rows of a decode step).  Returns False for sizes the kernel does not take: the caller then forms the logits with
        `linear` and calls `route_scores`."""
        _dev(x, router, correction, chosen, weights, gate)
        n_tokens, hidden = x.shape
        top = chosen.shape[1]
        _need(x.dtype == router.dtype and x.stride(1) == 1 and router.is_contiguous() and router.shape[1] == hidden
              and router.shape[0] == n_experts + (gate is not None), "router [E (+ 1), H]")
        _need(correction is None or (correction.dtype == torch.float32 and correction.numel() == n_experts), "the correction is float32 [E]")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32 and chosen.is_contiguous() and weights.is_contiguous()
              and tuple(chosen.shape) == (n_tokens, top) == tuple(weights.shape), "chosen int32 and weights float32 [T, top]")
        _need(gate is None or (gate.dtype == torch.float32 and gate.numel() == n_tokens), "the gate is float32 [T]")
        _need(0 < top <= min(n_experts, 64), "between one and 64 experts a token, no more than there are")
        _need(n_groups >= 0 and (n_groups == 0 or (n_experts % n_groups == 0 and 0 < keep_groups <= n_groups
                                                   and keep_groups * (n_experts // n_groups) >= top)),
              "the kept groups must hold the experts a token uses")
        status = self.lib.ta_route_rows_scores(_ptr(x), x.stride(0) if n_tokens > 1 else hidden, _ptr(router), _ptr(correction),
                                               n_tokens, hidden, n_experts, int(n_groups), int(keep_groups), top,
                                               int(bool(softmax)), int(bool(group_max)), _ptr(chosen), _ptr(weights),
                                               _ptr(gate), _code(x.dtype), self._stream())
        if status == -2:
            return False
        self._check(status, "route_rows_scores")
        return True

    def route_rows_sigmoid(self, x: torch.Tensor, router: torch.Tensor, correction: torch.Tensor, n_groups: int,
                           keep_groups: int, chosen: torch.Tensor, weights: torch.Tensor) -> bool:
        """`route_sigmoid` of the float32 logits x @ router.T without leaving them in memory: product and choice in one
        kernel, a token a workgroup (for the few rows of a decode step).  Returns False for sizes the kernel does not take
        (as `route_rows`): the caller then forms the logits with `linear` and calls `route_sigmoid`."""
        _dev(x, router, correction, chosen, weights)
        n_tokens, hidden = x.shape
        n_experts, top = router.shape[0], chosen.shape[1]
        _need(x.dtype == router.dtype and x.stride(1) == 1 and router.is_contiguous() and router.shape[1] == hidden, "router [E, H]")
        _need(correction.dtype == torch.float32 and correction.numel() == n_experts, "the correction is float32 [E]")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32 and chosen.is_contiguous() and weights.is_contiguous()
              and tuple(chosen.shape) == (n_tokens, top) == tuple(weights.shape), "chosen int32 and weights float32 [T, top]")
        _need(0 < top <= min(n_experts, 64), "between one and 64 experts a token, no more than there are")
        _need(n_groups >= 0 and (n_groups == 0 or (n_experts % n_groups == 0 and 0 < keep_groups <= n_groups
                                                   and keep_groups * (n_experts // n_groups) >= top)),
              "the kept groups must hold the experts a token uses")
        status = self.lib.ta_route_rows_sigmoid(_ptr(x), x.stride(0) if n_tokens > 1 else hidden, _ptr(router), _ptr(correction),
                                                n_tokens, hidden, n_experts, n_groups, keep_groups, top, _ptr(chosen),
                                                _ptr(weights), _code(x.dtype), self._stream())
        if status == -2:
            return False
        self._check(status, "route_rows_sigmoid")
        return True

    ROUTE_ROWS_FUSED = 64      # rows up to which the sigmoid router's product and choice are one kernel (a workgroup a row)

    # Routed feed-forwards over sorted tokens (bfloat16): tiles of `bm` slots that belong to one expert each.
    GROUPED_EXPERTS = 256

    @staticmethod
    def grouped_tiles(n_entries: int, n_experts: int, bm: int) -> int:
        """How many tiles of `bm` slots the (token, expert) pairs of a step can need at most."""
        return -(-n_entries // bm) + n_experts

    def expert_slots(self, chosen: torch.Tensor, n_experts: int, bm: int):
        """Sort a step's picks (chosen int32 [T, top]) by expert into tiles of `bm` slots: returns (slot_of int32
        [T * top], row_of int32 [tiles * bm] with -1 for slots that only fill a tile up, tile_expert int32 [tiles] with
        -1 for tiles past the last run), all on the device; nothing comes back to the host."""
        _dev(chosen)
        _need(chosen.dtype == torch.int32 and chosen.dim() == 2 and chosen.is_contiguous(), "chosen is int32 [T, top]")
        _need(0 < n_experts <= self.GROUPED_EXPERTS and bm in (64, 128), "up to 256 experts, tiles of 64 or 128 slots")
        n_entries = chosen.numel()
        tiles = self.grouped_tiles(n_entries, n_experts, bm)
        slot_of = torch.empty(n_entries, dtype=torch.int32, device=chosen.device)
        row_of = torch.empty(tiles * bm, dtype=torch.int32, device=chosen.device)
        tile_expert = torch.empty(tiles, dtype=torch.int32, device=chosen.device)
        self._check(self.lib.ta_expert_slots(_ptr(chosen), n_entries, chosen.shape[1], n_experts, bm, tiles, _ptr(slot_of),
                                             _ptr(row_of), _ptr(tile_expert), self._stream()), "expert_slots")
        return slot_of, row_of, tile_expert

    def grouped_linear(self, x: torch.Tensor, row_of: torch.Tensor | None, tile_expert: torch.Tensor, bm: int,
                       weight: torch.Tensor, expert_stride: int, n_out: int, k: int, out_dtype: torch.dtype) -> torch.Tensor:
        """out[slot] = x[row_of[slot]] (or x[slot] without `row_of`) @ W_e.T for every slot of every tile, W_e the
        [n_out, k] block of `weight` (contiguous [rows, ldw]) that starts `expert_stride` elements times the tile's
        expert into it.  bfloat16 operands, float32 sums; out [tiles * bm, n_out] bfloat16 or float32."""
        _dev(x, row_of, tile_expert, weight)
        tiles = tile_expert.numel()
        _need(x.dtype == torch.bfloat16 and weight.dtype == torch.bfloat16 and x.stride(1) == 1 and weight.is_contiguous(),
              "bfloat16 operands with contiguous rows")
        _need(x.shape[1] >= k and (row_of is not None or x.shape[0] >= tiles * bm), "rows of x for every slot")
        _need(row_of is None or (row_of.dtype == torch.int32 and row_of.numel() == tiles * bm), "row_of is int32 [tiles bm]")
        _need(tile_expert.dtype == torch.int32 and k % 8 == 0 and x.stride(0) % 8 == 0 and weight.shape[1] % 8 == 0
              and expert_stride % 8 == 0, "K, strides and the experts' offsets in eights")
        out = torch.empty((tiles * bm, n_out), dtype=out_dtype, device=x.device)
        self._check(self.lib.ta_grouped_gemm_bf16(_ptr(x), x.stride(0), _ptr(row_of), _ptr(tile_expert), tiles, bm, _ptr(weight),
                                                  int(expert_stride), weight.shape[1], _ptr(out), n_out, n_out, k,
                                                  _code(out_dtype), self._stream()), "grouped_linear")
        return out

    def expert_combine(self, rows: torch.Tensor, slot_of: torch.Tensor, weights: torch.Tensor, shared: torch.Tensor | None,
                       out: torch.Tensor, shared_weight: torch.Tensor | None = None) -> torch.Tensor:
        """out[t] = shared[t] (if given; times shared_weight[t], float32 [T], if that is given) + sum over the token's picks of weights[t, k] * rows[slot_of[t top + k]]; rows
        float32 [slots, H], weights float32 [T, top], shared and out [T, H] of one dtype."""
        _dev(rows, slot_of, weights, shared, out)
        n_tokens, top = weights.shape
        _need(rows.dtype == torch.float32 and rows.is_contiguous() and rows.shape[1] == out.shape[1], "rows are float32 [slots, H]")
        _need(slot_of.dtype == torch.int32 and slot_of.numel() == n_tokens * top and weights.dtype == torch.float32
              and weights.is_contiguous(), "slot_of int32 [T top], weights float32 [T, top]")
        _need(out.is_contiguous() and out.shape[0] == n_tokens and (shared is None or (shared.shape == out.shape
              and shared.dtype == out.dtype and shared.is_contiguous())), "shared and out are [T, H]")
        _dev(shared_weight)
        _need(shared_weight is None or (shared_weight.dtype == torch.float32 and shared_weight.numel() == n_tokens),
              "the shared expert's weights are float32 [T]")
        self._check(self.lib.ta_expert_combine(_ptr(rows), _ptr(slot_of), _ptr(weights), n_tokens, top, _ptr(shared), _ptr(out),
                                               out.shape[1], _code(out.dtype), _ptr(shared_weight), self._stream()), "expert_combine")
        return out

    def expert_gate(self, gate_up: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor, n_experts: int, inner: int,
                    shared: int, out: torch.Tensor, shared_weight: torch.Tensor | None = None) -> torch.Tensor:
        """gate_up [T, n_experts 2 inner + 2 shared] (every expert's gate rows, then its up rows; the shared expert
        last) -> out [T, >= n_experts inner + shared]: weight * silu(gate) * up in the columns of the experts a token
        chose, silu(gate) * up in the shared expert's (times shared_weight[t], float32 [T], if given), zero everywhere else."""
        _dev(gate_up, chosen, weights, out, shared_weight)
        _need(shared_weight is None or (shared_weight.dtype == torch.float32 and shared_weight.numel() == gate_up.shape[0]),
              "the shared expert's weights are float32 [T]")
        n_tokens = gate_up.shape[0]
        _need(gate_up.is_contiguous() and gate_up.shape[1] == n_experts * 2 * inner + 2 * shared, "gate_up width")
        _need(out.is_contiguous() and out.shape[0] == n_tokens and out.shape[1] >= n_experts * inner + shared
              and out.dtype == gate_up.dtype, "out is [T, >= E inner + shared]")
        _need(chosen.dtype == torch.int32 and weights.dtype == torch.float32 and chosen.shape == weights.shape
              and chosen.shape[0] == n_tokens and chosen.is_contiguous() and weights.is_contiguous(), "chosen and weights [T, top]")
        self._check(self.lib.ta_expert_gate(_ptr(gate_up), _ptr(chosen), _ptr(weights), n_tokens, chosen.shape[1], n_experts,
                                            inner, shared, out.shape[1], _ptr(out), _code(out.dtype), _ptr(shared_weight),
                                            self._stream()), "expert_gate")
        return out

    def side_gate(self, gate: torch.Tensor, table: torch.Tensor, token_ids: torch.Tensor, offset: int, dim: int,
                  out: torch.Tensor) -> torch.Tensor:
        """out[t, j] = gelu_tanh(gate[t, j]) * table[token_ids[t], offset + j] for j < dim, zero in further columns."""
        _dev(gate, table, token_ids, out)
        n_tokens, columns = gate.shape
        _need(gate.is_contiguous() and out.is_contiguous() and out.shape == gate.shape and out.dtype == gate.dtype == table.dtype,
              "gate and out are [T, columns] of the table's dtype")
        _need(table.dim() == 2 and table.is_contiguous() and 0 <= offset and offset + dim <= table.shape[1] and dim <= columns,
              "the table's slice")
        _need(token_ids.dtype == torch.int32 and token_ids.numel() == n_tokens, "token ids are int32 [T]")
        self._check(self.lib.ta_side_gate(_ptr(gate), _ptr(table), table.shape[1], _ptr(token_ids), offset, dim, columns,
                                          n_tokens, _ptr(out), _code(out.dtype), self._stream()), "side_gate")
        return out

    # ------------------------------------------------------------- gated activation
    def silu_gate(self, gate_up: torch.Tensor, out: torch.Tensor, act: tuple | None = None) -> torch.Tensor:
        """out = silu(gate_up[:, :I]) * gate_up[:, I:].  gate_up [T, 2I]; out [T, I].  With `act` = (alpha, limit,
        shift): g' = min(g, limit), u' = clamp(u, -limit, limit), out = g' * sigmoid(alpha g') * (u' + shift); with
        `act` = "gelu_tanh": out = 0.5 g (1 + tanh(sqrt(2/pi) (g + 0.044715 g^3))) * u."""
        _dev(gate_up, out)
        n_tokens, two_inner = gate_up.shape
        _need(two_inner % 2 == 0 and tuple(out.shape) == (n_tokens, two_inner // 2) and out.dtype == gate_up.dtype,
              "silu_gate shapes do not fit")
        if act == "gelu_tanh":
            self._check(self.lib.ta_gelu_gate(_ptr(gate_up), _ptr(out), n_tokens, two_inner // 2, _code(out.dtype),
                                              self._stream()), "gelu_gate")
            return out
        if act is not None:
            alpha, limit, shift = act
            self._check(self.lib.ta_capped_gate(_ptr(gate_up), _ptr(out), n_tokens, two_inner // 2, ctypes.c_float(alpha),
                                                ctypes.c_float(limit), ctypes.c_float(shift), _code(out.dtype),
                                                self._stream()), "capped_gate")
            return out
        self._check(self.lib.ta_silu_gate(_ptr(gate_up), _ptr(out), n_tokens, two_inner // 2,
                                          _code(out.dtype), self._stream()), "silu_gate")
        return out

    # ----------------------------------------------------------------------- rope
    def rope_store(self, qkv: torch.Tensor, bias: torch.Tensor | None, positions: torch.Tensor,
                   cos_sin: torch.Tensor | None, slots: torch.Tensor | None,
                   k_pages: torch.Tensor | None, v_pages: torch.Tensor | None,
                   n_q: int, n_kv: int, head_dim: int, value_dim: int | None = None) -> None:
        """Add bias, rotate q and k heads in place, store k and v heads into their pages.

        qkv [T, (n_q + n_kv) d + n_kv dv] (dv = `value_dim`, d if None); bias float32 or None; positions int32 [T];
        cos_sin float32 [P, d] (cos half, sin half) or None for no rotation;
        slots int32 [T] (page * page_size + offset, negative = skip) or None;
        key pages [n_pages, n_kv, page_size, d], value pages [n_pages, n_kv, d, page_size].
        """
        _dev(qkv, bias, positions, cos_sin, slots, k_pages, v_pages)
        n_tokens, width = qkv.shape
        value_dim = head_dim if value_dim is None else int(value_dim)
        _need(width == (n_q + n_kv) * head_dim + n_kv * value_dim, "qkv width does not match the head counts")
        _need(head_dim % 2 == 0 or cos_sin is None, "head size must be even")
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        page_size = 1
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == width, "bias must be float32 of the qkv width")
        if cos_sin is not None:
            _need(cos_sin.dtype == torch.float32 and cos_sin.shape[1] == head_dim, "cos_sin must be float32 [P, d]")
        if slots is not None:
            _need(slots.dtype == torch.int32 and slots.numel() == n_tokens, "slots must be int32 [T]")
            _need(k_pages is not None and v_pages is not None, "slots without pages")
            _need(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "pages must have the dtype of qkv")
            page_size = self._page_size(k_pages, v_pages, n_kv, head_dim, value_dim)
        self._check(self.lib.ta_rope_store(_ptr(qkv), width, _ptr(bias), _ptr(positions), _ptr(cos_sin),
                                           _ptr(slots), _ptr(k_pages), _ptr(v_pages), n_tokens, n_q, n_kv,
                                           head_dim, page_size, _code(qkv.dtype), value_dim, self._stream()), "rope_store")

    @staticmethod
    def _page_size(k_pages: torch.Tensor, v_pages: torch.Tensor, n_kv: int, head_dim: int,
                   value_dim: int | None = None, value_heads: int | None = None) -> int:
        value_dim = head_dim if value_dim is None else value_dim
        _need(k_pages.dim() == 4 and k_pages.shape[1] == n_kv and k_pages.shape[3] == head_dim,
              "key pages must be [n_pages, n_kv, page_size, d]")
        page_size = k_pages.shape[2]
        _need(tuple(v_pages.shape) == (k_pages.shape[0], n_kv if value_heads is None else value_heads, value_dim, page_size),
              "value pages must be [n_pages, n_kv, dv, page_size]")
        _need(k_pages.numel() < 2 ** 31 and v_pages.numel() < 2 ** 31, "a layer's pages must hold fewer than 2^31 elements")
        return page_size

    # ------------------------------------------------------------------ attention
    def paged_attention(self, qkv: torch.Tensor, out: torch.Tensor, k_pages: torch.Tensor,
                        v_pages: torch.Tensor, positions: torch.Tensor, entry_of_token: torch.Tensor,
                        block_table: torch.Tensor, n_q: int, n_kv: int, head_dim: int,
                        window: int | None, scale: float, max_position: int | None = None,
                        batch=None, value_dim: int | None = None, chunk: int | None = None,
                        slopes: torch.Tensor | None = None, sinks: torch.Tensor | None = None,
                        keep_first: int = 0, value_heads: int | None = None, softcap: float | None = None) -> torch.Tensor:
        """Causal attention of every token over the pages of its request.

        `softcap` c: a score (scaled, with its distance term) becomes c tanh(score / c) before the softmax.

        `keep_first` n (with a window): keys at positions below n stay visible behind the window.  `value_heads`
        (a divisor of n_kv): the value pages hold so many heads, and key head g reads value head
        g / (n_kv / value_heads).  Both run the generic kernel.

        Beyond the plain form: `value_dim` (value heads of dv elements; out is [T, n_q dv]), `chunk` (only keys
        of the query's own run of so many positions, counted from position 0), `slopes` (float32 [n_q]: head h's
        score loses slopes[h] per position of distance), `sinks` (float32 [n_q]: exp(sinks[h]) joins the
        denominator).  Scores and weights are float32.

        qkv [T, >= n_q d] (query heads first); out [T, n_q d]; key pages [n_pages, n_kv, page_size, d],
        value pages [n_pages, n_kv, d, page_size];
        positions, entry_of_token int32 [T]; block_table int32 [E, P]; a token at position p sees keys
        max(0, p - window)..p.  `max_position` (host) lets the wrapper check that the table is wide enough.
        `batch` (a StepContext of the same tokens) lets bfloat16 batches run the tiled kernel on prompt
        portions and the split kernel on single tokens; without it every token goes through the latter.
        """
        _dev(qkv, out, k_pages, v_pages, positions, entry_of_token, block_table)
        n_tokens = qkv.shape[0]
        value_dim = head_dim if value_dim is None else int(value_dim)
        _dev(slopes, sinks)
        for extra in (slopes, sinks):
            _need(extra is None or (extra.dtype == torch.float32 and extra.numel() == n_q), "slopes and sinks are float32 [n_q]")
        _need(chunk is None or chunk > 0, "a chunk has at least one position")
        plain = value_dim == head_dim and chunk is None and slopes is None and sinks is None
        value_heads = n_kv if value_heads is None else int(value_heads)
        keep_first = int(keep_first) if window is not None else 0
        _need(value_heads > 0 and n_kv % value_heads == 0 and keep_first >= 0, "value heads divide the key heads")
        _need(qkv.shape[1] >= n_q * head_dim, "qkv is narrower than the query heads")
        _need(tuple(out.shape) == (n_tokens, n_q * value_dim) and out.dtype == qkv.dtype, "attention output shape")
        _need(k_pages.dtype == qkv.dtype and v_pages.dtype == qkv.dtype, "pages must have the dtype of qkv")
        page_size = self._page_size(k_pages, v_pages, n_kv, head_dim, value_dim, value_heads)
        _need(positions.dtype == torch.int32 and positions.numel() == n_tokens, "positions must be int32 [T]")
        _need(entry_of_token.dtype == torch.int32 and entry_of_token.numel() == n_tokens, "entry_of_token must be int32 [T]")
        _need(block_table.dtype == torch.int32 and block_table.dim() == 2, "block_table must be int32 [E, P]")
        _need(n_kv > 0 and n_q % n_kv == 0, "query heads must be a multiple of kv heads")
        _need(0 < head_dim <= 512 and 0 < value_dim <= 512, "head sizes up to 512 are supported")
        if max_position is not None:
            _need(max_position // page_size < block_table.shape[1], "block table is too narrow for the positions")
        # The matrix-core kernels take chunks, slopes and sinks as they are; value heads of another size than the key
        # heads go to the generic kernel.
        plain = plain and keep_first == 0 and value_heads == n_kv
        if (value_dim == head_dim and qkv.dtype == torch.bfloat16 and head_dim in self.DECODE_HEAD_DIMS and page_size % 16 == 0
                and qkv.shape[1] % 8 == 0 and self.use_fast_attention
                and (keep_first == 0 or (chunk is None and slopes is None))):
            args = (qkv, out, k_pages, v_pages, positions, entry_of_token, block_table, n_q, n_kv, head_dim,
                    page_size, window, scale, max_position)
            plain = plain and not softcap
            extras = {} if plain else dict(chunk=chunk, slopes=slopes, sinks=sinks, keep_first=keep_first,
                                           value_heads=value_heads, softcap=softcap)
            if batch is None:
                return self._decode_attention(*args, **extras)
            if batch.q_tiles.numel() == 0:
                # One token per request: request e is row e, the kernel needs no entry-of-token lookup.
                return self._decode_attention(*args, identity_entries=batch.n_tokens == block_table.shape[0], **extras)
            _need(batch.n_tokens == n_tokens and batch.cu_q.numel() == block_table.shape[0] + 1,
                  "the batch description does not belong to these tokens")
            n_tiles, choice = batch.q_tiles.shape[0], (
                -1 if window is None else int(window), self.prefill_shape, int(batch.max_position) + 1,
                self.prefill_waves, self.prefill_shared)
            # A few tiles behind a long context: the launcher cuts each tile's keys over workgroups, whose states
            # a second kernel merges; it says into how many parts, and gets the buffers for them.
            parts = self.lib.ta_prefill_attention_key_splits(n_tiles, n_q, n_kv, head_dim, *choice) \
                if self.prefill_key_splits and plain else 1
            part_o = part_ml = None
            if parts > 1:
                part_o = torch.empty((n_tiles * 16, n_q, parts, head_dim), dtype=torch.float32, device=qkv.device)
                part_ml = torch.empty((n_tiles * 16, n_q, parts, 2), dtype=torch.float32, device=qkv.device)
            self._check(self.lib.ta_prefill_attention_bf16(
                _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(batch.q_tiles),
                n_tiles, _ptr(batch.cu_q), _ptr(batch.first_position), _ptr(block_table),
                block_table.shape[1], n_q, n_kv, head_dim, page_size, choice[0], ctypes.c_float(scale), *choice[1:],
                _ptr(part_o), _ptr(part_ml), 0 if chunk is None else int(chunk), _ptr(slopes), _ptr(sinks),
                keep_first, value_heads, ctypes.c_float(softcap or 0.0), self._stream()), "prefill_attention")
            if batch.decode_rows.numel():
                self._decode_attention(*args, rows=batch.decode_rows, **extras)
            return out
        self._check(self.lib.ta_paged_attention_generic(
            _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(positions),
            _ptr(entry_of_token), _ptr(block_table), block_table.shape[1], n_tokens, n_q, n_kv, head_dim,
            page_size, -1 if window is None else int(window), ctypes.c_float(scale), _code(qkv.dtype),
            value_dim, 0 if chunk is None else int(chunk), _ptr(slopes), _ptr(sinks), keep_first, value_heads,
            ctypes.c_float(softcap or 0.0), self._stream()), "paged_attention")
        return out

    DECODE_HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256)
    use_fast_attention = True     # tests switch it off to reach the generic kernel in bfloat16
    prefill_waves = 0             # waves that share a tile's keys in the per-wave prompt kernel: 0 lets the launcher choose;
    #                               asking for a number asks for that kernel
    prefill_shape = 0             # shape of the workgroup-shared prompt kernel when it is asked for: heads a wave
    #                               (1 or 2), + 10 for two key groups in a workgroup; 0: its own choice
    prefill_shared = 0            # the prompt kernel whose waves share a block of keys through LDS: 1 = wherever it has
    #                               an instance, -1 = never, 0 = where the launcher expects it to be the faster one
    prefill_key_splits = True     # whether the prompt kernel may cut a tile's keys over workgroups (tests switch it off)
    target_workgroups = 1024      # what the split of the key range aims at
    min_split_keys = 128          # ... in parts of at least so many keys (a block of 32 for each of a workgroup's four waves)
    PLAN_KEYS = 512               # launch shapes depend on the context only through its multiple of this

    def _decode_attention(self, qkv, out, k_pages, v_pages, positions, entry_of_token, block_table,
                          n_q, n_kv, head_dim, page_size, window, scale, max_position, rows=None,
                          identity_entries=False, chunk=None, slopes=None, sinks=None, keep_first=0, value_heads=None,
                          softcap=None):
        """Matrix-core attention of single tokens with the key range split over workgroups (kept first keys behind a
        window are further splits of their own)."""
        n_items = qkv.shape[0] if rows is None else rows.numel()
        max_keys = (block_table.shape[1] * page_size) if max_position is None else max_position + 1
        # The split is planned for the context rounded up to a multiple of 512 keys: a step that replays a
        # graph captured for a whole range of contexts then splits exactly as the same step run on its own.
        max_keys = -(-max_keys // self.PLAN_KEYS) * self.PLAN_KEYS
        if window is not None:
            max_keys = min(max_keys, window + 32)
        if chunk is not None:
            max_keys = min(max_keys, chunk + 32)
        head_blocks = -(-(n_q // n_kv) // 16)
        per_split = max(1, self.target_workgroups // max(1, n_items * n_kv * head_blocks))
        split_keys = max(self.min_split_keys, -(-max_keys // per_split))
        split_keys = -(-split_keys // 32) * 32
        splits = max(1, -(-(max_keys + 31) // split_keys))
        kept_splits = -(-int(keep_first) // split_keys) if keep_first and window is not None else 0
        splits += kept_splits
        part_o = part_ml = None
        if splits > 1:
            part_o = torch.empty((n_items, n_q, splits, head_dim), dtype=torch.float32, device=qkv.device)
            part_ml = torch.empty((n_items, n_q, splits, 2), dtype=torch.float32, device=qkv.device)
        self._check(self.lib.ta_decode_attention_bf16(
            _ptr(qkv), qkv.shape[1], _ptr(out), _ptr(k_pages), _ptr(v_pages), _ptr(rows), _ptr(positions),
            _ptr(None if identity_entries and rows is None else entry_of_token), _ptr(block_table),
            block_table.shape[1], _ptr(part_o), _ptr(part_ml), n_items,
            n_q, n_kv, head_dim, page_size, -1 if window is None else int(window), ctypes.c_float(scale),
            split_keys, splits, 0 if chunk is None else int(chunk), _ptr(slopes), _ptr(sinks),
            int(keep_first) if kept_splits else 0, kept_splits, n_kv if value_heads is None else int(value_heads),
            ctypes.c_float(softcap or 0.0), self._stream()), "decode_attention")
        return out

    # --------------------------------------------------------------------- linear
    takes_pending = True      # `linear(pending=True)` and `add_rmsnorm` with a `PendingSum` exist here

    def linear(self, x: torch.Tensor, weight: torch.Tensor, bias: torch.Tensor | None = None,
               out: torch.Tensor | None = None, out_dtype: torch.dtype | None = None,
               pending: bool = False) -> "torch.Tensor | PendingSum":
        """out = x @ weight.T (+ bias).  x [M, K] (rows may be strided); weight [N, K]; bias float32 [N].

        float32 operands run on plain multiply-adds; bfloat16 operands on the matrix cores with
        float accumulation and a bfloat16 or float32 result.  `pending=True` allows the result to come back
        as a `PendingSum` when K is cut over workgroups: whoever takes it next (the norm that follows) adds the
        parts in its own kernel and the addition's launch is saved.
        """
        _need(x.is_cuda and weight.is_cuda, "kernel operands must live on the GPU")
        _need(x.dim() == 2 and weight.dim() == 2 and x.shape[1] == weight.shape[1], "linear shapes do not fit")
        _need(x.stride(1) == 1 and weight.is_contiguous(), "linear operands must have contiguous rows")
        _need(x.dtype == weight.dtype, "x and weight must share a dtype")
        m, k = x.shape
        n = weight.shape[0]
        lda = x.stride(0) if m > 1 else k
        if out_dtype is None:
            out_dtype = x.dtype if out is None else out.dtype
        pending = pending and out is None and x.dtype == torch.bfloat16
        if out is None and not pending:
            out = torch.empty((m, n), dtype=out_dtype, device=x.device)
        if out is not None:
            _need(tuple(out.shape) == (m, n) and out.is_contiguous() and out.dtype == out_dtype, "linear output shape")
        if bias is not None:
            _need(bias.is_cuda and bias.dtype == torch.float32 and bias.numel() == n, "bias must be float32 [N]")
        if x.dtype == torch.float32:
            _need(out_dtype == torch.float32, "float32 products give float32")
            status = self.lib.ta_gemm_f32(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, lda, n,
                                          self._stream())
        else:
            _need(x.dtype == torch.bfloat16, "linear takes float32 or bfloat16")
            if k % 8 or lda % 8 or x.data_ptr() % 16:
                # The matrix-core kernels read K sixteen bytes at a time.  A K that is no multiple of eight is filled
                # up with zeros (the weight once, kept; the rows each time): the sums gain only zeros.
                fill = (-k) % 8
                x = torch.nn.functional.pad(x, (0, fill)) if fill or lda % 8 or x.data_ptr() % 16 else x
                x = x.contiguous()
                weight = self._filled_weight(weight, fill) if fill else weight
                m, k = x.shape
                lda = k
            _need(x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
            streaming_splits = self._streaming_splits(m, n, k, pending)
            if streaming_splits > 1 and self.split_k_kind == "streaming":
                # 17 to 64 rows, a long K and few output columns (the down projection of a decode batch): the
                # weight-streaming kernel with K cut over workgroups, so that every compute unit streams a share
                # of the weights; the parts are added in a fixed order by a second small kernel.
                parts = _parts_of_k(k, streaming_splits, 32)
                leave = pending and parts > 1
                if out is None and not leave:
                    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
                partial = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
                self._check(self.lib.ta_gemm_skinny_bf16_splitk(
                    _ptr(x), lda, _ptr(weight), _ptr(bias), _ptr(None if leave else out), n, _ptr(partial), m, n, k,
                    _code(out_dtype), streaming_splits, self.skinny_column_blocks, self._stream()), "linear")
                return PendingSum(self, partial, bias, out_dtype) if leave else out
            splits = self._k_splits(m, n, k, pending)
            if splits > 1:
                # The same with the tiled kernel.
                parts = _parts_of_k(k, splits, 64)
                leave = pending and parts > 1
                if out is None and not leave:
                    out = torch.empty((m, n), dtype=out_dtype, device=x.device)
                partial = torch.empty((parts, m, n), dtype=torch.float32, device=x.device)
                self._check(self.lib.ta_gemm_bf16_splitk(
                    _ptr(x), _ptr(weight), _ptr(bias), _ptr(None if leave else out), _ptr(partial), m, n, k, lda, n,
                    _code(out_dtype), splits, self._stream()), "linear")
                return PendingSum(self, partial, bias, out_dtype) if leave else out
            if out is None:
                out = torch.empty((m, n), dtype=out_dtype, device=x.device)
            if m > self.SKINNY_ROWS:
                to_library = self.capturing or m * n * k >= self.EAGER_LIBRARY_WORK
            else:
                to_library = m > self.FUSED_ROWS and ((k >= 2048 and n <= 4096) or n * k >= self.LIBRARY_WEIGHT)
            if to_library and self.use_library_gemm and out_dtype == torch.bfloat16:
                # Plain products of more than 64 rows go to the vendor's library (hipBLASLt, called from
                # library_gemm.hip), as the reference's engine uses a library for its matrix products: on the
                # device's own clock (launches recorded in a graph, weights cold) it is ahead of the tiled
                # kernel of this package for nearly every shape of the 0.5B to 7B models.  So do products of 17
                # to 64 rows with a big weight matrix (every tile of the weight-streaming kernel reads all the
                # rows again, which costs more than the weights once there are more than sixteen of them), and
                # those with a long K and few output columns that the kernels above did not take.  The float32 bias
                # joins the library's float accumulator as it joins the kernels' own.  A launch of the library
                # costs the host some 15 us against 4 us for a kernel of this package: outside graph capture,
                # products of more than 64 rows that are over on the device in about that time stay with the
                # tiled kernel (steps of small models with few tokens are bound by the host's launches).
                # In the run that warms a step up before it is recorded the library is told that the shape
                # will come again: it then times its candidates for a big product and keeps the fastest.
                space = self._workspace(x.device)
                status = self.lib.ta_library_gemm_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, lda, n,
                                                       _ptr(space), space.numel(), int(self.capturing),
                                                       self._stream())
                if status != -3:                  # -3: no algorithm for this shape, the kernels below take it
                    self._check(status, "linear (vendor library)")
                    return out
            if m <= self.FUSED_ROWS or (m <= self.SKINNY_ROWS and n < self.WIDE_OUTPUT):
                status = self.lib.ta_gemm_skinny_bf16(_ptr(x), lda, _ptr(weight), _ptr(bias), _ptr(out), n, m, n, k,
                                                      _code(out_dtype), 0, self.skinny_column_blocks, self._stream())
            else:
                status = self.lib.ta_gemm_bf16(_ptr(x), _ptr(weight), _ptr(bias), _ptr(out), m, n, k, lda, n,
                                               _code(out_dtype), self._stream())
        self._check(status, "linear")
        return out

    def _filled_weight(self, weight: torch.Tensor, fill: int) -> torch.Tensor:
        """`weight` with `fill` zero columns behind its K, made once per weight tensor and kept."""
        kept = self._filled.get(weight.data_ptr())
        if kept is None or kept[0] is not weight:
            kept = (weight, torch.nn.functional.pad(weight, (0, fill)).contiguous())
            self._filled[weight.data_ptr()] = kept
        return kept[1]

    use_split_k = True
    skinny_column_blocks = 0   # blocks of sixteen output columns per workgroup of the weight-streaming kernel: 0 = its choice

    def _k_splits(self, m: int, n: int, k: int, pending: bool = False) -> int:
        """Into how many parts the tiled kernel cuts K.  17 to 64 rows: more than one with a K so long, and so few
        output tiles of 64 x 64, that the library (which cuts K as well) falls behind.  65 to 256 rows (portions of
        prompts beside decoded tokens): few tiles again, far fewer than compute units, and a whole K for each is
        a long walk (137 rows x 896 columns over a K of 4,864: 32 us in one piece).  Where the parts may be left
        for the norm that follows (`pending`) and K is 2,048 or more, eight parts beat the library as well (the same
        product: 10 us against 10 us; 137 x 1,536 over 8,960: 17 us against 23 us).  Launched eagerly, small
        products do not go to the library at all (its launch costs the host more than they take): those are cut
        whenever K allows, into parts for the next norm or, with a long K, into four that the kernel adds itself
        (14 us)."""
        if not self.use_split_k or n % 4:
            return 1
        tiles = -(-m // 64) * -(-n // 64)
        if self.SKINNY_ROWS < m <= 256:
            if tiles >= 128:
                return 1
            if pending and k >= 2048:
                return min(8, k // 512)
            if self.capturing or m * n * k >= self.EAGER_LIBRARY_WORK:
                return 1                   # the library's
            if pending and k >= 768:
                return min(8, k // 384)
            return 4 if k >= 2048 else 1
        if not (self.FUSED_ROWS < m <= self.SKINNY_ROWS) or k < self.SPLIT_K_FROM:
            return 1
        if tiles >= self.compute_units:
            return 1
        return max(1, min(-(-2 * self.compute_units // tiles), k // 256))

    split_k_kind = "streaming"     # which kernel cuts K for 17 to 64 rows ("tiled": only the tiled one)

    def _streaming_splits(self, m: int, n: int, k: int, pending: bool = False) -> int:
        """Into how many parts the weight-streaming kernel cuts K for 17 to 64 rows and a K of 2,048 up to where
        the tiled kernel takes over: so many that its tiles of sixteen output columns times the parts give every
        compute unit a workgroup, each part at least 512 long.  (Measured with cold weights for the down
        projections of the 0.5B to 7B models: one of the two beats the library at every row count from 17 to 64,
        the streaming kernel while a part is a few steps per wave, the tiled one, which reads the rows a quarter
        as often, for longer K.)  When the parts may be left for the next norm to add (`pending`), the addition
        costs no launch, and a K from 512 on is cut as well, into parts of at least 224 (the output projection of
        a decode batch: every workgroup reads all the rows, and a quarter of K is a quarter of them)."""
        shortest, part = (self.PENDING_SHORTEST_K, 224) if pending else (2048, 512)
        if self.use_split_k and 0 < m <= self.FUSED_ROWS and k >= self.FEW_ROWS_LONG_K and n % 4 == 0 and -(-n // 16) < 128:
            # Up to sixteen rows, a very long K and few output columns (the down product over all experts of a routed
            # layer in a decode step: K is experts times the inner width): one workgroup a tile of sixteen columns would
            # leave most compute units without a share of the weights.
            # (8 rows x 896 columns over a K of 29,184: 50 us in one piece, 24 in five parts, 19 in eight to twelve; 1,536
            # columns over 53,760: 95, 45 in five to eight.)
            return max(1, min(-(-2 * self.compute_units // -(-n // 16)), k // 2048))
        if (not self.use_split_k or not (self.FUSED_ROWS < m <= self.SKINNY_ROWS) or n % 4
                or not (shortest <= k < self.SPLIT_K_FROM)):
            return 1
        tiles = -(-n // 16)
        if tiles >= 128:
            return 1
        if m > 32:
            tiles = -(-n // 32)        # more than 32 rows: a workgroup takes two blocks of sixteen columns
        return max(1, min(-(-self.compute_units // tiles), k // part))

    FEW_ROWS_LONG_K = 8192     # the shortest K that is cut for up to sixteen rows
    PENDING_SHORTEST_K = 512   # the shortest K that is cut when the parts may be left for the next norm
    SPLIT_K_FROM = 8192        # the shortest K that the tiled kernel cuts (shorter ones are the weight-streaming kernel's)

    EAGER_LIBRARY_WORK = 2 ** 30   # multiply-adds from which a product launched eagerly goes to the library
    capturing = False          # set while a graph is recorded (and in the run that warms it up): launches are free then
    LIBRARY_WEIGHT = 2 ** 21   # weight elements from which products of 17 to 64 rows go to the library
    GATED_LIBRARY_WEIGHT = 2 ** 24   # ... and the gated product (its activation then is a kernel of its own)
    SKINNY_ROWS = 64    # up to this many rows the weight-streaming kernel runs ...
    WIDE_OUTPUT = 32768  # ... unless there are more than 16 rows and this many output columns (the vocabulary
    #                      projection): there the rows' re-reading per tile of 16 columns costs more than tiling
    use_library_gemm = True

    def linear_silu_gate(self, x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor | None = None,
                         act: tuple | None = None) -> torch.Tensor:
        """out = silu(x @ Wg.T) * (x @ Wu.T) for weight = [Wg; Wu] of shape [2I, K]; out [M, I].  `act`: another
        gated activation than silu (see `silu_gate`).

        Few bfloat16 rows run in one kernel; otherwise the product and the gated activation are two."""
        _need(weight.dim() == 2 and weight.shape[0] % 2 == 0, "the joined gate and up matrix has an even row count")
        m, inner = x.shape[0], weight.shape[0] // 2
        if out is None:
            out = torch.empty((m, inner), dtype=x.dtype, device=x.device)
        _need(tuple(out.shape) == (m, inner) and out.dtype == x.dtype and out.is_contiguous(), "gated output shape")
        if act is not None and act != "gelu_tanh":
            return self.silu_gate(self.linear(x, weight), out, act=act)
        if (x.dtype == torch.bfloat16 and m <= self.SKINNY_ROWS and x.shape[1] % 8 == 0 and (m == 1 or x.stride(0) % 8 == 0)
                and not (self.use_library_gemm and m > self.FUSED_ROWS
                         and weight.shape[0] * weight.shape[1] >= self.GATED_LIBRARY_WEIGHT)):
            _need(x.is_cuda and weight.is_cuda and x.dim() == 2 and x.shape[1] == weight.shape[1], "linear shapes do not fit")
            _need(x.stride(1) == 1 and weight.is_contiguous() and weight.dtype == torch.bfloat16, "linear operands")
            k = x.shape[1]
            lda = x.stride(0) if m > 1 else k
            _need(k % 8 == 0 and lda % 8 == 0, "bfloat16 products need K and the row stride to be multiples of 8")
            _need(x.data_ptr() % 16 == 0 and weight.data_ptr() % 16 == 0, "operands must be 16-byte aligned")
            self._check(self.lib.ta_gemm_skinny_bf16(_ptr(x), lda, _ptr(weight), None, _ptr(out), inner, m, 2 * inner,
                                                     k, _BF16, 2 if act == "gelu_tanh" else 1, self.skinny_column_blocks,
                                                     self._stream()), "linear_silu_gate")
            return out
        return self.silu_gate(self.linear(x, weight), out, act=act)

    # ------------------------------------------------------- fused decode products
    FUSED_ROWS = 16
    use_fused_decode = True
    fused_rows = 0            # 0: the launcher picks the weight rows per workgroup (1..32; 16, 8, 4 with rotation) ...
    fused_waves = 0           # ... and how many waves share a tile's K (4, 8, 16)

    FUSED_LDS_BYTES = 140 * 1024     # what the norm prologue may take of a compute unit's 160 KB of LDS

    def can_fuse_decode(self, rows: int, dtype: torch.dtype, hidden: int = 0) -> bool:
        """Batches of few bfloat16 rows can run the products that take the norm, the rotation with the
        cache write, the gated activation and the residual add into the same kernel.  The norm prologue
        keeps sixteen normalised rows of `hidden` elements in LDS, which bounds `hidden`."""
        return (self.use_fused_decode and dtype == torch.bfloat16 and 0 < rows <= self.FUSED_ROWS
                and (not self.fold_norm(hidden) or 16 * (hidden + 8) * 2 <= self.FUSED_LDS_BYTES))

    FOLD_NORM_WIDTH = 2048    # up to this model width the decode products normalise their rows themselves

    def fold_norm(self, hidden: int) -> bool:
        """Whether the fused decode products should take the norm into their prologue: every workgroup then reads
        and normalises all rows again, which pays for narrow models (one kernel fewer) and costs more than the
        norm's own small kernel for wide ones."""
        return hidden <= self.FOLD_NORM_WIDTH

    def fused_norm_qkv_rope(self, residual, norm_weight, eps, weight, bias, positions, cos_sin, slots,
                            k_pages, v_pages, n_q: int, n_kv: int, head_dim: int) -> torch.Tensor:
        """q, k, v = rmsnorm(residual) @ weight.T + bias; q and k rotated; k and v stored into their pages
        (when `slots` is given); returns q [M, n_q * d] in bfloat16.  residual float32 [M, K]; or, with
        `norm_weight` None, `residual` holds the normalised rows in bfloat16 already."""
        _dev(norm_weight, weight, bias, positions, cos_sin, slots, k_pages, v_pages)
        _need(residual.is_cuda and residual.dim() == 2, "the rows must live on the GPU")
        m, k = residual.shape
        if norm_weight is None:
            _need(residual.dtype == torch.bfloat16 and residual.stride(1) == 1 and residual.stride(0) % 8 == 0
                  and residual.data_ptr() % 16 == 0, "normalised rows are bfloat16 with 16-byte aligned rows")
        else:
            _need(residual.dtype == torch.float32 and residual.is_contiguous() and norm_weight.dtype == torch.float32
                  and norm_weight.numel() == k, "the residual and the norm weight are float32")
        _need(weight.dtype == torch.bfloat16 and tuple(weight.shape) == ((n_q + 2 * n_kv) * head_dim, k),
              "the joined q/k/v matrix has the wrong shape")
        _need(k % 8 == 0 and head_dim % 32 == 0
              and (m <= self.FUSED_ROWS or (norm_weight is None and m <= self.SKINNY_ROWS)),
              "sizes the fused projection does not take")
        _need(positions.dtype == torch.int32 and positions.numel() == m, "positions must be int32 [M]")
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == weight.shape[0], "bias must be float32")
        if cos_sin is not None:
            _need(cos_sin.dtype == torch.float32 and cos_sin.shape[1] == head_dim, "cos_sin must be float32 [P, d]")
        page_size = 1
        if slots is not None:
            _need(slots.dtype == torch.int32 and slots.numel() == m, "slots must be int32 [M]")
            _need(k_pages.dtype == torch.bfloat16 and v_pages.dtype == torch.bfloat16, "pages must be bfloat16")
            page_size = self._page_size(k_pages, v_pages, n_kv, head_dim)
        q = torch.empty((m, n_q * head_dim), dtype=torch.bfloat16, device=residual.device)
        tail = (_ptr(weight), _ptr(bias), _ptr(q), _ptr(positions), _ptr(cos_sin), _ptr(slots),
                _ptr(k_pages if slots is not None else None), _ptr(v_pages if slots is not None else None),
                m, k, n_q, n_kv, head_dim, page_size, self.fused_rows, self.fused_waves, self._stream())
        if m > self.FUSED_ROWS:
            # 17 to 64 rows: the weight-streaming kernel with the same epilogue.
            status = self.lib.ta_gemm_skinny_qkv_rope(_ptr(residual), residual.stride(0), *tail[:-3], self._stream())
        elif norm_weight is None:
            status = self.lib.ta_fused_qkv_rope(_ptr(residual), residual.stride(0) if m > 1 else k, *tail)
        else:
            status = self.lib.ta_fused_norm_qkv_rope(_ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), *tail)
        self._check(status, "fused_norm_qkv_rope")
        return q

    ROPE_STORE_WEIGHT = 2 ** 22   # joined q/k/v matrices up to this many elements take the route below at 17-64 rows

    def can_rope_store(self, rows: int, dtype: torch.dtype, weight_elements: int = 0) -> bool:
        """Whether `fused_norm_qkv_rope` should take this many normalised bfloat16 rows: 17 to 64 go through the
        weight-streaming kernel, which then needs no rotation kernel after it.  That pays while the matrix is
        small (measured: 0.5B and 1.5B sizes); a big one is better off with the library's product and the
        rotation kernel."""
        return (self.use_fused_decode and dtype == torch.bfloat16 and self.FUSED_ROWS < rows <= self.SKINNY_ROWS
                and weight_elements <= self.ROPE_STORE_WEIGHT)

    def fused_norm_gated(self, residual, norm_weight, eps, weight, act: torch.Tensor | None = None) -> torch.Tensor:
        """silu(x @ Wg.T) * (x @ Wu.T) with x = rmsnorm(residual), weight = [Wg; Wu]; bfloat16 [M, I].  With
        `norm_weight` None, `residual` holds the normalised rows in bfloat16 already.  `act`: float32 [3] on the
        device (alpha, limit, shift) for the capped gated activation in place of silu (see `silu_gate`)."""
        _dev(norm_weight, weight, act)
        _need(act is None or (act.dtype == torch.float32 and act.numel() == 3), "act is float32 [3]")
        _need(residual.is_cuda and residual.dim() == 2, "the rows must live on the GPU")
        m, k = residual.shape
        if norm_weight is None:
            _need(residual.dtype == torch.bfloat16 and residual.stride(1) == 1 and residual.stride(0) % 8 == 0
                  and residual.data_ptr() % 16 == 0, "normalised rows are bfloat16 with 16-byte aligned rows")
        else:
            _need(residual.dtype == torch.float32 and residual.is_contiguous() and norm_weight.dtype == torch.float32
                  and norm_weight.numel() == k, "the residual and the norm weight are float32")
        _need(weight.dtype == torch.bfloat16 and weight.shape[1] == k and weight.shape[0] % 2 == 0, "gate/up matrix shape")
        _need(m <= self.FUSED_ROWS and k % 8 == 0, "sizes the fused product does not take")
        out = torch.empty((m, weight.shape[0] // 2), dtype=torch.bfloat16, device=residual.device)
        tail = (_ptr(weight), _ptr(out), m, weight.shape[0], k, self.fused_rows, self.fused_waves, _ptr(act), self._stream())
        if norm_weight is None:
            status = self.lib.ta_fused_gated(_ptr(residual), residual.stride(0) if m > 1 else k, *tail)
        else:
            status = self.lib.ta_fused_norm_gated(_ptr(residual), _ptr(norm_weight), ctypes.c_float(eps), *tail)
        self._check(status, "fused_norm_gated")
        return out

    def linear_add(self, x, weight, bias, residual) -> None:
        """residual += x @ weight.T (+ bias), in place, in float32.  x bfloat16 [M, K], M <= 16."""
        _dev(weight, bias, residual)
        _need(x.is_cuda and x.dim() == 2 and x.stride(1) == 1 and x.dtype == torch.bfloat16, "x must be bfloat16 rows")
        m, k = x.shape
        n = weight.shape[0]
        lda = x.stride(0) if m > 1 else k
        _need(weight.dtype == torch.bfloat16 and weight.shape[1] == k, "weight shape")
        _need(residual.dtype == torch.float32 and tuple(residual.shape) == (m, n), "the residual must be float32 [M, N]")
        _need(m <= self.FUSED_ROWS and k % 8 == 0 and lda % 8 == 0 and x.data_ptr() % 16 == 0, "sizes not taken")
        if bias is not None:
            _need(bias.dtype == torch.float32 and bias.numel() == n, "bias must be float32 [N]")
        self._check(self.lib.ta_fused_linear_residual(_ptr(x), lda, _ptr(weight), _ptr(bias), _ptr(residual), m, n, k,
                                                      self.fused_rows, self.fused_waves, self._stream()), "linear_add")

    # ------------------------------------------------------- several residual streams
    MAX_STREAMS = 16

    def embedding_streams(self, ids: torch.Tensor, table: torch.Tensor, positions: torch.Tensor,
                          rates: torch.Tensor | None, out: torch.Tensor) -> torch.Tensor:
        """out[t, s] = table[ids[t]] (+ the position vector of positions[t]: entry 2i sin(p rates[i]), entry 2i+1
        the cosine) for every stream s.  ids, positions int32 [T]; table [V, W]; rates float32 [W / 2] or None;
        out float32 [T, S, W]."""
        _dev(ids, table, positions, rates, out)
        n, (vocab, width) = ids.numel(), table.shape
        _need(ids.dtype == torch.int32 and positions.dtype == torch.int32 and positions.numel() == n, "ids, positions int32 [T]")
        _need(out.dtype == torch.float32 and out.dim() == 3 and out.shape[0] == n and out.shape[2] == width, "out float32 [T, S, W]")
        if rates is not None:
            _need(rates.dtype == torch.float32 and width % 2 == 0 and rates.numel() == width // 2, "rates float32 [W / 2]")
        self._check(self.lib.ta_embedding_streams(_ptr(ids), _ptr(table), _ptr(positions), _ptr(rates), _ptr(out), n, width,
                                                  vocab, out.shape[1], _code(table.dtype), self._stream()), "embedding_streams")
        return out

    fuses_single_shift = True     # `streams_step(shift=...)` exists here (steps of one token per request)

    def streams_step(self, streams: torch.Tensor, write, read: torch.Tensor, gain: torch.Tensor, eps: float,
                     out: torch.Tensor, rows: torch.Tensor | None = None, shift: tuple | None = None) -> torch.Tensor:
        """Apply a sub-layer's write to the streams and make the next normalised read, in one kernel.

        streams float32 [T, S, W].  `write` (or None): an object with y [T, W], mix float32 [S, S] (indexed [from,
        to]), out float32 [S], scale float32 [W] or None: x_t <- sum_s mix[s, t] x_s + out[t] * scale * y, stored
        back unless `rows` (int32 [R]) picks a subset.  Then u = sum_s read[s] x_s and
        out[i] = u / sqrt(mean(u^2) + eps) * gain[0], out [R or T, W] float32 or the dtype of y.
        `shift` = (mu float32 [W], state float32 [slots, W], ctx), for steps of one token per request: the row
        written is h + (state row - h) * mu (zeros for the state at position 0) and h becomes the state row."""
        _dev(streams, read, gain, out, rows)
        _need(streams.dtype == torch.float32 and streams.dim() == 3, "streams are float32 [T, S, W]")
        n_tokens, n_streams, width = streams.shape
        _need(n_streams <= self.MAX_STREAMS, f"at most {self.MAX_STREAMS} streams")
        _need(read.dtype == torch.float32 and read.numel() == n_streams and gain.dtype == torch.float32 and gain.numel() == 1,
              "read float32 [S], gain float32 [1]")
        n_rows = n_tokens if rows is None else rows.numel()
        _need(tuple(out.shape) == (n_rows, width), "the read has the wrong shape")
        if rows is not None:
            _need(rows.dtype == torch.int32 and shift is None, "rows must be int32 (and no shift over a subset)")
        y = mix = coef = scale = None
        y_code = _code(out.dtype)
        if write is not None:
            y, mix, coef, scale = write.y, write.mix, write.out, write.scale
            _dev(y, mix, coef, scale)
            _need(tuple(y.shape) == (n_tokens, width) and mix.dtype == torch.float32 and tuple(mix.shape) == (n_streams, n_streams)
                  and coef.dtype == torch.float32 and coef.numel() == n_streams, "the write does not fit the streams")
            _need(scale is None or (scale.dtype == torch.float32 and scale.numel() == width), "scale float32 [W]")
            y_code = _code(y.dtype)
        _need(out.dtype == torch.float32 or _code(out.dtype) == y_code, "the read is float32 or has the dtype of y")
        mu = state = entry_of_token = state_slots = positions = None
        if shift is not None:
            mu, state, ctx = shift
            entry_of_token, state_slots, positions = ctx.entry_of_token, ctx.state_slots, ctx.positions
            _dev(mu, state, entry_of_token, state_slots, positions)
            _need(mu.dtype == torch.float32 and mu.numel() == width and state.dtype == torch.float32 and state.dim() == 2
                  and state.shape[1] == width, "mu float32 [W], state float32 [slots, W]")
            _need(entry_of_token.numel() == n_tokens and positions.numel() == n_tokens, "the batch description does not fit")
        self._check(self.lib.ta_streams_step(_ptr(streams), _ptr(y), _ptr(mix), _ptr(coef), _ptr(scale), _ptr(read), _ptr(gain),
                                             ctypes.c_float(eps), _ptr(out), _ptr(rows), n_rows, width, n_streams, y_code,
                                             _code(out.dtype), _ptr(mu), _ptr(state), _ptr(entry_of_token),
                                             _ptr(state_slots), _ptr(positions), self._stream()), "streams_step")
        return out

    def token_shift(self, h: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
                    first_position: torch.Tensor, state_slots: torch.Tensor, entry_of_token: torch.Tensor,
                    out: torch.Tensor) -> torch.Tensor:
        """out[t] = h[t] + (before - h[t]) * mu, `before` = h[t - 1] within an entry's rows, the entry's state row for
        its first token (zeros if its first position is 0); the entry's last row of h becomes its state row.
        h float32 [T, W]; mu float32 [W]; state float32 [slots, W]; cu_q int32 [E + 1]; first_position, state_slots
        int32 [E]; entry_of_token int32 [T]; out [T, W]."""
        _dev(h, mu, state, cu_q, first_position, state_slots, entry_of_token, out)
        n_tokens, width = h.shape
        _need(h.dtype == torch.float32 and mu.dtype == torch.float32 and mu.numel() == width, "h float32 [T, W], mu float32 [W]")
        _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] == width, "state float32 [slots, W]")
        _need(tuple(out.shape) == (n_tokens, width) and entry_of_token.numel() == n_tokens, "token_shift shapes do not fit")
        _need(first_position.numel() == cu_q.numel() - 1 == state_slots.numel(), "one first position and slot per entry")
        self._check(self.lib.ta_token_shift(_ptr(h), _ptr(mu), _ptr(state), _ptr(cu_q), _ptr(first_position), _ptr(state_slots),
                                            _ptr(entry_of_token), _ptr(out), n_tokens, width, _code(out.dtype),
                                            self._stream()), "token_shift")
        return out

    # -------------------------------------------------------------- matrix memory
    MLSTM_CHUNKED_FROM = 48      # rows beyond one per entry from which the recurrence runs in chunks

    def mlstm_scan(self, qkvg: torch.Tensor, gates: torch.Tensor, state: torch.Tensor, cu_q: torch.Tensor,
                   first_position: torch.Tensor, state_slots: torch.Tensor, out: torch.Tensor,
                   heads: int, d: int, dv: int, cap: float) -> torch.Tensor:
        """The matrix-memory recurrence over every entry's rows, from and into the entries' state rows.

        qkvg [T, >= 2 heads d + heads dv]: q, k (heads of d) and v (heads of dv) side by side; gates float32
        [T, >= 2 heads]: pre-activations of the input and of the forget gate; state float32 [slots, heads d dv +
        heads d + heads] (C, n, m; an entry whose first position is 0 starts from zeros); out float32 [T, heads dv]."""
        _dev(qkvg, gates, state, cu_q, first_position, state_slots, out)
        n_tokens = qkvg.shape[0]
        _need(qkvg.shape[1] >= 2 * heads * d + heads * dv and d > 0 and dv > 0, "q, k, v do not fit the rows")
        _need(gates.dtype == torch.float32 and gates.shape[0] == n_tokens and gates.shape[1] >= 2 * heads, "gates float32 [T, 2 heads]")
        _need(state.dtype == torch.float32 and state.dim() == 2 and state.shape[1] >= heads * d * dv + heads * d + heads,
              "state rows are too short")
        _need(out.dtype == torch.float32 and tuple(out.shape) == (n_tokens, heads * dv), "out float32 [T, heads dv]")
        n_entries = cu_q.numel() - 1
        _need(first_position.numel() == n_entries == state_slots.numel(), "one first position and slot per entry")
        if n_tokens - n_entries >= self.MLSTM_CHUNKED_FROM or d > 256:
            # Portions of many rows: chunks of 64 tokens side by side, the state carried from chunk to chunk.  (Heads wider
            # than the 256 columns of n that the token-by-token kernels keep a thread each always go this way.)
            max_chunks = n_tokens // 64 + n_entries
            scratch = torch.empty(max_chunks * heads * (d * dv + d + 3), dtype=torch.float32, device=qkvg.device)
            self._check(self.lib.ta_mlstm_chunked(_ptr(qkvg), qkvg.shape[1], _ptr(gates), gates.shape[1], _ptr(state),
                                                  ctypes.c_long(state.shape[1]), _ptr(cu_q), _ptr(first_position),
                                                  _ptr(state_slots), _ptr(scratch), _ptr(out), n_entries, max_chunks, heads, d,
                                                  dv, ctypes.c_float(cap), _code(qkvg.dtype), self._stream()), "mlstm_chunked")
            return out
        coef = torch.empty((n_tokens, heads, 3), dtype=torch.float32, device=qkvg.device)
        self._check(self.lib.ta_mlstm_scan(_ptr(qkvg), qkvg.shape[1], _ptr(gates), gates.shape[1], _ptr(state),
                                           ctypes.c_long(state.shape[1]), _ptr(cu_q), _ptr(first_position), _ptr(state_slots),
                                           _ptr(coef), _ptr(out), n_entries, heads, d, dv, ctypes.c_float(cap),
                                           _code(qkvg.dtype), self._stream()), "mlstm_scan")
        return out

    def head_norm_gate(self, read: torch.Tensor, weight: torch.Tensor, gate_rows: torch.Tensor, gate_offset: int,
                       eps: float, heads: int, dv: int, out: torch.Tensor) -> torch.Tensor:
        """out[t, h] = read[t, h] / sqrt(mean(read[t, h]^2) + eps) * weight[h] * sigmoid(gate[t, h]), heads of dv; the gate
        lies in `gate_rows` from column `gate_offset` on.  read float32 [T, heads dv]; weight float32 [heads dv]."""
        _dev(read, weight, gate_rows, out)
        n_tokens = read.shape[0]
        _need(read.dtype == torch.float32 and read.shape[1] == heads * dv and weight.dtype == torch.float32
              and weight.numel() == heads * dv, "read float32 [T, heads dv], weight float32 [heads dv]")
        _need(gate_rows.shape[0] == n_tokens and gate_rows.shape[1] >= gate_offset + heads * dv and gate_rows.dtype == out.dtype
              and tuple(out.shape) == (n_tokens, heads * dv), "the gate's rows do not fit")
        self._check(self.lib.ta_head_norm_gate(_ptr(read), _ptr(weight), _ptr(gate_rows), gate_rows.shape[1], gate_offset,
                                               ctypes.c_float(eps), n_tokens, heads, dv, _ptr(out), _code(out.dtype),
                                               self._stream()), "head_norm_gate")
        return out

    # ------------------------------------------------------------------- sampling
    def argmax(self, logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """First maximum of each row.  logits float32 [B, V] -> int32 [B]."""
        _dev(logits, out)
        _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be float32 [B, V]")
        if out is None:
            out = torch.empty(logits.shape[0], dtype=torch.int32, device=logits.device)
        _need(out.dtype == torch.int32 and out.numel() == logits.shape[0], "argmax output must be int32 [B]")
        n_rows, vocab = logits.shape
        chunks = max(1, min(256, vocab // 2048, 2048 // max(1, n_rows)))
        partial_v = torch.empty((n_rows, chunks), dtype=torch.float32, device=logits.device)
        partial_i = torch.empty((n_rows, chunks), dtype=torch.int32, device=logits.device)
        self._check(self.lib.ta_argmax(_ptr(logits), _ptr(out), _ptr(partial_v), _ptr(partial_i), n_rows, vocab,
                                       chunks, self._stream()), "argmax")
        return out

    NEXT_STEP_GROUPS = 4          # cache groups `argmax_next_step` can advance

    def argmax_next_step(self, logits: torch.Tensor, token_ids: torch.Tensor, positions: torch.Tensor,
                         first_position: torch.Tensor, slots: list[torch.Tensor], block_tables: list[torch.Tensor],
                         page_size: int) -> torch.Tensor:
        """`argmax` for a decode step of one token per request (row i of the logits = request i), which also turns
        the step's description into the next step's, in place: the picked ids become `token_ids`, `positions` and
        `first_position` go up by one, and every cache group's `slots` are looked up for the new positions in its
        block table [B, width] (a position past the table's width takes the last entry; a page that is not there
        gives slot -1).  All int32 [B]."""
        _dev(logits, token_ids, positions, first_position, *slots, *block_tables)
        _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be float32 [B, V]")
        n_rows, vocab = logits.shape
        _need(len(slots) == len(block_tables) <= self.NEXT_STEP_GROUPS, "one table per group of slots, four at most")
        for t in (token_ids, positions, first_position, *slots):
            _need(t.dtype == torch.int32 and t.numel() == n_rows and t.is_contiguous(), "the description is int32 [B]")
        for table in block_tables:
            _need(table.dtype == torch.int32 and table.dim() == 2 and table.shape[0] == n_rows and table.shape[1] >= 1
                  and table.is_contiguous(), "block tables are int32 [B, width]")
        _need(page_size >= 1, "page size")
        out = torch.empty(n_rows, dtype=torch.int32, device=logits.device)
        chunks = max(1, min(256, vocab // 2048, 2048 // max(1, n_rows)))
        partial_v = torch.empty((n_rows, chunks), dtype=torch.float32, device=logits.device)
        partial_i = torch.empty((n_rows, chunks), dtype=torch.int32, device=logits.device)
        groups = []
        for g in range(self.NEXT_STEP_GROUPS):
            if g < len(slots):
                groups += [_ptr(slots[g]), _ptr(block_tables[g]), int(block_tables[g].shape[1])]
            else:
                groups += [_ptr(None), _ptr(None), 0]
        self._check(self.lib.ta_argmax_next_step(_ptr(logits), _ptr(out), _ptr(partial_v), _ptr(partial_i), n_rows, vocab,
                                                 chunks, _ptr(token_ids), _ptr(positions), _ptr(first_position),
                                                 int(page_size), len(slots), *groups, self._stream()), "argmax_next_step")
        return out

    def sample(self, logits: torch.Tensor, temperature: torch.Tensor, top_p: torch.Tensor, uniform: torch.Tensor,
               out: torch.Tensor | None = None, any_cut: bool = True) -> torch.Tensor:
        """Temperature / nucleus draw per row with the reference's rules (tokens by falling logit, lower
        index first among equals; the shortest prefix reaching top_p; the uniform number walks its mass).
        logits float32 [B, V]; temperature (> 0), top_p, uniform: float32 [B]; returns int32 [B].
        `any_cut=False` promises that no row has top_p < 1: the rounds that look for the nucleus's end are
        then not launched."""
        _dev(logits, temperature, top_p, uniform, out)
        _need(logits.dtype == torch.float32 and logits.dim() == 2, "logits must be float32 [B, V]")
        n_rows = logits.shape[0]
        for name, t in (("temperature", temperature), ("top_p", top_p), ("uniform", uniform)):
            _need(t.dtype == torch.float32 and t.numel() == n_rows, f"{name} must be float32 [B]")
        if out is None:
            out = torch.empty(n_rows, dtype=torch.int32, device=logits.device)
        _need(out.dtype == torch.int32 and out.numel() == n_rows, "sample output must be int32 [B]")
        workspace = torch.empty(max(1, n_rows) * self.lib.ta_sample_workspace_words(), dtype=torch.float32,
                                device=logits.device)
        self._check(self.lib.ta_sample(_ptr(logits), _ptr(temperature), _ptr(top_p), _ptr(uniform), _ptr(out),
                                       _ptr(workspace), n_rows, logits.shape[1], 1 if any_cut else 0, self._stream()),
                    "sample")
        return out


_OPS: Ops | None = None
_LOCK = threading.Lock()


def get_ops() -> Ops:
    """The loaded kernel library; builds it on first use if no built library is found."""
    global _OPS
    if _OPS is not None:
        return _OPS
    with _LOCK:
        if _OPS is None:
            if not torch.cuda.is_available():
                raise KernelError("tokenizer_amd runs on an AMD GPU through its HIP kernels; "
                                  "no GPU is visible and there is no CPU path")
            path = _build.find_library()
            if path is None:
                path = _build.build_library()
            _OPS = Ops(path)
    return _OPS


def default_scale(head_dim: int) -> float:
    return 1.0 / math.sqrt(head_dim)
