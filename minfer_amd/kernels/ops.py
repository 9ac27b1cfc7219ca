"""Python faces of the HIP kernels: each function checks its operands on the host (device,
type, shape, contiguity), then launches on torch's current stream.  Outputs are written
into tensors the caller allocated, so a captured step allocates nothing here except the
cached workspaces below.
"""
from __future__ import annotations

import ctypes
import sys
from ctypes import c_char_p, c_double, c_float, c_int, c_size_t, c_uint64, c_void_p
from typing import Dict, Optional, Tuple

import torch

from . import build, tuning
from ..cache.paged import v_page_shape

PAGE = 64          # tokens per cache page (MF_PAGE in csrc/common.h)
HAVE_PREFILL_ATTENTION = True
PREFILL_MAX_SHARES = 8  # workgroups that may take the pages of one block of queries of the prompt attention in turn
PREFILL_MIN_PAGES = 4   # ... each with at least this many pages
EPI_F32, EPI_ACC_F32, EPI_BF16, EPI_SWIGLU, EPI_XIELU = 0, 1, 2, 3, 4


class KernelError(RuntimeError):
    pass


_P = c_void_p
_PROTOTYPES = {
    "elementwise": {
        "mf_embed": [_P, c_int, _P, _P, c_int, c_int, c_int, _P],
        "mf_rmsnorm": [_P, _P, _P, _P, c_int, c_int, c_int, c_float, _P],
        "mf_rmsnorm_cols": [_P, c_int, _P, _P, c_int, c_int, c_int, c_float, _P],
        "mf_gather_rows": [_P, _P, _P, c_int, c_int, _P],
        "mf_swiglu": [_P, c_int, _P, c_int, c_int, c_int, _P],
        "mf_convert": [_P, c_int, _P, c_int, c_size_t, _P],
        "mf_rope_table": [_P, _P, c_int, c_int, c_double, c_double, _P],
        "mf_rope_kvwrite": [_P, _P, _P, _P, _P, _P, c_int, _P, _P, _P, c_int, c_int, c_int, c_int,
                            c_int, c_int, _P],
        "mf_rope_inplace": [_P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_fill_normal": [_P, c_int, c_size_t, c_uint64, c_float, c_int, _P],
        "mf_group_rmsnorm": [_P, _P, _P, _P, c_int, c_int, _P, c_int, c_int, c_int, c_float, _P],
        "mf_xielu": [_P, _P, c_int, c_size_t, c_float, c_float, _P],
        "mf_rope_table_freqs": [_P, _P, _P, c_int, c_int, c_double, _P],
        "mf_rope_pairs_inplace": [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_embed_pos": [_P, _P, c_int, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_gelu_tanh": [_P, _P, c_int, c_size_t, _P],
        "mf_softcap": [_P, c_float, c_size_t, _P],
        "mf_weighted_sum": [_P, c_int, c_int, _P, _P, _P, c_int, c_int, _P],
        "mf_add_rows": [_P, _P, c_size_t, _P],
    },
    "linear_attention": {
        "mf_la_chunk": [],
        "mf_lightning_scan": [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_lightning_scan_chunked": [_P, _P, c_int, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_gated_rmsnorm": [_P, _P, c_int, _P, _P, c_int, c_int, c_int, c_float, _P],
    },
    "attn_capped": {
        "mf_qkv_conv_prep": [_P, _P, c_int, _P, _P, _P, _P, _P, _P, _P, c_int, c_float, _P, _P, _P, c_int, _P, _P, _P,
                             c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_capped_attn": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_float, c_float, c_int, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, _P],
        "mf_rope_half_inplace": [_P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, _P],
    },
    "attn_capped_mfma": {
        "mf_capped_mfma": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_int, c_float, c_float, c_int, c_int, _P, _P, c_int, _P, c_int, _P],
    },
    "attn_normed": {
        "mf_qk_norm_prep": [_P, _P, _P, c_float, c_int, _P, _P, _P, _P, c_int, c_int, c_int, _P, _P, c_int, _P, c_int, _P, _P, _P,
                            c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_unrotate": [_P, c_int, _P, _P, _P, c_int, c_int, c_int, c_float, _P],
    },
    "gated_recurrence": {
        "mf_gr_chunk": [],
        "mf_gated_scan": [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_gated_scan_chunked": [_P, _P, _P, c_int, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
        "mf_head_rmsnorm": [_P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_float, _P],
    },
    "moe": {
        "mf_moe_route": [_P, c_int, _P, _P, c_int, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P, c_int, c_float, _P],
        "mf_moe_act": [_P, _P, _P, c_int, c_int, c_int, c_int, c_float, c_int, _P],
        "mf_moe_sparse": [_P, _P, _P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                          _P],
        "mf_moe_group": [_P, c_int, c_int, _P, _P, _P],
        "mf_moe_gather": [_P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, _P],
        "mf_moe_combine": [_P, _P, _P, _P, _P, _P, c_int, c_int, c_int, c_int, _P],
    },
    "recurrence": {
        "mf_mingru_scan": [_P, _P, _P, _P, _P, c_int, c_int, c_int, _P],
        "mf_mingru_scan_chunked": [_P, _P, c_int, _P, _P, _P, _P, _P, c_int, c_int, c_int, _P],
        "mf_scan_chunk": [],
    },
    "attn_latent": {
        "mf_latent_prep": [_P, c_int, c_int, c_int, c_int, _P, c_int, _P, c_float, _P, _P, c_int, _P, _P, _P, c_int, _P, _P,
                           _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_headwise_linear": [_P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_headwise_mfma": [_P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_latent_attn": [_P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                           c_int, c_int, _P],
    },
    "attn_latent_mfma": {
        "mf_latent_mfma": [_P, _P, _P, c_int, _P, _P, _P, _P, c_int, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                           c_float, c_int, c_int, c_int, _P],
    },
    "probe": {
        "mf_probe_read": [_P, c_size_t, _P, c_int, _P],
        "mf_probe_mfma": [c_int, _P, c_int, _P],
    },
    "host_random": {
        "mf_fill_normal_host": [_P, c_int, c_size_t, c_uint64, c_float, c_int, c_int],
    },
    "gemm_f32": {
        "mf_gemm_f32": [_P, c_int, _P, c_int, _P, _P, c_int, c_int, c_int, c_int, c_int, _P],
    },
    "gemm_bf16": {
        "mf_gemm_bf16": [_P, c_int, _P, c_int, _P, _P, c_int, c_int, c_int, c_int, c_int, c_int, _P],
        "mf_gemm_bf16_splitk": [_P, c_int, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int, c_int, c_int,
                                c_int, _P],
        "mf_gemm_bf16_skinny": [_P, c_int, _P, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int,
                                c_int, c_int, _P],
        "mf_gemm_bf16_normed": [_P, c_int, _P, _P, c_float, _P, _P, c_int, _P, _P, c_int, c_int, c_int, c_int,
                                c_int, _P],
        "mf_gemm_bf16_skinny_fused": [_P, c_int, _P, _P, c_int, _P, _P, c_int, _P, c_int, c_int, c_int, c_int,
                                      c_int, c_int, _P, c_int, c_float, _P, _P, _P, c_int, _P],
        "mf_gemm_bf16_plan": [c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_char_p, c_int],
        "mf_gemm_bf16_tile_plan": [c_int, c_int, c_int, c_int, c_int, c_int, _P],
    },
    "attn_tokens_f32": {
        "mf_attn_tokens_f32": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                               c_float, c_int, c_int, c_int, _P],
    },
    "attn_decode_bf16": {
        "mf_attn_decode_bf16": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int, c_int,
                                c_float, c_int, c_int, c_int, _P],
        "mf_attn_decode_rope_bf16": [_P, _P, _P, _P, _P, _P, c_int, _P, _P, _P, _P, c_int, c_int, c_int,
                                     c_int, c_float, c_int, c_int, c_int, c_int, _P],
    },
    "attn_prefill_bf16": {
        "mf_attn_prefill_bf16": [_P, _P, _P, _P, c_int, _P, _P, _P, _P, _P, _P, _P, c_int, _P, c_int, c_int, c_int,
                                 c_int, c_int, c_int, c_float, c_int, _P],
        "mf_attn_prefill_part_floats": [c_int],
        "mf_attn_prefill_rows": [c_int],
        "mf_attn_prefill_per_cu": [c_int],
    },
    "sampling": {
        "mf_argmax": [_P, c_int, c_int, c_int, _P, _P, c_int, _P],
        "mf_sample": [_P, c_int, c_int, c_int, c_float, _P, _P, _P, _P, _P],
        "mf_penalties": [_P, c_int, c_int, c_int, _P, c_int, _P, c_float, c_float, c_float, _P],
        "mf_top_k": [_P, c_int, c_int, c_int, c_int, _P],
        "mf_top_p": [_P, c_int, c_int, c_int, c_float, _P],
        "mf_sample_filtered": [_P, c_int, c_int, c_int, c_int, c_float, c_float, _P, _P, _P, _P, _P, _P],
        "mf_advance": [_P, _P, _P, _P, c_int, _P, c_int, _P, _P, _P],
    },
}
_functions: Dict[str, object] = {}


def _fn(lib: str, name: str, variant: Optional[str] = None):
    """`variant`: the name of a sized variant of `lib` (`build.variant`), whose functions have the
    prototypes of `lib`."""
    key = name if variant is None else f"{variant}:{name}"
    f = _functions.get(key)
    if f is None:
        f = getattr(build.load(variant or lib), name)
        f.argtypes = _PROTOTYPES[lib][name]
        f.restype = c_int
        _functions[key] = f
    return f


def _stream() -> c_void_p:
    return c_void_p(torch.cuda.current_stream().cuda_stream)


def _check(rc: int, what: str) -> None:
    """Raises on a launch error.  With MF_DEBUG_SYNC the stream is synchronised after every launch,
    so a fault inside a kernel is reported here, under the name of the launch that caused it
    (the reference's debug_sync, src/cuda.rs:378-395 of yusiwen/minfer)."""
    if rc != 0:
        raise KernelError(f"{what}: HIP error {rc}"
                          + (" (invalid argument: a size the kernel does not take)" if rc == 1 else ""))
    if _trace is not None:
        ev = torch.cuda.Event(enable_timing=True)
        ev.record()
        _trace.append((what, ev))
    if tuning.DEBUG_SYNC and not torch.cuda.is_current_stream_capturing():
        try:
            torch.cuda.current_stream().synchronize()
        except RuntimeError as e:
            raise KernelError(f"{what}: failed on the device: {e}") from None
        print(f"[minfer_amd] {what} OK", file=sys.stderr, flush=True)


def _ptr(t: Optional[torch.Tensor]) -> c_void_p:
    return c_void_p(0 if t is None else t.data_ptr())


# ------------------------------------------------------------------ per-launch timing
_trace: Optional[list] = None


def start_trace() -> None:
    """From here on every launch is followed by an event on the stream; `stop_trace` turns them
    into (launch name, microseconds) pairs.  The time of a launch is the time between the event
    behind the launch before it and its own, so the GPU must not run dry in between: queue
    enough work first (`probe_mfma`) that the host stays ahead."""
    global _trace
    first = torch.cuda.Event(enable_timing=True)
    first.record()
    _trace = [("", first)]


def stop_trace():
    global _trace
    events, _trace = _trace or [], None
    if len(events) < 2:
        return []
    events[-1][1].synchronize()
    return [(name, events[i - 1][1].elapsed_time(ev) * 1e3) for i, (name, ev) in enumerate(events) if i]


def _need(t: torch.Tensor, name: str, dtype=None, shape=None) -> None:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise KernelError(f"{name}: must be a tensor on the GPU (there is no CPU path)")
    if not t.is_contiguous():
        raise KernelError(f"{name}: must be contiguous, got strides {t.stride()} for shape {tuple(t.shape)}")
    if dtype is not None:
        ok = t.dtype in dtype if isinstance(dtype, (tuple, list)) else t.dtype == dtype
        if not ok:
            raise KernelError(f"{name}: dtype {t.dtype}, expected {dtype}")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise KernelError(f"{name}: shape {tuple(t.shape)}, expected {tuple(shape)}")


def _is_bf16(t: torch.Tensor) -> int:
    return 1 if t.dtype == torch.bfloat16 else 0


_FLOATS = (torch.float32, torch.bfloat16)

# ------------------------------------------------------------------ workspaces
# Scratch buffers are shared by all callers and replaced by larger ones on demand.  A captured
# graph holds the addresses of the buffers that were current when it was captured, so an outgrown
# buffer must stay allocated while such a graph may still be replayed.  One rule, kept here: whoever
# captures ops calls takes a `GraphLease` right after the capture and gives it back when the
# graph is dropped (`lease_graph`, `release_graph`); a buffer that is replaced is kept while any
# lease is older than its replacement, and freed otherwise.  `lease.stale()` tells an owner that
# a buffer was replaced since its capture: it may capture again (and so let the old one go), or go
# on replaying, which stays safe.
_workspaces: Dict[Tuple[str, int], torch.Tensor] = {}
_counters: Dict[Tuple[str, int], torch.Tensor] = {}
_workspace_generation = 0
_retired: list = []                  # (generation in which the buffer was last current, buffer)
_leases: Dict[int, "GraphLease"] = {}
_next_lease = 0


def _device_index(device) -> int:
    dev = torch.device(device)
    if dev.type != "cuda":
        return -1
    return dev.index if dev.index is not None else torch.cuda.current_device()


class GraphLease:
    """Held by the owner of a captured graph for as long as the graph may be replayed."""

    def __init__(self, token: int, generation: int):
        self.token, self.generation = token, generation

    def stale(self) -> bool:
        """A buffer whose address the graph may hold has been replaced since the capture."""
        return self.generation != _workspace_generation


def lease_graph() -> GraphLease:
    """To be called right after a capture that recorded ops calls."""
    global _next_lease
    _next_lease += 1
    lease = _leases[_next_lease] = GraphLease(_next_lease, _workspace_generation)
    return lease


def release_graph(lease: Optional[GraphLease]) -> None:
    """The graph is gone: buffers that only it could still address are freed."""
    if lease is not None and _leases.pop(lease.token, None) is not None:
        _drop_unreachable()


def _drop_unreachable() -> None:
    oldest = min((l.generation for l in _leases.values()), default=None)
    _retired[:] = [(g, b) for g, b in _retired if oldest is not None and oldest <= g]


def _retire(buffer: torch.Tensor) -> None:
    """`buffer` is being replaced: the generation moves on, and the buffer stays allocated if a
    leased graph was captured while it was current."""
    global _workspace_generation
    _retired.append((_workspace_generation, buffer))
    _workspace_generation += 1
    _drop_unreachable()


def workspace(tag: str, n_floats: int, device) -> torch.Tensor:
    """A float32 scratch tensor of at least n_floats, kept per (tag, device) and replaced by one at
    least twice as large when it is outgrown.  Kernels that use one run in stream order, so sharing
    it is safe."""
    key = (tag, _device_index(device))
    w = _workspaces.get(key)
    if w is None or w.numel() < n_floats:
        if w is not None:
            _retire(w)
            n_floats = max(n_floats, 2 * w.numel())
        w = torch.empty(max(n_floats, 1 << 16), dtype=torch.float32, device=device)
        _workspaces[key] = w
    return w


def _zeroed_counters(tag: str, n: int, device) -> torch.Tensor:
    """int32 counters for kernels whose workgroups count themselves in and leave the counters at
    zero again: zero when made, kept per (tag, device), replaced (see above) when more are needed."""
    key = (tag, _device_index(device))
    c = _counters.get(key)
    if c is None or c.numel() < n:
        if c is not None:
            _retire(c)
            n = max(n, 2 * c.numel())
        c = torch.zeros(max(n, 1024), dtype=torch.int32, device=torch.device(device))
        _counters[key] = c
    return c


def workspace_generation() -> int:
    return _workspace_generation


def note_replaced_buffer(old: Optional[torch.Tensor] = None) -> None:
    """For any other buffer whose address a captured graph may hold (a rotation table that was
    rebuilt longer): `old` is treated like an outgrown workspace."""
    _retire(old if old is not None else torch.empty(0))


# ------------------------------------------------------------------ element-wise
def embed(table: torch.Tensor, ids: torch.Tensor, out: torch.Tensor) -> None:
    _need(table, "embed.table", _FLOATS)
    _need(ids, "embed.ids", torch.int32)
    n, d = ids.numel(), table.shape[1]
    _need(out, "embed.out", torch.float32, (n, d))
    _check(_fn("elementwise", "mf_embed")(_ptr(table), _is_bf16(table), _ptr(ids), _ptr(out), n, d,
                                           table.shape[0], _stream()), "embed")


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out: torch.Tensor,
            row_idx: Optional[torch.Tensor] = None, cols: Optional[int] = None) -> None:
    """out = x / sqrt(mean(x^2) + eps) * weight, row by row (row r reads x[row_idx[r]] where given).  `cols`: the norm
    is taken over the first `cols` values of x's longer rows (the front of a product's stacked output)."""
    _need(x, "rmsnorm.x", torch.float32)
    if cols is not None and cols != x.shape[-1]:
        rows = x.shape[0]
        if row_idx is not None or not 1 <= cols < x.shape[1]:
            raise KernelError(f"rmsnorm: the first {cols} values of rows of {x.shape[1]}, with a row list or not")
        _need(out, "rmsnorm.out", _FLOATS, (rows, cols))
        if weight is not None:
            _need(weight, "rmsnorm.weight", torch.float32, (cols,))
        _check(_fn("elementwise", "mf_rmsnorm_cols")(_ptr(x), x.shape[1], _ptr(weight), _ptr(out), _is_bf16(out), rows, cols,
                                                      float(eps), _stream()), "rmsnorm")
        return
    d = x.shape[-1]
    rows = out.shape[0]
    _need(out, "rmsnorm.out", _FLOATS, (rows, d))
    if weight is not None:
        _need(weight, "rmsnorm.weight", torch.float32, (d,))
    if row_idx is not None:
        _need(row_idx, "rmsnorm.row_idx", torch.int32, (rows,))
    elif x.shape[0] != rows:
        raise KernelError(f"rmsnorm: x has {x.shape[0]} rows, out has {rows}")
    _check(_fn("elementwise", "mf_rmsnorm")(_ptr(x), _ptr(row_idx), _ptr(weight), _ptr(out),
                                             _is_bf16(out), rows, d, float(eps), _stream()), "rmsnorm")


def gather_rows(x: torch.Tensor, idx: torch.Tensor, out: torch.Tensor) -> None:
    _need(x, "gather_rows.x", torch.float32)
    _need(idx, "gather_rows.idx", torch.int32)
    _need(out, "gather_rows.out", torch.float32, (idx.numel(), x.shape[1]))
    _check(_fn("elementwise", "mf_gather_rows")(_ptr(x), _ptr(idx), _ptr(out), idx.numel(),
                                                 x.shape[1], _stream()), "gather_rows")


def swiglu(gate_up: torch.Tensor, out: torch.Tensor) -> None:
    _need(gate_up, "swiglu.gate_up", _FLOATS)
    rows, two_nf = gate_up.shape
    if two_nf % 2:
        raise KernelError(f"swiglu: gate_up has an odd width {two_nf}")
    _need(out, "swiglu.out", _FLOATS, (rows, two_nf // 2))
    if _is_bf16(gate_up) and not _is_bf16(out):
        raise KernelError("swiglu: bfloat16 input with float32 output is not provided")
    _check(_fn("elementwise", "mf_swiglu")(_ptr(gate_up), _is_bf16(gate_up), _ptr(out), _is_bf16(out),
                                            rows, two_nf // 2, _stream()), "swiglu")


def convert(src: torch.Tensor, dst: torch.Tensor) -> None:
    _need(src, "convert.src", _FLOATS)
    _need(dst, "convert.dst", _FLOATS)
    if src.numel() != dst.numel() or src.dtype == dst.dtype:
        raise KernelError("convert: needs equal sizes and different types")
    _check(_fn("elementwise", "mf_convert")(_ptr(src), _is_bf16(src), _ptr(dst), _is_bf16(dst),
                                             src.numel(), _stream()), "convert")


def fill_normal(out: torch.Tensor, seed: int, std: float, round_bf16: bool = True) -> None:
    """N(0, std) values that depend on (seed, index) only, the same bits as `fill_normal_host`
    gives.  `round_bf16`: a float32 tensor gets values that bfloat16 represents."""
    _need(out, "fill_normal.out", _FLOATS)
    _check(_fn("elementwise", "mf_fill_normal")(_ptr(out), _is_bf16(out), out.numel(),
                                                 seed & 0xFFFFFFFFFFFFFFFF, float(std), 1 if round_bf16 else 0,
                                                 _stream()), "fill_normal")


def fill_normal_host(out: torch.Tensor, seed: int, std: float, round_bf16: bool = True, threads: int = 0) -> None:
    """The same fill into a CPU tensor (host code only; no GPU is touched)."""
    import os
    if not isinstance(out, torch.Tensor) or out.is_cuda or not out.is_contiguous() or out.dtype not in _FLOATS:
        raise KernelError("fill_normal_host: needs a contiguous float32 or bfloat16 tensor on the CPU")
    threads = threads or max(1, min(16, os.cpu_count() or 1))
    rc = _fn("host_random", "mf_fill_normal_host")(c_void_p(out.data_ptr()), _is_bf16(out), out.numel(),
                                                    seed & 0xFFFFFFFFFFFFFFFF, float(std),
                                                    1 if round_bf16 else 0, threads)
    if rc != 0:
        raise KernelError(f"fill_normal_host: error {rc}")


def rope_table(n_pos: int, half: int, theta: float, freq_scale: float, device):
    cs = torch.empty((n_pos, half), dtype=torch.float32, device=device)
    sn = torch.empty((n_pos, half), dtype=torch.float32, device=device)
    _need(cs, "rope_table.out")
    _check(_fn("elementwise", "mf_rope_table")(_ptr(cs), _ptr(sn), n_pos, half, float(theta),
                                                float(freq_scale), _stream()), "rope_table")
    return cs, sn


def rope_inplace(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                 n_rot_heads: int, n_heads_total: int, head_dim: int) -> None:
    """The half-split rotation alone: the first `n_rot_heads` heads of every token's
    `[n_heads_total][head_dim]` row of 32-bit values are rotated in place."""
    n_tok = positions.numel()
    _need(qkv, "rope_inplace.qkv", torch.float32, (n_tok, n_heads_total * head_dim))
    _need(cos, "rope_inplace.cos", torch.float32)
    _need(sin, "rope_inplace.sin", torch.float32, tuple(cos.shape))
    if cos.shape[1] != head_dim // 2 or head_dim % 2 or n_rot_heads > n_heads_total:
        raise KernelError(f"rope_inplace: table {tuple(cos.shape)}, head_dim {head_dim}, {n_rot_heads} of {n_heads_total} heads")
    _need(positions, "rope_inplace.positions", torch.int32, (n_tok,))
    _check(_fn("elementwise", "mf_rope_inplace")(_ptr(qkv), _ptr(cos), _ptr(sin), _ptr(positions), n_tok,
                                                  n_rot_heads, n_heads_total, head_dim, _stream()), "rope_inplace")


def rope_kvwrite(qkv: torch.Tensor, cos: Optional[torch.Tensor], sin: Optional[torch.Tensor],
                 positions: torch.Tensor, seq_of_tok: torch.Tensor, page_table: torch.Tensor, q_out: torch.Tensor,
                 kcache: Optional[torch.Tensor], vcache: Optional[torch.Tensor], n_heads: int,
                 n_kv_heads: int, head_dim: int, write_kv: bool = True) -> None:
    """Rotates q and k, and stores k and v of the tokens at their positions in the cache pages
    (`v_page_shape` says how V lies in a page).  Without tables (cos and sin None) nothing is
    rotated: q is rounded into q_out and k, v are stored as they come."""
    n_tok = positions.numel()
    _need(qkv, "rope.qkv", torch.float32, (n_tok, (n_heads + 2 * n_kv_heads) * head_dim))
    if (cos is None) != (sin is None):
        raise KernelError("rope: cos and sin come together or not at all")
    if cos is not None:
        _need(cos, "rope.cos", torch.float32)
        _need(sin, "rope.sin", torch.float32, tuple(cos.shape))
        if cos.shape[1] != head_dim // 2:
            raise KernelError(f"rope: table has {cos.shape[1]} frequencies, head_dim {head_dim} needs {head_dim // 2}")
    _need(positions, "rope.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "rope.seq_of_tok", torch.int32, (n_tok,))
    _need(page_table, "rope.page_table", torch.int32)
    _need(q_out, "rope.q_out", _FLOATS, (n_tok, n_heads * head_dim))
    if write_kv:
        _need_caches("rope", kcache, vcache, q_out.dtype, n_kv_heads, head_dim)
    _check(_fn("elementwise", "mf_rope_kvwrite")(
        _ptr(qkv), _ptr(cos), _ptr(sin), _ptr(positions), _ptr(seq_of_tok), _ptr(page_table),
        page_table.shape[1], _ptr(q_out), _ptr(kcache if write_kv else None),
        _ptr(vcache if write_kv else None), _is_bf16(q_out), n_tok, n_heads, n_kv_heads, head_dim,
        1 if write_kv else 0, _stream()), "rope_kvwrite")


# ------------------------------------------------------------------ norm in groups, xIELU, frequency tables
def group_rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], eps: float, groups: int, out: torch.Tensor,
                  row_idx: Optional[torch.Tensor] = None, add: bool = False,
                  cast_out: Optional[torch.Tensor] = None) -> None:
    """The RMS norm taken over `groups` equal consecutive parts of each row, times `weight`.
    `out` gets the normed rows (run type); with `add` they are added into the float32 `out` instead
    (a residual stream taking a branch's normed result), and `cast_out` (bfloat16) then also gets the
    new rows rounded.  `x` and `out` may be the same tensor."""
    _need(x, "group_rmsnorm.x", torch.float32)
    d = x.shape[-1]
    rows = out.shape[0]
    _need(out, "group_rmsnorm.out", torch.float32 if add else _FLOATS, (rows, d))
    if groups < 1 or d % groups:
        raise KernelError(f"group_rmsnorm: {d} values do not split into {groups} equal parts")
    if weight is not None:
        _need(weight, "group_rmsnorm.weight", torch.float32, (d,))
    if row_idx is not None:
        _need(row_idx, "group_rmsnorm.row_idx", torch.int32, (rows,))
    elif x.shape[0] != rows:
        raise KernelError(f"group_rmsnorm: x has {x.shape[0]} rows, out has {rows}")
    if cast_out is not None:
        _need(cast_out, "group_rmsnorm.cast_out", torch.bfloat16, (rows, d))
    _check(_fn("elementwise", "mf_group_rmsnorm")(_ptr(x), _ptr(row_idx), _ptr(weight), _ptr(out), _is_bf16(out),
                                                   1 if add else 0, _ptr(cast_out), rows, d, int(groups), float(eps),
                                                   _stream()), "group_rmsnorm")


def xielu(x: torch.Tensor, out: torch.Tensor, a_pos: float, a_neg: float) -> None:
    """out = a_pos x^2 + x/2 where x > 0, a_neg (e^x - 1 - x) + x/2 elsewhere; x float32, out run type."""
    _need(x, "xielu.x", torch.float32)
    _need(out, "xielu.out", _FLOATS, tuple(x.shape))
    _check(_fn("elementwise", "mf_xielu")(_ptr(x), _ptr(out), _is_bf16(out), x.numel(), float(a_pos), float(a_neg),
                                           _stream()), "xielu")


def rope_table_freqs(n_pos: int, freqs, magnitude: float, device):
    """(cos, sin) float32 `[n_pos][len(freqs)]` of position * freqs[i], both times `magnitude`;
    the frequencies are given in double and the angles are formed in double on the device."""
    f = torch.tensor([float(v) for v in freqs], dtype=torch.float64).to(device)
    half = f.numel()
    cs = torch.empty((n_pos, half), dtype=torch.float32, device=device)
    sn = torch.empty((n_pos, half), dtype=torch.float32, device=device)
    _need(cs, "rope_table_freqs.out")
    _check(_fn("elementwise", "mf_rope_table_freqs")(_ptr(cs), _ptr(sn), _ptr(f), n_pos, half, float(magnitude),
                                                      _stream()), "rope_table_freqs")
    return cs, sn


def rope_pairs_inplace(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                       n_rot_heads: int, n_heads_total: int, head_dim: int) -> None:
    """The rotation in neighbouring pairs alone: values (2i, 2i+1), i below the tables' width, of the
    first `n_rot_heads` heads of every token's `[n_heads_total][head_dim]` row of 32-bit values are
    rotated in place; the rest of a head passes unchanged."""
    n_tok = positions.numel()
    _need(qkv, "rope_pairs_inplace.qkv", torch.float32, (n_tok, n_heads_total * head_dim))
    _need(cos, "rope_pairs_inplace.cos", torch.float32)
    _need(sin, "rope_pairs_inplace.sin", torch.float32, tuple(cos.shape))
    if 2 * cos.shape[1] > head_dim or n_rot_heads > n_heads_total:
        raise KernelError(f"rope_pairs_inplace: table {tuple(cos.shape)}, head_dim {head_dim}, "
                          f"{n_rot_heads} of {n_heads_total} heads")
    _need(positions, "rope_pairs_inplace.positions", torch.int32, (n_tok,))
    _check(_fn("elementwise", "mf_rope_pairs_inplace")(_ptr(qkv), _ptr(cos), _ptr(sin), _ptr(positions), n_tok,
                                                        n_rot_heads, n_heads_total, head_dim, cos.shape[1],
                                                        _stream()), "rope_pairs_inplace")


# ------------------------------------------------------------------ recurrences

# ------------------------------------------------------------------ table row plus position row, gelu, weighted sums
def embed_pos(table: torch.Tensor, pos_table: torch.Tensor, ids: torch.Tensor, positions: torch.Tensor,
              out: torch.Tensor) -> None:
    """out[r] = table[ids[r]] + pos_table[positions[r]], added in 32-bit."""
    _need(table, "embed_pos.table", _FLOATS)
    _need(pos_table, "embed_pos.pos_table", table.dtype)
    n, d = ids.numel(), table.shape[1]
    if pos_table.dim() != 2 or pos_table.shape[1] != d:
        raise KernelError(f"embed_pos: position table {tuple(pos_table.shape)} for rows of {d}")
    _need(ids, "embed_pos.ids", torch.int32)
    _need(positions, "embed_pos.positions", torch.int32, (n,))
    _need(out, "embed_pos.out", torch.float32, (n, d))
    _check(_fn("elementwise", "mf_embed_pos")(_ptr(table), _ptr(pos_table), _is_bf16(table), _ptr(ids), _ptr(positions),
                                               _ptr(out), n, d, table.shape[0], pos_table.shape[0], _stream()), "embed_pos")


def gelu_tanh(x: torch.Tensor, out: torch.Tensor) -> None:
    """out = 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) from 32-bit values, rounded once."""
    _need(x, "gelu_tanh.x", torch.float32)
    _need(out, "gelu_tanh.out", _FLOATS, tuple(x.shape))
    _check(_fn("elementwise", "mf_gelu_tanh")(_ptr(x), _ptr(out), _is_bf16(out), x.numel(), _stream()), "gelu_tanh")


def softcap(x: torch.Tensor, cap: float) -> None:
    """x <- cap tanh(x / cap), in place, 32-bit."""
    _need(x, "softcap.x", torch.float32)
    if not cap > 0:
        raise KernelError(f"softcap: cap {cap} must be positive")
    _check(_fn("elementwise", "mf_softcap")(_ptr(x), float(cap), x.numel(), _stream()), "softcap")


def weighted_sum(buffers, weights: torch.Tensor, out: torch.Tensor, row_idx: Optional[torch.Tensor] = None,
                 n_indexed: int = 0) -> None:
    """out[r] = sum_j weights[j] buffers[j][row(j, r)], added in the order of j in 32-bit.  The first
    `n_indexed` buffers are read at row `row_idx[r]`, the others at row r."""
    n = len(buffers)
    rows, d = out.shape
    _need(out, "weighted_sum.out", torch.float32)
    _need(weights, "weighted_sum.weights", torch.float32, (n,))
    if n_indexed:
        _need(row_idx, "weighted_sum.row_idx", torch.int32, (rows,))
    for j, b in enumerate(buffers):
        _need(b, f"weighted_sum.buffers[{j}]", torch.float32)
        if b.shape[1] != d or (j >= n_indexed and b.shape[0] != rows):
            raise KernelError(f"weighted_sum: buffer {j} is {tuple(b.shape)}, out is {tuple(out.shape)}")
        if rows and b.data_ptr() == out.data_ptr():
            raise KernelError("weighted_sum: the output is one of the inputs")
    if rows == 0:
        return
    ptrs = (c_void_p * n)(*[b.data_ptr() for b in buffers])
    _check(_fn("elementwise", "mf_weighted_sum")(ptrs, n, int(n_indexed), _ptr(row_idx if n_indexed else None),
                                                  _ptr(weights), _ptr(out), rows, d, _stream()), "weighted_sum")


def add_rows(h: torch.Tensor, x: torch.Tensor) -> None:
    """h += x, both float32 of one shape."""
    _need(h, "add_rows.h", torch.float32)
    _need(x, "add_rows.x", torch.float32, tuple(h.shape))
    _check(_fn("elementwise", "mf_add_rows")(_ptr(h), _ptr(x), h.numel(), _stream()), "add_rows")


# ------------------------------------------------------------------ gated linear recurrence
GR_CHUNK = 64            # tokens of a chunk of the chunked form (MF_GR_CHUNK in csrc/gated_recurrence.hip)


def gr_chunks(host_new):
    """The chunk table of the chunked gated recurrence for a step whose sequences bring `host_new` tokens:
    int32 `[4][n_chunks]` (first token, tokens, sequence, last of its sequence or not) followed by `[n_seqs + 1]`
    first chunks; and the number of chunks."""
    t0s, ns, seqs, lasts, firsts = [], [], [], [], [0]
    t = 0
    for b, n in enumerate(host_new):
        for c0 in range(0, n, GR_CHUNK):
            t0s.append(t + c0)
            ns.append(min(GR_CHUNK, n - c0))
            seqs.append(b)
            lasts.append(1 if c0 + GR_CHUNK >= n else 0)
        firsts.append(len(t0s))
        t += n
    return torch.tensor(t0s + ns + seqs + lasts + firsts, dtype=torch.int32), len(t0s)


def gated_scan(proj: torch.Tensor, lower: torch.Tensor, cu_seqlens: torch.Tensor, slot_ids: torch.Tensor,
               state: torch.Tensor, out: torch.Tensor, n_heads: int, dim: int, v_dim: int, chunks=None) -> None:
    """The recurrence S_t = diag(a_t) S_(t-1) + (1 - a_t) v_t^T, o_t = S_t^T silu(q_t), with
    a_t = lower + (1 - lower) sigmoid(f_t), over a ragged step.  `proj` float32 `[tokens][2 H dim + H v_dim]`:
    q | f | v; `lower` float32 `[H dim]`; `state` float32 `[slots][H][dim][v_dim]`, read and left at each
    sequence's last token for the rows `slot_ids`; `out` float32 `[tokens][H v_dim]`.  With `chunks`
    (`gr_chunks`, the table on the device and its number of chunks) the sequences are walked in chunks side by
    side."""
    n_tok = proj.shape[0]
    n_seqs = slot_ids.numel()
    _need(proj, "gated_scan.proj", torch.float32, (n_tok, n_heads * (2 * dim + v_dim)))
    _need(lower, "gated_scan.lower", torch.float32, (n_heads * dim,))
    _need(cu_seqlens, "gated_scan.cu_seqlens", torch.int32, (n_seqs + 1,))
    _need(slot_ids, "gated_scan.slot_ids", torch.int32, (n_seqs,))
    _need(state, "gated_scan.state", torch.float32)
    if tuple(state.shape[1:]) != (n_heads, dim, v_dim):
        raise KernelError(f"gated_scan: state {tuple(state.shape)} for {n_heads} heads of {dim} x {v_dim}")
    _need(out, "gated_scan.out", torch.float32, (n_tok, n_heads * v_dim))
    if dim > 256:
        raise KernelError(f"gated_scan: key width {dim} is beyond 256")
    if chunks is None:
        _check(_fn("gated_recurrence", "mf_gated_scan")(_ptr(proj), _ptr(lower), _ptr(cu_seqlens), _ptr(slot_ids),
                                                        _ptr(state), _ptr(out), n_seqs, n_heads, dim, v_dim, _stream()),
               "gated_scan")
        return
    table, n_chunks = chunks
    _need(table, "gated_scan.chunks", torch.int32, (4 * n_chunks + n_seqs + 1,))
    per = n_heads * dim * v_dim
    ws = workspace("gr_chunks", n_chunks * (per + n_heads * dim), proj.device)
    _check(_fn("gated_recurrence", "mf_gated_scan_chunked")(
        _ptr(proj), _ptr(lower), _ptr(table), n_chunks, c_void_p(table.data_ptr() + 16 * n_chunks), _ptr(slot_ids),
        _ptr(state), _ptr(ws), c_void_p(ws.data_ptr() + 4 * n_chunks * per), _ptr(out), n_seqs, n_heads, dim, v_dim,
        _stream()), "gated_scan_chunked")


def head_rmsnorm(o: torch.Tensor, weight: Optional[torch.Tensor], eps: float, out: torch.Tensor, n_heads: int,
                 scale: float = 1.0) -> None:
    """out[t][h] = o[t][h] / sqrt(mean(o[t][h]^2) + eps) * weight * scale: every head of a row normed over its
    own values, with one gain vector for all heads; o float32 `[tokens][H V]`, out in the run type."""
    rows, n = o.shape
    _need(o, "head_rmsnorm.o", torch.float32)
    if n % n_heads:
        raise KernelError(f"head_rmsnorm: rows of {n} values are not {n_heads} equal heads")
    if weight is not None:
        _need(weight, "head_rmsnorm.weight", torch.float32, (n // n_heads,))
    _need(out, "head_rmsnorm.out", _FLOATS, (rows, n))
    _check(_fn("gated_recurrence", "mf_head_rmsnorm")(_ptr(o), _ptr(weight), _ptr(out), _is_bf16(out), rows, n_heads,
                                                      n // n_heads, float(eps), float(scale), _stream()), "head_rmsnorm")


# ------------------------------------------------------------------ normed, pair-rotated queries and keys
def qk_norm_prep(qkv: torch.Tensor, q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                 normed: bool, seq_of_tok: torch.Tensor, positions: torch.Tensor, rot_tables, value_tables,
                 v_from_k: bool, page_table: torch.Tensor, q_out: torch.Tensor, kcache: torch.Tensor,
                 vcache: torch.Tensor, n_heads: int, n_kv_heads: int, dim: int, v_dim: int,
                 write_cache: bool = True, halves: bool = False, q_only: bool = False) -> None:
    """From the 32-bit q|k|v rows of one product (q|k alone with `v_from_k`): with `normed`, every q and k head
    over its root mean square (eps inside the root), times `q_gain` / `k_gain` (float32 `[dim]`) where given; the
    rotation in neighbouring pairs over the first 2 x columns values of a head (`rot_tables` = (cos, sin) or
    None); the value heads (their own projection, or with `v_from_k` the key heads as projected) rotated in pairs
    over all their values (`value_tables` = (cos, sin) `[positions][v_dim / 2]` or None); k and v into the cache
    pages at the tokens' positions and q rounded into `q_out`.  `halves`: the rotation turns value i with value
    i + columns instead (the half-split layout).  `q_only`: the rows hold the query heads alone (a layer that
    reads another layer's keys and values); nothing is written to the cache."""
    n_tok = positions.numel()
    C = n_heads * dim if q_only else n_heads * dim + n_kv_heads * dim + (0 if v_from_k else n_kv_heads * v_dim)
    _need(qkv, "qk_norm_prep.qkv", torch.float32, (n_tok, C))
    for name, g in (("q_gain", q_gain), ("k_gain", k_gain)):
        if g is not None:
            _need(g, "qk_norm_prep." + name, torch.float32, (dim,))
    rot, cos_r, sin_r = 0, None, None
    if rot_tables is not None:
        cos_r, sin_r = rot_tables
        _need(cos_r, "qk_norm_prep.cos", torch.float32)
        _need(sin_r, "qk_norm_prep.sin", torch.float32, tuple(cos_r.shape))
        rot = 2 * cos_r.shape[1]
        if rot > dim:
            raise KernelError(f"qk_norm_prep: {rot} rotated values in heads of {dim}")
    cos_v = sin_v = None
    if value_tables is not None:
        cos_v, sin_v = value_tables
        _need(cos_v, "qk_norm_prep.value cos", torch.float32)
        _need(sin_v, "qk_norm_prep.value sin", torch.float32, tuple(cos_v.shape))
        if 2 * cos_v.shape[1] != v_dim:
            raise KernelError(f"qk_norm_prep: value tables of {cos_v.shape[1]} pairs for values of {v_dim}")
    if v_from_k and v_dim != dim:
        raise KernelError(f"qk_norm_prep: values taken from keys of {dim} cannot have {v_dim} values")
    _need(q_out, "qk_norm_prep.q_out", _FLOATS, (n_tok, n_heads * dim))
    _need_kv_pages("qk_norm_prep", kcache, vcache, q_out.dtype, n_kv_heads, dim, v_dim)
    _need(page_table, "qk_norm_prep.page_table", torch.int32)
    _need(seq_of_tok, "qk_norm_prep.seq_of_tok", torch.int32, (n_tok,))
    _need(positions, "qk_norm_prep.positions", torch.int32, (n_tok,))
    _check(_fn("attn_normed", "mf_qk_norm_prep")(
        _ptr(qkv), _ptr(q_gain), _ptr(k_gain), float(eps), 1 if normed else 0, _ptr(seq_of_tok), _ptr(positions),
        _ptr(cos_r), _ptr(sin_r), rot, 1 if halves else 0, 1 if q_only else 0, _ptr(cos_v), _ptr(sin_v),
        1 if v_from_k else 0, _ptr(page_table),
        page_table.shape[1], _ptr(q_out), _ptr(kcache), _ptr(vcache), _is_bf16(q_out), n_tok, n_heads, n_kv_heads, dim,
        v_dim, 1 if write_cache else 0, _stream()), "qk_norm_prep")


def unrotate(rows: torch.Tensor, value_tables, positions: torch.Tensor, n_heads: int, scale: float = 1.0) -> None:
    """Rows `[tokens][H v_dim]` of the run type, in place: pair m of every head turns back by the token's angle m
    (`value_tables` = (cos, sin) `[positions][v_dim / 2]`; None: no turn), and everything is multiplied by
    `scale`."""
    n_tok = positions.numel()
    _need(rows, "unrotate.rows", _FLOATS)
    if rows.shape[0] != n_tok or rows.shape[1] % n_heads or (rows.shape[1] // n_heads) % 2:
        raise KernelError(f"unrotate: rows {tuple(rows.shape)} for {n_tok} tokens of {n_heads} heads")
    v_dim = rows.shape[1] // n_heads
    cos_v = sin_v = None
    if value_tables is not None:
        cos_v, sin_v = value_tables
        _need(cos_v, "unrotate.cos", torch.float32)
        _need(sin_v, "unrotate.sin", torch.float32, tuple(cos_v.shape))
        if 2 * cos_v.shape[1] != v_dim:
            raise KernelError(f"unrotate: tables of {cos_v.shape[1]} pairs for values of {v_dim}")
    _need(positions, "unrotate.positions", torch.int32, (n_tok,))
    _check(_fn("attn_normed", "mf_unrotate")(_ptr(rows), _is_bf16(rows), _ptr(cos_v), _ptr(sin_v), _ptr(positions), n_tok,
                                              n_heads, v_dim, float(scale), _stream()), "unrotate")


# ------------------------------------------------------------------ linear attention with decay
LA_CHUNK = 64            # tokens of a chunk of the chunked form (MF_LA_CHUNK in csrc/linear_attention.hip)
LA_CHUNKED_MAX_DIM = 128  # key width up to which the chunked form's tiles fit into LDS


def la_chunks(host_new):
    """The chunk table of the chunked linear attention for a step whose sequences bring `host_new`
    tokens: int32 `[2][n_chunks]` (first token, tokens) followed by `[n_seqs + 1]` first chunks."""
    t0s, ns, firsts = [], [], [0]
    t = 0
    for n in host_new:
        for c0 in range(0, n, LA_CHUNK):
            t0s.append(t + c0)
            ns.append(min(LA_CHUNK, n - c0))
        firsts.append(len(t0s))
        t += n
    return torch.tensor(t0s + ns + firsts, dtype=torch.int32), len(t0s)


def lightning_scan(proj: torch.Tensor, cu_seqlens: torch.Tensor, slot_ids: torch.Tensor, decays: torch.Tensor,
                   state: torch.Tensor, out: torch.Tensor, n_heads: int, dim: int, v_dim: int,
                   chunks=None) -> None:
    """Linear attention with a decay per head over a ragged step.  `proj` float32
    `[tokens][2 H dim + 2 H v_dim]`: q | k | v | gate pre-activations (the gate is not read here);
    `state` float32 `[slots][H][dim][v_dim]`, read and left at each sequence's last token for the rows
    `slot_ids`; `out` float32 `[tokens][H v_dim]`.  With `chunks` (`la_chunks`, the table on the device
    and its number of chunks) the sequences are walked in chunks side by side."""
    n_tok = proj.shape[0]
    n_seqs = slot_ids.numel()
    _need(proj, "lightning_scan.proj", torch.float32, (n_tok, 2 * n_heads * (dim + v_dim)))
    _need(cu_seqlens, "lightning_scan.cu_seqlens", torch.int32, (n_seqs + 1,))
    _need(slot_ids, "lightning_scan.slot_ids", torch.int32, (n_seqs,))
    _need(decays, "lightning_scan.decays", torch.float32, (n_heads,))
    _need(state, "lightning_scan.state", torch.float32)
    if tuple(state.shape[1:]) != (n_heads, dim, v_dim):
        raise KernelError(f"lightning_scan: state {tuple(state.shape)} for {n_heads} heads of {dim} x {v_dim}")
    _need(out, "lightning_scan.out", torch.float32, (n_tok, n_heads * v_dim))
    if dim > 256:
        raise KernelError(f"lightning_scan: key width {dim} is beyond 256")
    if chunks is None or dim > LA_CHUNKED_MAX_DIM:
        _check(_fn("linear_attention", "mf_lightning_scan")(_ptr(proj), _ptr(cu_seqlens), _ptr(slot_ids), _ptr(decays),
                                                            _ptr(state), _ptr(out), n_seqs, n_heads, dim, v_dim,
                                                            _stream()), "lightning_scan")
        return
    table, n_chunks = chunks
    _need(table, "lightning_scan.chunks", torch.int32, (2 * n_chunks + n_seqs + 1,))
    ws = workspace("la_chunks", n_chunks * n_heads * dim * v_dim, proj.device)
    first = c_void_p(table.data_ptr() + 8 * n_chunks)
    _check(_fn("linear_attention", "mf_lightning_scan_chunked")(
        _ptr(proj), _ptr(table), n_chunks, first, _ptr(slot_ids), _ptr(decays), _ptr(state), _ptr(ws), _ptr(out),
        n_seqs, n_heads, dim, v_dim, _stream()), "lightning_scan_chunked")


def gated_rmsnorm(o: torch.Tensor, proj: torch.Tensor, gate_offset: int, weight: torch.Tensor, eps: float,
                  out: torch.Tensor) -> None:
    """out = o / sqrt(mean(o^2) + eps) * weight * sigmoid(gate), the gate being the columns
    `gate_offset ..` of the 32-bit rows `proj`."""
    rows, n = o.shape
    _need(o, "gated_rmsnorm.o", torch.float32)
    _need(proj, "gated_rmsnorm.proj", torch.float32)
    if proj.shape[0] != rows or gate_offset + n > proj.shape[1]:
        raise KernelError(f"gated_rmsnorm: gate columns {gate_offset}..{gate_offset + n} of rows {tuple(proj.shape)}")
    _need(weight, "gated_rmsnorm.weight", torch.float32, (n,))
    _need(out, "gated_rmsnorm.out", _FLOATS, (rows, n))
    _check(_fn("linear_attention", "mf_gated_rmsnorm")(_ptr(o), c_void_p(proj.data_ptr() + 4 * gate_offset), proj.shape[1],
                                                       _ptr(weight), _ptr(out), _is_bf16(out), rows, n, float(eps),
                                                       _stream()), "gated_rmsnorm")


# ------------------------------------------------------------------ capped attention with a convolution in front
CONV_MAX_TAPS = 16


def rope_half_inplace(rows: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor,
                      n_rot_heads: int, n_heads_total: int, head_dim: int) -> None:
    """Half-split rotation over the first 2 x cos.shape[1] values of the first `n_rot_heads` heads of
    32-bit rows `[tokens][n_heads_total head_dim]`, in place."""
    n_tok = positions.numel()
    rot = 2 * cos.shape[1]
    _need(rows, "rope_half.rows", torch.float32, (n_tok, n_heads_total * head_dim))
    _need(cos, "rope_half.cos", torch.float32)
    _need(sin, "rope_half.sin", torch.float32, tuple(cos.shape))
    _need(positions, "rope_half.positions", torch.int32)
    if rot > head_dim:
        raise KernelError(f"rope_half: {rot} rotated values in heads of {head_dim}")
    _check(_fn("attn_capped", "mf_rope_half_inplace")(_ptr(rows), _ptr(cos), _ptr(sin), _ptr(positions), n_tok,
                                                      n_rot_heads, n_heads_total, head_dim, rot, _stream()), "rope_half_inplace")


def qkv_conv_prep(qkv: torch.Tensor, conv_w: Optional[torch.Tensor], conv_state: Optional[torch.Tensor],
                  cu_seqlens: torch.Tensor, seq_of_tok: torch.Tensor, slot_ids: torch.Tensor, positions: torch.Tensor,
                  cos: Optional[torch.Tensor], sin: Optional[torch.Tensor], blend: float,
                  v_first: Optional[torch.Tensor], v_own: Optional[torch.Tensor], page_table: torch.Tensor,
                  q_out: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, n_heads: int, n_kv_heads: int,
                  dim: int, v_dim: int, write_cache: bool = True) -> None:
    """From the 32-bit q|k|v rows of one product: the short causal convolution over time on every
    channel (`conv_w` `[channels][taps]`; the rows before a sequence's part of the step come from
    `conv_state` `[slots][taps - 1][channels]`, which is moved on afterwards), the half-split rotation of
    q and k over the tables' 2 x columns first values of a head, v <- (1 - blend) v + blend v_first
    where `v_first` is given, the convolved v into `v_own` where given, k and v into the cache pages
    at the tokens' positions and q rounded into `q_out`."""
    n_tok = positions.numel()
    n_seqs = slot_ids.numel()
    C = n_heads * dim + n_kv_heads * (dim + v_dim)
    _need(qkv, "qkv_conv_prep.qkv", torch.float32, (n_tok, C))
    taps = 1
    if conv_w is not None:
        _need(conv_w, "qkv_conv_prep.conv_w", torch.float32)
        if conv_w.dim() != 2 or conv_w.shape[0] != C or not 1 <= conv_w.shape[1] <= CONV_MAX_TAPS:
            raise KernelError(f"qkv_conv_prep: convolution weights {tuple(conv_w.shape)} for {C} channels")
        taps = conv_w.shape[1]
    if taps > 1:
        _need(conv_state, "qkv_conv_prep.conv_state", torch.float32)
        if tuple(conv_state.shape[1:]) != (taps - 1, C):
            raise KernelError(f"qkv_conv_prep: state {tuple(conv_state.shape)} for {taps} taps of {C} channels")
    rot = 0
    if cos is not None:
        _need(cos, "qkv_conv_prep.cos", torch.float32)
        _need(sin, "qkv_conv_prep.sin", torch.float32, tuple(cos.shape))
        rot = 2 * cos.shape[1]
        if rot > dim:
            raise KernelError(f"qkv_conv_prep: {rot} rotated values in heads of {dim}")
    for name, t in (("v_first", v_first), ("v_own", v_own)):
        if t is not None:
            _need(t, "qkv_conv_prep." + name, torch.float32, (n_tok, n_kv_heads * v_dim))
    _need(q_out, "qkv_conv_prep.q_out", _FLOATS, (n_tok, n_heads * dim))
    _need_kv_pages("qkv_conv_prep", kcache, vcache, q_out.dtype, n_kv_heads, dim, v_dim)
    _need(page_table, "qkv_conv_prep.page_table", torch.int32)
    for name, t, shape in (("cu_seqlens", cu_seqlens, (n_seqs + 1,)), ("seq_of_tok", seq_of_tok, (n_tok,)),
                           ("slot_ids", slot_ids, (n_seqs,)), ("positions", positions, (n_tok,))):
        _need(t, "qkv_conv_prep." + name, torch.int32, shape)
    _check(_fn("attn_capped", "mf_qkv_conv_prep")(
        _ptr(qkv), _ptr(conv_w), taps, _ptr(conv_state if taps > 1 else None), _ptr(cu_seqlens), _ptr(seq_of_tok),
        _ptr(slot_ids), _ptr(positions), _ptr(cos), _ptr(sin), rot, float(blend), _ptr(v_first), _ptr(v_own),
        _ptr(page_table), page_table.shape[1], _ptr(q_out), _ptr(kcache), _ptr(vcache), _is_bf16(q_out), n_tok, n_seqs,
        n_heads, n_kv_heads, dim, v_dim, 1 if write_cache else 0, _stream()), "qkv_conv_prep")


def _need_kv_pages(what: str, kcache: torch.Tensor, vcache: torch.Tensor, dtype, n_kv_heads: int, dim: int,
                   v_dim: int) -> None:
    _need(kcache, what + ".kcache", dtype)
    _need(vcache, what + ".vcache", dtype)
    if tuple(kcache.shape[1:]) != (n_kv_heads, PAGE, dim):
        raise KernelError(f"{what}.kcache: shape {tuple(kcache.shape)}, expected [pages, {n_kv_heads}, {PAGE}, {dim}]")
    want = v_page_shape(n_kv_heads, v_dim, dtype)
    if tuple(vcache.shape[1:]) != want or vcache.shape[0] != kcache.shape[0]:
        raise KernelError(f"{what}.vcache: shape {tuple(vcache.shape)}, expected {[kcache.shape[0]] + list(want)}")


def capped_attn(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, page_table: torch.Tensor,
                positions: torch.Tensor, seq_of_tok: torch.Tensor, temp: torch.Tensor, out: torch.Tensor,
                n_heads: int, n_kv_heads: int, dim: int, v_dim: int, scale: float, cap: float, window: int,
                max_len: int, chunk: int = 0, far=None, keep_first: int = 0, bias: Optional[torch.Tensor] = None) -> None:
    """Each query token attends to its sequence's cache rows lo..position with
    s = cap tanh(q . k scale temp[head] / cap) (no cap where `cap` is 0), ordinary softmax; keys of
    `dim` and values of `v_dim` values.  `chunk`: a token sees only the keys of its own chunk of that many
    positions, counted from 0.  `far` = (a, b), float32 per head: s -= a[h] ln(1 + b[h] (position - key)).
    `keep_first`: with a window, the sequence's first so many positions stay in sight of every later token.
    `bias` float32 `[heads][n]`: s += bias[h][min(position - key, n - 1)]."""
    n_tok = positions.numel()
    _need(q, "capped_attn.q", _FLOATS, (n_tok, n_heads * dim))
    _need(out, "capped_attn.out", q.dtype, (n_tok, n_heads * v_dim))
    _need_kv_pages("capped_attn", kcache, vcache, q.dtype, n_kv_heads, dim, v_dim)
    _need(page_table, "capped_attn.page_table", torch.int32)
    _need(positions, "capped_attn.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "capped_attn.seq_of_tok", torch.int32, (n_tok,))
    _need(temp, "capped_attn.temp", torch.float32, (n_heads,))
    if n_heads % n_kv_heads or dim > 512 or v_dim > 256:
        raise KernelError(f"capped_attn: {n_heads} heads over {n_kv_heads}, keys of {dim} (at most 512), values of "
                          f"{v_dim} (at most 256)")
    if max_len > page_table.shape[1] * PAGE:
        raise KernelError(f"capped_attn: max_len {max_len} exceeds the page table ({page_table.shape[1]} pages)")
    far_a, far_b = _far_pair("capped_attn", far, n_heads)
    keep_first, n_bias = _kept_and_bias("capped_attn", keep_first, window, chunk, bias, n_heads)
    # keys split over workgroups where tokens x kv heads alone do not fill the chip: at least 256 keys a split;
    # a windowed token's splits start at its window's first key
    reach = min(max_len, window) if window else max_len
    if chunk:
        reach = min(reach, int(chunk))
    blocks = n_tok * n_kv_heads * ((n_heads // n_kv_heads + 7) // 8)
    n_splits = max(1, min(1024 // max(1, blocks), (reach + 255) // 256, 64))
    split_len = ((reach + n_splits - 1) // n_splits + PAGE - 1) // PAGE * PAGE
    n_splits = (reach + split_len - 1) // split_len
    part = workspace("attn", n_tok * n_heads * n_splits * (v_dim + 2), q.device) if n_splits > 1 else None
    _check(_fn("attn_capped", "mf_capped_attn")(
        _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(positions), _ptr(seq_of_tok),
        _ptr(temp), _ptr(out), _ptr(part), _is_bf16(q), n_tok, n_heads, n_kv_heads, dim, v_dim, float(scale),
        float(cap or 0.0), int(window or 0), int(chunk or 0), _ptr(far_a), _ptr(far_b), keep_first, _ptr(bias), n_bias,
        n_splits, split_len, _stream()), "capped_attn")


def _kept_and_bias(what: str, keep_first, window, chunk, bias: Optional[torch.Tensor], n_heads: int):
    """(keep_first, columns of the bias table) as the attention kernels take them, checked."""
    keep_first = int(keep_first or 0)
    if keep_first < 0 or (keep_first and chunk):
        raise KernelError(f"{what}: keep_first {keep_first} with chunk {chunk}: kept first positions go with a window")
    if not window:
        keep_first = 0          # every earlier position is in sight anyway
    if bias is None:
        return keep_first, 0
    _need(bias, what + ".bias", torch.float32)
    if bias.dim() != 2 or bias.shape[0] != n_heads or bias.shape[1] < 1:
        raise KernelError(f"{what}.bias: shape {tuple(bias.shape)}, expected [{n_heads}][distances]")
    return keep_first, bias.shape[1]


def _far_pair(what: str, far, n_heads: int):
    """The two per-head vectors of the penalty on distance, checked; (None, None) without one."""
    if far is None:
        return None, None
    a, b = far
    _need(a, what + ".far[0]", torch.float32, (n_heads,))
    _need(b, what + ".far[1]", torch.float32, (n_heads,))
    return a, b


CAPPED_MFMA_ROWS = 16        # consecutive tokens of a sequence that a wave of the matrix-core form takes


def capped_mfma_takes(dtype, dim: int, v_dim: int) -> bool:
    """Whether the matrix-core form of the capped attention takes these sizes (it is compiled for them)."""
    return dtype == torch.bfloat16 and dim % 16 == 0 and v_dim % 16 == 0 and 16 <= dim <= 256 and 16 <= v_dim <= 256


def capped_attn_prefill(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, page_table: torch.Tensor, ctx,
                        temp: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv_heads: int, dim: int, v_dim: int,
                        scale: float, cap: float, window: int, chunk: int = 0, far=None, keep_first: int = 0,
                        bias: Optional[torch.Tensor] = None) -> None:
    """`capped_attn` in bfloat16 on the matrix cores: blocks of 16 consecutive new tokens of a sequence
    (`ctx.query_tiles`) times the query heads of a kv head.  A decode step (one token a sequence) splits every
    token's keys over several waves (at least 128 keys a split) and merges the parts in their order."""
    n_tok = ctx.n_tokens
    if not capped_mfma_takes(q.dtype, dim, v_dim):
        raise KernelError(f"capped_attn_prefill: bfloat16 with keys and values of multiples of 16 up to 256; got "
                          f"{q.dtype}, {dim}, {v_dim}")
    _need(q, "capped_attn_prefill.q", torch.bfloat16, (n_tok, n_heads * dim))
    _need(out, "capped_attn_prefill.out", torch.bfloat16, (n_tok, n_heads * v_dim))
    _need_kv_pages("capped_attn_prefill", kcache, vcache, q.dtype, n_kv_heads, dim, v_dim)
    _need(page_table, "capped_attn_prefill.page_table", torch.int32)
    _need(temp, "capped_attn_prefill.temp", torch.float32, (n_heads,))
    _need(ctx.cu_seqlens, "capped_attn_prefill.cu_seqlens", torch.int32, (ctx.n_seqs + 1,))
    _need(ctx.start_pos, "capped_attn_prefill.start_pos", torch.int32, (ctx.n_seqs,))
    if n_heads % n_kv_heads:
        raise KernelError(f"capped_attn_prefill: {n_heads} heads over {n_kv_heads} kv heads")
    if ctx.max_len > page_table.shape[1] * PAGE:
        raise KernelError(f"capped_attn_prefill: max_len {ctx.max_len} exceeds the page table")
    far_a, far_b = _far_pair("capped_attn_prefill", far, n_heads)
    keep_first, n_bias = _kept_and_bias("capped_attn_prefill", keep_first, window, chunk, bias, n_heads)
    n_splits, split_len, part = 1, 0, None
    if ctx.all_decode:
        # every sequence is a tile of one token; nothing comes from the host (the step may be captured)
        tile_seq = ctx.seq_of_tok
        tile_q0 = torch.zeros(n_tok, dtype=torch.int32, device=q.device)
        reach = min(ctx.max_len, window) if window else ctx.max_len
        if chunk:
            reach = min(reach, int(chunk))
        waves = n_tok * n_kv_heads * max(1, (n_heads // n_kv_heads) // 2)
        n_splits = max(1, min(4 * cu_count() // max(1, waves), (reach + 31 + 127) // 128, 64))
        split_len = (((reach + 31 + n_splits - 1) // n_splits) + 31) // 32 * 32
        n_splits = (reach + 31 + split_len - 1) // split_len
        if n_splits > 1:
            part = workspace("attn", n_tok * n_heads * n_splits * (v_dim + 2), q.device)
    else:
        tile_seq, tile_q0 = ctx.query_tiles(CAPPED_MFMA_ROWS)
    lib = build.variant("attn_capped_mfma", MF_CAPM_D=dim, MF_CAPM_V=v_dim)
    _check(_fn("attn_capped_mfma", "mf_capped_mfma", lib)(
        _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(ctx.cu_seqlens),
        _ptr(ctx.start_pos), _ptr(tile_seq), _ptr(tile_q0), tile_seq.numel(), _ptr(temp), _ptr(out), _ptr(part), n_splits,
        split_len, n_tok, n_heads, n_kv_heads, dim, v_dim, float(scale), float(cap or 0.0), int(window or 0),
        int(chunk or 0), _ptr(far_a), _ptr(far_b), keep_first, _ptr(bias), n_bias, _stream()),
        "capped_attn_decode" if ctx.all_decode else "capped_attn_prefill")


# ------------------------------------------------------------------ mixture of experts
MOE_MAX_EXPERTS = 1024
MOE_SPARSE_TOKENS, MOE_SPARSE_PAIRS = 16, 128     # what `moe_sparse` takes in one step (csrc/moe.hip)


def moe_route(x: torch.Tensor, router: torch.Tensor, dense: Optional[torch.Tensor], chosen: torch.Tensor,
              weights: torch.Tensor, n_groups: int, keep: int, bias: Optional[torch.Tensor] = None,
              score: str = "softmax", correction: Optional[torch.Tensor] = None, group_top: int = 1,
              weight_scale: float = 1.0) -> None:
    """The router: logits = router x in 32-bit (`router` float32 `[experts][K]`, `x` `[tokens][K]` in the run
    type), softmax scores, the `keep` best of `n_groups` groups of neighbouring experts (a group's score is
    its best expert's), the `chosen.shape[1]` best experts of those groups, weighted by their scores over
    their sum.  `dense` `[tokens][experts]`, where given, gets the weights at the chosen experts and 0
    elsewhere; `chosen`, `weights` `[tokens][top]`.  `bias` float32 `[experts]` is added to the logits.  With one
    group the weights are the softmax over the chosen logits alone.  `score` "sigmoid": the scores are
    sigmoid(logits).  `correction` float32 `[experts]` joins the scores where groups and experts are chosen, not in
    the weights.  `group_top`: a group's score is the sum of its so many best (corrected) scores.  `weight_scale`
    multiplies the weights."""
    n_tok, K = x.shape
    E = router.shape[0]
    top = chosen.shape[1]
    _need(x, "moe_route.x", _FLOATS)
    _need(router, "moe_route.router", torch.float32, (E, K))
    if dense is not None:
        _need(dense, "moe_route.dense", torch.float32, (n_tok, E))
    _need(chosen, "moe_route.chosen", torch.int32, (n_tok, top))
    _need(weights, "moe_route.weights", torch.float32, (n_tok, top))
    if E > MOE_MAX_EXPERTS or E % n_groups or not 1 <= keep <= n_groups or not 1 <= top <= min(64, keep * (E // n_groups)):
        raise KernelError(f"moe_route: {E} experts in {n_groups} groups, {keep} kept, {top} chosen")
    if bias is not None:
        _need(bias, "moe_route.bias", torch.float32, (E,))
    if correction is not None:
        _need(correction, "moe_route.correction", torch.float32, (E,))
    if score not in MOE_SCORES or group_top < 1:
        raise KernelError(f"moe_route: scores {score!r} (one of {sorted(MOE_SCORES)}), group_top {group_top}")
    _check(_fn("moe", "mf_moe_route")(_ptr(x), _is_bf16(x), _ptr(router), _ptr(bias), K, _ptr(dense), _ptr(chosen), _ptr(weights),
                                       n_tok, E, n_groups, keep, top, MOE_SCORES[score], _ptr(correction), int(group_top),
                                       float(weight_scale), _stream()), "moe_route")


MOE_ACTS = {"clamped_swish": 0, "silu": 1}      # the experts' activations (MF_MOE_ACT_* in csrc/moe.hip)
MOE_SCORES = {"softmax": 0, "sigmoid": 1}       # how a router turns logits into scores (MF_MOE_SCORE_*)


def moe_act(gu: torch.Tensor, dense: torch.Tensor, out: torch.Tensor, limit: float, act: int = 0) -> None:
    """`gu` float32 `[tokens][experts][2 F]` (gate sums, then up sums): out `[tokens][experts F]` =
    dense[t][e] g sigmoid(1.702 g) (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit); with `act` 1,
    dense[t][e] silu(gate) up."""
    n_tok, E = dense.shape
    _need(dense, "moe_act.dense", torch.float32)
    _need(gu, "moe_act.gu", torch.float32)
    if gu.shape[0] != n_tok or gu.shape[1] % (2 * E):
        raise KernelError(f"moe_act: rows {tuple(gu.shape)} for {E} experts")
    F = gu.shape[1] // (2 * E)
    _need(out, "moe_act.out", _FLOATS, (n_tok, E * F))
    _check(_fn("moe", "mf_moe_act")(_ptr(gu), _ptr(dense), _ptr(out), _is_bf16(out), n_tok, E, F, float(limit),
                                     int(act), _stream()), "moe_act")


def moe_sparse(x: torch.Tensor, gate_up: torch.Tensor, down: torch.Tensor, chosen: torch.Tensor, weights: torch.Tensor,
               out: torch.Tensor, n_experts: int, limit: float, act: int = 0) -> None:
    """The chosen experts only, for steps of few tokens: `gate_up` `[experts][2 F][K]` (an expert's gate
    rows, then its up rows), `down` `[experts][N][F]`; out `[tokens][N]` float32 += the weighted sum of the
    chosen experts' outputs, choices added in their order."""
    n_tok, K = x.shape
    top = chosen.shape[1]
    _, N, F = down.shape
    _need(x, "moe_sparse.x", _FLOATS)
    _need(gate_up, "moe_sparse.gate_up", x.dtype, (n_experts, 2 * F, K))
    _need(down, "moe_sparse.down", x.dtype, (n_experts, N, F))
    _need(chosen, "moe_sparse.chosen", torch.int32, (n_tok, top))
    _need(weights, "moe_sparse.weights", torch.float32, (n_tok, top))
    _need(out, "moe_sparse.out", torch.float32, (n_tok, N))
    if n_tok > MOE_SPARSE_TOKENS or n_tok * top > MOE_SPARSE_PAIRS:
        raise KernelError(f"moe_sparse: {n_tok} tokens with {top} experts each; it takes {MOE_SPARSE_TOKENS} tokens and "
                          f"{MOE_SPARSE_PAIRS} pairs")
    y = torch.empty((n_tok, top, F), dtype=x.dtype, device=x.device)
    rows = torch.empty((n_tok * top, N), dtype=torch.float32, device=x.device)
    _check(_fn("moe", "mf_moe_sparse")(_ptr(x), _ptr(gate_up), _ptr(down), _ptr(chosen), _ptr(weights), _ptr(y), _ptr(rows), _ptr(out),
                                        _is_bf16(x), n_tok, top, n_experts, F, K, N, float(limit), int(act), _stream()), "moe_sparse")

SCAN_CHUNK = 32          # tokens of a chunk of the chunked scan (MF_SCAN_CHUNK in csrc/recurrence.hip)


def scan_chunks(host_new):
    """The chunk table of the chunked scan for a step whose sequences bring `host_new` tokens:
    int32 `[5][n_chunks]` (first token, tokens, sequence, first chunk of the sequence, last or not)."""
    t0s, ns, seqs, firsts, lasts = [], [], [], [], []
    t = 0
    for b, n in enumerate(host_new):
        first = len(t0s)
        for c0 in range(0, n, SCAN_CHUNK):
            t0s.append(t + c0)
            ns.append(min(SCAN_CHUNK, n - c0))
            seqs.append(b)
            firsts.append(first)
            lasts.append(1 if c0 + SCAN_CHUNK >= n else 0)
        t += n
    return torch.tensor([t0s, ns, seqs, firsts, lasts], dtype=torch.int32)


def mingru_scan(zug: torch.Tensor, cu_seqlens: torch.Tensor, slot_ids: torch.Tensor, state: torch.Tensor,
                out: torch.Tensor, chunks: Optional[torch.Tensor] = None) -> None:
    """The minGRU recurrence over a ragged step.  `zug` float32 `[tokens][3 W]`: gate, candidate and
    output-gate pre-activations; `state` float32 `[slots][W]`, read and left at each sequence's
    last token for the rows `slot_ids`; `out` `[tokens][W]` (run type) = state * silu(g).  With
    `chunks` (`scan_chunks`, on the device) the sequences are walked in chunks side by side."""
    _need(zug, "mingru_scan.zug", torch.float32)
    n_tok, w3 = zug.shape
    if w3 % 3:
        raise KernelError(f"mingru_scan: rows of {w3} values are not three equal parts")
    w = w3 // 3
    n_seqs = slot_ids.numel()
    _need(cu_seqlens, "mingru_scan.cu_seqlens", torch.int32, (n_seqs + 1,))
    _need(slot_ids, "mingru_scan.slot_ids", torch.int32, (n_seqs,))
    _need(state, "mingru_scan.state", torch.float32)
    if state.dim() != 2 or state.shape[1] != w:
        raise KernelError(f"mingru_scan: state {tuple(state.shape)} for a width of {w}")
    _need(out, "mingru_scan.out", _FLOATS, (n_tok, w))
    if chunks is None:
        _check(_fn("recurrence", "mf_mingru_scan")(_ptr(zug), _ptr(cu_seqlens), _ptr(slot_ids), _ptr(state), _ptr(out),
                                                    _is_bf16(out), n_seqs, w, _stream()), "mingru_scan")
        return
    _need(chunks, "mingru_scan.chunks", torch.int32)
    if chunks.dim() != 2 or chunks.shape[0] != 5:
        raise KernelError(f"mingru_scan: chunk table {tuple(chunks.shape)}")
    n_chunks = chunks.shape[1]
    ws = workspace("scan", (2 * n_chunks + n_seqs) * w, zug.device)
    _check(_fn("recurrence", "mf_mingru_scan_chunked")(
        _ptr(zug), _ptr(chunks), n_chunks, _ptr(slot_ids), _ptr(state), _ptr(ws), c_void_p(ws.data_ptr() + 8 * n_chunks * w),
        _ptr(out), _is_bf16(out), n_seqs, w, _stream()), "mingru_scan_chunked")


# ------------------------------------------------------------------ latent attention
def latent_prep(proj: torch.Tensor, off_dkv: int, off_gate: int, latent_weight: torch.Tensor, eps: float,
                cos: torch.Tensor, sin: torch.Tensor, positions: torch.Tensor, seq_of_tok: torch.Tensor,
                page_table: torch.Tensor, cache: torch.Tensor, q_plain: torch.Tensor, q_abs: torch.Tensor,
                gate: torch.Tensor, n_heads: int, dim: int, rot_dim: int, rank: int, write_cache: bool = True,
                q_rows: Optional[torch.Tensor] = None) -> None:
    """From the 32-bit rows [q | dkv | gates] of one product: the normed latent and the rotated
    shared key part into the cache rows `[pages][64][rank + rot_dim]` at the tokens' positions, the
    plain query parts into `q_plain` `[tokens][heads][dim]`, the rotated query parts into the last
    `rot_dim` columns of `q_abs` `[tokens][heads][rank + rot_dim]`, sigmoid of the gates into `gate`
    (`[tokens][heads]`: one gate a head; `[tokens][heads][w]`: one for each of a head's w values).
    The tables have one column per rotated pair (2i, 2i+1); values behind the pairs pass unchanged.
    `q_rows`: the queries as 32-bit rows `[tokens][heads (dim + rot_dim)]` of their own, where they are not the
    first columns of `proj`."""
    n_tok = positions.numel()
    ld = proj.shape[1]
    dk = rank + rot_dim
    _need(proj, "latent_prep.proj", torch.float32, (n_tok, ld))
    gate_w = 1 if gate.dim() == 2 else gate.shape[2]
    if q_rows is None:
        if off_dkv < n_heads * (dim + rot_dim):
            raise KernelError(f"latent_prep: the queries do not fit in front of column {off_dkv}")
        q_src = proj
    else:
        _need(q_rows, "latent_prep.q_rows", torch.float32, (n_tok, n_heads * (dim + rot_dim)))
        q_src = q_rows
    if off_dkv < 0 or off_dkv + dk > ld or off_gate + n_heads * gate_w > ld or off_gate < 0:
        raise KernelError(f"latent_prep: offsets {off_dkv}, {off_gate} do not fit rows of {ld}")
    _need(latent_weight, "latent_prep.latent_weight", torch.float32, (rank,))
    _need(cos, "latent_prep.cos", torch.float32)
    _need(sin, "latent_prep.sin", torch.float32, tuple(cos.shape))
    rd = 2 * cos.shape[1]
    if rd > rot_dim:
        raise KernelError(f"latent_prep: {rd} rotated values in a part of {rot_dim}")
    _need(positions, "latent_prep.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "latent_prep.seq_of_tok", torch.int32, (n_tok,))
    _need(page_table, "latent_prep.page_table", torch.int32)
    _need(q_plain, "latent_prep.q_plain", _FLOATS, (n_tok, n_heads, dim))
    _need(q_abs, "latent_prep.q_abs", q_plain.dtype, (n_tok, n_heads, dk))
    _need(gate, "latent_prep.gate", torch.float32, (n_tok, n_heads) if gate.dim() == 2 else (n_tok, n_heads, gate_w))
    _need(cache, "latent_prep.cache", q_plain.dtype)
    if cache.dim() < 2 or cache.shape[-1] != dk or cache.numel() % (PAGE * dk):
        raise KernelError(f"latent_prep: cache {tuple(cache.shape)} does not hold pages of {PAGE} rows of {dk}")
    _check(_fn("attn_latent", "mf_latent_prep")(
        _ptr(proj), ld, off_dkv, off_gate, gate_w, _ptr(q_src), q_src.shape[1], _ptr(latent_weight), float(eps), _ptr(cos),
        _ptr(sin), rd, _ptr(positions),
        _ptr(seq_of_tok), _ptr(page_table), page_table.shape[1], _ptr(cache), _ptr(q_plain), _ptr(q_abs), _ptr(gate),
        _is_bf16(q_plain), n_tok, n_heads, dim, rot_dim, rank, 1 if write_cache else 0, _stream()), "latent_prep")


def _gate_width(what: str, gate: Optional[torch.Tensor], n_tok: int, heads: int, n_out: int) -> int:
    """1 for a gate a head (`[tokens][heads]`) or none, `n_out` for a gate a value (`[tokens][heads][n_out]`)."""
    if gate is None or gate.dim() == 2:
        if gate is not None:
            _need(gate, what + ".gate", torch.float32, (n_tok, heads))
        return 1
    _need(gate, what + ".gate", torch.float32, (n_tok, heads, n_out))
    return n_out


def headwise_linear(x: torch.Tensor, n_in: int, wt: torch.Tensor, out: torch.Tensor, n_out: int,
                    gate: Optional[torch.Tensor] = None) -> None:
    """out[t][h][:n_out] = (gate[t][h] *) wt[h]^T x[t][h][:n_in] for `wt` `[heads][n_in][n_out]` (each
    head's matrix stored input-major); x and out are `[tokens][heads][row]` with rows at least that
    long, everything in the run type, sums in 32-bit.  A gate `[tokens][heads][n_out]` multiplies value by
    value."""
    _need(x, "headwise_linear.x", _FLOATS)
    if x.dim() != 3 or out.dim() != 3:
        raise KernelError("headwise_linear: x and out are [tokens][heads][row]")
    n_tok, heads, in_stride = x.shape
    _need(wt, "headwise_linear.wt", x.dtype, (heads, n_in, n_out))
    _need(out, "headwise_linear.out", x.dtype)
    if tuple(out.shape[:2]) != (n_tok, heads) or out.shape[2] < n_out or in_stride < n_in:
        raise KernelError(f"headwise_linear: x {tuple(x.shape)}, out {tuple(out.shape)}, matrix {tuple(wt.shape)}")
    if n_in * 32 > 64 * 1024:
        raise KernelError(f"headwise_linear: inputs of {n_in} values do not fit the kernel's staging")
    gate_w = _gate_width("headwise_linear", gate, n_tok, heads, n_out)
    _check(_fn("attn_latent", "mf_headwise_linear")(_ptr(x), in_stride, _ptr(wt), _ptr(out), out.shape[2], _ptr(gate),
                                                     gate_w, _is_bf16(x), n_tok, heads, n_in, n_out, _stream()),
           "headwise_linear")


def headwise_mfma_takes(dtype, n_in: int, in_stride: int) -> bool:
    """Whether `headwise_linear_mfma` runs these sizes: bfloat16 and inputs in 16-byte pieces."""
    return dtype == torch.bfloat16 and n_in % 8 == 0 and in_stride % 8 == 0


def headwise_linear_mfma(x: torch.Tensor, n_in: int, wo: torch.Tensor, out: torch.Tensor, n_out: int,
                         gate: Optional[torch.Tensor] = None) -> None:
    """`headwise_linear` on the matrix cores: `wo` is `[heads][n_out][n_in]` (each head's matrix
    output-major), everything bfloat16, n_in and x's row length multiples of 8."""
    _need(x, "headwise_linear_mfma.x", torch.bfloat16)
    if x.dim() != 3 or out.dim() != 3:
        raise KernelError("headwise_linear_mfma: x and out are [tokens][heads][row]")
    n_tok, heads, in_stride = x.shape
    _need(wo, "headwise_linear_mfma.wo", torch.bfloat16, (heads, n_out, n_in))
    _need(out, "headwise_linear_mfma.out", torch.bfloat16)
    if tuple(out.shape[:2]) != (n_tok, heads) or out.shape[2] < n_out or in_stride < n_in:
        raise KernelError(f"headwise_linear_mfma: x {tuple(x.shape)}, out {tuple(out.shape)}, matrix {tuple(wo.shape)}")
    if not headwise_mfma_takes(x.dtype, n_in, in_stride):
        raise KernelError(f"headwise_linear_mfma: inputs of {n_in} in rows of {in_stride} are not 16-byte pieces")
    gate_w = _gate_width("headwise_linear_mfma", gate, n_tok, heads, n_out)
    _check(_fn("attn_latent", "mf_headwise_mfma")(_ptr(x), in_stride, _ptr(wo), _ptr(out), out.shape[2], _ptr(gate),
                                                   gate_w, n_tok, heads, n_in, n_out, _stream()), "headwise_linear_mfma")


def latent_split_plan(n_blocks: int, max_len: int, target_blocks: Optional[int] = None, most: int = 64) -> Tuple[int, int]:
    """(n_splits, split_len) of the latent attention's keys: as many splits (whole pages, at most
    `most`) as it takes to give every CU a block where the step's `n_blocks` alone do not."""
    target = target_blocks or cu_count()
    pages = (max_len + PAGE - 1) // PAGE
    want = max(1, min(most, pages, target // max(1, n_blocks)))
    per = (pages + want - 1) // want
    return (pages + per - 1) // per, per * PAGE


LATENT_MFMA_ROWS = 64        # (token, head) rows of a workgroup of the matrix-core latent attention
LATENT_MFMA_MAX = (640, 512)  # padded row and rank up to which its registers hold queries and accumulators


def latent_mfma_takes(dtype, rank: int, dk: int) -> bool:
    """Whether the matrix-core kernel is built for these sizes: bfloat16, rows and rank multiples
    of 8 (16-byte pieces), padded sizes within what a wave's registers hold."""
    pad = lambda v: (v + 31) // 32 * 32
    return (dtype == torch.bfloat16 and rank % 8 == 0 and dk % 8 == 0 and pad(dk) <= LATENT_MFMA_MAX[0]
            and pad(rank) <= LATENT_MFMA_MAX[1] and not tuning.NO_LATENT_MFMA)


def latent_attn(q_abs: torch.Tensor, cache: torch.Tensor, page_table: torch.Tensor, positions: torch.Tensor,
                seq_of_tok: torch.Tensor, out: torch.Tensor, rank: int, scale: float, window: int,
                max_len: int, ctx=None) -> None:
    """out[t][h][:] = sum_j softmax_j(scale q_abs[t][h] . row_j) row_j[:rank] over the cached rows
    j <= position of the token's sequence (the last `window` of them when window > 0).  With the
    step's context (`ctx`: its ragged layout) and sizes the matrix-core kernel is built for, that
    kernel runs: a workgroup per 64 (token, head) rows that share their keys."""
    _need(q_abs, "latent_attn.q_abs", _FLOATS)
    if q_abs.dim() != 3:
        raise KernelError("latent_attn: q_abs is [tokens][heads][rank + rot_dim]")
    n_tok, heads, dk = q_abs.shape
    _need(cache, "latent_attn.cache", q_abs.dtype)
    if cache.shape[-1] != dk or cache.numel() % (PAGE * dk) or not 0 < rank <= dk:
        raise KernelError(f"latent_attn: cache {tuple(cache.shape)}, queries of {dk}, rank {rank}")
    _need(out, "latent_attn.out", q_abs.dtype, (n_tok, heads, rank))
    _need(page_table, "latent_attn.page_table", torch.int32)
    _need(positions, "latent_attn.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "latent_attn.seq_of_tok", torch.int32, (n_tok,))
    if page_table.shape[1] * PAGE < max_len:
        raise KernelError(f"latent_attn: page table of {page_table.shape[1]} columns for {max_len} positions")
    if ctx is not None and latent_mfma_takes(q_abs.dtype, rank, dk):
        hc = min(heads, LATENT_MFMA_ROWS)
        tq = LATENT_MFMA_ROWS // hc
        if ctx.all_decode:
            tile_seq = tile_q0 = cu = None
            n_tiles = n_tok
        else:
            tile_seq, tile_q0 = ctx.query_tiles(tq)
            n_tiles = tile_seq.numel()
            cu = ctx.cu_seqlens
            _need(cu, "latent_attn.cu_seqlens", torch.int32, (page_table.shape[0] + 1,))
        n_splits, split_len = latent_split_plan(n_tiles * ((heads + hc - 1) // hc), max_len, target_blocks=2 * cu_count(), most=32)
        part = workspace("latent_attn", n_tok * heads * n_splits * (rank + 2), q_abs.device) if n_splits > 1 else None
        lib = build.variant("attn_latent_mfma", MF_LAT_DKP=(dk + 31) // 32 * 32, MF_LAT_RP=(rank + 31) // 32 * 32)
        _check(_fn("attn_latent_mfma", "mf_latent_mfma", lib)(
            _ptr(q_abs), _ptr(cache), _ptr(page_table), page_table.shape[1], _ptr(positions), _ptr(cu),
            _ptr(tile_seq), _ptr(tile_q0), n_tiles, _ptr(out), _ptr(part), n_tok, heads, rank, dk, hc, tq, float(scale),
            int(window), n_splits, split_len, _stream()), "latent_attn_mfma")
        return
    if rank > 1024 or (4 * dk + 4 * 256 + 4) * 4 > 64 * 1024:
        raise KernelError(f"latent_attn: rank {rank} / row {dk} beyond what the kernel holds")
    n_splits, split_len = latent_split_plan(n_tok * ((heads + 3) // 4), max_len)
    part = workspace("latent_attn", n_tok * heads * n_splits * (rank + 2), q_abs.device) if n_splits > 1 else None
    _check(_fn("attn_latent", "mf_latent_attn")(
        _ptr(q_abs), _ptr(cache), _ptr(page_table), page_table.shape[1], _ptr(positions), _ptr(seq_of_tok), _ptr(out),
        _ptr(part), _is_bf16(q_abs), n_tok, heads, rank, dk, float(scale), int(window), n_splits, split_len,
        _stream()), "latent_attn")


# ------------------------------------------------------------------ matrix products
_CU_COUNT: Optional[int] = None


def cu_count() -> int:
    """Compute units of the current device (256 on MI355X)."""
    global _CU_COUNT
    if _CU_COUNT is None:
        _CU_COUNT = int(torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count)
    return _CU_COUNT


# K = 256 NS for which the register-resident decode product is instantiated
# (MF_STATIONARY_NS in csrc/gemm_bf16.hip; `plan_linear` asks the library itself)
STATIONARY_NS = (4, 6, 8, 10, 12, 14, 16, 20, 24, 28, 32)
STATIONARY_K7 = 896      # and this K, which runs as seven waves of four steps (the narrowest model of the family)


def stationary_shape(n: int, k: int, folded: bool = False) -> bool:
    """True where the register-resident decode product is built for [n][k] weights (aligned
    operands given): K = 256 NS for one of the NS above, or 896, and at least 128 tiles of 16 weight rows;
    a K above 5120 only with a norm or SwiGLU folded in (`folded`)."""
    if k == STATIONARY_K7:
        return (n + 15) // 16 >= 64
    return k % 256 == 0 and k // 256 in STATIONARY_NS and (n + 15) // 16 >= 128 and (k <= 5120 or folded)


def skinny_plan(m: int, n: int, k: int, target_blocks: Optional[int] = None,
                swiglu: bool = False, tiled: bool = False) -> Tuple[int, int]:
    """(splits, k_per_split) of a product with at most 64 rows.  One split: one kernel, K divided
    between the waves of a block.  More: blocks of 128 weight rows with the activations staged in
    LDS, K split so that there is about one block per CU, and a second kernel that adds the parts.

    At most 16 rows take the one-kernel form, except against a K of 8192 and more that the
    register-resident kernel does not hold, where it does badly from 9 rows on (every block reads
    its own copy of the activations from L2; from 13 rows on where it reads the tiled copy of the
    weights: the down product of the 7B shape at 12 rows 28.9 us against 29.9, at 16 rows 32.4
    against 30.4) and where a CU's share of the weight rows fills its 16-row tiles poorly, unless
    the matrix is small (the down product of the 3B shape, 2048 x 11008, at 8 rows: 13.5 us in one
    kernel, half-filled tiles and all, against 15.0 in two; at 16 rows 17.1 against 15.4)."""
    if target_blocks is None:
        target_blocks = tuning.SKINNY_TARGET or cu_count()
    if m <= 16:
        share = (n + target_blocks - 1) // target_blocks          # weight rows of a block in the one-kernel form
        fill = share / float((share + 15) // 16 * 16)
        small = m <= 8 and n * k <= 24 << 20          # up to 48 MB of weights: the second kernel's few microseconds count
        if k < 8192 or (m <= (12 if tiled else 8) and fill >= 0.8) or small or stationary_shape(n, k, swiglu):
            return 1, (k + 255) // 256 * 256
    n_blocks = (n + 127) // 128
    chunks = (k + 255) // 256
    splits = max(1, min(chunks, target_blocks // max(1, n_blocks)))
    per = (chunks + splits - 1) // splits
    return (chunks + per - 1) // per, per * 256


def tile_plan(m: int, n: int, k: int, epi: int, aligned: bool = True, n_cu: Optional[int] = None) -> Tuple[int, int, int]:
    """(variant, splits, k_per_split) of a bfloat16 product of more than 64 rows, as the library
    chooses among its tile kernels (an estimate of the rounds their tiles take over the CUs); with
    splits > 1, K is cut over blocks and a second kernel adds the parts."""
    out = (c_int * 3)()
    rc = _fn("gemm_bf16", "mf_gemm_bf16_tile_plan")(m, n, k, 1 if aligned else 0, epi, n_cu or cu_count(), out)
    if rc != 0:
        raise KernelError(f"tile_plan: error {rc} for m {m}, n {n}, k {k}")
    return out[0], out[1], out[2]


def _k_split(m: int, n: int, k: int, swiglu: bool, aligned: bool, n_cu: Optional[int] = None,
             tiled: bool = False) -> Tuple[int, int]:
    """(splits, k_per_split) as `linear` and `linear_swiglu` cut a bfloat16 product of at most 64 rows."""
    target = tuning.SKINNY_TARGET or n_cu
    return skinny_plan(m, n, k, target_blocks=target, swiglu=swiglu, tiled=tiled)


def plan_linear(m: int, n: int, k: int, swiglu: bool = False, normed: bool = False, aligned: bool = True,
                out_bf16: bool = False, accumulate: bool = False, n_cu: Optional[int] = None,
                tiled: bool = False) -> Dict[str, object]:
    """Which kernel `linear` / `linear_swiglu` / `linear_normed` runs for a bfloat16 product of
    `m` rows against `[n][k]` weights, as the library itself decides it, without launching
    anything: {'kernel': name, 'splits': s, 'k_per_split': per}.  With `normed` an empty name
    means that no kernel folds the norm in at this shape (norm and product then run one after
    the other).  `n` counts the interleaved gate|up rows for `swiglu`; `tiled`: the product is
    given the tiled copy of the weights (it moves the row count from which K is cut over blocks)."""
    n_cu = n_cu or cu_count()
    epi = EPI_SWIGLU if swiglu else (EPI_BF16 if out_bf16 else (EPI_ACC_F32 if accumulate else EPI_F32))
    splits, per = 1, k
    if normed:
        if m > 16 or tuning.NO_FOLD:
            return dict(kernel="", splits=1, k_per_split=k)
    elif m <= 64:
        splits, per = _k_split(m, n, k, swiglu, aligned, n_cu, tiled)
    else:
        _, splits, per = tile_plan(m, n, k, epi, aligned, n_cu)
    name = ctypes.create_string_buffer(64)
    rc = _fn("gemm_bf16", "mf_gemm_bf16_plan")(m, n, k, 1 if aligned else 0, epi, splits, per,
                                               1 if normed else 0, n_cu, name, 64)
    if rc != 0:
        raise KernelError(f"plan_linear: error {rc} for m {m}, n {n}, k {k}")
    return dict(kernel=name.value.decode(), splits=splits, k_per_split=per)


def tile_weight(weight: torch.Tensor) -> torch.Tensor:
    """The tiled copy of a bfloat16 `[n][k]` matrix, k a multiple of 32: `[ceil(n / 16)][k / 32][16][32]`,
    rows padded with zeros to a multiple of 16.  The products of at most 64 rows read their
    weights a tile (a contiguous kilobyte) per wave and step from it; made once, when a model is
    loaded, where memory allows a second copy."""
    _need(weight, "tile_weight.weight", torch.bfloat16)
    n, k = weight.shape
    if k % 32:
        raise KernelError(f"tile_weight: k {k} is not a multiple of 32")
    n16 = (n + 15) // 16 * 16
    if n16 != n:
        weight = torch.cat([weight, torch.zeros((n16 - n, k), dtype=weight.dtype, device=weight.device)])
    return weight.view(n16 // 16, 16, k // 32, 32).permute(0, 2, 1, 3).contiguous()


def _need_tiled(tiled: Optional[torch.Tensor], name: str, n: int, k: int) -> None:
    if tiled is not None:
        _need(tiled, name, torch.bfloat16, ((n + 15) // 16, k // 32, 16, 32))


def linear(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
           accumulate: bool = False, variant: int = 0, tiled: Optional[torch.Tensor] = None,
           xielu: bool = False) -> None:
    """out (+)= x @ weight^T (+ bias).  weight is [out][in].  float32 weights take the true
    32-bit kernel; bfloat16 weights take the matrix-core kernels (a few rows: the streaming
    kernel).  `out` is float32, or bfloat16 for a bfloat16 product that is stored.  `tiled`:
    `tile_weight(weight)`, which the kernels for at most 64 rows read instead where they can."""
    _need(x, "linear.x", _FLOATS)
    _need(weight, "linear.weight", x.dtype)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear: x is [{m},{k}], weight is {tuple(weight.shape)}")
    _need(out, "linear.out", _FLOATS, (m, n))
    if xielu:
        if bias is None or x.dtype != torch.bfloat16 or out.dtype != torch.bfloat16 or accumulate:
            raise KernelError("linear(xielu): needs bfloat16 operands and output, and the biases with the two constants")
        _need(bias, "linear.bias", torch.float32, (n + 2,))
    elif bias is not None:
        _need(bias, "linear.bias", torch.float32, (n,))
    if m == 0:
        return
    if x.dtype == torch.float32:
        _need(out, "linear.out", torch.float32)
        _check(_fn("gemm_f32", "mf_gemm_f32")(_ptr(x), k, _ptr(weight), k, _ptr(bias), _ptr(out), n, m,
                                               n, k, 1 if accumulate else 0, _stream()), f"gemm_f32 {m}x{n}x{k}")
        return
    if accumulate and out.dtype != torch.float32:
        raise KernelError("linear: accumulation needs a float32 output")
    epi = EPI_XIELU if xielu else (EPI_BF16 if out.dtype == torch.bfloat16 else (EPI_ACC_F32 if accumulate else EPI_F32))
    aligned = not (x.data_ptr() % 16 or weight.data_ptr() % 16 or k % 8)
    if m <= 64 and variant == 0:
        splits, per = _k_split(m, n, k, False, aligned, tiled=tiled is not None)
        part = workspace("skinny", splits * m * n, x.device) if splits > 1 else None
        _need_tiled(tiled, "linear.tiled", n, k)
        _check(_fn("gemm_bf16", "mf_gemm_bf16_skinny")(_ptr(x), k, _ptr(weight), _ptr(tiled), k, _ptr(bias),
                                                        _ptr(out), n, _ptr(part), m, n, k, splits, per,
                                                        epi, _stream()), f"gemm_bf16_skinny {m}x{n}x{k}")
        return
    if variant == 0:
        variant, splits, per = tile_plan(m, n, k, epi, aligned)
        if splits > 1:
            part = workspace("skinny", splits * m * n, x.device)
            _check(_fn("gemm_bf16", "mf_gemm_bf16_splitk")(_ptr(x), k, _ptr(weight), k, _ptr(bias), _ptr(out), n,
                                                            _ptr(part), m, n, k, splits, per, epi, variant,
                                                            _stream()), f"gemm_bf16_splitk {m}x{n}x{k}")
            return
    _check(_fn("gemm_bf16", "mf_gemm_bf16")(_ptr(x), k, _ptr(weight), k, _ptr(bias), _ptr(out), n, m,
                                             n, k, epi, variant, _stream()), f"gemm_bf16 {m}x{n}x{k}")


def interleave_gate_up(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """Rows of gate and up `[nf][k]` in groups of 64: 32 gate rows, then the 32 up rows of the
    same outputs; the last group is padded with zero rows.  The layout `linear_swiglu` reads."""
    nf, k = gate.shape
    groups = (nf + 31) // 32
    pad = groups * 32 - nf
    if pad:
        z = torch.zeros((pad, k), dtype=gate.dtype, device=gate.device)
        gate, up = torch.cat([gate, z]), torch.cat([up, z])
    return torch.stack([gate.view(groups, 32, k), up.view(groups, 32, k)], dim=1).reshape(groups * 64, k).contiguous()


def linear_swiglu(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, variant: int = 0,
                  tiled: Optional[torch.Tensor] = None) -> None:
    """out = silu(x @ Wg^T) * (x @ Wu^T) in one kernel; `weight` is `interleave_gate_up(Wg, Wu)`,
    everything bfloat16, `out` is [rows][nf].  `tiled`: `tile_weight(weight)`."""
    _need(x, "linear_swiglu.x", torch.bfloat16)
    _need(weight, "linear_swiglu.weight", torch.bfloat16)
    m, k = x.shape
    n = weight.shape[0]
    nf = out.shape[1]
    if weight.shape[1] != k or n % 64 or not n // 2 - 32 < nf <= n // 2:
        raise KernelError(f"linear_swiglu: x {tuple(x.shape)}, weight {tuple(weight.shape)}, out {tuple(out.shape)}")
    _need(out, "linear_swiglu.out", torch.bfloat16, (m, nf))
    if m == 0:
        return
    aligned = not (x.data_ptr() % 16 or weight.data_ptr() % 16 or k % 8)
    if m <= 64 and variant == 0:
        splits, per = _k_split(m, n, k, True, aligned, tiled=tiled is not None)
        part = workspace("skinny", splits * m * n, x.device) if m > 16 or splits > 1 else None
        _need_tiled(tiled, "linear_swiglu.tiled", n, k)
        _check(_fn("gemm_bf16", "mf_gemm_bf16_skinny")(_ptr(x), k, _ptr(weight), _ptr(tiled), k, _ptr(None), _ptr(out), nf,
                                                        _ptr(part), m, n, k, splits, per, EPI_SWIGLU, _stream()),
               f"gemm_bf16_skinny(swiglu) {m}x{n}x{k}")
        return
    if variant == 0:
        variant, splits, per = tile_plan(m, n, k, EPI_SWIGLU, aligned)
        if splits > 1:
            part = workspace("skinny", splits * m * n, x.device)
            _check(_fn("gemm_bf16", "mf_gemm_bf16_splitk")(_ptr(x), k, _ptr(weight), k, _ptr(None), _ptr(out), nf,
                                                            _ptr(part), m, n, k, splits, per, EPI_SWIGLU, variant,
                                                            _stream()), f"gemm_bf16_splitk(swiglu) {m}x{n}x{k}")
            return
    _check(_fn("gemm_bf16", "mf_gemm_bf16")(_ptr(x), k, _ptr(weight), k, _ptr(None), _ptr(out), nf, m, n, k,
                                             EPI_SWIGLU, variant, _stream()), f"gemm_bf16(swiglu) {m}x{n}x{k}")


NOT_BUILT = -2      # an entry point's answer for a shape it has no kernel for; nothing was launched


def linear_normed(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, row_idx: Optional[torch.Tensor],
                  weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                  accumulate: bool = False, swiglu: bool = False, tiled: Optional[torch.Tensor] = None) -> bool:
    """out (+)= rmsnorm(x[row_idx]) @ weight^T (+ bias) in one kernel, for the few-row shapes
    the register-resident decode product covers; with `swiglu`, `weight` is
    `interleave_gate_up(Wg, Wu)` and out = silu(gate) * up.  x is the float32 residual stream,
    weight bfloat16.  Returns False, having done nothing, when there is no such kernel for
    the shape: the caller then norms and multiplies in two steps.  `tiled`: `tile_weight(weight)`."""
    _need(x, "linear_normed.x", torch.float32)
    _need(weight, "linear_normed.weight", torch.bfloat16)
    k = x.shape[1]
    n = weight.shape[0]
    m = x.shape[0] if row_idx is None else row_idx.numel()
    if weight.shape[1] != k:
        raise KernelError(f"linear_normed: x is {tuple(x.shape)}, weight is {tuple(weight.shape)}")
    _need(norm_weight, "linear_normed.norm_weight", torch.float32, (k,))
    if row_idx is not None:
        _need(row_idx, "linear_normed.row_idx", torch.int32)
    if bias is not None:
        _need(bias, "linear_normed.bias", torch.float32, (n,))
    if swiglu:
        nf = out.shape[1]
        if n % 64 or not n // 2 - 32 < nf <= n // 2 or bias is not None or accumulate:
            raise KernelError(f"linear_normed(swiglu): weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        _need(out, "linear_normed.out", torch.bfloat16, (m, nf))
        epi, ldc = EPI_SWIGLU, nf
    else:
        _need(out, "linear_normed.out", _FLOATS, (m, n))
        if accumulate and out.dtype != torch.float32:
            raise KernelError("linear_normed: accumulation needs a float32 output")
        epi = EPI_BF16 if out.dtype == torch.bfloat16 else (EPI_ACC_F32 if accumulate else EPI_F32)
        ldc = n
    if m == 0:
        return True
    if m > 16 or tuning.NO_FOLD:
        return False
    _need_tiled(tiled, "linear_normed.tiled", n, k)
    rc = _fn("gemm_bf16", "mf_gemm_bf16_normed")(_ptr(x), k, _ptr(row_idx), _ptr(norm_weight), float(eps),
                                                 _ptr(weight), _ptr(tiled), k, _ptr(bias), _ptr(out), ldc, m, n, k,
                                                 epi, _stream())
    if rc == NOT_BUILT:
        return False
    _check(rc, f"gemm_bf16_normed{'(swiglu)' if swiglu else ''} {m}x{n}x{k}")
    return True


NORM_SUM_RUN = 256       # columns a partial sum of squares covers (a block of the kernel that adds a K split's parts)


# Steps of at most 16 rows prepare the next norm in a product's epilogue only for rows of this many
# values: measured at batch 8 (a decode step with it against without), width 896: 10 % slower (the
# reading product waits for the rows' sums, a trip to memory, where the whole kernel is 7 us), 1536
# and 2048: 0.5 % slower, 3584: 0.7 % faster (2.4 % at batch 1), 5120: 4.5 % faster; from 5121 on
# the register-resident product has no form that reads bfloat16 activations.
NORM_AHEAD_16_WIDTHS = (3072, 5120)


def norm_sum_parts(n: int, m: int = 64) -> int:
    """Partial sums of squares a row of `n` values comes with from a product of `m` rows (see
    `linear_fused`): one per run of 256 columns from 17 rows on (the kernel that adds the parts of a K
    split writes them), one per workgroup of the product's one kernel for at most 16 rows."""
    runs = (n + NORM_SUM_RUN - 1) // NORM_SUM_RUN
    return max(cu_count(), runs) if m <= 16 else runs


def linear_fused(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], out: torch.Tensor,
                 accumulate: bool = False, tiled: Optional[torch.Tensor] = None, swiglu: bool = False,
                 scale_in=None, norm_out=None) -> bool:
    """A bfloat16 product of at most 64 rows with an RMS norm folded in on either side, across two
    products: the norm is no kernel of its own between them (17 to 64 rows), and the product behind
    it reads its activations in bfloat16, half the bytes, with nothing to convert (at most 16 rows,
    where the norm is otherwise folded into that product's prologue):

    * `norm_out` = (g `[n]`, xg `[m][n]` bfloat16, sums `[m][norm_sum_parts(n, m)]`): the product stores
      or adds into the 32-bit `out` as `linear` does and leaves, beside it, bf16(out g) and the sums
      of out^2 in parts, for the norm with weight g that reads `out` next;
    * `scale_in` = (sums `[m][parts]`, eps): `x` is such an xg, and the product's sums are multiplied
      by the row's 1 / sqrt(sum / k + eps) before the bias and the epilogue; with `swiglu`, `weight`
      is `interleave_gate_up(Wg, Wu)` and out = silu(gate) * up, bfloat16.

    Returns False, having launched nothing, where the kernels the shape takes have no place for it
    (the caller then runs norm and product one after the other)."""
    _need(x, "linear_fused.x", torch.bfloat16)
    _need(weight, "linear_fused.weight", torch.bfloat16)
    m, k = x.shape
    n = weight.shape[0]
    if weight.shape[1] != k:
        raise KernelError(f"linear_fused: x is [{m},{k}], weight is {tuple(weight.shape)}")
    if m == 0 or m > 64 or (scale_in is None and norm_out is None):
        return False
    if swiglu:
        nf = out.shape[1]
        if n % 64 or not n // 2 - 32 < nf <= n // 2 or bias is not None or accumulate or norm_out is not None:
            raise KernelError(f"linear_fused(swiglu): weight {tuple(weight.shape)}, out {tuple(out.shape)}")
        _need(out, "linear_fused.out", torch.bfloat16, (m, nf))
        epi, ldc = EPI_SWIGLU, nf
    else:
        _need(out, "linear_fused.out", _FLOATS, (m, n))
        if accumulate and out.dtype != torch.float32:
            raise KernelError("linear_fused: accumulation needs a float32 output")
        epi = EPI_BF16 if out.dtype == torch.bfloat16 else (EPI_ACC_F32 if accumulate else EPI_F32)
        ldc = n
    if bias is not None:
        _need(bias, "linear_fused.bias", torch.float32, (n,))
    in_ssq, in_parts, in_eps = None, 0, 0.0
    if scale_in is not None:
        in_ssq, in_eps = scale_in
        _need(in_ssq, "linear_fused.scale_in", torch.float32)
        if in_ssq.dim() != 2 or in_ssq.shape[0] != m or in_ssq.shape[1] < 1:
            raise KernelError(f"linear_fused.scale_in: sums {tuple(in_ssq.shape)} for {m} rows")
        in_parts = in_ssq.shape[1]
    out_g = out_xg = out_ssq = None
    if norm_out is not None:
        out_g, out_xg, out_ssq = norm_out
        if out.dtype != torch.float32:
            raise KernelError("linear_fused.norm_out: the product's own output must be float32")
        _need(out_g, "linear_fused.norm_out.g", torch.float32, (n,))
        _need(out_xg, "linear_fused.norm_out.xg", torch.bfloat16, (m, n))
        _need(out_ssq, "linear_fused.norm_out.sums", torch.float32, (m, norm_sum_parts(n, m)))
    aligned = not (x.data_ptr() % 16 or weight.data_ptr() % 16 or k % 8)
    splits, per = _k_split(m, n, k, swiglu, aligned, tiled=tiled is not None)
    part = workspace("skinny", splits * m * n, x.device) if (splits > 1 or (swiglu and m > 16)) else None
    _need_tiled(tiled, "linear_fused.tiled", n, k)
    rc = _fn("gemm_bf16", "mf_gemm_bf16_skinny_fused")(
        _ptr(x), k, _ptr(weight), _ptr(tiled), k, _ptr(bias), _ptr(out), ldc, _ptr(part), m, n, k, splits, per, epi,
        _ptr(in_ssq), in_parts, float(in_eps), _ptr(out_g), _ptr(out_xg), _ptr(out_ssq),
        out_ssq.shape[1] if out_ssq is not None else 0, _stream())
    if rc == NOT_BUILT:
        return False
    _check(rc, f"gemm_bf16_skinny_fused{'(swiglu)' if swiglu else ''} {m}x{n}x{k}")
    return True


# ------------------------------------------------------------------ attention
def split_plan(n_tok: int, n_kv_heads: int, group: int, head_dim: int, max_len: int,
               target_blocks: int = 1024) -> Tuple[int, int]:
    """(n_splits, split_len) for the per-token attention: split the keys when tokens x kv
    heads alone do not fill the chip.  Depends on the capacity, not on current lengths;
    split_len is a multiple of the page size and at least four pages; at most 64 splits."""
    gc = 8 if head_dim <= 128 else 4
    blocks = n_tok * n_kv_heads * ((group + gc - 1) // gc)
    n_splits = max(1, min(target_blocks // max(1, blocks), (max_len + 4 * PAGE - 1) // (4 * PAGE), 64))
    split_len = ((max_len + n_splits - 1) // n_splits + PAGE - 1) // PAGE * PAGE
    return (max_len + split_len - 1) // split_len, split_len


def _need_caches(what: str, kcache: torch.Tensor, vcache: torch.Tensor, dtype, n_kv_heads: int,
                 head_dim: int) -> None:
    _need(kcache, what + ".kcache", dtype)
    _need(vcache, what + ".vcache", dtype)
    if tuple(kcache.shape[1:]) != (n_kv_heads, PAGE, head_dim):
        raise KernelError(f"{what}.kcache: shape {tuple(kcache.shape)}, expected "
                          f"[pages, {n_kv_heads}, {PAGE}, {head_dim}]")
    want = v_page_shape(n_kv_heads, head_dim, dtype)
    if tuple(vcache.shape[1:]) != want or vcache.shape[0] != kcache.shape[0]:
        raise KernelError(f"{what}.vcache: shape {tuple(vcache.shape)}, expected "
                          f"{[kcache.shape[0]] + list(want)}")


# Sequences that can be this long share their step's key splits by length: working the shares out
# costs a block about a microsecond, which shorter ones do not gain back.  (This threshold, the cap
# of four times the even share and the 32 places were tuned on an MI355X: 256 CUs in 8 dies.)
SHARED_SPLITS_FROM = 8192


def decode_split_plan(n_tok: int, n_kv_heads: int, group: int, max_len: int,
                      target_blocks: Optional[int] = None) -> Tuple[int, int]:
    """(places, splits) of the bfloat16 decode attention's key splits.  `splits`: about one block
    per CU, at least 256 keys of the longest possible sequence per split, at most 32.  A step of
    one token, of more than 64, of sequences that cannot be long, or without splits, gives every
    token that many (`places` = `splits`); otherwise the
    step's tokens share tokens x splits between them in proportion to their keys, a token taking
    at most `places` = 4 x splits (at most 32), so that a long sequence among short ones is cut
    finer and the blocks have about equal work.  The kernel divides a token's keys in rounds of
    128; a place without keys is marked empty and the merge passes it over."""
    if target_blocks is None:
        target_blocks = cu_count()
    blocks = n_tok * n_kv_heads * ((group + 15) // 16)
    splits = tuning.ATTN_SPLITS or max(1, min(target_blocks // max(1, blocks), (max_len + 255) // 256, 32))
    if n_tok == 1 or n_tok > 64 or splits == 1 or max_len < SHARED_SPLITS_FROM or tuning.ATTN_EQUAL_SPLITS:
        return splits, splits
    return max(splits, min(4 * splits, 32)), splits


def attn_tokens(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, page_table: torch.Tensor,
                positions: torch.Tensor, seq_of_tok: torch.Tensor, out: torch.Tensor, n_heads: int,
                n_kv_heads: int, head_dim: int, scale: float, window: int, max_len: int) -> None:
    """Each query token attends to its sequence's cache rows lo..position.  `max_len` bounds
    position + 1 for every token (it only shapes the launch).  bfloat16 runs on the matrix
    cores, 32-bit on plain FMA."""
    n_tok = positions.numel()
    _need(q, "attn.q", _FLOATS, (n_tok, n_heads * head_dim))
    _need(out, "attn.out", q.dtype, (n_tok, n_heads * head_dim))
    _need_caches("attn", kcache, vcache, q.dtype, n_kv_heads, head_dim)
    _need(page_table, "attn.page_table", torch.int32)
    _need(positions, "attn.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "attn.seq_of_tok", torch.int32, (n_tok,))
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention: head_dim {head_dim} is not a multiple of 16 in [16, 256]")
    if n_heads % n_kv_heads:
        raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
    if max_len > page_table.shape[1] * PAGE:
        raise KernelError(f"attention: max_len {max_len} exceeds the page table ({page_table.shape[1]} pages)")
    if q.dtype == torch.bfloat16:
        n_splits, base = decode_split_plan(n_tok, n_kv_heads, n_heads // n_kv_heads, max_len)
        part = workspace("attn", n_tok * n_heads * n_splits * (head_dim + 2), q.device) if n_splits > 1 else None
        _check(_fn("attn_decode_bf16", "mf_attn_decode_bf16")(
            _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(positions),
            _ptr(seq_of_tok), _ptr(out), _ptr(part), n_tok, n_heads, n_kv_heads, head_dim, float(scale),
            int(window or 0), n_splits, base, _stream()), "attn_decode_bf16")
        return
    n_splits, split_len = split_plan(n_tok, n_kv_heads, n_heads // n_kv_heads, head_dim, max_len)
    part = workspace("attn", n_tok * n_heads * n_splits * (head_dim + 2), q.device) if n_splits > 1 else None
    _check(_fn("attn_tokens_f32", "mf_attn_tokens_f32")(
        _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(positions),
        _ptr(seq_of_tok), _ptr(out), _ptr(part), n_tok, n_heads, n_kv_heads, head_dim, float(scale),
        int(window or 0), n_splits, split_len, _stream()), "attn_tokens_f32")


def attn_decode_rope(qkv: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, kcache: torch.Tensor,
                     vcache: torch.Tensor, page_table: torch.Tensor, positions: torch.Tensor,
                     seq_of_tok: torch.Tensor, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int,
                     scale: float, window: int, max_len: int, write_kv: bool = True) -> None:
    """A bfloat16 decode step's rotation, cache write and attention in one kernel: qkv is the
    float32 `[tokens][(heads + 2 kv_heads) head_dim]` output of the q|k|v product; every token is
    the next position of its sequence.  Same result as `rope_kvwrite` then `attn_tokens`."""
    n_tok = positions.numel()
    _need(qkv, "attn_decode_rope.qkv", torch.float32, (n_tok, (n_heads + 2 * n_kv_heads) * head_dim))
    _need(cos, "attn_decode_rope.cos", torch.float32)
    _need(sin, "attn_decode_rope.sin", torch.float32, tuple(cos.shape))
    if cos.shape[1] != head_dim // 2:
        raise KernelError(f"rope: table has {cos.shape[1]} frequencies, head_dim {head_dim} needs {head_dim // 2}")
    _need(out, "attn_decode_rope.out", torch.bfloat16, (n_tok, n_heads * head_dim))
    _need_caches("attn_decode_rope", kcache, vcache, torch.bfloat16, n_kv_heads, head_dim)
    _need(page_table, "attn_decode_rope.page_table", torch.int32)
    _need(positions, "attn_decode_rope.positions", torch.int32, (n_tok,))
    _need(seq_of_tok, "attn_decode_rope.seq_of_tok", torch.int32, (n_tok,))
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention: head_dim {head_dim} is not a multiple of 16 in [16, 256]")
    if n_heads % n_kv_heads:
        raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
    if max_len > page_table.shape[1] * PAGE or max_len > cos.shape[0]:
        raise KernelError(f"attention: max_len {max_len} exceeds the page table ({page_table.shape[1]} pages) "
                          f"or the rotation table ({cos.shape[0]} positions)")
    n_splits, base = decode_split_plan(n_tok, n_kv_heads, n_heads // n_kv_heads, max_len)
    part = workspace("attn", n_tok * n_heads * n_splits * (head_dim + 2), qkv.device) if n_splits > 1 else None
    _check(_fn("attn_decode_bf16", "mf_attn_decode_rope_bf16")(
        _ptr(qkv), _ptr(cos), _ptr(sin), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1],
        _ptr(positions), _ptr(seq_of_tok), _ptr(out), _ptr(part), n_tok, n_heads, n_kv_heads, head_dim,
        float(scale), int(window or 0), n_splits, base, 1 if write_kv else 0, _stream()), "attn_decode_rope_bf16")


def prefill_tile(n_heads: int, n_kv_heads: int, head_dim: int):
    """(tq, gh, workgroups per block of queries): a workgroup of the prompt attention takes `gh` heads
    of a kv head's group (all of them, unless there are more than it has rows) times `tq` consecutive
    new tokens, so that a page of keys it brings in serves every head that reads it."""
    rows = _fn("attn_prefill_bf16", "mf_attn_prefill_rows")(head_dim)
    group = n_heads // n_kv_heads
    gh = min(group, rows)
    return rows // gh, gh, n_kv_heads * (-(-group // gh))


def attn_prefill(q: torch.Tensor, kcache: torch.Tensor, vcache: torch.Tensor, page_table: torch.Tensor,
                 ctx, out: torch.Tensor, n_heads: int, n_kv_heads: int, head_dim: int, scale: float,
                 window: int) -> None:
    """bfloat16 attention of a step that brings several tokens per sequence: every new token
    attends to its sequence's cache rows up to its own position (the step's keys are already
    stored).  `ctx` gives the ragged layout (cu_seqlens, start_pos, the query blocks)."""
    n_tok = ctx.n_tokens
    _need(q, "attn_prefill.q", torch.bfloat16, (n_tok, n_heads * head_dim))
    _need(out, "attn_prefill.out", torch.bfloat16, (n_tok, n_heads * head_dim))
    _need_caches("attn_prefill", kcache, vcache, torch.bfloat16, n_kv_heads, head_dim)
    _need(page_table, "attn_prefill.page_table", torch.int32)
    if not scale > 0.0:
        raise KernelError(f"attn_prefill: scale {scale} must be positive")
    _need(ctx.cu_seqlens, "attn_prefill.cu_seqlens", torch.int32, (ctx.n_seqs + 1,))
    _need(ctx.start_pos, "attn_prefill.start_pos", torch.int32, (ctx.n_seqs,))
    if head_dim % 16 or not 16 <= head_dim <= 256:
        raise KernelError(f"attention: head_dim {head_dim} is not a multiple of 16 in [16, 256]")
    if n_heads % n_kv_heads:
        raise KernelError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
    if ctx.max_len > page_table.shape[1] * PAGE or page_table.shape[0] != ctx.n_seqs:
        raise KernelError(f"attention: page table {tuple(page_table.shape)} does not cover "
                          f"{ctx.n_seqs} sequences of up to {ctx.max_len} positions")
    # Where the kernel's time is that of the block with the most pages (a few new tokens on a long
    # context, few short prompts), blocks of queries with more pages than a workgroup's even share
    # of all of them (two workgroups fit a CU up to a head size of 128) are given to several
    # workgroups, which take the pages in turn.
    window = int(window or 0)
    tq, gh, per_tile = prefill_tile(n_heads, n_kv_heads, head_dim)
    per_cu = _fn("attn_prefill_bf16", "mf_attn_prefill_per_cu")(head_dim)
    shared = None if tuning.NO_SHARED_PAGES else ctx.shared_query_tiles(
        tq, PAGE, window, per_tile, cu_count(), per_cu, PREFILL_MIN_PAGES, PREFILL_MAX_SHARES)
    if shared is None:
        tile_seq, tile_q0 = ctx.query_tiles(tq)
        tile_share = parts = arrived = None
    else:
        tile_seq, tile_q0, tile_share, n_slots, most_shares = shared
        part = _fn("attn_prefill_bf16", "mf_attn_prefill_part_floats")(head_dim)
        parts = workspace("prefill_parts", n_slots * per_tile * most_shares * part, q.device)
        arrived = _zeroed_counters("prefill_arrived", n_slots * per_tile, q.device)
    rc = _fn("attn_prefill_bf16", "mf_attn_prefill_bf16")(
        _ptr(q), _ptr(kcache), _ptr(vcache), _ptr(page_table), page_table.shape[1], _ptr(ctx.cu_seqlens),
        _ptr(ctx.start_pos), _ptr(tile_seq), _ptr(tile_q0), _ptr(tile_share), _ptr(parts), _ptr(arrived),
        most_shares if shared is not None else 1, _ptr(out), tile_seq.numel(), n_heads, n_kv_heads, head_dim,
        gh, tq, float(scale), window, _stream())
    if rc != 0 and arrived is not None:
        arrived.zero_()                  # a launch that failed may have left workgroups counted in
    _check(rc, "attn_prefill_bf16")


# ------------------------------------------------------------------ sampling
def _logit_rows(logits: torch.Tensor, name: str):
    _need(logits, name, torch.float32)
    if logits.dim() != 2:
        raise KernelError(f"{name}: expected [rows][vocab], got {tuple(logits.shape)}")
    return logits.shape


def argmax(logits: torch.Tensor, out: torch.Tensor) -> None:
    rows, vocab = _logit_rows(logits, "argmax.logits")
    _need(out, "argmax.out", torch.int32, (rows,))
    chunks = 1
    if vocab >= 16384 and rows < 256:          # few long rows: several blocks per row
        chunks = max(1, min(64, 512 // rows, vocab // 4096))
    work = workspace("argmax", 2 * rows * chunks, logits.device) if chunks > 1 else None
    _check(_fn("sampling", "mf_argmax")(_ptr(logits), vocab, rows, vocab, _ptr(out), _ptr(work), chunks,
                                         _stream()), "argmax")


def sample(logits: torch.Tensor, temp: float, streams: torch.Tensor, steps: torch.Tensor,
           out: torch.Tensor, forced_r: Optional[torch.Tensor] = None) -> None:
    """Temperature draw per row (greedy when temp < 1e-6).  The uniform of row i is
    `rng.uniform(seed, key_i, steps[i])` for streams[i] = `rng.stream_i64(seed, key_i)`, or
    forced_r[i] when given (tests)."""
    rows, vocab = _logit_rows(logits, "sample.logits")
    _need(streams, "sample.streams", torch.int64, (rows,))
    _need(steps, "sample.steps", torch.int32, (rows,))
    _need(out, "sample.out", torch.int32, (rows,))
    if forced_r is not None:
        _need(forced_r, "sample.forced_r", torch.float32, (rows,))
    _check(_fn("sampling", "mf_sample")(_ptr(logits), vocab, rows, vocab, float(temp), _ptr(streams),
                                         _ptr(steps), _ptr(forced_r), _ptr(out), _stream()), "sample")


def penalties(logits: torch.Tensor, prev: torch.Tensor, n_prev: torch.Tensor, repeat: float,
              frequency: float, presence: float) -> None:
    rows, vocab = _logit_rows(logits, "penalties.logits")
    _need(prev, "penalties.prev", torch.int32)
    if prev.dim() != 2 or prev.shape[0] != rows:
        raise KernelError(f"penalties.prev: expected [{rows}][window], got {tuple(prev.shape)}")
    _need(n_prev, "penalties.n_prev", torch.int32, (rows,))
    _check(_fn("sampling", "mf_penalties")(_ptr(logits), vocab, rows, vocab, _ptr(prev), prev.shape[1],
                                            _ptr(n_prev), float(repeat), float(frequency),
                                            float(presence), _stream()), "penalties")


def top_k(logits: torch.Tensor, k: int) -> None:
    rows, vocab = _logit_rows(logits, "top_k.logits")
    _check(_fn("sampling", "mf_top_k")(_ptr(logits), vocab, rows, vocab, int(k), _stream()), "top_k")


def top_p(logits: torch.Tensor, p: float) -> None:
    rows, vocab = _logit_rows(logits, "top_p.logits")
    _check(_fn("sampling", "mf_top_p")(_ptr(logits), vocab, rows, vocab, float(p), _stream()), "top_p")


FILTERED_K_MAX = 48            # the largest top-k that `sample_filtered` takes
FILTERED_VOCAB_MAX = 64 * 64 * 64


def sample_filtered_takes(vocab: int, k: int, temp: float) -> bool:
    """Whether `sample_filtered` covers these settings (else: top_k, top_p, sample one after the other)."""
    return 1 <= k <= FILTERED_K_MAX and k < vocab <= FILTERED_VOCAB_MAX and temp >= 1e-6


def sample_filtered(logits: torch.Tensor, k: int, p: float, temp: float, streams: torch.Tensor,
                    steps: torch.Tensor, out: torch.Tensor, forced_r: Optional[torch.Tensor] = None) -> None:
    """top-k, then top-p (off unless 0 < p < 1), then the temperature draw, as `top_k`, `top_p` and
    `sample` one after the other give it, but reading each row once: its k largest entries and their
    ties are picked out by 64 waves a row and the rest runs on those few.  The logits stay as they
    are, except for rows with more equal values than the lists hold, which take the whole-row
    kernels in place."""
    rows, vocab = _logit_rows(logits, "sample_filtered.logits")
    if not sample_filtered_takes(vocab, k, temp):
        raise KernelError(f"sample_filtered: k {k}, vocabulary {vocab}, temperature {temp} are outside what it takes")
    _need(streams, "sample_filtered.streams", torch.int64, (rows,))
    _need(steps, "sample_filtered.steps", torch.int32, (rows,))
    _need(out, "sample_filtered.out", torch.int32, (rows,))
    if forced_r is not None:
        _need(forced_r, "sample_filtered.forced_r", torch.float32, (rows,))
    work = workspace("sample_filtered", rows * 64 * (2 * 64 + 2), logits.device)
    _check(_fn("sampling", "mf_sample_filtered")(_ptr(logits), vocab, rows, vocab, int(k), float(p), float(temp),
                                                  _ptr(streams), _ptr(steps), _ptr(forced_r), _ptr(work),
                                                  _ptr(out), _stream()),
           "sample_filtered")


def advance(next_ids: torch.Tensor, sampled: torch.Tensor, positions: torch.Tensor, steps: torch.Tensor,
            prev: Optional[torch.Tensor] = None, n_prev: Optional[torch.Tensor] = None,
            cursor: Optional[torch.Tensor] = None) -> None:
    """After a decode step: next_ids = sampled, positions and steps move on by one; with `prev`
    `[n][window]` the sampled token also enters the window of recent tokens (n_prev entries in
    use, cursor = where the next one goes)."""
    n = next_ids.numel()
    for name, t in (("next_ids", next_ids), ("sampled", sampled), ("positions", positions), ("steps", steps)):
        _need(t, "advance." + name, torch.int32, (n,))
    max_prev = 0
    if prev is not None:
        _need(prev, "advance.prev", torch.int32)
        if prev.dim() != 2 or prev.shape[0] != n:
            raise KernelError(f"advance.prev: shape {tuple(prev.shape)}, expected [{n}, window]")
        max_prev = prev.shape[1]
        _need(n_prev, "advance.n_prev", torch.int32, (n,))
        _need(cursor, "advance.cursor", torch.int32, (n,))
    _check(_fn("sampling", "mf_advance")(_ptr(next_ids), _ptr(sampled), _ptr(positions), _ptr(steps), n,
                                          _ptr(prev), max_prev, _ptr(n_prev if prev is not None else None),
                                          _ptr(cursor if prev is not None else None), _stream()), "advance")


# ------------------------------------------------------------------ measuring kernels
def probe_read(buffer: torch.Tensor, blocks: Optional[int] = None) -> None:
    """Launches one plain streaming read of the whole buffer (for the benchmark's measured
    memory bandwidth; time it from outside)."""
    _need(buffer, "probe_read.buffer")
    nbytes = buffer.numel() * buffer.element_size() // 16 * 16
    blocks = blocks or cu_count()
    sink = workspace("probe", blocks, buffer.device)
    _check(_fn("probe", "mf_probe_read")(_ptr(buffer), nbytes, _ptr(sink), blocks, _stream()), "probe_read")


def probe_mfma(rounds: int, blocks: Optional[int] = None, device="cuda") -> float:
    """Launches a register-resident loop of bfloat16 matrix-core products and returns the number
    of floating-point operations it performs (time it from outside)."""
    blocks = blocks or cu_count()
    sink = workspace("probe", blocks, device)
    _check(_fn("probe", "mf_probe_mfma")(int(rounds), _ptr(sink), blocks, _stream()), "probe_mfma")
    return float(blocks) * 8 * rounds * 8 * 2 * 32 * 32 * 16


def moe_group(chosen: torch.Tensor, n_experts: int, rank: torch.Tensor, counts: torch.Tensor) -> None:
    """`rank[t][k]`: how many earlier (token, choice) pairs of the step chose the same expert; `counts[e]`:
    the pairs of expert e."""
    _need(chosen, "moe_group.chosen", torch.int32)
    _need(rank, "moe_group.rank", torch.int32, tuple(chosen.shape))
    _need(counts, "moe_group.counts", torch.int32, (n_experts,))
    _check(_fn("moe", "mf_moe_group")(_ptr(chosen), chosen.numel(), n_experts, _ptr(rank), _ptr(counts), _stream()), "moe_group")


def moe_gather(x: torch.Tensor, chosen: torch.Tensor, rank: torch.Tensor, offsets: torch.Tensor, xs: torch.Tensor) -> None:
    """xs[offsets[chosen[t][k]] + rank[t][k]] = x[t]: the tokens of every expert side by side, one expert after
    the other."""
    n_tok, K = x.shape
    top = chosen.shape[1]
    _need(x, "moe_gather.x", _FLOATS)
    _need(chosen, "moe_gather.chosen", torch.int32, (n_tok, top))
    _need(rank, "moe_gather.rank", torch.int32, (n_tok, top))
    _need(offsets, "moe_gather.offsets", torch.int32)
    _need(xs, "moe_gather.xs", x.dtype, (n_tok * top, K))
    _check(_fn("moe", "mf_moe_gather")(_ptr(x), _is_bf16(x), _ptr(chosen), _ptr(rank), _ptr(offsets), _ptr(xs), n_tok * top,
                                        top, K, _stream()), "moe_gather")


def moe_combine(rows: torch.Tensor, chosen: torch.Tensor, rank: torch.Tensor, offsets: torch.Tensor, weights: torch.Tensor,
                out: torch.Tensor, accumulate: bool = True) -> None:
    """out[t] (+)= sum_k weights[t][k] rows[offsets[chosen[t][k]] + rank[t][k]], a token's choices in their order."""
    n_tok, top = chosen.shape
    N = out.shape[1]
    _need(rows, "moe_combine.rows", torch.float32, (n_tok * top, N))
    _need(chosen, "moe_combine.chosen", torch.int32)
    _need(rank, "moe_combine.rank", torch.int32, (n_tok, top))
    _need(offsets, "moe_combine.offsets", torch.int32)
    _need(weights, "moe_combine.weights", torch.float32, (n_tok, top))
    _need(out, "moe_combine.out", torch.float32, (n_tok, N))
    _check(_fn("moe", "mf_moe_combine")(_ptr(rows), _ptr(chosen), _ptr(rank), _ptr(offsets), _ptr(weights), _ptr(out), n_tok,
                                         top, N, 1 if accumulate else 0, _stream()), "moe_combine")
