"""Python faces of the HIP kernels: each checks operand shapes, dtypes and contiguity on the host,
then launches on torch's current stream through the family's ``extern "C"`` entry point.
A non-zero return of a launcher raises ``KernelError``; nothing falls back to another path.
"""
from __future__ import annotations

import ctypes
import logging
from typing import Optional

import torch

from . import build, dispatch

F32, BF16 = 0, 1
logger = logging.getLogger("ullm_amd")


class KernelError(RuntimeError):
    pass


_ERR_NAMES = {-1: "unsupported dtype combination", -2: "operand shape outside what the kernel takes",
              -3: "unsupported argument combination", -4: "partial results exceed the fixed scratch array"}


def _check(rc: int, what: str) -> None:
    if rc != 0:
        reason = _ERR_NAMES.get(rc, f"HIP error {rc}")
        raise KernelError(f"{what}: {reason}")


def _dt(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return F32
    if t.dtype == torch.bfloat16:
        return BF16
    raise KernelError(f"dtype {t.dtype} is not float32 or bfloat16")


def _stream() -> ctypes.c_void_p:
    return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)


def _p(t: Optional[torch.Tensor]) -> ctypes.c_void_p:
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _need(cond: bool, msg: str) -> None:
    if not cond:
        raise KernelError(msg)


def _i32(t: torch.Tensor, name: str, n: Optional[int] = None) -> None:
    _need(t.dtype == torch.int32 and t.is_contiguous(), f"{name} must be contiguous int32")
    if n is not None:
        _need(t.numel() >= n, f"{name} holds {t.numel()} entries, {n} needed")


_c_int, _c_float = ctypes.c_int, ctypes.c_float


def _check_pools(k_pool, v_pool, nkv: int, page_size: int, hd: int, dtype) -> None:
    """Keys are [pages, nkv, page_size, hd]; values are kept transposed inside a page: [pages, nkv, hd, page_size]."""
    _need(k_pool is not None and k_pool.dim() == 4 and tuple(k_pool.shape[1:]) == (nkv, page_size, hd)
          and k_pool.is_contiguous() and k_pool.dtype == dtype,
          f"k_pool must be contiguous [pages, {nkv}, {page_size}, {hd}] of {dtype}")
    _need(v_pool is not None and v_pool.dim() == 4 and tuple(v_pool.shape[1:]) == (nkv, hd, page_size)
          and v_pool.is_contiguous() and v_pool.dtype == dtype and v_pool.shape[0] == k_pool.shape[0],
          f"v_pool must be contiguous [pages, {nkv}, {hd}, {page_size}] of {dtype}")


# ---------------------------------------------------------------------------------- elementwise

def embedding(ids: torch.Tensor, table: torch.Tensor, out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """float32 [T, H] rows of ``table`` [V, H] at ``ids`` [T] (int32), times ``scale``."""
    T = ids.numel()
    V, H = table.shape
    _i32(ids, "ids")
    _need(table.is_contiguous(), "embedding table must be contiguous")
    if out is None:
        out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    _need(out.dtype == torch.float32 and out.is_contiguous() and out.shape == (T, H), "bad embedding output")
    lib = build.load("elementwise")
    _check(lib.ullm_embedding(_p(ids), _p(table), _p(out), _c_int(T), _c_int(H), _c_int(V),
                              _c_int(_dt(table)), _c_float(scale), _stream()), "embedding")
    return out


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x = cap * tanh(x / cap) in place, float32 [rows, cols]."""
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1 and cap > 0, "softcap takes float32 [rows, cols] and a cap > 0")
    _check(build.load("elementwise").ullm_softcap(_p(x), _c_int(x.shape[0]), _c_int(x.shape[1]), _c_int(x.stride(0)),
                                                  _c_float(cap), _stream()), "softcap")
    return x


def feed_tokens(ids: torch.Tensor, feed: torch.Tensor, source: torch.Tensor) -> None:
    """ids[t] = source[feed[t]] wherever feed[t] >= 0 (all int32): token ids that the step before has
    sampled and the host has not yet seen are taken from that step's output on the device."""
    n = ids.numel()
    _i32(ids, "ids")
    _i32(feed, "feed", n)
    _i32(source, "source")
    _check(build.load("elementwise").ullm_feed_tokens(_p(ids), _p(feed), _p(source), _c_int(n),
                                                      _c_int(source.numel()), _stream()), "feed_tokens")


def zero_fresh_rows(state: torch.Tensor, entry_slot: torch.Tensor, entry_start: torch.Tensor, n_entries: int) -> None:
    """state[entry_slot[b]] = 0 for every entry b < n_entries with entry_start[b] == 0: the per-request state
    rows (``state`` contiguous [slots, anything]) of requests that step from their first token.  Takes
    everything from device tensors, so it can be part of a captured step."""
    _need(state.is_contiguous() and state.dim() >= 1, "state must be contiguous [slots, ...]")
    _i32(entry_slot, "entry_slot", n_entries)
    _i32(entry_start, "entry_start", n_entries)
    rows = state.shape[0]
    row_bytes = (state.numel() // max(1, rows)) * state.element_size()
    _check(build.load("elementwise").ullm_zero_fresh_rows(_p(state), ctypes.c_longlong(row_bytes), _c_int(rows),
                                                         _p(entry_slot), _p(entry_start), _c_int(n_entries), _stream()),
           "zero_fresh_rows")


def gather_rows(src: torch.Tensor, index: torch.Tensor) -> torch.Tensor:
    """src[index] for float32 ``src`` [n, cols] and int32 ``index`` on the device: no index travels from the
    host and nothing waits for the device."""
    _need(src.dtype == torch.float32 and src.dim() == 2 and src.stride(1) == 1, "gather_rows takes float32 [n, cols]")
    _i32(index, "index")
    n, cols = index.numel(), src.shape[1]
    out = torch.empty((n, cols), dtype=torch.float32, device=src.device)
    _check(build.load("elementwise").ullm_gather_rows(_p(src), ctypes.c_longlong(src.stride(0)), _c_int(src.shape[0]),
                                                     _p(index), _p(out), _c_int(n), _c_int(cols), _stream()), "gather_rows")
    return out


def stream_read(src: torch.Tensor, blocks: int = 0) -> torch.Tensor:
    """Read ``src`` (contiguous, a multiple of 16 bytes) once with a kernel that does nothing else; returns the
    words the blocks stored (their xor of what they read).  For measuring what a read-only kernel reaches."""
    nbytes = src.numel() * src.element_size()
    _need(src.is_contiguous() and nbytes % 16 == 0 and src.data_ptr() % 16 == 0, "stream_read takes contiguous, 16-byte aligned memory")
    n_blocks = blocks if blocks > 0 else 8 * compute_units(src.device)
    sink = torch.empty(n_blocks * 4, dtype=torch.int32, device=src.device)
    _check(build.load("elementwise").ullm_stream_read(_p(src), ctypes.c_longlong(nbytes), _p(sink), _c_int(n_blocks), _stream()),
           "stream_read")
    return sink


def add_rmsnorm(branch: Optional[torch.Tensor], residual: torch.Tensor, gain: torch.Tensor, eps: float,
                out_dtype: torch.dtype, rows: Optional[torch.Tensor] = None,
                out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """residual (float32 [T, H], updated in place unless ``rows``) += branch; returns the RMS-normed
    sum times ``gain`` (float32 [H]) in ``out_dtype``.  With ``rows`` (int32 [n]) only those rows are
    produced and the residual stays untouched.  ``branch`` may be a stack [S, T, H] of partial sums
    (see :func:`gemm_partial_sums`): they are added in order."""
    T, H = residual.shape
    _need(residual.dtype == torch.float32 and residual.is_contiguous(), "residual must be contiguous float32")
    _need(gain.dtype == torch.float32 and gain.numel() == H and gain.is_contiguous(), "gain must be float32 [H]")
    n_branch, branch_stride = 1, 0
    if branch is not None:
        _need(branch.shape[-2:] == (T, H) and branch.dim() in (2, 3) and branch.is_contiguous(),
              "branch must be contiguous [T, H] or a stack [S, T, H]")
        if branch.dim() == 3:
            n_branch, branch_stride = branch.shape[0], T * H
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    if out is None:
        out = torch.empty((n, H), dtype=out_dtype, device=residual.device)
    _need(out.shape == (n, H) and out.is_contiguous() and out.dtype == out_dtype, "bad norm output")
    lib = build.load("elementwise")
    bdt = _dt(branch) if branch is not None else _dt(out)
    _check(lib.ullm_add_rmsnorm(_p(branch), _p(residual), _p(gain), _c_float(eps), _p(out), _p(rows),
                                _c_int(n), _c_int(H), _c_int(bdt), _c_int(_dt(out)),
                                _c_int(0 if rows is not None else 1), _c_int(n_branch),
                                ctypes.c_longlong(branch_stride), _stream()), "add_rmsnorm")
    return out


def residual_add(branch: torch.Tensor, residual: torch.Tensor) -> None:
    """residual (float32, contiguous) += branch (same shape, contiguous)."""
    _need(residual.dtype == torch.float32 and residual.is_contiguous() and branch.is_contiguous()
          and branch.shape == residual.shape, "residual_add takes contiguous tensors of one shape")
    lib = build.load("elementwise")
    _check(lib.ullm_residual_add(_p(branch), _p(residual), ctypes.c_longlong(residual.numel()), _c_int(_dt(branch)),
                                 _stream()), "residual_add")


def branch_sum(a: torch.Tensor, b: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [T, H]: the sum of two branches, each one tensor [T, H] or a stack of partial sums [S, T, H]
    (contiguous, float32 or bfloat16), added slice by slice, ``a``'s first; ``b`` None: ``a``'s slices alone."""
    shape = tuple(a.shape[-2:])
    for t in (a, b):
        _need(t is None or (t.is_contiguous() and t.dim() in (2, 3) and tuple(t.shape[-2:]) == shape),
              "branch_sum takes contiguous [T, H] or [S, T, H] of one row shape")
    out = torch.empty(shape, dtype=torch.float32, device=a.device)
    sa = a.shape[0] if a.dim() == 3 else 1
    sb = 0 if b is None else (b.shape[0] if b.dim() == 3 else 1)
    _check(build.load("elementwise").ullm_branch_sum(_p(a), _c_int(sa), _c_int(_dt(a)), _p(b), _c_int(sb),
                                                     _c_int(_dt(b) if b is not None else F32), _p(out),
                                                     ctypes.c_longlong(out.numel()), _stream()), "branch_sum")
    return out


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y [T, N] += bias (float32 [N]) in place, the sum taken in 32-bit; returns y."""
    T, N = y.shape
    _need(y.stride(1) == 1, "y must have unit stride along its rows")
    _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    _check(build.load("elementwise").ullm_add_bias(_p(y), _p(bias), _c_int(T), _c_int(N), ctypes.c_longlong(y.stride(0)),
                                                   _c_int(_dt(y)), _stream()), "add_bias")
    return y


def silu_mul(gate_up: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """silu(gate_up[:, :I]) * gate_up[:, I:] for a contiguous [T, 2I] input."""
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and gate_up.is_contiguous(), "gate_up must be contiguous [T, 2I]")
    inter = two_i // 2
    if out is None:
        out = torch.empty((T, inter), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.shape == (T, inter) and out.is_contiguous() and out.dtype == gate_up.dtype, "bad silu_mul output")
    lib = build.load("elementwise")
    _check(lib.ullm_silu_mul(_p(gate_up), _p(out), _c_int(T), _c_int(inter), _c_int(_dt(gate_up)), _stream()),
           "silu_mul")
    return out


ACT_RELU2, ACT_GELU_TANH, ACT_TANH = 0, 1, 2       # activations behind a product


def activation(x: torch.Tensor, kind: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """act(x) element by element, computed in 32-bit: ACT_RELU2 max(x, 0)^2, ACT_GELU_TANH the tanh form of GELU,
    ACT_TANH tanh."""
    _need(x.is_contiguous(), "activation takes a contiguous tensor")
    if out is None:
        out = torch.empty_like(x)
    _need(out.shape == x.shape and out.is_contiguous() and out.dtype == x.dtype, "bad activation output")
    _check(build.load("elementwise").ullm_activation(_p(x), _p(out), ctypes.c_longlong(x.numel()), _c_int(kind),
                                                     _c_int(_dt(x)), _stream()), "activation")
    return out


def stream_pair(branch: Optional[torch.Tensor], mult: float, residual: torch.Tensor, other: torch.Tensor,
                out_dtype: torch.dtype) -> torch.Tensor:
    """residual (float32 [T, H], in place) += mult * branch ([T, H] or None); returns [residual | other] as
    [T, 2 H] of ``out_dtype`` for ``other`` float32 [T, H]."""
    T, H = residual.shape
    _need(residual.dtype == torch.float32 and residual.is_contiguous(), "residual must be contiguous float32")
    _need(other.dtype == torch.float32 and other.is_contiguous() and other.shape == (T, H), "other must be float32 [T, H]")
    if branch is not None:
        _need(branch.shape == (T, H) and branch.is_contiguous(), "branch must be contiguous [T, H]")
    out = torch.empty((T, 2 * H), dtype=out_dtype, device=residual.device)
    _check(build.load("elementwise").ullm_stream_pair(
        _p(branch), _c_int(_dt(branch) if branch is not None else F32), _c_float(mult), _p(residual), _p(other), _p(out),
        _c_int(T), _c_int(H), _c_int(_dt(out)), _stream()), "stream_pair")
    return out


def glu_clamped(gate_up: torch.Tensor, limit: float, alpha: float, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """g * sigmoid(alpha * g) * (u + 1) with g = min(gate, limit), u = clamp(up, -limit, limit), for a contiguous
    [T, 2I] input gate | up."""
    T, two_i = gate_up.shape
    _need(two_i % 2 == 0 and gate_up.is_contiguous(), "gate_up must be contiguous [T, 2I]")
    inter = two_i // 2
    if out is None:
        out = torch.empty((T, inter), dtype=gate_up.dtype, device=gate_up.device)
    _need(out.shape == (T, inter) and out.is_contiguous() and out.dtype == gate_up.dtype, "bad glu_clamped output")
    _check(build.load("elementwise").ullm_glu_clamped(_p(gate_up), _p(out), _c_int(T), _c_int(inter), _c_float(limit),
                                                      _c_float(alpha), _c_int(_dt(gate_up)), _stream()), "glu_clamped")
    return out


def sum_stacks(stacks: torch.Tensor, bias: Optional[torch.Tensor] = None,
               out_dtype: torch.dtype = torch.bfloat16) -> torch.Tensor:
    """The sum over the first dimension of float32 ``stacks`` [S, M, N] (what :func:`gemm_partial_sums` leaves), added
    in order, plus ``bias`` [N], as [M, N] of ``out_dtype``."""
    _need(stacks.dtype == torch.float32 and stacks.dim() == 3 and stacks.is_contiguous() and stacks.shape[2] % 4 == 0,
          "stacks must be contiguous float32 [S, M, N] with N a multiple of 4")
    S, M, N = stacks.shape
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    out = torch.empty((M, N), dtype=out_dtype, device=stacks.device)
    lib = build.load("elementwise")
    _check(lib.ullm_sum_stacks(_p(stacks), _c_int(S), _p(bias), _p(out), _c_int(M), _c_int(N), _c_int(_dt(out)), _stream()),
           "sum_stacks")
    return out


def qk_norm_rope_write(qkv: torch.Tensor, q_out: torch.Tensor, q_gain: Optional[torch.Tensor],
                       k_gain: Optional[torch.Tensor], eps: float, cos_sin: Optional[torch.Tensor],
                       rotary_dim: int, style: int, positions: torch.Tensor, token_entry: torch.Tensor,
                       block_table: torch.Tensor, k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor],
                       page_size: int, nq: int, nkv: int, hd: int, write_kv: bool,
                       values_from_keys: bool = False, norm_dim: int = 0) -> None:
    """Per-head norm and rotation of q (to ``q_out`` [T, nq*hd]) and k, and the cache write of k and v.
    ``qkv`` is [T, (nq + 2 nkv) * hd]; key pool [pages, nkv, page_size, hd], value pool
    [pages, nkv, hd, page_size]; ``block_table`` is
    int32 [B, stride] with one row per batch entry.  With ``values_from_keys`` the row is [T, (nq + nkv) * hd]
    and the values written are the keys as projected, before norm and rotation.  ``norm_dim``: the size the norm's
    mean of squares is taken over (heads stored padded with zeros to ``hd``; 0: ``hd``)."""
    T = qkv.shape[0]
    _need(qkv.dim() == 2 and qkv.shape[1] == (nq + (1 if values_from_keys else 2) * nkv) * hd and qkv.stride(1) == 1,
          "bad qkv shape")
    _need(q_out.shape == (T, nq * hd) and q_out.is_contiguous() and q_out.dtype == qkv.dtype, "bad q_out")
    _need(hd <= 512, f"head_dim {hd} exceeds 512")
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    for g, nm in ((q_gain, "q_gain"), (k_gain, "k_gain")):
        if g is not None:
            _need(g.dtype == torch.float32 and g.numel() == hd and g.is_contiguous(), f"{nm} must be float32 [hd]")
    table_rows = 0
    if style != 0 and rotary_dim > 0:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.dim() == 2
              and cos_sin.shape[1] == rotary_dim and cos_sin.is_contiguous(),
              "cos_sin must be float32 [positions, rotary_dim]")
        table_rows = cos_sin.shape[0]
    if write_kv:
        _check_pools(k_pool, v_pool, nkv, page_size, hd, qkv.dtype)
    lib = build.load("elementwise")
    _check(lib.ullm_qk_norm_rope_write(
        _p(qkv), _c_int(qkv.stride(0)), _p(q_out), _c_int(q_out.stride(0)), _p(q_gain), _p(k_gain),
        _c_float(eps), _p(cos_sin), _c_int(table_rows), _c_int(rotary_dim), _c_int(style), _p(positions),
        _p(token_entry), _p(block_table), _c_int(block_table.stride(0)), _p(k_pool), _p(v_pool),
        _c_int(page_size), _c_int(T), _c_int(nq), _c_int(nkv), _c_int(hd), _c_int(1 if write_kv else 0),
        _c_int(nq if values_from_keys else nq + nkv), _c_int(norm_dim or hd), _c_int(_dt(qkv)), _stream()), "qk_norm_rope_write")



def scale_(x: torch.Tensor, s: float) -> torch.Tensor:
    """x *= s in place, float32 [rows, cols]."""
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.stride(1) == 1, "scale_ takes float32 [rows, cols]")
    _check(build.load("elementwise").ullm_scale(_p(x), _c_int(x.shape[0]), _c_int(x.shape[1]), _c_int(x.stride(0)),
                                                _c_float(s), _stream()), "scale")
    return x


def embedding_sum(ids: torch.Tensor, table: torch.Tensor, scale: float, pair_table: Optional[torch.Tensor],
                  mul_prev: int, mul_cur: int, position_table: Optional[torch.Tensor], positions: torch.Tensor,
                  token_entry: torch.Tensor, q_start: torch.Tensor, entry_slot: torch.Tensor,
                  last_id: Optional[torch.Tensor]) -> torch.Tensor:
    """float32 [T, H]: ``scale`` * table[ids] + pair_table[row] + position_table[positions].  ``pair_table``
    [buckets + 1, H] is read at (previous id * mul_prev + id * mul_cur) mod buckets, at row ``buckets`` for a
    request's first token; the id before an entry's first token comes from ``last_id`` (int32 [slots, 1], row =
    the entry's slot), where the entry's last id is left afterwards.  Either table may be None."""
    T = ids.numel()
    V, H = table.shape
    _i32(ids, "ids")
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _i32(q_start, "q_start")
    _i32(entry_slot, "entry_slot")
    _need(table.is_contiguous(), "embedding table must be contiguous")
    pair_rows = 0
    if pair_table is not None:
        _need(pair_table.is_contiguous() and pair_table.dim() == 2 and pair_table.shape[1] == H
              and pair_table.dtype == table.dtype and pair_table.shape[0] >= 2, "pair table must be [buckets + 1, H]")
        _need(last_id is not None and last_id.dtype == torch.int32 and last_id.is_contiguous()
              and last_id.numel() == last_id.shape[0], "last_id must be contiguous int32 [slots, 1]")
        pair_rows = pair_table.shape[0] - 1
    if position_table is not None:
        _need(position_table.dtype == torch.float32 and position_table.is_contiguous() and position_table.dim() == 2
              and position_table.shape[1] == H, "position table must be float32 [positions, H]")
    out = torch.empty((T, H), dtype=torch.float32, device=table.device)
    ll = ctypes.c_longlong
    _check(build.load("elementwise").ullm_embedding_sum(
        _p(ids), _p(table), _c_float(scale), _p(pair_table), ll(pair_rows), ll(int(mul_prev)), ll(int(mul_cur)),
        _p(position_table), _c_int(0 if position_table is None else position_table.shape[0]), _p(positions),
        _p(token_entry), _p(q_start), _p(entry_slot), _p(last_id), _p(out), _c_int(T), _c_int(H), _c_int(V),
        _c_int(_dt(table)), _stream()), "embedding_sum")
    return out


NORM_RMS, NORM_LAYER = 0, 1       # kinds of norm the general add + norm kernel knows


def add_norm_general(branch: Optional[torch.Tensor], residual: torch.Tensor, gain: Optional[torch.Tensor], eps: float,
                     kind: int, out_dtype: Optional[torch.dtype], rows: Optional[torch.Tensor] = None,
                     post_gain: Optional[torch.Tensor] = None, post_eps: float = 0.0, post_kind: int = NORM_RMS,
                     mult: float = 1.0) -> Optional[torch.Tensor]:
    """residual (float32 [T, H], in place unless ``rows``) += mult * b, where b is ``branch`` [T, H] or, with
    ``post_gain``, the norm of the branch (``post_kind``, ``post_eps``) times that gain; returns the norm
    (``kind``: NORM_RMS or NORM_LAYER, the layer norm without a bias) of the sum times ``gain`` in ``out_dtype``,
    or None with ``gain`` None (then only the stream is updated).  Everything is computed in 32-bit."""
    T, H = residual.shape
    _need(residual.dtype == torch.float32 and residual.is_contiguous(), "residual must be contiguous float32")
    for g, nm in ((gain, "gain"), (post_gain, "post_gain")):
        if g is not None:
            _need(g.dtype == torch.float32 and g.numel() == H and g.is_contiguous(), f"{nm} must be float32 [H]")
    if branch is not None:
        _need(branch.shape == (T, H) and branch.is_contiguous(), "branch must be contiguous [T, H]")
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    out = None
    if gain is not None:
        out = torch.empty((n, H), dtype=out_dtype, device=residual.device)
    bdt = _dt(branch) if branch is not None else F32
    _check(build.load("elementwise").ullm_add_norm_general(
        _p(branch), _p(residual), _p(post_gain), _c_float(post_eps), _c_int(post_kind), _c_float(mult), _p(gain),
        _c_float(eps), _c_int(kind), _p(out), _p(rows), _c_int(n), _c_int(H), _c_int(bdt),
        _c_int(_dt(out) if out is not None else F32), _c_int(0 if rows is not None else 1), _stream()), "add_norm_general")
    return out


def qk_whole_norm_write(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, q_out: torch.Tensor,
                        q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float, q_count: int,
                        k_count: int, positions: torch.Tensor, token_entry: torch.Tensor, block_table: torch.Tensor,
                        k_pool: Optional[torch.Tensor], v_pool: Optional[torch.Tensor], page_size: int, nq: int,
                        nkv: int, hd: int, has_kv: bool) -> None:
    """q (columns ``q_off``.. of ``proj``, nq*hd values) and, with ``has_kv``, k (``k_off``.., nkv*hd values) are
    divided by the root mean square over all their values of a token at once (sum of squares / ``q_count`` resp.
    ``k_count``, eps inside the root) and multiplied by a gain per value (float32 [nq*hd], [nkv*hd]; None: no norm);
    q goes to ``q_out`` [T, nq*hd], k and v (``v_off``..) to the paged pools."""
    T = proj.shape[0]
    width = proj.shape[1]
    _need(proj.dim() == 2 and proj.stride(1) == 1, "proj must be [T, columns]")
    _need(0 <= q_off and q_off + nq * hd <= width, "q columns outside the projection")
    _need(q_out.shape == (T, nq * hd) and q_out.is_contiguous() and q_out.dtype == proj.dtype, "bad q_out")
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    for g, nm, n in ((q_gain, "q_gain", nq * hd), (k_gain, "k_gain", nkv * hd)):
        if g is not None:
            _need(g.dtype == torch.float32 and g.numel() == n and g.is_contiguous(), f"{nm} must be float32 [{n}]")
    if has_kv:
        _need(0 <= k_off and k_off + nkv * hd <= width and 0 <= v_off and v_off + nkv * hd <= width,
              "k or v columns outside the projection")
        _check_pools(k_pool, v_pool, nkv, page_size, hd, proj.dtype)
    _check(build.load("elementwise").ullm_qk_whole_norm_write(
        _p(proj), _c_int(proj.stride(0)), _c_int(q_off), _c_int(k_off), _c_int(v_off), _p(q_out), _c_int(q_out.stride(0)),
        _p(q_gain), _p(k_gain), _c_float(eps), _c_float(float(q_count)), _c_float(float(k_count)), _p(positions),
        _p(token_entry), _p(block_table), _c_int(block_table.stride(0)), _p(k_pool if has_kv else None),
        _p(v_pool if has_kv else None), _c_int(page_size), _c_int(T), _c_int(nq), _c_int(nkv), _c_int(hd),
        _c_int(1 if has_kv else 0), _c_int(_dt(proj)), _stream()), "qk_whole_norm_write")


def head_gate_(x: torch.Tensor, gate: torch.Tensor, nq: int, hd: int) -> torch.Tensor:
    """x [T, nq*hd] *= sigmoid(gate [T, >= nq])[:, head] in place (``gate`` may be columns of a wider row)."""
    T = x.shape[0]
    _need(x.shape == (T, nq * hd) and x.is_contiguous(), "x must be contiguous [T, nq*hd]")
    _need(gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= nq and gate.stride(1) == 1 and gate.dtype == x.dtype,
          "gate must be [T, >= nq] of x's dtype")
    _check(build.load("elementwise").ullm_head_gate(_p(x), _p(gate), _c_int(gate.stride(0)), _c_int(T), _c_int(nq),
                                                    _c_int(hd), _c_int(_dt(x)), _stream()), "head_gate")
    return x


# ---------------------------------------------------------------------------------- recurrent mixers

CONV_MAX_TAPS = 16


def conv_silu(proj: torch.Tensor, in_off: int, channels: int, weight: torch.Tensor, bias: Optional[torch.Tensor],
              carry: torch.Tensor, token_entry: torch.Tensor, q_start: torch.Tensor, entry_slot: torch.Tensor,
              n_entries: int, update_carry: bool = True) -> torch.Tensor:
    """silu of a causal convolution per channel over each entry's tokens: float32 [T, channels] from columns
    ``in_off``.. of ``proj`` (float32 [T, columns]), ``weight`` float32 [channels, taps] (the last column is the
    current token's), ``bias`` float32 [channels].  ``carry`` (float32 [slots, >= (taps-1)*channels]; may be a view
    of wider rows) holds the inputs of the taps-1 tokens before the step in the entry's slot row and takes those
    of the entry's last tokens afterwards."""
    T = proj.shape[0]
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, columns]")
    _need(weight.dtype == torch.float32 and weight.dim() == 2 and weight.shape[0] == channels and weight.is_contiguous(),
          "conv weight must be contiguous float32 [channels, taps]")
    taps = weight.shape[1]
    _need(1 <= taps <= CONV_MAX_TAPS, f"a convolution of {taps} taps: at most {CONV_MAX_TAPS}")
    _need(in_off >= 0 and in_off + channels <= proj.shape[1], "convolution channels outside the projection")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == channels and bias.is_contiguous(), "conv bias must be float32 [channels]")
    _need(carry.dtype == torch.float32 and carry.dim() == 2 and carry.stride(1) == 1
          and carry.shape[1] >= (taps - 1) * channels, "carry must be float32 [slots, >= (taps-1)*channels]")
    _i32(token_entry, "token_entry", T)
    _i32(q_start, "q_start", n_entries + 1)
    _i32(entry_slot, "entry_slot", n_entries)
    out = torch.empty((T, channels), dtype=torch.float32, device=proj.device)
    _check(build.load("recurrent").ullm_conv_silu(
        _p(proj), _c_int(proj.stride(0)), _c_int(in_off), _p(weight), _p(bias), _p(carry), ctypes.c_longlong(carry.stride(0)),
        _p(token_entry), _p(q_start), _p(entry_slot), _p(out), _c_int(T), _c_int(n_entries), _c_int(channels), _c_int(taps),
        _c_int(1 if update_carry else 0), _stream()), "conv_silu")
    return out


def ssm_scan(xbc: torch.Tensor, proj: torch.Tensor, dt_off: int, dt_bias: torch.Tensor, a_log: torch.Tensor,
             d_skip: torch.Tensor, state: torch.Tensor, state_off: int, q_start: torch.Tensor, entry_slot: torch.Tensor,
             n_entries: int, heads: int, groups: int, n_state: int, head_dim: int, write_state: bool = True) -> torch.Tensor:
    """The selective state-space recurrence over each entry's tokens: per head h with state S [n_state, head_dim]
    (float32, at ``state[slot, state_off + h * n_state * head_dim ..]``), dt = softplus(proj[t, dt_off + h] + dt_bias[h]),
    S = exp(-exp(a_log[h]) dt) S + dt B x^T, y = S^T C + d_skip[h] x, with x | B | C the columns of ``xbc``
    (float32 [T, heads*head_dim + 2*groups*n_state]).  Returns y float32 [T, heads*head_dim]."""
    T = xbc.shape[0]
    channels = heads * head_dim + 2 * groups * n_state
    _need(xbc.dtype == torch.float32 and xbc.shape == (T, channels) and xbc.is_contiguous(), "xbc must be contiguous float32 [T, x|B|C]")
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[0] == T
          and 0 <= dt_off and dt_off + heads <= proj.shape[1], "proj must be float32 [T, columns] with the dt columns inside")
    for v, nm in ((dt_bias, "dt_bias"), (a_log, "a_log"), (d_skip, "d_skip")):
        _need(v.dtype == torch.float32 and v.numel() == heads and v.is_contiguous(), f"{nm} must be float32 [heads]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1
          and state_off >= 0 and state_off + heads * n_state * head_dim <= state.shape[1], "state must be float32 [slots, row] holding the heads' states")
    _need(heads % groups == 0 and head_dim <= 256, "heads must be a multiple of groups and head_dim at most 256")
    _i32(q_start, "q_start", n_entries + 1)
    _i32(entry_slot, "entry_slot", n_entries)
    y = torch.empty((T, heads * head_dim), dtype=torch.float32, device=xbc.device)
    ll = ctypes.c_longlong
    _check(build.load("recurrent").ullm_ssm_scan(
        _p(xbc), _p(proj), _c_int(proj.stride(0)), _c_int(dt_off), _p(dt_bias), _p(a_log), _p(d_skip), _p(state),
        ll(state.stride(0)), ll(state_off), _p(q_start), _p(entry_slot), _p(y), _c_int(n_entries), _c_int(heads),
        _c_int(groups), _c_int(n_state), _c_int(head_dim), _c_int(1 if write_state else 0), _stream()), "ssm_scan")
    return y


def gated_group_norm(y: torch.Tensor, proj: torch.Tensor, z_off: int, gain: torch.Tensor, eps: float, parts: int,
                     out_dtype: torch.dtype) -> torch.Tensor:
    """(y * silu(z)) cut into ``parts`` equal parts, each divided by its own root mean square (eps inside the root),
    times ``gain``: y float32 [T, width], z = columns ``z_off``.. of ``proj`` (float32), result in ``out_dtype``."""
    T, width = y.shape
    _need(y.dtype == torch.float32 and y.is_contiguous(), "y must be contiguous float32")
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1 and proj.shape[0] == T
          and 0 <= z_off and z_off + width <= proj.shape[1], "proj must be float32 [T, columns] with the gate columns inside")
    _need(gain.dtype == torch.float32 and gain.numel() == width and gain.is_contiguous(), "gain must be float32 [width]")
    _need(parts >= 1 and width % parts == 0, f"{width} values do not cut into {parts} equal parts")
    out = torch.empty((T, width), dtype=out_dtype, device=y.device)
    _check(build.load("recurrent").ullm_gated_group_norm(
        _p(y), _p(proj), _c_int(proj.stride(0)), _c_int(z_off), _p(gain), _c_float(eps), _p(out), _c_int(T), _c_int(width),
        _c_int(parts), _c_int(_dt(out)), _stream()), "gated_group_norm")
    return out


# ---------------------------------------------------------------------------------- several copies of the stream

STREAMS_MAX = 8          # the most copies of the residual stream the kernels take


def streams_spread(x: torch.Tensor, copies: int) -> torch.Tensor:
    """float32 [copies, T, H] whose every slice is ``x`` (float32 [T, H])."""
    _need(x.dtype == torch.float32 and x.dim() == 2 and x.is_contiguous(), "x must be contiguous float32 [T, H]")
    _need(1 <= copies <= STREAMS_MAX, f"{copies} copies of the stream: 1 to {STREAMS_MAX}")
    out = torch.empty((copies,) + tuple(x.shape), dtype=torch.float32, device=x.device)
    _check(build.load("streams").ullm_streams_spread(_p(x), _p(out), ctypes.c_longlong(x.numel()), _c_int(copies), _stream()),
           "streams_spread")
    return out


def streams_step(streams: torch.Tensor, branch: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                 out_w: Optional[torch.Tensor] = None, mult: float = 1.0, in_w: Optional[torch.Tensor] = None,
                 gain: Optional[torch.Tensor] = None, eps: float = 0.0, kind: int = NORM_RMS,
                 out_dtype: Optional[torch.dtype] = None, rows: Optional[torch.Tensor] = None,
                 second: Optional[torch.Tensor] = None, a: float = 1.0, b: float = 1.0) -> Optional[torch.Tensor]:
    """What lies between two sublayers of a model that keeps ``streams`` (float32 [S, T, H]) copies of its residual
    stream.  With ``branch`` ([T, H]; with ``second`` the branch is ``a * branch + b * second``): every copy t becomes
    sum_s mix[s, t] * copy_s + mult * out_w[t] * branch, all from the old copies (``mix`` float32 [S, S] indexed
    [from, to], ``out_w`` float32 [S]); written back in place unless ``rows``.  With ``gain``: returns the norm
    (``kind``: NORM_RMS or NORM_LAYER, the layer norm without a bias) of sum_s in_w[s] * copy_s times ``gain`` in
    ``out_dtype``, for all tokens or the ones ``rows`` (int32) lists.  Everything is computed in 32-bit."""
    _need(streams.dtype == torch.float32 and streams.dim() == 3 and streams.is_contiguous(), "streams must be contiguous float32 [S, T, H]")
    S, T, H = streams.shape
    _need(1 <= S <= STREAMS_MAX, f"{S} copies of the stream: 1 to {STREAMS_MAX}")
    y_dt = F32
    if branch is not None:
        _need(branch.shape == (T, H) and branch.is_contiguous(), "the branch must be contiguous [T, H]")
        _need(mix is not None and mix.dtype == torch.float32 and mix.shape == (S, S) and mix.is_contiguous(), "mix must be float32 [S, S]")
        _need(out_w is not None and out_w.dtype == torch.float32 and out_w.numel() == S and out_w.is_contiguous(), "out_w must be float32 [S]")
        y_dt = _dt(branch)
        if second is not None:
            _need(second.shape == (T, H) and second.is_contiguous() and second.dtype == branch.dtype, "the second branch must match the first")
    else:
        _need(second is None, "a second branch needs a first")
    n = T
    if rows is not None:
        _i32(rows, "rows")
        n = rows.numel()
    out = None
    if gain is not None:
        _need(gain.dtype == torch.float32 and gain.numel() == H and gain.is_contiguous(), "gain must be float32 [H]")
        _need(in_w is not None and in_w.dtype == torch.float32 and in_w.numel() == S and in_w.is_contiguous(), "in_w must be float32 [S]")
        out = torch.empty((n, H), dtype=out_dtype or torch.float32, device=streams.device)
    _check(build.load("streams").ullm_streams_step(
        _p(streams), _p(branch), _p(second), _c_float(a), _c_float(b), _c_int(y_dt), _p(mix), _p(out_w), _c_float(mult),
        _p(in_w), _p(gain), _c_float(eps), _c_int(kind), _p(out), _c_int(_dt(out) if out is not None else F32), _p(rows),
        _c_int(n), _c_int(T), _c_int(H), _c_int(S), _stream()), "streams_step")
    return out


def weighted_sum(x: torch.Tensor, y: torch.Tensor, a: float, b: float) -> torch.Tensor:
    """float32 a * x + b * y for two contiguous tensors of one shape."""
    _need(x.shape == y.shape and x.is_contiguous() and y.is_contiguous(), "weighted_sum takes two contiguous tensors of one shape")
    out = torch.empty(x.shape, dtype=torch.float32, device=x.device)
    _check(build.load("streams").ullm_weighted_sum(_p(x), _c_int(_dt(x)), _p(y), _c_int(_dt(y)), _c_float(a), _c_float(b),
                                                   _p(out), ctypes.c_longlong(x.numel()), _stream()), "weighted_sum")
    return out


# ---------------------------------------------------------------------------------- recurrences with decays

DECAY_PER_HEAD, DECAY_SIGMOID_ROOT, DECAY_EXP_EXP, DECAY_READY = 0, 1, 2, 3      # how a recurrence's decays come about
GATE_SILU, GATE_SIGMOID = 0, 1
DECAY_SCAN_MAX_KEYS = 512


def _f32_rows(t: torch.Tensor, name: str, T: int, cols: int) -> None:
    _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape == (T, cols) and t.stride(1) == 1,
          f"{name} must be float32 [{T}, {cols}] with unit stride along its rows")


def decay_scan(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor, decay_kind: int,
               state: torch.Tensor, state_off: int, q_start: torch.Tensor, entry_slot: torch.Tensor, n_entries: int,
               heads: int, key_dim: int, value_dim: int, tau: float = 1.0, bonus: Optional[torch.Tensor] = None,
               silu_inputs: bool = False, q_scale: float = 1.0, write_state: bool = True, max_len: int = 0) -> torch.Tensor:
    """A recurrence per head over each entry's tokens, with the head's state S [key_dim, value_dim] (float32, at
    ``state[slot, state_off + head * key_dim * value_dim ..]``): S = diag(d) S + k v^T and o = S^T q after the
    update, or with ``bonus`` (float32 [heads, key_dim]) o = (S + diag(bonus) k v^T)^T q before it.  ``q``, ``k``
    (float32 [T, heads * key_dim]) and ``v`` (float32 [T, heads * value_dim]) may be column ranges of wider rows; with
    ``silu_inputs`` they go through silu first; q is multiplied by ``q_scale``.  The decays d: ``decay`` float32
    [heads] (DECAY_PER_HEAD: one constant a head) or raw values z float32 [T, heads * key_dim] with d =
    sigmoid(z)^(1/tau) (DECAY_SIGMOID_ROOT) or exp(-exp(z)) (DECAY_EXP_EXP), or the decays themselves (DECAY_READY:
    :func:`decay_prepare` has been over them).  ``max_len``: the most tokens any entry brings, if known (1: a step of
    single tokens takes a variant of the kernel made for it).  Returns o float32 [T, heads * value_dim]."""
    T = q.shape[0]
    _f32_rows(q, "q", T, heads * key_dim)
    _f32_rows(k, "k", T, heads * key_dim)
    _f32_rows(v, "v", T, heads * value_dim)
    _need(1 <= key_dim <= DECAY_SCAN_MAX_KEYS, f"{key_dim} key channels a head: at most {DECAY_SCAN_MAX_KEYS}")
    if decay_kind == DECAY_PER_HEAD:
        _need(decay.dtype == torch.float32 and decay.numel() == heads and decay.is_contiguous(), "decay must be float32 [heads]")
        z_ld = 0
    else:
        _need(decay_kind in (DECAY_SIGMOID_ROOT, DECAY_EXP_EXP, DECAY_READY), "unknown kind of decay")
        _f32_rows(decay, "decay", T, heads * key_dim)
        z_ld = decay.stride(0)
    if bonus is not None:
        _need(bonus.dtype == torch.float32 and bonus.numel() == heads * key_dim and bonus.is_contiguous(), "bonus must be float32 [heads, key_dim]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and state_off >= 0
          and state_off + heads * key_dim * value_dim <= state.shape[1], "state must be float32 [slots, row] holding the heads' states")
    _i32(q_start, "q_start", n_entries + 1)
    _i32(entry_slot, "entry_slot", n_entries)
    ll = ctypes.c_longlong
    out = torch.empty((T, heads * value_dim), dtype=torch.float32, device=q.device)
    _check(build.load("decay_scan").ullm_decay_scan(
        _p(q), _c_int(q.stride(0)), _p(k), _c_int(k.stride(0)), _p(v), _c_int(v.stride(0)), _p(decay), _c_int(z_ld),
        _c_int(decay_kind), _c_float(tau), _p(bonus), _c_int(1 if silu_inputs else 0), _c_float(q_scale),
        _c_int(1 if bonus is not None else 0), _p(state), ll(state.stride(0)), ll(state_off), _p(q_start), _p(entry_slot),
        _p(out), _c_int(n_entries), _c_int(heads), _c_int(key_dim), _c_int(value_dim), _c_int(1 if write_state else 0),
        _c_int(max_len), _stream()), "decay_scan")
    return out


DECAY_PREPARE_FROM = 16      # from this many tokens a step on, a pass of its own applies the inputs' functions


def decay_prepare(x: Optional[torch.Tensor], decay: Optional[torch.Tensor] = None, decay_kind: int = DECAY_EXP_EXP,
                  tau: float = 1.0) -> None:
    """In place, ahead of :func:`decay_scan` in a step of many tokens: silu over ``x`` (float32 [T, columns], may be a
    column range of wider rows) and the decay's function (``decay_kind``) over the raw decays ``decay`` (float32
    [T, columns]); either may be None.  The recurrence is then called without ``silu_inputs`` and with DECAY_READY."""
    T = (x if x is not None else decay).shape[0]
    for t, nm in ((x, "x"), (decay, "decay")):
        if t is not None:
            _need(t.dtype == torch.float32 and t.dim() == 2 and t.shape[0] == T and t.stride(1) == 1, f"{nm} must be float32 [T, columns]")
    _check(build.load("decay_scan").ullm_decay_prepare(
        _p(x), _c_int(x.stride(0) if x is not None else 0), _c_int(x.shape[1] if x is not None else 0), _p(decay),
        _c_int(decay.stride(0) if decay is not None else 0), _c_int(decay.shape[1] if decay is not None else 0),
        _c_int(decay_kind), _c_float(tau), _c_int(T), _stream()), "decay_prepare")


def token_shift(x: torch.Tensor, mu: torch.Tensor, state: torch.Tensor, state_off: int, token_entry: torch.Tensor,
                q_start: torch.Tensor, entry_slot: torch.Tensor, n_entries: int, write_state: bool = True) -> torch.Tensor:
    """[M, T, H] of x's dtype: slice m is x[t] + (prev(t) - x[t]) * mu[m] (``mu`` float32 [M, H]) with prev(t) the row
    before t in its entry or, for an entry's first token, ``state[slot, state_off .. + H]`` (float32: the last row
    of the step before); that part of the state row then takes the entry's last row."""
    T, H = x.shape
    _need(x.is_contiguous(), "x must be contiguous [T, H]")
    _need(mu.dtype == torch.float32 and mu.dim() == 2 and mu.shape[1] == H and mu.is_contiguous(), "mu must be float32 [M, H]")
    _need(state.dtype == torch.float32 and state.dim() == 2 and state.stride(1) == 1 and 0 <= state_off
          and state_off + H <= state.shape[1], "state must be float32 [slots, row] holding a row of H values")
    _i32(token_entry, "token_entry", T)
    _i32(q_start, "q_start", n_entries + 1)
    _i32(entry_slot, "entry_slot", n_entries)
    M = mu.shape[0]
    out = torch.empty((M, T, H), dtype=x.dtype, device=x.device)
    ll = ctypes.c_longlong
    _check(build.load("decay_scan").ullm_token_shift(
        _p(x), _p(mu), _p(state), ll(state.stride(0)), ll(state_off), _p(token_entry), _p(q_start), _p(entry_slot), _p(out),
        _c_int(T), _c_int(H), _c_int(M), _c_int(1 if write_state else 0), _c_int(_dt(x)), _stream()), "token_shift")
    return out


def gated_unit_norm(o: torch.Tensor, gate: torch.Tensor, gain: torch.Tensor, eps: float, parts: int, gate_kind: int,
                    out_dtype: torch.dtype) -> torch.Tensor:
    """Rows ``o`` (float32 [T, width], or [slices, T, width] whose slices are added first, in their order) cut into ``parts`` equal parts, each divided by its root mean square (eps inside
    the root), times ``gain`` (float32; as long as a part, shared by the parts, or as long as the row) and times
    silu or sigmoid (``gate_kind``) of ``gate`` (float32 [T, width], may be a column range of wider rows)."""
    slices = 1
    if o.dim() == 3:
        slices = o.shape[0]
    T, width = o.shape[-2:]
    _need(o.dtype == torch.float32 and o.is_contiguous(), "o must be contiguous float32 [T, width] or [slices, T, width]")
    _f32_rows(gate, "gate", T, width)
    _need(parts >= 1 and width % parts == 0, f"{width} values do not cut into {parts} equal parts")
    _need(gain.dtype == torch.float32 and gain.is_contiguous() and gain.numel() in (width // parts, width),
          "gain must be float32, as long as a part or as the row")
    out = torch.empty((T, width), dtype=out_dtype, device=o.device)
    _check(build.load("decay_scan").ullm_gated_unit_norm(
        _p(o), _p(gate), _c_int(gate.stride(0)), _p(gain), _c_int(gain.numel()), _c_float(eps), _c_int(gate_kind), _p(out),
        _c_int(T), _c_int(width), _c_int(parts), _c_int(slices), _c_int(_dt(out)), _stream()), "gated_unit_norm")
    return out


# ---------------------------------------------------------------------------------- attention

def _check_gate(gate: Optional[torch.Tensor], T: int, nq: int) -> None:
    if gate is not None:
        _need(gate.dtype == torch.bfloat16 and gate.dim() == 2 and gate.shape[0] == T and gate.shape[1] >= nq
              and gate.stride(1) == 1, f"a head gate must be bfloat16 [T, >= {nq}]")


def _check_distance_bias(bias: Optional[torch.Tensor], nq: int) -> int:
    """Rows of a distance-bias table (0 for none) after checking that it is float32 [nq, rows]."""
    if bias is None:
        return 0
    _need(bias.dtype == torch.float32 and bias.dim() == 2 and bias.shape[0] == nq and bias.shape[1] >= 1
          and bias.is_contiguous(), f"a distance bias must be contiguous float32 [{nq}, rows]")
    return bias.shape[1]


def _check_sink(sink: Optional[torch.Tensor], nq: int) -> None:
    if sink is not None:
        _need(sink.dtype == torch.float32 and sink.numel() == nq and sink.is_contiguous(),
              f"attention sinks must be contiguous float32 [{nq}]")


def paged_attention_generic(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor,
                            positions: torch.Tensor, token_entry: torch.Tensor, block_table: torch.Tensor,
                            page_size: int, nq: int, nkv: int, hd: int, scale: float, window: int,
                            out: Optional[torch.Tensor] = None, bias: Optional[torch.Tensor] = None,
                            sink: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``bias`` (float32 [nq, rows]): bias[h, min(distance, rows - 1)] is added to the scaled score of a key
    ``distance`` positions behind the query.  ``sink`` (float32 [nq]): exp(sink[h]) is one more term of the
    softmax's denominator, with no key and no value."""
    _check_sink(sink, nq)
    T = q.shape[0]
    _need(q.shape == (T, nq * hd) and q.stride(1) == 1, "q must be [T, nq*hd]")
    _need(hd <= 1024 and nq % nkv == 0, "head_dim > 1024 or heads not a multiple of kv heads")
    _check_pools(k_pool, v_pool, nkv, page_size, hd, q.dtype)
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    if out is None:
        out = torch.empty((T, nq * hd), dtype=q.dtype, device=q.device)
    _need(out.shape == (T, nq * hd) and out.is_contiguous() and out.dtype == q.dtype, "bad attention output")
    lib = build.load("attention_generic")
    _check(lib.ullm_paged_attention_generic(
        _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(positions),
        _p(token_entry), _p(block_table), _c_int(block_table.stride(0)), _c_int(page_size), _c_int(T),
        _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window), _p(bias),
        _c_int(_check_distance_bias(bias, nq)), _p(sink), _c_int(_dt(q)), _stream()),
        "paged_attention_generic")
    return out


# ---------------------------------------------------------------------------------- matrix products

def gemm_simple(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """a [M, K] times w [N, K] transposed (+ bias float32 [N]); 32-bit multiply-add in fixed K order."""
    M, K = a.shape
    N, K2 = w.shape
    _need(K == K2, f"inner sizes differ: a is [{M}, {K}], w is [{N}, {K2}]")
    _need(a.stride(1) == 1 and w.stride(1) == 1, "a and w must have unit stride along K")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "bad gemm output")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    lib = build.load("gemm_simple")
    _check(lib.ullm_gemm_simple(_p(a), _c_int(a.stride(0)), _p(w), _c_int(w.stride(0)), _p(bias), _p(out),
                                _c_int(out.stride(0)), _c_int(M), _c_int(N), _c_int(K), _c_int(_dt(a)),
                                _c_int(_dt(w)), _c_int(_dt(out)), _stream()), "gemm_simple")
    return out


def _skinny_ok(M: int, K: int, x: torch.Tensor, w: torch.Tensor) -> bool:
    return (w.dtype == torch.bfloat16 and 1 <= M <= 64 and K % 8 == 0 and K >= 8 and x.stride(1) == 1
            and w.stride(1) == 1 and x.stride(0) % 8 == 0 and w.stride(0) % 8 == 0 and x.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0)


def gemm_skinny_supports(a: torch.Tensor, w: torch.Tensor) -> bool:
    return a.dtype == torch.bfloat16 and _skinny_ok(a.shape[0], a.shape[1], a, w)


def _gemm_skinny(x, w, bias, c, M, N, K, epi, c_dtype, nt=0, waves=0, gain=None, eps=0.0, rows=0,
                 ahead=None, squares=None, unit_limit=0.0, unit_alpha=0.0, act=0) -> None:
    """``ahead``: (next gain, next x, next squares) that an adding product leaves for the norm after it;
    ``squares``: the [parts, M] sums such a product left, which scale this product's rows."""
    lib = build.load("gemm_skinny")
    next_gain, next_x, next_sq = ahead if ahead is not None else (None, None, None)
    _check(lib.ullm_gemm_skinny(_p(x), _c_int(x.stride(0)), _p(w), _c_int(w.stride(0)), _p(bias),
                                _p(c), _c_int(c.stride(0)), _c_int(M), _c_int(N), _c_int(K),
                                _c_int(epi), _c_int(c_dtype), _c_int(nt), _c_int(waves), _p(gain),
                                ctypes.c_float(eps), _c_int(rows), _p(next_gain), _p(next_x),
                                _c_int(next_x.stride(0) if next_x is not None else 0), _p(next_sq), _p(squares),
                                _c_int(squares.shape[1] if squares is not None else 0), _c_float(unit_limit),
                                _c_float(unit_alpha), _c_int(act), _stream()),
           "gemm_skinny")


def _check_squares(squares: Optional[torch.Tensor], M: int) -> None:
    if squares is not None:
        _need(M <= 16 and squares.dtype == torch.float32 and squares.dim() == 2 and squares.shape[0] == M
              and squares.shape[1] >= 4 and squares.shape[1] % 4 == 0 and squares.is_contiguous()
              and squares.data_ptr() % 16 == 0, f"row squares must be float32 [{M} <= 16, a multiple of 4]")


def gemm_skinny(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
                out_dtype: Optional[torch.dtype] = None, out: Optional[torch.Tensor] = None,
                nt: int = 0, waves: int = 0, rows: int = 0, squares: Optional[torch.Tensor] = None,
                eps: float = 0.0, act: Optional[int] = None) -> torch.Tensor:
    """a [M <= 64, K] times w [N, K] transposed, bfloat16 operands streamed once through the matrix
    cores, 32-bit accumulation; output bfloat16 or float32; ``act`` (ACT_RELU2, ACT_GELU_TANH): that activation of
    the 32-bit sums (+ bias) on store.  With ``squares`` (float32 [M <= 16, parts], see
    :func:`gemm_skinny_add`) row m of the product is scaled by rsqrt(sum of squares[m] / K + eps) before
    the bias: a is then a stream times a norm's gain and the result the product of the normed stream."""
    M, K = a.shape
    N, K2 = w.shape
    _need(K == K2, f"inner sizes differ: a is [{M}, {K}], w is [{N}, {K2}]")
    _need(gemm_skinny_supports(a, w), "gemm_skinny takes bfloat16, M <= 64, K a multiple of 8, 16-byte aligned rows")
    if out is None:
        out = torch.empty((M, N), dtype=out_dtype or a.dtype, device=a.device)
    _need(out.shape == (M, N) and out.stride(1) == 1, "bad gemm output")
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    _check_squares(squares, M)
    _gemm_skinny(a, w, bias, out, M, N, K, 0, _dt(out), nt, waves, eps=float(eps), rows=rows, squares=squares,
                 act=0 if act is None else act + 1)
    return out


def gemm_skinny_add(a: torch.Tensor, w: torch.Tensor, residual: torch.Tensor, nt: int = 0, waves: int = 0,
                    rows: int = 0, next_gain: Optional[torch.Tensor] = None):
    """residual (float32 [M, N]) += a (bfloat16 [M, K]) times w transposed.
    With ``next_gain`` (float32 [N], the gain of the RMS norm that is applied to the residual next) the kernel
    also leaves what that norm needs and returns it: (scaled, squares) with scaled = residual * next_gain in
    bfloat16 [M, N] and squares float32 [M, parts], every block's sum of the squares of its columns of a row
    (zeros behind them up to a multiple of four).
    The norm of row m is scaled[m] * rsqrt(squares[m].sum() / N + eps), which a product after it applies
    to its own results (``squares=`` of :func:`gemm_skinny`, :func:`gemm_skinny_silu`, :func:`gemm_rows`)."""
    M = a.shape[0]
    N, K = w.shape
    _need(a.dtype == torch.bfloat16 and a.shape[1] == K and _skinny_ok(M, K, a, w),
          "gemm_skinny_add takes bfloat16 activations [M <= 64, K]")
    _need(residual.dtype == torch.float32 and residual.shape == (M, N) and residual.stride(1) == 1
          and residual.stride(0) % 4 == 0 and residual.data_ptr() % 16 == 0, "residual must be float32 [M, N]")
    if next_gain is None:
        _gemm_skinny(a, w, None, residual, M, N, K, 1, F32, nt, waves, rows=rows)
        return None
    _need(next_gain.dtype == torch.float32 and next_gain.numel() == N and next_gain.is_contiguous()
          and next_gain.data_ptr() % 16 == 0 and N % 4 == 0, "the next norm's gain must be float32 [N], N a multiple of 4")
    blocks = int(build.load("gemm_skinny").ullm_gemm_skinny_blocks(
        _c_int(M), _c_int(N), _c_int(K), _c_int(a.stride(0)), _c_int(w.stride(0)), _c_int(1), _c_int(nt), _c_int(waves),
        _c_int(rows)))
    _check(min(blocks, 0), "gemm_skinny_blocks")
    scaled = torch.empty((M, N), dtype=torch.bfloat16, device=a.device)
    squares = torch.empty((M, -(-blocks // 4) * 4), dtype=torch.float32, device=a.device)
    _gemm_skinny(a, w, None, residual, M, N, K, 1, F32, nt, waves, rows=rows, ahead=(next_gain, scaled, squares))
    return scaled, squares


def gemm_skinny_silu(a: torch.Tensor, w_gate_up: torch.Tensor, nt: int = 0, waves: int = 0, rows: int = 0,
                     squares: Optional[torch.Tensor] = None, eps: float = 0.0, limit: float = 0.0,
                     alpha: float = 0.0) -> torch.Tensor:
    """silu(a g^T) * (a u^T) as bfloat16 [M, I] for a (bfloat16 [M, K]) and the stacked weights
    g | u (bfloat16 [2 I, K]); the activation is applied to the 32-bit sums (with ``squares``: to the sums
    scaled as in :func:`gemm_skinny`).  With ``limit`` > 0 the clamped gated unit of :func:`glu_clamped` instead."""
    M, K = a.shape
    two_i, K2 = w_gate_up.shape
    _need(K == K2 and two_i % 2 == 0, f"gate|up weights must be [2 I, {K}]")
    _need(a.dtype == torch.bfloat16 and _skinny_ok(M, K, a, w_gate_up), "gemm_skinny_silu takes bfloat16 [M <= 64, K]")
    out = torch.empty((M, two_i // 2), dtype=torch.bfloat16, device=a.device)
    _check_squares(squares, M)
    _gemm_skinny(a, w_gate_up, None, out, M, two_i // 2, K, 2, BF16, nt, waves, eps=float(eps), rows=rows, squares=squares,
                 unit_limit=float(limit), unit_alpha=float(alpha))
    return out


NORMED_MAX_ROWS = 16


def gemm_skinny_normed_supports(stream: torch.Tensor, gain: torch.Tensor, w: torch.Tensor) -> bool:
    M, K = stream.shape
    return (stream.dtype == torch.float32 and gain.dtype == torch.float32 and w.dtype == torch.bfloat16
            and M <= NORMED_MAX_ROWS and gain.numel() == K and gain.is_contiguous() and gain.data_ptr() % 16 == 0
            and _skinny_ok(M, K, stream, w))


def gemm_skinny_normed(stream: torch.Tensor, gain: torch.Tensor, eps: float, w: torch.Tensor,
                       bias: Optional[torch.Tensor] = None, out_dtype: torch.dtype = torch.bfloat16,
                       silu: bool = False, nt: int = 0, waves: int = 0, rows: int = 0) -> torch.Tensor:
    """rmsnorm(stream) times w transposed for the float32 residual stream [M <= 16, K], the norm
    (gain float32 [K], eps) folded into the product: the kernel rounds stream * gain to bfloat16 for
    the matrix cores, sums the squares of the rows it reads anyway and scales the 32-bit sums by
    rsqrt(mean + eps).  With silu, w is gate | up [2 I, K] and the result silu(gate) * up [M, I]."""
    M, K = stream.shape
    N, K2 = w.shape
    _need(K == K2, f"inner sizes differ: the stream is [{M}, {K}], w is [{N}, {K2}]")
    _need(gemm_skinny_normed_supports(stream, gain, w),
          "gemm_skinny_normed takes a float32 stream [M <= 16, K], a float32 gain [K] and bfloat16 weights")
    if silu:
        _need(N % 2 == 0 and bias is None and out_dtype == torch.bfloat16, "gate|up weights must be [2 I, K], no bias")
        N //= 2
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == N and bias.is_contiguous(), "bias must be float32 [N]")
    out = torch.empty((M, N), dtype=out_dtype, device=stream.device)
    _gemm_skinny(stream, w, bias, out, M, N, K, 2 if silu else 0, _dt(out), nt, waves, gain, float(eps), rows)
    return out


PARTIAL_SUMS_MAX_ROWS = 256


def gemm_partial_sums_supports(a: torch.Tensor, w: torch.Tensor) -> bool:
    M, K = a.shape
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.stride(1) == 1 and w.stride(1) == 1
            and a.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0 and w.shape[1] == K
            and bool(build.load("gemm_mid").ullm_gemm_partial_sums_supports(
                _c_int(M), _c_int(w.shape[0]), _c_int(K), _c_int(a.stride(0)), _c_int(w.stride(0)))))


def gemm_partial_sums(a: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    """a (bfloat16 [M <= 256, K]) times w (bfloat16 [N, K]) transposed as a stack [S, M, N] of float32
    partial sums over S slices of K; the product is their sum.  S depends on the matrix alone.  For
    17 to 256 rows of the projections that end in the residual stream: the add + norm kernel adds the
    stack (:func:`add_rmsnorm`), so the slices cost no kernel of their own."""
    M, K = a.shape
    N = w.shape[0]
    _need(gemm_partial_sums_supports(a, w), "gemm_partial_sums takes bfloat16, M <= 256, K a multiple of 8, N of 4")
    lib = build.load("gemm_mid")
    slices = int(lib.ullm_gemm_partial_sums_slices(_c_int(N), _c_int(K)))
    out = torch.empty((slices, M, N), dtype=torch.float32, device=a.device)
    _check(lib.ullm_gemm_partial_sums(_p(a), _c_int(a.stride(0)), _p(w), _c_int(w.stride(0)), _p(out), _c_int(M),
                                      _c_int(N), _c_int(K), _stream()), "gemm_partial_sums")
    return out


ROWS_MAX_ROWS = 128       # most rows the kernel takes (which matrices it is chosen for: dispatch.limits)


def gemm_rows_supports(a: torch.Tensor, w: torch.Tensor, silu: bool = False) -> bool:
    M, K = a.shape
    n_out = w.shape[0] // 2 if silu else w.shape[0]
    return (a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.stride(1) == 1 and w.stride(1) == 1
            and w.shape[1] == K and (not silu or w.shape[0] % 2 == 0) and a.data_ptr() % 16 == 0
            and w.data_ptr() % 16 == 0 and n_out % 4 == 0
            and bool(build.load("gemm_rows").ullm_gemm_rows_supports(
                _c_int(M), _c_int(n_out), _c_int(K), _c_int(a.stride(0)), _c_int(w.stride(0)), _c_int(n_out),
                _c_int(1 if silu else 0))))


def gemm_rows(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None, silu: bool = False,
              squares: Optional[torch.Tensor] = None, eps: float = 0.0, limit: float = 0.0,
              alpha: float = 0.0, act: Optional[int] = None) -> torch.Tensor:
    """a (bfloat16 [M <= 128, K]) times w (bfloat16 [N, K]) transposed (+ bias float32 [N]) as bfloat16 [M, N];
    with ``silu``, w is gate | up [2 I, K] and the result silu(gate) * up [M, I] on the 32-bit sums.  The
    matrix is cut into one block per compute unit and every wave keeps several stages of its rows of w in
    flight: for the row counts between the few-rows kernel and the library.  ``squares``, ``eps``: as in
    :func:`gemm_skinny`.  With ``silu`` and ``limit`` > 0 the clamped gated unit of :func:`glu_clamped` instead;
    without ``silu``, ``act`` (ACT_RELU2, ACT_GELU_TANH) is applied to the 32-bit sums (+ bias) on store."""
    _need(silu or limit <= 0, "the clamped unit needs gate | up weights")
    _need(act is None or not silu, "an ungated activation and the gated unit exclude each other")
    M, K = a.shape
    _need(gemm_rows_supports(a, w, silu), "gemm_rows takes bfloat16, M <= 128, K a multiple of 64, N a multiple of 4")
    n_out = w.shape[0] // 2 if silu else w.shape[0]
    if bias is not None:
        _need(not silu and bias.dtype == torch.float32 and bias.numel() == n_out and bias.is_contiguous(),
              "bias must be float32 [N] (and there is none with silu)")
    _check_squares(squares, M)
    out = torch.empty((M, n_out), dtype=torch.bfloat16, device=a.device)
    _check(build.load("gemm_rows").ullm_gemm_rows(_p(a), _c_int(a.stride(0)), _p(w), _c_int(w.stride(0)), _p(bias), _p(out),
                                                  _c_int(n_out), _c_int(M), _c_int(n_out), _c_int(K),
                                                  _c_int(1 if silu else 0), _p(squares),
                                                  _c_int(squares.shape[1] if squares is not None else 0),
                                                  ctypes.c_float(float(eps)), _c_float(float(limit)), _c_float(float(alpha)),
                                                  _c_int(0 if act is None else act + 1), _stream()), "gemm_rows")
    return out


# torch.mm(..., out_dtype=float32) stores the 32-bit accumulator of a bfloat16 product; older torch lacks it
_MM_TAKES_OUT_DTYPE = "out_dtype" in (torch.mm.__doc__ or "")


def gemm_bf16(a: torch.Tensor, w: torch.Tensor, bias: Optional[torch.Tensor] = None,
              out_dtype: Optional[torch.dtype] = None, act: Optional[int] = None) -> torch.Tensor:
    """bfloat16 operands, 32-bit accumulation.  Few rows go to the weight-streaming kernels (up to how many
    for this matrix: :func:`dispatch.limits`), some more, where that was measured to be ahead, to the partial-sums
    kernel and a kernel that adds its stacks; many rows go through the library product (as the reference's
    linears do, ullm/layers/linear.py:165), which for 32-bit output (logits) stores the accumulator unrounded.
    ``act`` (ACT_RELU2, ACT_GELU_TANH): that activation of the result, on store in the few-rows and rows kernels, by
    the activation kernel behind the others."""
    out_dtype = out_dtype or a.dtype
    M = a.shape[0]
    if act is not None:
        lim = dispatch.limits(w.shape[0], w.shape[1])
        if M <= (lim.f32_skinny if out_dtype == torch.float32 else lim.skinny) and gemm_skinny_supports(a, w):
            return gemm_skinny(a, w, bias, out_dtype=out_dtype, act=act)
        if out_dtype == torch.bfloat16 and M <= min(lim.rows, ROWS_MAX_ROWS) and gemm_rows_supports(a, w):
            return gemm_rows(a, w, bias, act=act)
        y = gemm_bf16(a, w, bias, out_dtype)
        return activation(y, act, out=y)
    library = a.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and a.is_cuda
    lim = dispatch.limits(w.shape[0], w.shape[1])
    few = lim.f32_skinny if out_dtype == torch.float32 else lim.skinny
    if M <= few and gemm_skinny_supports(a, w):
        return gemm_skinny(a, w, bias, out_dtype=out_dtype)
    if out_dtype == torch.bfloat16 and M <= min(lim.rows, ROWS_MAX_ROWS) and gemm_rows_supports(a, w):
        return gemm_rows(a, w, bias)
    if (out_dtype == torch.bfloat16 and 0 < lim.sums_from <= M <= lim.sums_to and w.shape[0] % 4 == 0
            and gemm_partial_sums_supports(a, w)):
        return sum_stacks(gemm_partial_sums(a, w), bias)
    if library and out_dtype == torch.float32 and a.is_contiguous() and w.is_contiguous() and _MM_TAKES_OUT_DTYPE:
        y = torch.mm(a, w.t(), out_dtype=torch.float32)
        return y if bias is None else add_bias(y, bias)
    if library and out_dtype == torch.bfloat16:
        y = torch.nn.functional.linear(a, w)
        return y if bias is None else add_bias(y, bias)
    if out_dtype == torch.float32 and M <= 64 and gemm_skinny_supports(a, w):
        return gemm_skinny(a, w, bias, out_dtype=out_dtype)
    return gemm_simple(a, w, bias, out_dtype=out_dtype)


def attention_mfma_supports(dtype: torch.dtype, hd: int, page_size: int, nq: int, nkv: int) -> bool:
    """True if the matrix-core attention kernels take this shape (bfloat16, head_dim in
    {32, 64, 96, 128, 256}, page size a multiple of 16)."""
    if dtype != torch.bfloat16:
        return False
    return bool(build.load("attention_mfma").ullm_attention_mfma_supports(
        _c_int(hd), _c_int(page_size), _c_int(nq), _c_int(nkv)))


_units_of_device = {}


def compute_units(device=None) -> int:
    """Compute units of the device the kernels run on (256 on an MI355X)."""
    index = torch.cuda.current_device() if device is None else torch.device(device).index or 0
    n = _units_of_device.get(index)
    if n is None:
        n = _units_of_device[index] = int(torch.cuda.get_device_properties(index).multi_processor_count)
    return n


def decode_split(n_items: int, nkv: int, groups: int, max_kv: int, hd: int = 128, window: int = 0, units: int = 256):
    """(waves, num_splits) of the decode attention launch.  A wave walks its keys one 32-key tile after
    the other, each a round trip to memory, so few (token, kv head) pairs with many keys are cut over
    several blocks, up to one block per compute unit (more would run in a second round), and a second
    small kernel adds the blocks' partial results; that kernel costs about as much as walking eight more
    tiles, so short contexts are not cut.  Mostly a block is a single wave (several are resident on a
    SIMD, they start and end independently and one's start overlaps the others' streaming, and their number
    need not be a multiple of the compute units); four waves a block where few pairs have very many keys.
    With a window a token reads at most the window's keys (and up to 31 before them, to the tile's edge),
    however long its context is.  ``units``: the device's compute units, four SIMDs each."""
    pairs = max(1, n_items * nkv * groups)
    simds = 4 * units
    if pairs >= simds:
        return 1, 1
    if window > 0:
        max_kv = min(max_kv, window + 31)
    tiles = -(-max_kv // 32)
    if pairs > units:
        # single waves, two to four to a SIMD, so that the launch has no rounds of whole blocks (four-wave blocks,
        # one to a compute unit, take 49 us at 264 pairs against 30 us at 256); up to 2.25 pairs a unit cut in three
        # where that still gives at most one wave per SIMD and compute unit, else in two
        return 1, (max(2, min(3, simds // pairs)) if pairs <= units * 9 // 4 and tiles > 16 else 1)
    if pairs == units:
        return (4 if tiles > 16 else 1), 1
    # up to 16 blocks a pair; up to 32 where very few pairs have very many keys (one request at 4 096 keys and
    # more: 134 MB of cache at 32 768 keys in 34 us against 49 us with 16; three or four requests at 32 000 keys:
    # 70 and 89 us against 89 and 93 us; two requests are better off with 16 blocks of four waves)
    most = 32 if ((pairs * 128 <= simds and tiles >= 128) or (16 < pairs <= simds // 32 and tiles >= 512)) else 16
    splits = min(most, max(1, 2 * units // pairs), tiles)
    if tiles > 8 * splits:
        splits = min(most, max(1, simds // pairs), tiles)
    waves = 4 if (tiles > 4 * splits and pairs * splits * 4 <= simds) else 1
    return waves, splits


def attention_decode_mfma(q, out, k_pool, v_pool, token_list: Optional[torch.Tensor], n_items: int,
                          positions, token_entry, block_table, page_size: int, nq: int, nkv: int, hd: int,
                          scale: float, window: int, max_kv: int, splits: int = 0, waves: int = 0,
                          bias_log2: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                          sink_log2: Optional[torch.Tensor] = None) -> None:
    """One query token per item (``token_list`` int32 [n_items] names the tokens, None = tokens
    0..n_items-1) against its request's cache; with ``splits`` > 1 the keys go to several blocks whose
    partial results a second small kernel adds up.  ``bias_log2`` (float32 [nq, rows], a distance bias times
    log2(e)) is added to the scores, ``gate`` (bfloat16 [T, >= nq]) gates every head's output by its sigmoid,
    ``sink_log2`` (float32 [nq], sinks times log2(e)) adds 2^sink to every head's sum of weights."""
    _check_pools(k_pool, v_pool, nkv, page_size, hd, torch.bfloat16)
    _need(q.dtype == torch.bfloat16 and q.stride(1) == 1 and q.shape[1] == nq * hd, "q must be bfloat16 [T, nq*hd]")
    _need(out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.shape == q.shape, "bad attention output")
    _i32(positions, "positions")
    _i32(token_entry, "token_entry")
    if token_list is not None:
        _i32(token_list, "token_list", n_items)
    else:
        _need(n_items <= q.shape[0], "more items than tokens")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    _need(-(-max_kv // page_size) <= block_table.shape[1], "block table narrower than the longest context")
    groups = -(-(nq // nkv) // 16)
    auto_waves, auto_splits = decode_split(n_items, nkv, groups, max_kv, hd, window, compute_units(q.device))
    waves = waves or auto_waves
    if hd == 256 and waves == 8:
        waves = 4
    splits = splits or auto_splits
    lib = build.load("attention_mfma")
    ws = None
    if splits > 1:
        ws = torch.empty(n_items * nq * splits * (hd + 4), dtype=torch.float32, device=q.device)
    if bias_log2 is not None or gate is not None or sink_log2 is not None:
        _check_gate(gate, q.shape[0], nq)
        _check_sink(sink_log2, nq)
        _check(lib.ullm_attention_decode_extras(
            _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(token_list),
            _c_int(n_items), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
            _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
            _c_int(splits), _c_int(waves), _p(ws), _p(bias_log2), _c_int(_check_distance_bias(bias_log2, nq)), _p(gate),
            _c_int(gate.stride(0) if gate is not None else 0), _p(sink_log2), _stream()), "attention_decode_extras")
        return
    _check(lib.ullm_attention_decode(
        _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(token_list),
        _c_int(n_items), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
        _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
        _c_int(splits), _c_int(waves), _p(ws), _stream()), "attention_decode")


def attention_decode_fused_supports(dtype: torch.dtype, hd: int, page_size: int, nq: int, nkv: int,
                                    rotary_dim: int, style: int) -> bool:
    """Whether the decode kernel can also do the step's per-head norm, rotation and cache write."""
    if dtype != torch.bfloat16:
        return False
    lib = build.load("attention_mfma")
    return bool(lib.ullm_attention_decode_fused_supports(_c_int(hd), _c_int(page_size), _c_int(nq), _c_int(nkv),
                                                         _c_int(rotary_dim), _c_int(style)))


def attention_decode_fused(qkv, out, q_gain: Optional[torch.Tensor], k_gain: Optional[torch.Tensor], eps: float,
                           cos_sin: Optional[torch.Tensor], rotary_dim: int, style: int, k_pool, v_pool,
                           token_list: Optional[torch.Tensor], n_items: int, positions, token_entry, block_table,
                           page_size: int, nq: int, nkv: int, hd: int, scale: float, window: int, max_kv: int,
                           write_kv: bool, splits: int = 0, waves: int = 0) -> None:
    """``attention_decode_mfma`` for a step in which every item is its request's newest token, with what
    ``qk_norm_rope_write`` does folded in: ``qkv`` [T, (nq + 2 nkv) * hd] is the fused projection as the
    matrix product left it; the kernel norms and rotates q and k itself and writes k and v to the cache."""
    _check_pools(k_pool, v_pool, nkv, page_size, hd, torch.bfloat16)
    _need(qkv.dtype == torch.bfloat16 and qkv.dim() == 2 and qkv.stride(1) == 1 and qkv.shape[1] == (nq + 2 * nkv) * hd,
          "qkv must be bfloat16 [T, (nq + 2 nkv) * hd]")
    _need(out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.shape == (qkv.shape[0], nq * hd), "bad attention output")
    _i32(positions, "positions")
    _i32(token_entry, "token_entry")
    if token_list is not None:
        _i32(token_list, "token_list", n_items)
    else:
        _need(n_items <= qkv.shape[0], "more items than tokens")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    _need(-(-max_kv // page_size) <= block_table.shape[1], "block table narrower than the longest context")
    for gn, nm in ((q_gain, "q_gain"), (k_gain, "k_gain")):
        if gn is not None:
            _need(gn.dtype == torch.float32 and gn.numel() == hd and gn.is_contiguous(), f"{nm} must be float32 [hd]")
    table_rows = 0
    if style != 0 and rotary_dim > 0:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.dim() == 2
              and cos_sin.shape[1] == rotary_dim and cos_sin.is_contiguous(),
              "cos_sin must be float32 [positions, rotary_dim]")
        table_rows = cos_sin.shape[0]
    groups = -(-(nq // nkv) // 16)
    auto_waves, auto_splits = decode_split(n_items, nkv, groups, max_kv, hd, window, compute_units(qkv.device))
    waves = waves or auto_waves
    if hd == 256 and waves == 8:
        waves = 4
    splits = splits or auto_splits
    lib = build.load("attention_mfma")
    ws = None
    if splits > 1:
        ws = torch.empty(n_items * nq * splits * (hd + 4), dtype=torch.float32, device=qkv.device)
    _check(lib.ullm_attention_decode_fused(
        _p(qkv), _c_int(qkv.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(token_list),
        _c_int(n_items), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
        _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
        _c_int(splits), _c_int(waves), _p(ws), _p(q_gain), _p(k_gain), _c_float(eps), _p(cos_sin),
        _c_int(table_rows), _c_int(rotary_dim), _c_int(style), _c_int(1 if write_kv else 0), _stream()),
        "attention_decode_fused")


PREFILL_TILE = 32      # tokens of one request per prompt tile (two groups of 16 columns for every wave of a block)


def attention_prefill_mfma(q, out, k_pool, v_pool, tiles: torch.Tensor, n_tiles: int, positions, token_entry,
                           block_table, page_size: int, nq: int, nkv: int, hd: int, scale: float,
                           window: int, halves: int = 0, keys_total: int = 0, keys_max: int = 0,
                           bias_log2: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None,
                           sink_log2: Optional[torch.Tensor] = None) -> None:
    """Tiles (first token, count <= PREFILL_TILE) of consecutive tokens of one request each, every
    token against the keys up to its own position.  ``halves``: 2 = two halves of a block share a
    tile's keys, 1 = one block takes them all, 0 = chosen from ``keys_total`` (the sum over the tiles of
    the keys each sees) and ``keys_max`` (the most any tile sees), or from the number of tiles if
    these are 0.  Every choice computes the same function."""
    _check_pools(k_pool, v_pool, nkv, page_size, hd, torch.bfloat16)
    _need(q.dtype == torch.bfloat16 and q.stride(1) == 1 and q.shape[1] == nq * hd, "q must be bfloat16 [T, nq*hd]")
    _need(out.dtype == torch.bfloat16 and out.stride(1) == 1 and out.shape == q.shape, "bad attention output")
    _need(tiles.dtype == torch.int32 and tiles.is_contiguous() and tiles.numel() >= 2 * n_tiles, "tiles must be int32 [n, 2]")
    _i32(positions, "positions")
    _i32(token_entry, "token_entry")
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    lib = build.load("attention_mfma")
    if bias_log2 is not None or gate is not None or sink_log2 is not None:
        _check_gate(gate, q.shape[0], nq)
        _check_sink(sink_log2, nq)
        _check(lib.ullm_attention_prefill_extras(
            _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(tiles),
            _c_int(n_tiles), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
            _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
            _c_int(halves), ctypes.c_longlong(int(keys_total)), _c_int(keys_max), _p(bias_log2),
            _c_int(_check_distance_bias(bias_log2, nq)), _p(gate), _c_int(gate.stride(0) if gate is not None else 0),
            _p(sink_log2), _stream()), "attention_prefill_extras")
        return
    _check(lib.ullm_attention_prefill(
        _p(q), _c_int(q.stride(0)), _p(out), _c_int(out.stride(0)), _p(k_pool), _p(v_pool), _p(tiles),
        _c_int(n_tiles), _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)),
        _c_int(page_size), _c_int(nq), _c_int(nkv), _c_int(hd), _c_float(scale), _c_int(window),
        _c_int(halves), ctypes.c_longlong(int(keys_total)), _c_int(keys_max), _stream()),
        "attention_prefill")


_warned_general_attention = set()


def _warn_general_attention(hd: int, page_size: int) -> None:
    """Said once per shape: bfloat16 attention that the matrix-core kernels do not take runs on the general
    kernel (one block per token and head), which is right but many times slower."""
    if (hd, page_size) in _warned_general_attention:
        return
    _warned_general_attention.add((hd, page_size))
    why = []
    if hd not in (32, 64, 96, 128, 256):
        why.append(f"head_dim {hd} is not one of 32, 64, 96, 128, 256")
    if page_size % 16:
        why.append(f"page size {page_size} is not a multiple of 16")
    logger.warning("bfloat16 attention runs on the general kernel, not on the matrix cores (%s): expect it to be "
                   "many times slower", "; ".join(why) or "shape not supported")


def paged_attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, ctx, group, nq: int,
                    nkv: int, hd: int, scale: float, window: int, plan=None,
                    bias: Optional[torch.Tensor] = None, bias_log2: Optional[torch.Tensor] = None,
                    gate: Optional[torch.Tensor] = None, sink: Optional[torch.Tensor] = None,
                    sink_log2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of the batch's queries over their requests' cached keys and values (the new
    tokens' rows included).  bfloat16 shapes the matrix-core kernels take go there (one launch for
    the one-token entries, one for the tiles of longer entries, both listed in ``plan``: arrays
    ``decode_tokens`` and ``tiles``, numbers ``num_decode``, ``max_decode_kv``, ``num_tiles``,
    ``tile_keys_total``, ``tile_keys_max``); everything else, and float32 always, takes the general
    kernel.  Every choice computes the same function.  ``bias`` (float32 [nq, rows]) is a bias by distance on the
    scores (``bias_log2``: the same times log2(e), which the matrix-core kernels add to their exponents of two);
    ``gate`` [T, >= nq]: every head's output is multiplied by the sigmoid of its gate; ``sink`` (float32 [nq]):
    exp(sink[head]) joins the softmax's denominator (``sink_log2``: the same times log2(e))."""
    if not attention_mfma_supports(q.dtype, hd, group.page_size, nq, nkv):
        if q.dtype == torch.bfloat16:
            _warn_general_attention(hd, group.page_size)
        out = paged_attention_generic(q, k_pool, v_pool, ctx.positions, ctx.token_entry, group.block_table,
                                      group.page_size, nq, nkv, hd, scale, window, bias=bias, sink=sink)
        return out if gate is None else head_gate_(out, gate, nq, hd)
    if bias is not None:
        _need(bias_log2 is not None and bias_log2.shape == bias.shape, "the matrix-core kernels take the bias times log2(e)")
    if sink is not None:
        _need(sink_log2 is not None and sink_log2.shape == sink.shape, "the matrix-core kernels take the sinks times log2(e)")
    _need(plan is not None, "the matrix-core attention kernels need the step's work lists (a step plan)")
    out = torch.empty((q.shape[0], nq * hd), dtype=q.dtype, device=q.device)
    n = plan.facts
    if n["num_decode"]:
        attention_decode_mfma(q, out, k_pool, v_pool, plan.arrays["decode_tokens"], n["num_decode"], ctx.positions,
                              ctx.token_entry, group.block_table, group.page_size, nq, nkv, hd, scale, window,
                              n["max_decode_kv"], bias_log2=bias_log2 if bias is not None else None, gate=gate,
                              sink_log2=sink_log2 if sink is not None else None)
    if n["num_tiles"]:
        attention_prefill_mfma(q, out, k_pool, v_pool, plan.arrays["tiles"], n["num_tiles"], ctx.positions,
                               ctx.token_entry, group.block_table, group.page_size, nq, nkv, hd, scale, window,
                               keys_total=n["tile_keys_total"], keys_max=n["tile_keys_max"],
                               bias_log2=bias_log2 if bias is not None else None, gate=gate,
                               sink_log2=sink_log2 if sink is not None else None)
    return out


# ---------------------------------------------------------------------------------- latent attention

def latent_prepare(proj: torch.Tensor, q_off: int, q_rank: int, kv_off: int, kv_rank: int, kr_off: int, rot: int,
                   g_off: int, n_gate: int, q_gain: Optional[torch.Tensor], kv_gain: torch.Tensor, eps: float,
                   cos_sin: Optional[torch.Tensor], positions: torch.Tensor, token_entry: torch.Tensor,
                   block_table: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, page_size: int, hd: int,
                   write_kv: bool, dtype: torch.dtype):
    """What a latent-attention layer does with its first product ``proj`` (float32 [T, columns]: q latent at ``q_off``,
    kv latent at ``kv_off``, the rotated key part at ``kr_off``, gate logits at ``g_off``): returns (cq, gate) with
    cq = rmsnorm(q latent) * ``q_gain`` as [T, q_rank] and gate = the logits as [T, n_gate rounded up to 8], both of
    ``dtype``; with ``write_kv`` the token's cache row [rmsnorm(kv latent) * ``kv_gain`` | rotated key part] goes to
    ``k_pool`` ([pages, 1, page_size, hd]) and the normed latent to ``v_pool`` ([pages, 1, hd, page_size])."""
    T = proj.shape[0]
    _need(proj.dtype == torch.float32 and proj.dim() == 2 and proj.stride(1) == 1, "proj must be float32 [T, columns]")
    _i32(positions, "positions", T)
    _i32(token_entry, "token_entry", T)
    _need(block_table.dtype == torch.int32 and block_table.dim() == 2 and block_table.stride(1) == 1,
          "block_table must be int32 [B, stride]")
    for g, nm, n in ((q_gain, "q_gain", q_rank), (kv_gain, "kv_gain", kv_rank)):
        _need((g is None and n == 0) or (g is not None and g.dtype == torch.float32 and g.numel() == n and g.is_contiguous()),
              f"{nm} must be float32 [{n}]")
    table_rows = 0
    if rot > 0:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.dim() == 2 and cos_sin.shape[1] == rot
              and cos_sin.is_contiguous(), "cos_sin must be float32 [positions, rot]")
        table_rows = cos_sin.shape[0]
    if write_kv:
        _check_pools(k_pool, v_pool, 1, page_size, hd, dtype)
    cq = torch.empty((T, q_rank), dtype=dtype, device=proj.device)
    ldg = -(-n_gate // 8) * 8
    gate = torch.empty((T, ldg), dtype=dtype, device=proj.device) if n_gate else None    # the kernel writes all ldg columns
    _check(build.load("latent").ullm_latent_prepare(
        _p(proj), _c_int(proj.stride(0)), _c_int(q_off), _c_int(q_rank), _c_int(kv_off), _c_int(kv_rank), _c_int(kr_off),
        _c_int(rot), _c_int(g_off), _c_int(n_gate), _p(q_gain), _p(kv_gain), _c_float(eps), _p(cos_sin), _c_int(table_rows),
        _p(positions), _p(token_entry), _p(block_table), _c_int(block_table.stride(0)), _p(k_pool), _p(v_pool),
        _c_int(page_size), _c_int(hd), _c_int(1 if write_kv else 0), _p(cq), _p(gate), _c_int(ldg), _c_int(T),
        _c_int(F32 if dtype == torch.float32 else BF16), _stream()), "latent_prepare")
    return cq, gate


HEAD_LINEAR_MAX_K = 1024          # the widest rows the per-head kernel keeps in shared memory
HEAD_LINEAR_LIBRARY_FROM = 128    # from this many rows on a bfloat16 product per head is the library's batched product


def head_linear(x: torch.Tensor, w: torch.Tensor, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[t, h] = w[h]^T x[t, h] for x [T, heads, K] (unit stride along K, any strides otherwise), w contiguous
    [heads, K, N] of x's dtype; y [T, heads, N] (``out`` may be a strided view with unit stride along N; without
    ``out`` the result may be one).  Few rows, and float32 always, take the hand-written kernel (32-bit sums in an
    order that depends on the row alone); many bfloat16 rows the library's batched product."""
    T, heads, K = x.shape
    _need(w.dim() == 3 and w.shape[0] == heads and w.shape[1] == K and w.is_contiguous() and w.dtype == x.dtype
          and w.data_ptr() % 8 == 0, "w must be contiguous [heads, K, N] of x's dtype")
    _need(x.stride(2) == 1, "x must have unit stride along K")
    N = w.shape[2]
    if out is not None:
        _need(out.shape == (T, heads, N) and out.stride(2) == 1 and out.dtype == x.dtype, "bad head_linear output")
    if x.dtype == torch.bfloat16 and T >= HEAD_LINEAR_LIBRARY_FROM and x.is_cuda:
        y = torch.bmm(x.transpose(0, 1), w).transpose(0, 1)          # [heads, T, N] seen as [T, heads, N]
        if out is None:
            return y
        out.copy_(y)
        return out
    _need(K <= HEAD_LINEAR_MAX_K, f"head_linear takes rows of up to {HEAD_LINEAR_MAX_K} values")
    if out is None:
        out = torch.empty((T, heads, N), dtype=x.dtype, device=x.device)
    ll = ctypes.c_longlong
    _check(build.load("latent").ullm_head_linear(_p(x), ll(x.stride(0)), ll(x.stride(1)), _p(w), _p(out), ll(out.stride(0)),
                                                 ll(out.stride(1)), _c_int(T), _c_int(heads), _c_int(N), _c_int(K),
                                                 _c_int(_dt(x)), _stream()), "head_linear")
    return out


def latent_query(qa: torch.Tensor, q: torch.Tensor, plain: int, rot: int, hd: int, cos_sin: Optional[torch.Tensor],
                 positions: torch.Tensor) -> torch.Tensor:
    """The query rows [T, heads * hd] a latent-attention layer hands the attention kernels: per head
    [qa[t, h] (rank values) | the head's last ``rot`` dims of ``q`` turned by the token's position | zeros], for
    qa [T, heads, rank] (unit stride along rank) and q [T, heads * (plain + rot)]."""
    T, heads, rank = qa.shape
    _need(qa.stride(2) == 1 and q.dtype == qa.dtype and q.dim() == 2 and q.stride(1) == 1
          and q.shape == (T, heads * (plain + rot)), "qa must be [T, heads, rank], q [T, heads * (plain + rot)]")
    _i32(positions, "positions", T)
    table_rows = 0
    if rot > 0:
        _need(cos_sin is not None and cos_sin.dtype == torch.float32 and cos_sin.dim() == 2 and cos_sin.shape[1] == rot
              and cos_sin.is_contiguous(), "cos_sin must be float32 [positions, rot]")
        table_rows = cos_sin.shape[0]
    out = torch.empty((T, heads * hd), dtype=qa.dtype, device=qa.device)
    ll = ctypes.c_longlong
    _check(build.load("latent").ullm_latent_query(_p(qa), ll(qa.stride(0)), ll(qa.stride(1)), _p(q), _c_int(q.stride(0)),
                                                  _c_int(plain), _c_int(rot), _c_int(rank), _c_int(heads), _c_int(hd),
                                                  _p(cos_sin), _c_int(table_rows), _p(positions), _p(out),
                                                  _c_int(out.stride(0)), _c_int(T), _c_int(_dt(qa)), _stream()),
           "latent_query")
    return out


# ---------------------------------------------------------------------------------- routed feed-forward

MOE_MAX_ROUTER, MOE_MAX_TOP = 1024, 32
MOE_TILE_ROWS = (16, 32, 64, 128)     # grouped rows a block of the matrix-core expert products takes


ROUTE_SOFTMAX_ALL, ROUTE_TOP_LOGITS, ROUTE_SIGMOID = 0, 1, 2      # how a router turns logits into experts and weights


def moe_route(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, mode: int = ROUTE_SOFTMAX_ALL,
              weight_scale: float = 1.0):
    """(ids int32 [T, top], weights float32 [T, top]) from router logits float32 [T, R]: the softmax over all R, the
    ``top`` largest of softmax + ``correction`` (float32 [R] or None; ties go to the lower index), and as weights the
    chosen outputs' softmax values over their sum (+ 1e-20).  With ``mode`` ROUTE_TOP_LOGITS: the ``top`` largest of
    logits + ``correction`` (a bias on the logits), weighed by the softmax over those alone.  With ROUTE_SIGMOID the
    scores are the sigmoids of the logits, each on its own; choice and weights as with the softmax.  Every weight is
    multiplied by ``weight_scale``."""
    T, R = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "router logits must be float32 [T, R]")
    _need(1 <= top <= min(R, MOE_MAX_TOP) and R <= MOE_MAX_ROUTER, f"top {top} of {R} router outputs: at most "
          f"{MOE_MAX_TOP} of {MOE_MAX_ROUTER}")
    if correction is not None:
        _need(correction.dtype == torch.float32 and correction.numel() == R and correction.is_contiguous(),
              "the router's correction must be float32 [R]")
    ids = torch.empty((T, top), dtype=torch.int32, device=logits.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=logits.device)
    _check(build.load("moe").ullm_moe_route(_p(logits), _c_int(logits.stride(0)), _p(correction), _c_int(T), _c_int(R),
                                            _c_int(top), _p(ids), _p(weights), _c_int(mode), _c_float(weight_scale),
                                            _stream()), "moe_route")
    return ids, weights


MOE_ROUTER_MAX_WIDTH = 12288      # widest row the fused router kernel keeps in shared memory


def moe_router(x: torch.Tensor, w_router: torch.Tensor, correction: Optional[torch.Tensor], top: int,
               mode: int = ROUTE_SOFTMAX_ALL, weight_scale: float = 1.0):
    """:func:`moe_route` of the 32-bit product of ``x`` [T, H] with ``w_router`` (float32 [R, H]), in one kernel: every
    router output is summed along the row in an order that depends on nothing but the row."""
    T, H = x.shape
    R = w_router.shape[0]
    _need(x.stride(1) == 1 and H <= MOE_ROUTER_MAX_WIDTH, f"x must be [T, H <= {MOE_ROUTER_MAX_WIDTH}] with unit stride")
    _need(w_router.dtype == torch.float32 and w_router.shape == (R, H) and w_router.is_contiguous(),
          "the router's matrix must be contiguous float32 [R, H]")
    _need(1 <= top <= min(R, MOE_MAX_TOP) and R <= MOE_MAX_ROUTER, f"top {top} of {R} router outputs: at most "
          f"{MOE_MAX_TOP} of {MOE_MAX_ROUTER}")
    if correction is not None:
        _need(correction.dtype == torch.float32 and correction.numel() == R and correction.is_contiguous(),
              "the router's correction must be float32 [R]")
    ids = torch.empty((T, top), dtype=torch.int32, device=x.device)
    weights = torch.empty((T, top), dtype=torch.float32, device=x.device)
    _check(build.load("moe").ullm_moe_router(_p(x), _c_int(x.stride(0)), _p(w_router), _p(correction), _c_int(T), _c_int(H),
                                             _c_int(R), _c_int(top), _p(ids), _p(weights), _c_int(mode), _c_float(weight_scale),
                                             _c_int(_dt(x)),
                                             _stream()), "moe_router")
    return ids, weights


def moe_max_tiles(n_pairs: int, n_experts: int, tile_rows: int) -> int:
    """The most tiles of ``tile_rows`` rows that ``n_pairs`` (token, expert) pairs over ``n_experts`` experts can fill."""
    return max(1, n_pairs // tile_rows + min(n_experts, n_pairs))


def moe_sort(ids: torch.Tensor, n_experts: int, tile_rows: int):
    """Groups the pairs (token, k) of ``ids`` int32 [T, top] by expert.  Returns (slot_of_pair int32 [T * top], -1 for
    a pair whose expert index is >= ``n_experts``; token_of_slot int32 [T * top]; tiles int32 [max_tiles + 1, 3] =
    (expert, first slot, rows <= tile_rows), rows 0 in unused tiles, and behind the list one entry whose first number
    counts the tiles in use; offsets int32 [n_experts + 1])."""
    _i32(ids, "ids")
    T, top = ids.shape
    n_pairs = T * top
    dev = ids.device
    max_tiles = moe_max_tiles(n_pairs, n_experts, tile_rows)
    slot_of_pair = torch.empty(n_pairs, dtype=torch.int32, device=dev)
    token_of_slot = torch.empty(n_pairs, dtype=torch.int32, device=dev)
    tiles = torch.empty((max_tiles + 1, 3), dtype=torch.int32, device=dev)     # behind the list: the tiles in use
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=dev)
    _check(build.load("moe").ullm_moe_sort(_p(ids), _c_int(n_pairs), _c_int(top), _c_int(n_experts), _c_int(tile_rows),
                                           _p(offsets), _p(slot_of_pair), _p(token_of_slot), _p(tiles), _c_int(max_tiles),
                                           _stream()), "moe_sort")
    return slot_of_pair, token_of_slot, tiles, offsets


def moe_rows(x: torch.Tensor, row_index: Optional[torch.Tensor], w: torch.Tensor, tiles: torch.Tensor, tile_rows: int,
             n_slots: int, gated: bool, limit: float = 0.0, alpha: float = 0.0) -> torch.Tensor:
    """The experts' products over grouped rows.  ``w`` is [experts, 2 n_out, K] (``gated``: gate rows, then up rows) or
    [experts, n_out, K]; row ``slot`` of the result comes from row ``row_index[slot]`` of ``x`` (``slot`` itself
    without an index) and the expert of the tile that holds the slot.  Gated: the clamped gated unit of the two
    products in x's dtype [n_slots, n_out]; else the product in float32.  Rows of slots no tile holds stay
    unwritten."""
    _need(w.dim() == 3 and w.is_contiguous() and w.dtype == x.dtype, "expert matrices must be contiguous [experts, rows, K] of x's dtype")
    K = w.shape[2]
    n_out = w.shape[1] // 2 if gated else w.shape[1]
    _need(x.dim() == 2 and x.shape[1] == K and x.stride(1) == 1, "x must be [rows, K]")
    _need(not gated or w.shape[1] % 2 == 0, "gated expert matrices hold gate rows, then as many up rows")
    _need(tiles.dtype == torch.int32 and tiles.dim() == 2 and tiles.shape[1] == 3 and tiles.is_contiguous(), "tiles must be int32 [n, 3]")
    if row_index is not None:
        _i32(row_index, "row_index", n_slots)
    else:
        _need(x.shape[0] >= n_slots, "fewer rows than slots")
    out = torch.empty((n_slots, n_out), dtype=x.dtype if gated else torch.float32, device=x.device)
    _need(tiles.shape[0] >= 2, "the tile list ends with the entry that counts the tiles in use")
    _check(build.load("moe").ullm_moe_rows(_p(x), _c_int(x.stride(0)), _p(row_index), _p(w), _p(tiles),
                                           _c_int(tiles.shape[0] - 1), _c_int(tile_rows), _p(out), _c_int(out.stride(0)),
                                           _c_int(n_out), _c_int(K), _c_int(1 if gated else 0), _c_float(limit),
                                           _c_float(alpha), _c_int(_dt(x)), _stream()), "moe_rows")
    return out


def moe_combine(y: Optional[torch.Tensor], x: torch.Tensor, ids: torch.Tensor, weights: torch.Tensor,
                slot_of_pair: torch.Tensor, n_experts: int, base: Optional[torch.Tensor] = None,
                bias: Optional[torch.Tensor] = None, shared: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [T, H]: ``base`` + ``bias`` + ``shared`` + the sum over a token's chosen experts, in their order, of
    weight times the expert's row of ``y`` (float32 [slots, H]) or, for an expert index >= ``n_experts``, times the
    token's own row of ``x``."""
    T, H = x.shape
    top = ids.shape[1]
    _need(x.stride(1) == 1, "x must have unit stride along its rows")
    _need(y is None or (y.dtype == torch.float32 and y.dim() == 2 and y.shape[1] == H and y.is_contiguous()), "y must be float32 [slots, H]")
    _need(y is not None or n_experts == 0, "experts with weights need their rows")
    _i32(ids, "ids", T * top)
    _i32(slot_of_pair, "slot_of_pair", T * top)
    _need(weights.dtype == torch.float32 and weights.is_contiguous() and weights.numel() == T * top, "weights must be float32 [T, top]")
    base_dt = F32
    if base is not None:
        _need(base.shape == (T, H) and base.is_contiguous(), "base must be contiguous [T, H]")
        base_dt = _dt(base)
    if bias is not None:
        _need(bias.dtype == torch.float32 and bias.numel() == H and bias.is_contiguous(), "bias must be float32 [H]")
    if shared is not None:
        _need(shared.shape == (T, H) and shared.is_contiguous() and shared.dtype == x.dtype, "shared must be [T, H] of x's dtype")
    out = torch.empty((T, H), dtype=torch.float32, device=x.device)
    _check(build.load("moe").ullm_moe_combine(_p(y), _p(x), _c_int(x.stride(0)), _p(ids), _p(weights), _p(slot_of_pair),
                                              _c_int(top), _c_int(n_experts), _p(base), _c_int(base_dt), _p(bias),
                                              _p(shared), _p(out), _c_int(T), _c_int(H), _c_int(_dt(x)), _stream()),
           "moe_combine")
    return out


# ---------------------------------------------------------------------------------- sampling

SAMPLE_PARTS_TOP_K = 64     # the largest top-k that the sampling kernels serve from parts of a row (PART_K_MAX)


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           min_p: torch.Tensor, seed_lo: torch.Tensor, seed_hi: torch.Tensor, position: torch.Tensor,
           out: Optional[torch.Tensor] = None, parts: bool = True) -> torch.Tensor:
    """One token id per row of float32 ``logits`` [n, V].  Per-row parameters: temperature (0 =
    greedy), top_k (<= 0 = all), top_p, min_p (float32), seed halves and position (int32).  ``parts``: a first
    kernel cuts the rows into parts over many blocks where the settings allow (False: one block per row does
    everything)."""
    n, V = logits.shape
    _need(logits.dtype == torch.float32 and logits.stride(1) == 1, "logits must be float32 with unit stride")
    for t, nm, dt in ((temperature, "temperature", torch.float32), (top_k, "top_k", torch.int32),
                      (top_p, "top_p", torch.float32), (min_p, "min_p", torch.float32),
                      (seed_lo, "seed_lo", torch.int32), (seed_hi, "seed_hi", torch.int32),
                      (position, "position", torch.int32)):
        _need(t.dtype == dt and t.numel() >= n and t.is_contiguous(), f"{nm} must be contiguous {dt} [n]")
    if out is None:
        out = torch.empty((n,), dtype=torch.int32, device=logits.device)
    _need(out.dtype == torch.int32 and out.numel() >= n and out.is_contiguous(), "bad sample output")
    lib = build.load("sampling")
    lib.ullm_sample_workspace.restype = ctypes.c_longlong
    need = int(lib.ullm_sample_workspace(_c_int(n), _c_int(V), _c_int(logits.stride(0)))) if parts else 0
    ws = torch.empty(need, dtype=torch.float32, device=logits.device) if need > 0 else None
    _check(lib.ullm_sample(_p(logits), _c_int(n), _c_int(V), _c_int(logits.stride(0)), _p(temperature), _p(top_k),
                           _p(top_p), _p(min_p), _p(seed_lo), _p(seed_hi), _p(position), _p(out), _p(ws), _stream()),
           "sample")
    return out
