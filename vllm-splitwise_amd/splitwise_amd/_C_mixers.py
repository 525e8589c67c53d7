"""ctypes binding of libsplitwise_mixers.so: the operators of recurrent / windowed token mixers
(``include/splitwise_mixers.h``).  Same rules as ``_C``: raw device pointers, torch's current HIP
stream, RuntimeError when the library is missing or an entry point refuses its arguments; no fallback.

Every operator takes the step's ragged layout as a ``RaggedBatch``-like object with the int32 device
tensors ``q_start`` [B + 1], ``ctx_len`` [B], ``token_seq`` [rows], ``state_slot`` [B] and
``block_tables`` [B, width].
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from types import SimpleNamespace
from typing import Optional

import torch

_PKG_DIR = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_PKG_DIR, "libsplitwise_mixers.so")
ABI_VERSION = 5

SW_F32, SW_BF16 = 0, 2
_ACT = {torch.float32: SW_F32, torch.bfloat16: SW_BF16}

_p, _i, _l, _f = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_float
_SIGNATURES = {
    "swm_scalar_norm_add": [_p, _p, _p, _f, _p, _l, _i, _l, _i, _i, _p],
    "swm_scalar_norm": [_p, _p, _p, _f, _l, _i, _i, _p],
    "swm_qk_norm_cache": [_p, _p, _p, _p, _l, _p, _p, _f, _p, _p, _p, _l, _i, _i, _i, _i, _p],
    "swm_window_attention": [_p, _p, _p, _p, _p, _p, _i, _p, _p, _p, _l, _i, _i, _i, _i, _i, _i, _f, _i, _i, _i,
                             _p, _i, _p],
    "swm_short_conv": [_p, _p, _l, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _p],
    "swm_short_conv_advance": [_p, _p, _l, _p, _p, _p, _i, _i, _i, _i, _p],
    "swm_channel_delta": [_p, _p, _p, _l, _p, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _i, _p],
    "swm_general_delta": [_p, _p, _p, _p, _l, _p, _l, _p, _p, _l, _p, _p, _p, _p, _p, _l, _i, _i, _i, _p, _i, _p],
    "swm_head_norm_gate": [_p, _p, _p, _l, _p, _i, _f, _l, _i, _i, _i, _p],
    "swm_expert_up_gelu": [_p, _p, _p, _p, _p, _i, _l, _i, _i, _i, _i, _p],
    "swm_expert_down": [_p, _p, _p, _p, _p, _i, _l, _i, _i, _i, _f, _i, _p],
    "swm_expert_up": [_p, _p, _p, _p, _p, _i, _l, _i, _i, _i, _i, _i, _p],
    "swm_expert_down_weighted": [_p, _p, _p, _p, _p, _i, _l, _i, _i, _i, _f, _p, _i, _p],
    "swm_stream_add_norm": [_p, _p, _l, _p, _l, _p, _p, _f, _f, _p, _l, _i, _i, _p],
    "swm_clamped_glu": [_p, _p, _l, _l, _i, _f, _f, _f, _i, _p],
    "swm_relu2": [_p, _p, _l, _l, _i, _i, _p],
    "swm_rope_cache": [_p, _p, _p, _p, _l, _p, _p, _i, _i, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p],
    "swm_group_router": [_p, _p, _p, _p, _l, _i, _i, _i, _i, _f, _p],
    "swm_group_pairs": [_p, _p, _p, _l, _i, _p],
    "swm_capped_attention": [_p, _p, _p, _p, _p, _l, _p, _i, _p, _p, _l, _i, _i, _i, _i, _i, _i, _i, _f, _f, _i, _i,
                             _p],
    "swm_masked_attention": [_p, _p, _p, _p, _p, _l, _p, _i, _p, _p, _l, _i, _i, _i, _i, _i, _i, _i, _f, _f, _i, _i,
                             _i, _l, _l, _p, _i, _p],
    "swm_gated_stream_step": [_p, _p, _l, _p, _l, _f, _p, _l, _p, _i, _p, _p, _p, _p, _l, _i, _i, _p],
    "swm_poly_norm": [_p, _p, _l, _p, _f, _l, _i, _i, _p],
    "swm_gate_mul": [_p, _p, _l, _l, _p, _l, _l, _i, _i, _i, _i, _p],
    "swm_latent_rope_cache": [_p, _p, _l, _l, _p, _l, _l, _p, _l, _p, _f, _p, _p, _p, _p, _l, _i, _i, _i, _i, _p],
    "swm_head_norm_gate_act": [_p, _p, _p, _l, _p, _i, _f, _l, _i, _i, _i, _i, _p],
    "swm_gla": [_p, _p, _p, _p, _l, _p, _l, _p, _f, _f, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _i, _p],
    "swm_lightning": [_p, _p, _p, _p, _l, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _i, _p],
    "swm_group_norm_add": [_p, _p, _l, _f, _p, _l, _f, _i, _p, _p, _p, _p, _i, _i, _f, _l, _i, _p],
    "swm_causal_conv": [_p, _i, _p, _i, _l, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p],
    "swm_gated_delta": [_p, _p, _p, _l, _p, _l, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _i, _p],
    "swm_gated_delta_chunked": [_p, _p, _p, _l, _p, _l, _p, _p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _i, _p],
    "swm_norm_rope_cache": [_p, _p, _p, _p, _l, _p, _p, _f, _p, _p, _i, _i, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p],
    "swm_sigmoid_attention": [_p, _p, _p, _p, _p, _l, _p, _p, _i, _p, _p, _l, _i, _i, _i, _i, _i, _i, _i, _f, _i, _p,
                              _i, _p],
    "swm_group_router_as": [_p, _p, _p, _p, _l, _i, _i, _i, _i, _f, _i, _i, _i, _p],
    "swm_expert_up_as": [_p, _p, _p, _p, _p, _i, _l, _i, _i, _i, _i, _f, _f, _f, _i, _p],
}
ACT_GELU, ACT_RELU2, ACT_NONE, ACT_CLAMPED_GLU = 0, 1, 2, 3

_lib = None


def library_path() -> str:
    return _LIB_PATH


def build_library() -> None:
    """Compiles only this library (``make mixers``): what a fresh checkout needs before its first step."""
    subprocess.run(["make", "-C", os.path.dirname(_PKG_DIR), "mixers", "-j", str(min(8, os.cpu_count() or 1))],
                   check=True, stdout=subprocess.DEVNULL)


def load_library() -> ctypes.CDLL:
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(_LIB_PATH):
        raise RuntimeError(f"native library not built: {_LIB_PATH} is missing (run `make -C vllm-splitwise_amd mixers`)")
    lib = ctypes.CDLL(_LIB_PATH)
    lib.swm_last_error.restype, lib.swm_last_error.argtypes = ctypes.c_char_p, []
    lib.swm_abi_version.restype, lib.swm_abi_version.argtypes = _i, []
    lib.swm_lightning_workspace_floats.restype = _l
    lib.swm_lightning_workspace_floats.argtypes = [_l, _i, _i, _i, _i, _i]
    lib.swm_masked_attention_workspace_floats.restype = _l
    lib.swm_masked_attention_workspace_floats.argtypes = [_l, _i, _i, _i, _i, _i, _i, _i, _i, _i]
    lib.swm_gated_delta_chunked_workspace_floats.restype = _l
    lib.swm_gated_delta_chunked_workspace_floats.argtypes = [_l, _i, _i, _i, _i]
    lib.swm_gla_workspace_floats.restype = _l
    lib.swm_gla_workspace_floats.argtypes = [_l, _i, _i, _i, _i, _i]
    if lib.swm_abi_version() != ABI_VERSION:
        raise RuntimeError(f"{_LIB_PATH} implements interface version {lib.swm_abi_version()}, this binding needs "
                           f"{ABI_VERSION}: rebuild it (`make -C vllm-splitwise_amd mixers`)")
    for name, argtypes in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes, fn.restype = argtypes, _i
    _lib = lib
    return lib


def _check(status: int) -> None:
    if status != 0:
        raise RuntimeError(load_library().swm_last_error().decode("utf-8", "replace")
                           or f"splitwise_mixers call failed with status {status}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t: torch.Tensor) -> int:
    """torch's current HIP stream on ``t``'s device (the raw handle; a step makes a hundred of these calls)."""
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


class _SameDevice:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_SAME_DEVICE = _SameDevice()


def _on_device_of(t: torch.Tensor):
    """Context that makes ``t``'s device current; free when it already is (an eager step makes some seventy
    of these calls, and switching devices costs more than the launch)."""
    if t.device.index == torch.cuda.current_device():
        return _SAME_DEVICE
    return torch.cuda.device(t.device)


def _act(t: torch.Tensor) -> int:
    try:
        return _ACT[t.dtype]
    except KeyError:
        raise RuntimeError(f"Unsupported data type: {t.dtype}") from None


def _need(cond: bool, what: str) -> None:
    if not cond:
        raise RuntimeError(what)


def _dev(*tensors: Optional[torch.Tensor]) -> None:
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError("splitwise_mixers operators need tensors on a HIP device")


def _f32c(t: torch.Tensor, what: str) -> None:
    _need(t.dtype == torch.float32 and t.is_contiguous(), f"{what} must be a contiguous fp32 tensor")


def _rows(t: torch.Tensor, what: str) -> int:
    """Row stride (elements) of a 2-D view whose rows are contiguous."""
    _need(t.dim() == 2 and t.stride(1) == 1, f"{what} must be 2-D with contiguous rows")
    return t.stride(0)


def scalar_norm_add(residual: torch.Tensor, y: torch.Tensor, gain: torch.Tensor, eps: float,
                    cast_out: Optional[torch.Tensor] = None) -> None:
    """residual (fp32, in place) += y / rms(y) * gain; cast_out = the new residual in cast_out's dtype."""
    _dev(residual, y, gain, cast_out)
    _f32c(residual, "residual")
    _f32c(gain, "gain")
    _need(residual.shape == y.shape and gain.numel() == 1, "scalar_norm_add: shapes")
    stride = _rows(y, "y")
    if cast_out is not None:
        _need(cast_out.is_contiguous() and cast_out.shape == y.shape, "scalar_norm_add: cast_out")
    with _on_device_of(y):
        _check(load_library().swm_scalar_norm_add(
            residual.data_ptr(), y.data_ptr(), gain.data_ptr(), eps,
            None if cast_out is None else cast_out.data_ptr(), y.shape[0], y.shape[1], stride, _act(y),
            _act(y if cast_out is None else cast_out), _stream(y)))


def scalar_norm(out: torch.Tensor, x: torch.Tensor, gain: torch.Tensor, eps: float) -> None:
    _dev(out, x, gain)
    _f32c(x, "x")
    _f32c(gain, "gain")
    _need(out.is_contiguous() and out.shape == x.shape and x.dim() == 2 and gain.numel() == 1, "scalar_norm: shapes")
    with _on_device_of(x):
        _check(load_library().swm_scalar_norm(out.data_ptr(), x.data_ptr(), gain.data_ptr(), eps, x.shape[0],
                                              x.shape[1], _act(out), _stream(x)))


def qk_norm_cache(q_out: torch.Tensor, q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
                  q_gain: torch.Tensor, k_gain: Optional[torch.Tensor], eps: float,
                  key_cache: Optional[torch.Tensor], value_cache: Optional[torch.Tensor],
                  slot_mapping: Optional[torch.Tensor]) -> None:
    """q, k, v: column ranges of ONE projection output (same row stride).  Caches: [pages, page, kv * size]."""
    _dev(q_out, q, k, v, q_gain, k_gain, key_cache, value_cache, slot_mapping)
    _f32c(q_out, "q_out")
    _f32c(q_gain, "q_gain")
    stride = _rows(q, "q")
    rows, q_size = q.shape
    _need(q_out.shape == q.shape and q_gain.numel() == q_size, "qk_norm_cache: query shapes")
    k_size = v_size = 0
    if k is not None:
        _need(v is not None and k_gain is not None and key_cache is not None and value_cache is not None
              and slot_mapping is not None, "qk_norm_cache: keys need values, a gain, caches and slots")
        _f32c(k_gain, "k_gain")
        k_size, v_size = k.shape[1], v.shape[1]
        _need(_rows(k, "k") == stride and _rows(v, "v") == stride and k.dtype == q.dtype and v.dtype == q.dtype
              and k.shape[0] == rows and v.shape[0] == rows, "qk_norm_cache: q, k, v must share rows and stride")
        _need(k_gain.numel() == k_size and key_cache.dtype == q.dtype and value_cache.dtype == q.dtype
              and key_cache.is_contiguous() and value_cache.is_contiguous()
              and key_cache.shape[-1] == k_size and value_cache.shape[-1] == v_size, "qk_norm_cache: cache shapes")
        _need(slot_mapping.dtype == torch.int64 and slot_mapping.numel() == rows and slot_mapping.is_contiguous(),
              "qk_norm_cache: slot_mapping must be int64 [rows]")
        slots = key_cache.shape[0] * key_cache.shape[1]
        _need(value_cache.shape[0] * value_cache.shape[1] == slots, "qk_norm_cache: caches differ in slots")
    with _on_device_of(q):
        _check(load_library().swm_qk_norm_cache(
            q_out.data_ptr(), q.data_ptr(), None if k is None else k.data_ptr(), None if v is None else v.data_ptr(),
            stride, q_gain.data_ptr(), None if k is None else k_gain.data_ptr(), eps,
            None if k is None else key_cache.data_ptr(), None if k is None else value_cache.data_ptr(),
            None if k is None else slot_mapping.data_ptr(), rows, q_size, k_size, v_size, _act(q), _stream(q)))


def _ragged_ok(batch, rows: int) -> int:
    n = batch.ctx_len.numel()
    for name in ("q_start", "ctx_len", "token_seq", "state_slot"):
        t = getattr(batch, name)
        _need(t is not None and t.dtype == torch.int32 and t.is_contiguous() and t.is_cuda, f"ragged batch: {name}")
    _need(batch.q_start.numel() == n + 1 and batch.token_seq.numel() == rows and batch.state_slot.numel() == n,
          "ragged batch: lengths")
    return n


def window_attention(out: torch.Tensor, q: torch.Tensor, key_cache: torch.Tensor, value_cache: torch.Tensor,
                     talk: torch.Tensor, batch, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                     window: int, keep_first: int, splits: Optional[int] = None) -> None:
    """out [rows, heads * vdim] (cache dtype); q fp32 [rows, heads * dim]; caches [pages, page, kv_heads * size].
    ``splits``: runs that a token's keys are cut into (default: enough to fill the GPU when the step has few
    tokens, 1 otherwise)."""
    _dev(out, q, key_cache, value_cache, talk)
    _f32c(q, "q")
    _f32c(talk, "talk")
    rows = q.shape[0]
    n = _ragged_ok(batch, rows)
    tables = batch.block_tables
    _need(tables.dtype == torch.int32 and tables.is_contiguous() and tables.dim() == 2 and tables.shape[0] == n,
          "window_attention: block tables")
    _need(q.shape[1] == heads * dim and out.shape == (rows, heads * vdim) and out.is_contiguous()
          and out.dtype == key_cache.dtype == value_cache.dtype and talk.shape == (heads, heads)
          and key_cache.is_contiguous() and value_cache.is_contiguous()
          and key_cache.shape[1:] == (value_cache.shape[1], kv_heads * dim)
          and value_cache.shape[2] == kv_heads * vdim and key_cache.shape[0] == value_cache.shape[0],
          "window_attention: shapes")
    _need(batch.max_pages_used <= tables.shape[1] and batch.max_page_id < key_cache.shape[0],
          "window_attention: block tables exceed the cache")
    if splits is None:
        most_keys = min(window + keep_first, batch.max_pages_used * key_cache.shape[1])
        splits = max(1, min(8, 512 // rows, most_keys // 64))
    partial = None
    if splits > 1:
        partial = torch.empty(rows * splits * (2 * heads + heads * kv_heads * vdim), dtype=torch.float32, device=q.device)
    with _on_device_of(q):
        _check(load_library().swm_window_attention(
            out.data_ptr(), q.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), talk.data_ptr(),
            tables.data_ptr(), tables.shape[1], batch.q_start.data_ptr(), batch.ctx_len.data_ptr(),
            batch.token_seq.data_ptr(), rows, n, heads, kv_heads, dim, vdim, key_cache.shape[1], scale, window,
            keep_first, splits, None if partial is None else partial.data_ptr(), _act(out), _stream(q)))


def short_conv(out: torch.Tensor, x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, batch) -> None:
    """out fp32 [rows, channels] = silu(causal conv of x with the sequence's carried inputs); the state
    [slots, taps - 1, channels] is read here and moved on by ``short_conv_advance``."""
    _dev(out, x, taps, state)
    _f32c(out, "out")
    _f32c(taps, "taps")
    _f32c(state, "state")
    stride = _rows(x, "x")
    rows, channels = x.shape
    n = _ragged_ok(batch, rows)
    k = taps.shape[1]
    _need(out.shape == x.shape and taps.shape[0] == channels and state.shape[1:] == (k - 1, channels)
          and batch.max_state_slot < state.shape[0], "short_conv: shapes")
    with _on_device_of(x):
        lib = load_library()
        _check(lib.swm_short_conv(out.data_ptr(), x.data_ptr(), stride, taps.data_ptr(), state.data_ptr(),
                                  batch.q_start.data_ptr(), batch.ctx_len.data_ptr(), batch.token_seq.data_ptr(),
                                  batch.state_slot.data_ptr(), rows, channels, k, _act(x), _stream(x)))
        _check(lib.swm_short_conv_advance(state.data_ptr(), x.data_ptr(), stride, batch.q_start.data_ptr(),
                                          batch.ctx_len.data_ptr(), batch.state_slot.data_ptr(), n, channels, k,
                                          _act(x), _stream(x)))


def causal_conv(out: torch.Tensor, x: torch.Tensor, taps: torch.Tensor, state: torch.Tensor, batch,
                silu: bool = False, residual: bool = True) -> None:
    """out [rows, channels] (any activation dtype) = act(conv(x) + x) (``residual``) or act(conv(x)), act = silu or
    none; x: a 2-D view, fp32 or bf16; the state [slots, taps - 1, channels] (fp32: the sequence's last inputs) is read
    and moved past the step's tokens in the same launch."""
    _dev(out, x, taps, state)
    _f32c(taps, "taps")
    _f32c(state, "state")
    stride = _rows(x, "x")
    rows, channels = x.shape
    n = _ragged_ok(batch, rows)
    k = taps.shape[1]
    _need(out.shape == x.shape and out.is_contiguous() and taps.shape[0] == channels
          and state.shape[1:] == (k - 1, channels) and batch.max_state_slot < state.shape[0], "causal_conv: shapes")
    with _on_device_of(x):
        lib = load_library()
        _check(lib.swm_causal_conv(out.data_ptr(), _act(out), x.data_ptr(), _act(x), stride, taps.data_ptr(),
                                   state.data_ptr(), batch.q_start.data_ptr(), batch.ctx_len.data_ptr(),
                                   batch.token_seq.data_ptr(), batch.state_slot.data_ptr(), rows, channels, k,
                                   1 if silu else 0, 1 if residual else 0, 1, _stream(x)))


def gated_delta(out: torch.Tensor, qkv: torch.Tensor, beta_pre: torch.Tensor, decay_pre: torch.Tensor,
                dt_bias: torch.Tensor, a_log: torch.Tensor, state: torch.Tensor, batch, heads: int, kv_heads: int,
                dim: int, vdim: int, chunked: Optional[bool] = None) -> None:
    """The delta rule with ONE decay per head: decay_pre, beta_pre [rows, heads] (2-D views in the activation dtype),
    dt_bias, a_log fp32 [heads]; qkv fp32 [rows, 2 * kv_heads * dim + heads * vdim] from the short convolution;
    state fp32 [slots, heads, dim, vdim]; out fp32 [rows, heads * vdim].  ``chunked``: chunks of 32 tokens on the matrix
    cores instead of token by token (default: when some sequence brings at least 32 tokens; key sizes up to 224)."""
    _dev(out, qkv, beta_pre, decay_pre, dt_bias, a_log, state)
    for t, what in ((out, "out"), (qkv, "qkv"), (dt_bias, "dt_bias"), (a_log, "a_log"), (state, "state")):
        _f32c(t, what)
    rows = qkv.shape[0]
    n = _ragged_ok(batch, rows)
    _need(qkv.shape[1] == 2 * kv_heads * dim + heads * vdim and out.shape == (rows, heads * vdim)
          and beta_pre.shape == (rows, heads) and decay_pre.shape == (rows, heads)
          and decay_pre.dtype == beta_pre.dtype and dt_bias.numel() == heads and a_log.numel() == heads
          and state.shape[1:] == (heads, dim, vdim) and batch.max_state_slot < state.shape[0],
          "gated_delta: shapes")
    if chunked is None:
        chunked = int(getattr(batch, "max_query_len", 0) or 0) >= 32
    if chunked and dim <= 224:                                 # larger keys: the chunks' operands outgrow the LDS
        with _on_device_of(qkv):
            lib = load_library()
            need = lib.swm_gated_delta_chunked_workspace_floats(rows, n, heads, dim, vdim)
            work = torch.empty(need, dtype=torch.float32, device=qkv.device)
            _check(lib.swm_gated_delta_chunked(
                out.data_ptr(), qkv.data_ptr(), beta_pre.data_ptr(), _rows(beta_pre, "beta_pre"), decay_pre.data_ptr(),
                _rows(decay_pre, "decay_pre"), dt_bias.data_ptr(), a_log.data_ptr(), state.data_ptr(),
                batch.q_start.data_ptr(), batch.ctx_len.data_ptr(), batch.state_slot.data_ptr(), rows, n, heads,
                kv_heads, dim, vdim, work.data_ptr(), _act(decay_pre), _stream(qkv)))
        return
    work = torch.empty(rows * heads * (3 * (-(-dim // 4) * 4) + 1), dtype=torch.float32, device=qkv.device)
    with _on_device_of(qkv):
        _check(load_library().swm_gated_delta(
            out.data_ptr(), qkv.data_ptr(), beta_pre.data_ptr(), _rows(beta_pre, "beta_pre"), decay_pre.data_ptr(),
            _rows(decay_pre, "decay_pre"), dt_bias.data_ptr(), a_log.data_ptr(), state.data_ptr(),
            batch.q_start.data_ptr(), batch.ctx_len.data_ptr(), batch.state_slot.data_ptr(), rows, n, heads, kv_heads,
            dim, vdim, work.data_ptr(), _act(decay_pre), _stream(qkv)))


def channel_delta(out: torch.Tensor, qkv: torch.Tensor, beta_pre: torch.Tensor, decay_pre: torch.Tensor,
                  dt_bias: torch.Tensor, a_log: torch.Tensor, state: torch.Tensor, batch, heads: int, kv_heads: int,
                  dim: int, vdim: int) -> None:
    _dev(out, qkv, beta_pre, decay_pre, dt_bias, a_log, state)
    for t, what in ((out, "out"), (qkv, "qkv"), (dt_bias, "dt_bias"), (a_log, "a_log"), (state, "state")):
        _f32c(t, what)
    rows = qkv.shape[0]
    n = _ragged_ok(batch, rows)
    _need(qkv.shape[1] == 2 * kv_heads * dim + heads * vdim and out.shape == (rows, heads * vdim)
          and beta_pre.shape == (rows, heads) and decay_pre.shape == (rows, heads * dim) and decay_pre.is_contiguous()
          and decay_pre.dtype == beta_pre.dtype and dt_bias.numel() == heads * dim and a_log.numel() == heads
          and state.shape[1:] == (heads, dim, vdim) and batch.max_state_slot < state.shape[0],
          "channel_delta: shapes")
    with _on_device_of(qkv):
        _check(load_library().swm_channel_delta(
            out.data_ptr(), qkv.data_ptr(), beta_pre.data_ptr(), _rows(beta_pre, "beta_pre"), decay_pre.data_ptr(),
            dt_bias.data_ptr(), a_log.data_ptr(), state.data_ptr(), batch.q_start.data_ptr(),
            batch.ctx_len.data_ptr(), batch.state_slot.data_ptr(), rows, n, heads, kv_heads, dim, vdim,
            torch.empty(rows * heads * (3 * (-(-dim // 4) * 4) + 1), dtype=torch.float32, device=qkv.device).data_ptr(),
            _act(decay_pre), _stream(qkv)))


def general_delta(out: torch.Tensor, r: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay_pre: torch.Tensor,
                  w0: torch.Tensor, rate_pre: torch.Tensor, a_bias: torch.Tensor, state: torch.Tensor, batch,
                  heads: int, dim: int) -> None:
    _dev(out, r, k, v, decay_pre, w0, rate_pre, a_bias, state)
    for t, what in ((out, "out"), (w0, "w0"), (a_bias, "a_bias"), (state, "state")):
        _f32c(t, what)
    rows = r.shape[0]
    n = _ragged_ok(batch, rows)
    stride = _rows(r, "r")
    size = heads * dim
    _need(all(t.shape == (rows, size) and t.dtype == r.dtype for t in (r, k, v, decay_pre, rate_pre))
          and _rows(k, "k") == stride and _rows(v, "v") == stride and out.shape == (rows, size)
          and w0.numel() == size and a_bias.numel() == size and state.shape[1:] == (heads, dim, dim)
          and batch.max_state_slot < state.shape[0], "general_delta: shapes")
    with _on_device_of(r):
        _check(load_library().swm_general_delta(
            out.data_ptr(), r.data_ptr(), k.data_ptr(), v.data_ptr(), stride, decay_pre.data_ptr(),
            _rows(decay_pre, "decay_pre"), w0.data_ptr(), rate_pre.data_ptr(), _rows(rate_pre, "rate_pre"),
            a_bias.data_ptr(), state.data_ptr(), batch.q_start.data_ptr(), batch.ctx_len.data_ptr(),
            batch.state_slot.data_ptr(), rows, n, heads, dim,
            torch.empty(rows * heads * 4 * (-(-dim // 4) * 4), dtype=torch.float32, device=r.device).data_ptr(), _act(r),
            _stream(r)))


def head_norm_gate(out: torch.Tensor, o: torch.Tensor, gate: torch.Tensor, weight: torch.Tensor, per_head_weight: bool,
                   eps: float, heads: int, vdim: int, gate_silu: bool = False) -> None:
    """``per_head_weight``: weight is [heads * vdim]; otherwise [vdim], shared by the heads.  ``gate_silu``: the
    normed output is multiplied by gate * sigmoid(gate) instead of sigmoid(gate)."""
    _dev(out, o, gate, weight)
    _f32c(o, "o")
    _f32c(weight, "weight")
    rows = o.shape[0]
    _need(o.shape == (rows, heads * vdim) and gate.shape == o.shape and out.shape == o.shape and out.is_contiguous()
          and out.dtype == gate.dtype and weight.numel() == (heads * vdim if per_head_weight else vdim),
          "head_norm_gate: shapes")
    with _on_device_of(o):
        _check(load_library().swm_head_norm_gate_act(out.data_ptr(), o.data_ptr(), gate.data_ptr(),
                                                     _rows(gate, "gate"), weight.data_ptr(),
                                                     vdim if per_head_weight else 0, eps, rows, heads, vdim,
                                                     1 if gate_silu else 0, _act(out), _stream(o)))


def expert_ffn(out: torch.Tensor, x: torch.Tensor, up: torch.Tensor, down: torch.Tensor, order: torch.Tensor,
               expert_start: torch.Tensor, top: int, weight: float, activation: int = ACT_GELU,
               pair_weight: Optional[torch.Tensor] = None, glu: Optional[tuple] = None) -> None:
    """out (fp32 [rows, width], zeroed by the caller) += weight * sum over each row's experts of
    pair_weight[row, choice] * down[e] act(up[e] x[row]); ``order`` / ``expert_start``: the (row, choice) pairs
    sorted by expert and every expert's first sorted pair; ``activation``: ACT_GELU (exact gelu) or ACT_RELU2;
    ``pair_weight`` fp32 [rows, top] (None: all 1).  ``glu`` = (alpha, limit, shift): a gated hidden layer,
    g sigmoid(alpha g) (u + shift) with g = min(gate x, limit), u = clamp(up x, -limit, limit), worked out in the
    up-projection's epilogue -- ``up`` then holds gate and up rows in runs of 16 (``glu_rows``)."""
    _dev(out, x, up, down, order, expert_start, pair_weight)
    _f32c(out, "out")
    rows, width = x.shape
    experts, ff = up.shape[0], up.shape[1]
    alpha, limit, shift = 1.0, float("inf"), 0.0
    if glu is not None:
        ff = down.shape[2]
        _need(up.shape[1] == 32 * (-(-ff // 16)), "expert_ffn: a gated hidden layer takes gate and up rows in runs of 16")
        activation = ACT_CLAMPED_GLU
        alpha, limit, shift = (float(v) for v in glu)
    _need(x.is_contiguous() and up.is_contiguous() and down.is_contiguous() and up.dtype == x.dtype == down.dtype
          and up.shape[::2] == (experts, width) and (glu is not None or up.shape[1] == ff) and out.shape == (rows, width)
          and down.shape == (experts, width, ff)
          and order.dtype == torch.int32 and order.numel() == rows * top and order.is_contiguous()
          and expert_start.dtype == torch.int32 and expert_start.numel() == experts + 1
          and expert_start.is_contiguous(), "expert_ffn: shapes")
    if pair_weight is not None:
        _f32c(pair_weight, "pair_weight")
        _need(pair_weight.numel() == rows * top, "expert_ffn: one weight per (row, choice)")
    pairs = rows * top
    hidden = torch.empty(pairs, ff, dtype=x.dtype, device=x.device)
    with _on_device_of(x):
        lib = load_library()
        _check(lib.swm_expert_up_as(hidden.data_ptr(), x.data_ptr(), up.data_ptr(), order.data_ptr(),
                                    expert_start.data_ptr(), experts, pairs, width, ff, top, activation, alpha, limit,
                                    shift, _act(x), _stream(x)))
        _check(lib.swm_expert_down_weighted(out.data_ptr(), hidden.data_ptr(), down.data_ptr(), order.data_ptr(),
                                            expert_start.data_ptr(), experts, pairs, width, ff, top, weight,
                                            None if pair_weight is None else pair_weight.data_ptr(), _act(x),
                                            _stream(x)))


def glu_rows(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """gate, up [..., ff, width] -> [..., 32 * ceil(ff / 16), width]: per run of 16 hidden channels the 16 gate rows, then
    the 16 up rows (a shorter last run padded with zero rows): what ``expert_ffn(glu=...)`` takes as ``up``."""
    ff, width = gate.shape[-2:]
    runs = -(-ff // 16)
    pad = runs * 16 - ff
    if pad:
        zeros = gate.new_zeros(gate.shape[:-2] + (pad, width))
        gate, up = torch.cat([gate, zeros], -2), torch.cat([up, zeros], -2)
    both = torch.stack([gate.unflatten(-2, (runs, 16)), up.unflatten(-2, (runs, 16))], -3)     # [..., runs, 2, 16, width]
    return both.flatten(-4, -2).contiguous()


def _opt_ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def stream_add_norm(residual: torch.Tensor, weight: Optional[torch.Tensor], offset: float, eps: float,
                    out: Optional[torch.Tensor], a: Optional[torch.Tensor] = None, b: Optional[torch.Tensor] = None,
                    c: Optional[torch.Tensor] = None) -> None:
    """residual (fp32, in place) += a + b + c (a, b: the activation dtype, 2-D views; c: fp32), then
    out = residual / rms(residual) * (offset + weight) in out's dtype (``out`` None: only the sum)."""
    _dev(residual, weight, out, a, b, c)
    _f32c(residual, "residual")
    rows, width = residual.shape
    act = out if out is not None else (a if a is not None else b)
    _need(act is not None or c is not None, "stream_add_norm: nothing to do")
    for t in (a, b):
        if t is not None:
            _need(t.shape == residual.shape and t.dtype == act.dtype, "stream_add_norm: addend")
    if c is not None:
        _f32c(c, "c")
        _need(c.shape == residual.shape, "stream_add_norm: fp32 addend")
    if out is not None:
        _f32c(weight, "weight")
        _need(out.shape == residual.shape and out.is_contiguous() and weight.numel() == width, "stream_add_norm: out")
    with _on_device_of(residual):
        _check(load_library().swm_stream_add_norm(
            residual.data_ptr(), _opt_ptr(a), 0 if a is None else _rows(a, "a"), _opt_ptr(b),
            0 if b is None else _rows(b, "b"), _opt_ptr(c), _opt_ptr(weight), offset, eps, _opt_ptr(out), rows, width,
            SW_F32 if act is None else _act(act), _stream(residual)))


def group_norm_add(residual: torch.Tensor, groups: int, eps: float, y1: Optional[torch.Tensor] = None,
                   post_weight: Optional[torch.Tensor] = None, layer_scale: Optional[torch.Tensor] = None,
                   y2: Optional[torch.Tensor] = None, s1: float = 1.0, s2: float = 1.0,
                   weight: Optional[torch.Tensor] = None, out: Optional[torch.Tensor] = None) -> None:
    """N(u; w): a row in ``groups`` equal runs, each over its own root mean square, the row times w.
    residual (fp32, in place) += layer_scale * N(s1 * y1 + s2 * y2; post_weight) (y1, y2: 2-D views of one dtype,
    fp32 or bf16), then out = N(residual; weight) in out's dtype (fp32 or bf16)."""
    _dev(residual, y1, y2, post_weight, layer_scale, weight, out)
    _f32c(residual, "residual")
    rows, width = residual.shape
    _need(y1 is not None or out is not None, "group_norm_add: nothing to do")
    if y1 is not None:
        _f32c(post_weight, "post_weight")
        _need(y1.shape == residual.shape and post_weight.numel() == width, "group_norm_add: addend")
        if y2 is not None:
            _need(y2.shape == residual.shape and y2.dtype == y1.dtype, "group_norm_add: second addend")
        if layer_scale is not None:
            _f32c(layer_scale, "layer_scale")
            _need(layer_scale.numel() == width, "group_norm_add: layer scale")
    else:
        _need(y2 is None, "group_norm_add: a second addend without a first")
    if out is not None:
        _f32c(weight, "weight")
        _need(out.shape == residual.shape and out.is_contiguous() and weight.numel() == width, "group_norm_add: out")
    with _on_device_of(residual):
        _check(load_library().swm_group_norm_add(
            residual.data_ptr(), _opt_ptr(y1), 0 if y1 is None else _rows(y1, "y1"), s1, _opt_ptr(y2),
            0 if y2 is None else _rows(y2, "y2"), s2, SW_F32 if y1 is None else _act(y1), _opt_ptr(post_weight),
            _opt_ptr(layer_scale), _opt_ptr(weight), _opt_ptr(out), SW_F32 if out is None else _act(out), groups, eps,
            rows, width, _stream(residual)))


def clamped_glu(out: torch.Tensor, gate_up: torch.Tensor, alpha: float, limit: float, shift: float) -> None:
    """gate_up [rows, 2 * ff] = gate | up -> out [rows, ff] = g sigmoid(alpha g) (u + shift) with g = min(gate, limit),
    u = clamp(up, -limit, limit)."""
    _dev(out, gate_up)
    rows, ff = out.shape
    _need(out.is_contiguous() and gate_up.shape == (rows, 2 * ff) and gate_up.dtype == out.dtype, "clamped_glu: shapes")
    with _on_device_of(out):
        _check(load_library().swm_clamped_glu(out.data_ptr(), gate_up.data_ptr(), _rows(gate_up, "gate_up"), rows, ff,
                                              alpha, limit, shift, _act(out), _stream(out)))


def relu2(out: torch.Tensor, x: torch.Tensor) -> None:
    _dev(out, x)
    _need(out.is_contiguous() and x.shape == out.shape and x.dtype == out.dtype and out.dim() == 2, "relu2: shapes")
    with _on_device_of(out):
        _check(load_library().swm_relu2(out.data_ptr(), x.data_ptr(), _rows(x, "x"), out.shape[0], out.shape[1],
                                        _act(out), _stream(out)))


def rope_cache(q_out: torch.Tensor, q: torch.Tensor, k: Optional[torch.Tensor], v: Optional[torch.Tensor],
               positions: torch.Tensor, inv_freq: Optional[torch.Tensor], heads: int, kv_heads: int, dim: int, vdim: int,
               key_cache: Optional[torch.Tensor], value_cache: Optional[torch.Tensor],
               slot_mapping: Optional[torch.Tensor], pair_halves: bool = False,
               q_norm: Optional[torch.Tensor] = None, k_norm: Optional[torch.Tensor] = None,
               norm_eps: float = 0.0) -> None:
    """q, k, v: column ranges of ONE projection output.  q_out fp32 = rotated q; rotated k and v go to the caches
    [pages, page, kv_heads * size] (k None: a layer that reads another layer's keys).  ``pair_halves``: coordinate i
    turns with coordinate i + rot / 2 instead of neighbours (2i, 2i + 1).  ``q_norm`` / ``k_norm`` (fp32 [dim]): every
    query / key head first gets an RMS norm over its coordinates with that weight."""
    _dev(q_out, q, k, v, positions, inv_freq, key_cache, value_cache, slot_mapping, q_norm, k_norm)
    if q_norm is not None:
        _f32c(q_norm, "q_norm")
        _need(q_norm.numel() == dim, "rope_cache: query norm weight")
        if k is not None:
            _f32c(k_norm, "k_norm")
            _need(k_norm.numel() == dim, "rope_cache: key norm weight")
    _f32c(q_out, "q_out")
    stride = _rows(q, "q")
    rows = q.shape[0]
    rot = 0
    if inv_freq is not None and inv_freq.numel() > 0:
        _f32c(inv_freq, "inv_freq")
        rot = 2 * inv_freq.numel()
    _need(q.shape[1] == heads * dim and q_out.shape == q.shape and rot <= dim, "rope_cache: query shapes")
    _need(positions.dtype == torch.int64 and positions.numel() == rows and positions.is_contiguous(),
          "rope_cache: positions must be int64 [rows]")
    if k is not None:
        _need(v is not None and key_cache is not None and value_cache is not None and slot_mapping is not None,
              "rope_cache: keys need values, caches and slots")
        _need(_rows(k, "k") == stride and _rows(v, "v") == stride and k.dtype == q.dtype and v.dtype == q.dtype
              and k.shape == (rows, kv_heads * dim) and v.shape == (rows, kv_heads * vdim),
              "rope_cache: q, k, v must share rows and stride")
        _need(key_cache.dtype == q.dtype and value_cache.dtype == q.dtype and key_cache.is_contiguous()
              and value_cache.is_contiguous() and key_cache.shape[-1] == kv_heads * dim
              and value_cache.shape[-1] == kv_heads * vdim
              and key_cache.shape[0] * key_cache.shape[1] == value_cache.shape[0] * value_cache.shape[1],
              "rope_cache: cache shapes")
        _need(slot_mapping.dtype == torch.int64 and slot_mapping.numel() == rows and slot_mapping.is_contiguous(),
              "rope_cache: slot_mapping must be int64 [rows]")
    with _on_device_of(q):
        _check(load_library().swm_norm_rope_cache(
            q_out.data_ptr(), q.data_ptr(), _opt_ptr(k), _opt_ptr(v), stride, _opt_ptr(q_norm),
            _opt_ptr(k_norm) if q_norm is not None else None, norm_eps, positions.data_ptr(),
            _opt_ptr(inv_freq) if rot else None, rot, 1 if pair_halves else 0,
            None if k is None else key_cache.data_ptr(),
            None if k is None else value_cache.data_ptr(), None if k is None else slot_mapping.data_ptr(), rows, heads,
            kv_heads, dim, vdim, _act(q), _stream(q)))


def group_router(logits: torch.Tensor, correction: Optional[torch.Tensor], top: int, groups: int, keep: int,
                 scale: float, softmax: bool = False, group_best_one: bool = False, normalize: bool = True):
    """logits fp32 [rows, experts] -> (chosen int32 [rows, top], weights fp32 [rows, top]).  Scores: sigmoid of the
    logits, or with ``softmax`` their softmax over all experts; a group scores the sum of its two best choice scores,
    or with ``group_best_one`` its best; the chosen experts' scores are divided by their sum unless ``normalize`` is
    off; all times ``scale``."""
    _dev(logits, correction)
    _f32c(logits, "logits")
    rows, experts = logits.shape
    if correction is not None:
        _f32c(correction, "correction")
        _need(correction.numel() == experts, "group_router: correction")
    chosen = torch.empty(rows, top, dtype=torch.int32, device=logits.device)
    weights = torch.empty(rows, top, dtype=torch.float32, device=logits.device)
    with _on_device_of(logits):
        _check(load_library().swm_group_router_as(chosen.data_ptr(), weights.data_ptr(), logits.data_ptr(),
                                                  _opt_ptr(correction), rows, experts, top, groups, keep, scale,
                                                  1 if softmax else 0, 1 if group_best_one else 0,
                                                  1 if normalize else 0, _stream(logits)))
    return chosen, weights


def group_pairs(chosen: torch.Tensor, experts: int):
    """chosen int32 [rows, top] -> (order int32 [rows * top]: pair indices row * top + choice grouped by expert,
    expert_start int32 [experts + 1]); one launch, nothing travels to the host."""
    _dev(chosen)
    _need(chosen.dtype == torch.int32 and chosen.is_contiguous(), "group_pairs: chosen must be contiguous int32")
    pairs = chosen.numel()
    order = torch.empty(pairs, dtype=torch.int32, device=chosen.device)
    start = torch.empty(experts + 1, dtype=torch.int32, device=chosen.device)
    with _on_device_of(chosen):
        _check(load_library().swm_group_pairs(order.data_ptr(), start.data_ptr(), chosen.data_ptr(), pairs, experts,
                                              _stream(chosen)))
    return order, start


def capped_attention(out: torch.Tensor, q: torch.Tensor, key_cache: torch.Tensor, value_cache: Optional[torch.Tensor],
                     gate: Optional[torch.Tensor], batch, heads: int, kv_heads: int, dim: int, vdim: int, scale: float,
                     softcap: float = 0.0, window: int = 0, chunk: int = 0, sink: bool = False,
                     score_bias: Optional[torch.Tensor] = None) -> None:
    """out [rows, heads * vdim] (cache dtype); q fp32 [rows, heads * dim]; caches [pages, page, kv_heads * size];
    gate (None: no gate): a 2-D view [rows, heads * vdim] in the cache dtype.  ``window`` / ``chunk``: the mask (a
    sliding window, or chunks counted from position 0; neither: plain causal); ``sink``: one more term exp(0) in the
    softmax's denominator.  ``value_cache`` None: a token's values are the first kv_heads * vdim elements of its
    key row (attention over a shared latent).  ``score_bias`` (fp32 [heads]): no softmax -- a seen key weighs
    sigmoid(score + score_bias[head]) and the weights are not normalised (window mask only)."""
    _dev(out, q, key_cache, value_cache, gate, score_bias)
    if score_bias is not None:
        _f32c(score_bias, "score_bias")
        _need(score_bias.numel() == heads and not softcap and not chunk and not sink,
              "capped_attention: sigmoid weights take a bias per head and no cap, chunks or sink")
    _f32c(q, "q")
    rows = q.shape[0]
    n = _ragged_ok(batch, rows)
    tables = batch.block_tables
    _need(tables.dtype == torch.int32 and tables.is_contiguous() and tables.dim() == 2 and tables.shape[0] == n,
          "capped_attention: block tables")
    _need(q.shape[1] == heads * dim and out.shape == (rows, heads * vdim) and out.is_contiguous()
          and out.dtype == key_cache.dtype and key_cache.is_contiguous() and key_cache.dim() == 3
          and key_cache.shape[2] >= kv_heads * dim, "capped_attention: shapes")
    k_stride = key_cache.shape[2]
    if value_cache is None:
        _need(kv_heads * vdim <= k_stride and (kv_heads == 1 or vdim == dim),
              "capped_attention: values inside the key rows need value size <= key size (equal with several heads)")
        value_cache, v_stride = key_cache, k_stride
    else:
        _need(value_cache.dtype == out.dtype and value_cache.is_contiguous() and value_cache.dim() == 3
              and value_cache.shape[:2] == key_cache.shape[:2] and value_cache.shape[2] >= kv_heads * vdim,
              "capped_attention: value cache")
        v_stride = value_cache.shape[2]
    _need(batch.max_pages_used <= tables.shape[1] and batch.max_page_id < key_cache.shape[0],
          "capped_attention: block tables exceed the cache")
    if gate is not None:
        _need(gate.shape == out.shape and gate.dtype == out.dtype, "capped_attention: gate")
    longest = int(getattr(batch, "max_query_len", 0) or 0)
    with _on_device_of(q):
        lib = load_library()
        need = lib.swm_masked_attention_workspace_floats(rows, n, longest, heads, kv_heads, vdim, key_cache.shape[1],
                                                         tables.shape[1], int(window), int(chunk))
        work = torch.empty(need, dtype=torch.float32, device=q.device) if need > 0 else None
        if score_bias is not None:
            _need(k_stride == kv_heads * dim and v_stride == kv_heads * vdim and value_cache is not key_cache,
                  "capped_attention: sigmoid weights read plain key and value caches")
            _check(lib.swm_sigmoid_attention(
                out.data_ptr(), q.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), _opt_ptr(gate),
                0 if gate is None else _rows(gate, "gate"), score_bias.data_ptr(), tables.data_ptr(), tables.shape[1],
                batch.q_start.data_ptr(), batch.ctx_len.data_ptr(), rows, n, longest, heads, kv_heads, dim, vdim,
                key_cache.shape[1], scale, int(window), _opt_ptr(work), _act(out), _stream(q)))
            return
        _check(lib.swm_masked_attention(
            out.data_ptr(), q.data_ptr(), key_cache.data_ptr(), value_cache.data_ptr(), _opt_ptr(gate),
            0 if gate is None else _rows(gate, "gate"), tables.data_ptr(), tables.shape[1], batch.q_start.data_ptr(),
            batch.ctx_len.data_ptr(), rows, n, longest, heads, kv_heads, dim, vdim, key_cache.shape[1], scale, softcap,
            int(window), int(chunk), 1 if sink else 0, k_stride, v_stride, _opt_ptr(work), _act(out), _stream(q)))


def gated_stream_step(stream: torch.Tensor, y: Optional[torch.Tensor], gate: Optional[torch.Tensor], mult: float,
                      history: Optional[torch.Tensor] = None, depth_weights: Optional[torch.Tensor] = None,
                      norm=None, out: Optional[torch.Tensor] = None) -> None:
    """stream (fp32 [rows, width], in place) += mult * y * sigmoid(gate) (y, gate: 2-D views in the activation
    dtype; y None: nothing is added; gate None: no gate).  ``history`` fp32 [entries, rows, width] with
    ``depth_weights`` fp32 [entries]: the sum is filed as the last entry and the stream becomes the entries'
    weighted sum.  ``norm`` = (alpha [1], weight [width], bias [width]) fp32 with ``out``: out = tanh(alpha * stream)
    * weight + bias in out's dtype."""
    _dev(stream, y, gate, history, depth_weights, out)
    _f32c(stream, "stream")
    rows, width = stream.shape
    act = out if out is not None else y
    _need(act is not None or history is not None, "gated_stream_step: nothing to do")
    if y is not None:
        _need(y.shape == stream.shape and (gate is None or (gate.shape == stream.shape and gate.dtype == y.dtype)),
              "gated_stream_step: addend and gate")
    entries = 0
    if history is not None:
        _f32c(history, "history")
        _f32c(depth_weights, "depth_weights")
        entries = depth_weights.numel()
        _need(history.dim() == 3 and history.shape[1:] == stream.shape and 1 <= entries <= history.shape[0],
              "gated_stream_step: history")
    alpha = weight = bias = None
    if out is not None:
        alpha, weight, bias = norm
        for t, what in ((alpha, "alpha"), (weight, "norm weight"), (bias, "norm bias")):
            _f32c(t, what)
        _need(out.shape == stream.shape and out.is_contiguous() and alpha.numel() == 1 and weight.numel() == width
              and bias.numel() == width and (y is None or y.dtype == out.dtype), "gated_stream_step: norm")
    with _on_device_of(stream):
        _check(load_library().swm_gated_stream_step(
            stream.data_ptr(), _opt_ptr(y), 0 if y is None else _rows(y, "y"), _opt_ptr(gate),
            0 if gate is None else _rows(gate, "gate"), mult, _opt_ptr(history), rows * width, _opt_ptr(depth_weights),
            entries, _opt_ptr(alpha), _opt_ptr(weight), _opt_ptr(bias), _opt_ptr(out), rows, width,
            SW_F32 if act is None else _act(act), _stream(stream)))


def poly_norm(out: torch.Tensor, z: torch.Tensor, coef: torch.Tensor, eps: float) -> None:
    """out [rows, ff] = c0 U(z) + c1 U(z^2) + c2 U(z^3) + c3 with U = division of a row by its root mean square;
    coef fp32 [4]."""
    _dev(out, z, coef)
    _f32c(coef, "coef")
    _need(out.is_contiguous() and out.shape == z.shape and out.dtype == z.dtype and coef.numel() == 4 and z.dim() == 2,
          "poly_norm: shapes")
    with _on_device_of(out):
        _check(load_library().swm_poly_norm(out.data_ptr(), z.data_ptr(), _rows(z, "z"), coef.data_ptr(), eps,
                                            z.shape[0], z.shape[1], _act(out), _stream(out)))


def gate_mul(out: torch.Tensor, y: torch.Tensor, gate: torch.Tensor, silu: bool = False) -> None:
    """out [rows, heads * size] = y * sigmoid(gate) (``silu``: y * gate * sigmoid(gate)); y is [rows, heads * size]
    or a strided [rows, heads, size] view (e.g. the transpose of a batched product), gate a 2-D view."""
    _dev(out, y, gate)
    rows, n = out.shape
    if y.dim() == 2:
        y = y.unsqueeze(1)
    _need(y.dim() == 3 and y.shape[0] == rows and y.shape[1] * y.shape[2] == n and y.stride(2) == 1
          and gate.shape == out.shape and gate.dtype == out.dtype == y.dtype and out.is_contiguous(), "gate_mul: shapes")
    with _on_device_of(out):
        _check(load_library().swm_gate_mul(out.data_ptr(), y.data_ptr(), y.stride(0), y.stride(1), gate.data_ptr(),
                                           _rows(gate, "gate"), rows, y.shape[1], y.shape[2], 1 if silu else 0,
                                           _act(out), _stream(out)))


def latent_rope_cache(q_out: torch.Tensor, q_latent: torch.Tensor, q_rot: torch.Tensor, down: Optional[torch.Tensor],
                      norm_weight: Optional[torch.Tensor], eps: float, positions: torch.Tensor, inv_freq: torch.Tensor,
                      cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor]) -> None:
    """q_latent [rows, heads, rank], q_rot [rows, heads, rot]: strided views in the activation dtype; down [rows,
    rank + rot]: a 2-D view; cache [pages, page, rank + rot].  q_out fp32 [rows, heads * (rank + rot)]."""
    _dev(q_out, q_latent, q_rot, down, norm_weight, positions, inv_freq, cache, slot_mapping)
    _f32c(q_out, "q_out")
    rows, heads, rank = q_latent.shape
    rot = q_rot.shape[2]
    _need(q_rot.shape[:2] == (rows, heads) and q_latent.stride(2) == 1 and (rot == 0 or q_rot.stride(2) == 1)
          and q_rot.dtype == q_latent.dtype and q_out.shape == (rows, heads * (rank + rot)), "latent_rope_cache: queries")
    _need(positions.dtype == torch.int64 and positions.numel() == rows and positions.is_contiguous(),
          "latent_rope_cache: positions must be int64 [rows]")
    if rot:
        _f32c(inv_freq, "inv_freq")
        _need(2 * inv_freq.numel() == rot, "latent_rope_cache: one frequency per rotated pair")
    if down is not None:
        _f32c(norm_weight, "norm_weight")
        _need(down.shape == (rows, rank + rot) and down.dtype == q_latent.dtype and norm_weight.numel() == rank
              and cache.dtype == down.dtype and cache.is_contiguous() and cache.shape[-1] == rank + rot
              and slot_mapping.dtype == torch.int64 and slot_mapping.numel() == rows and slot_mapping.is_contiguous(),
              "latent_rope_cache: cache write")
    with _on_device_of(q_out):
        _check(load_library().swm_latent_rope_cache(
            q_out.data_ptr(), q_latent.data_ptr(), q_latent.stride(0), q_latent.stride(1), q_rot.data_ptr(),
            q_rot.stride(0), q_rot.stride(1), _opt_ptr(down), 0 if down is None else _rows(down, "down"),
            _opt_ptr(norm_weight), eps, positions.data_ptr(), _opt_ptr(inv_freq) if rot else None,
            None if down is None else cache.data_ptr(), None if down is None else slot_mapping.data_ptr(), rows, heads,
            rank, rot, _act(q_latent), _stream(q_out)))


def gla(out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay_pre: torch.Tensor,
        decay_bias: Optional[torch.Tensor], tau: float, q_scale: float, state: torch.Tensor, batch, heads: int,
        dim: int, vdim: int) -> None:
    """out fp32 [rows, heads * vdim]; q, k, v: column ranges of one projection output; decay_pre [rows, heads * dim]
    in the same dtype; decay_bias fp32 [heads * dim]; state fp32 [slots, heads, dim, vdim]."""
    _dev(out, q, k, v, decay_pre, decay_bias, state)
    for t, what in ((out, "out"), (state, "state")):
        _f32c(t, what)
    rows = q.shape[0]
    n = _ragged_ok(batch, rows)
    stride = _rows(q, "q")
    _need(q.shape == (rows, heads * dim) and k.shape == q.shape and v.shape == (rows, heads * vdim)
          and _rows(k, "k") == stride and _rows(v, "v") == stride and k.dtype == q.dtype and v.dtype == q.dtype
          and decay_pre.shape == q.shape and decay_pre.dtype == q.dtype and out.shape == (rows, heads * vdim)
          and state.shape[1:] == (heads, dim, vdim) and batch.max_state_slot < state.shape[0], "gla: shapes")
    if decay_bias is not None:
        _f32c(decay_bias, "decay_bias")
        _need(decay_bias.numel() == heads * dim, "gla: one bias per head and key channel")
    longest = int(getattr(batch, "max_query_len", 0) or 0)
    with _on_device_of(q):
        lib = load_library()
        need = lib.swm_gla_workspace_floats(rows, n, longest, heads, dim, vdim)
        work = torch.empty(need, dtype=torch.float32, device=q.device) if need > 0 else None
        _check(lib.swm_gla(out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), stride, decay_pre.data_ptr(),
                           _rows(decay_pre, "decay_pre"), _opt_ptr(decay_bias), tau, q_scale, state.data_ptr(),
                           batch.q_start.data_ptr(), batch.ctx_len.data_ptr(), batch.state_slot.data_ptr(), rows, n,
                           longest, heads, dim, vdim, _opt_ptr(work), _act(q), _stream(q)))


def lightning(out: torch.Tensor, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, decay: torch.Tensor,
              state: torch.Tensor, batch, heads: int, dim: int, vdim: int) -> None:
    """out fp32 [rows, heads * vdim]; q, k, v: column ranges of one projection output (before their silu);
    decay fp32 [heads]; state fp32 [slots, heads, dim, vdim]."""
    _dev(out, q, k, v, decay, state)
    for t, what in ((out, "out"), (decay, "decay"), (state, "state")):
        _f32c(t, what)
    rows = q.shape[0]
    n = _ragged_ok(batch, rows)
    stride = _rows(q, "q")
    _need(q.shape == (rows, heads * dim) and k.shape == q.shape and v.shape == (rows, heads * vdim)
          and _rows(k, "k") == stride and _rows(v, "v") == stride and k.dtype == q.dtype and v.dtype == q.dtype
          and out.shape == (rows, heads * vdim) and decay.numel() == heads and state.shape[1:] == (heads, dim, vdim)
          and batch.max_state_slot < state.shape[0], "lightning: shapes")
    longest = int(getattr(batch, "max_query_len", 0) or 0)
    with _on_device_of(q):
        lib = load_library()
        need = lib.swm_lightning_workspace_floats(rows, n, longest, heads, dim, vdim)
        work = torch.empty(need, dtype=torch.float32, device=q.device) if need > 0 else None
        _check(lib.swm_lightning(out.data_ptr(), q.data_ptr(), k.data_ptr(), v.data_ptr(), stride, decay.data_ptr(),
                                 state.data_ptr(), batch.q_start.data_ptr(), batch.ctx_len.data_ptr(),
                                 batch.state_slot.data_ptr(), rows, n, longest, heads, dim, vdim, _opt_ptr(work),
                                 _act(q), _stream(q)))


ops = SimpleNamespace(expert_ffn=expert_ffn, ACT_GELU=ACT_GELU, ACT_RELU2=ACT_RELU2,
    scalar_norm_add=scalar_norm_add, scalar_norm=scalar_norm, qk_norm_cache=qk_norm_cache,
    window_attention=window_attention, short_conv=short_conv, channel_delta=channel_delta,
    general_delta=general_delta, head_norm_gate=head_norm_gate, stream_add_norm=stream_add_norm,
    clamped_glu=clamped_glu, relu2=relu2, rope_cache=rope_cache, group_router=group_router, group_pairs=group_pairs,
    capped_attention=capped_attention, lightning=lightning, gated_stream_step=gated_stream_step, poly_norm=poly_norm,
    gate_mul=gate_mul, latent_rope_cache=latent_rope_cache, gla=gla, ACT_NONE=ACT_NONE, glu_rows=glu_rows,
    group_norm_add=group_norm_add, causal_conv=causal_conv, gated_delta=gated_delta)
