"""Python faces of the HIP kernels.  Each wrapper checks on the host that operand shapes,
dtypes and strides are what its kernel and grid assume, then launches on torch's current
stream.  There is no fallback: without the compiled library every call raises.
"""

from __future__ import annotations

import ctypes
import functools
from ctypes import c_double, c_float, c_int, c_longlong, c_void_p
from typing import Optional, Sequence, Tuple

import torch

from . import build as _build

EPI_F32, EPI_BF16, EPI_ADD_F32, EPI_SWIGLU_BF16 = 0, 1, 2, 3
ATT_PART = 64          # keys per partition of the bfloat16 attention fold


def fold_group_tiles(head_dim: int) -> int:
    """Tiles (of 16 query columns) one wave of the fold kernel owns; a wave's tiles must belong
    to one sequence, so the host pads every sequence's tile list to a multiple of this."""
    return int(_fn("bw_attention_fold_group_tiles")(int(head_dim)))
HEAD_DIMS = (16, 32, 48, 64, 80, 96, 112, 128, 160, 192, 224, 256)
PAGE_SIZES = (8, 16, 32, 64)       # tokens in a page that the attention kernels and the cache writes take

_ERRORS = {
    -2: "sizes or strides out of the kernel's range",
    -3: "misaligned pointer or stride",
    -4: f"head size not compiled in (supported: {HEAD_DIMS})",
    -5: "page size not supported (a power of two from 4 to 64 is needed)",
    -6: "scratch smaller than attention_decode_scratch asks for",
    -8: "the workgroup's partials do not fit the compute unit's LDS",
    -7: "sizes beyond what the library's static scratch holds",
}

_SIGS = {
    "bw_embed": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_rmsnorm": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float, c_void_p],
    "bw_add": [c_void_p, c_void_p, c_longlong, c_void_p],
    "bw_add_bias": [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_convert": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_swiglu_f32": [c_void_p, c_void_p, c_int, c_int, c_void_p],
    "bw_gather_rows_f32": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_rope_kvwrite": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p,
                        c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_f32": [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_clamped_glu_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p],
    "bw_gemm_add_scratch": [c_int, c_int, c_int, c_void_p, c_void_p],
    "bw_gemm_add_bf16": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_longlong, c_void_p,
                         c_int, c_void_p],
    "bw_gemm_add_bf16_static": [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_gemm_add_bf16_static_max": [c_void_p, c_void_p],
    "bw_gemm_qkv_rope_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                              c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_attention_f32_tiles": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_void_p,
                               c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_int, c_float, c_void_p],
    "bw_attention_f32": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                         c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_void_p, c_int, c_float, c_void_p],
    "bw_attention_bf16": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_longlong,
                          c_void_p, c_int, c_void_p, c_int, c_float, c_void_p],
    "bw_attention_decode_scratch": [c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p],
    "bw_attention_fold_group_tiles": [c_int],
    "bw_norm_gemm_supported": [c_int, c_int],
    "bw_norm_gemm_wide_supported": [c_int, c_int, c_int, c_int],
    "bw_norm_gemm_bf16": [c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                          c_int, c_void_p],
    "bw_norm_qkv_rope_bf16": [c_void_p, c_int, c_void_p, c_int, c_float, c_void_p, c_void_p, c_void_p, c_void_p,
                              c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                              c_int, c_int, c_int, c_void_p],
    "bw_chain_sync_words": [],
    "bw_chain_begin": [c_void_p, c_int, c_void_p, c_int],
    "bw_chain_flush": [c_void_p],
    "bw_chain_end": [c_void_p],
    "bw_sample": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    "bw_fingerprint": [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p],
    "bw_norm_shift": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_longlong, c_void_p, c_void_p, c_void_p, c_void_p,
                      c_void_p, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
    "bw_rotate_halves_rows": [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p],
    "bw_tanh_rows": [c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_norm_mean": [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "bw_norm_mean_add": [c_void_p, c_void_p, c_void_p, c_int, c_float, c_void_p, c_float, c_float, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_linear_recurrence": [c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p,
                             c_float, c_float, c_float, c_void_p, c_longlong, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int,
                             c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_longlong, c_void_p],
    "bw_head_norm_gate": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_void_p, c_int,
                          c_int, c_int, c_float, c_void_p],
    "bw_glu": [c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_float, c_float, c_void_p, c_int, c_void_p],
    "bw_embed_sum": [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                     c_float, c_int, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_void_p],
    "bw_whole_norm_kv": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_float, c_void_p, c_int,
                         c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                         c_int, c_int, c_void_p],
    "bw_shared_key_attention_mfma": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_int,
                                     c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_int, c_int,
                                     c_void_p, c_longlong, c_void_p],
    "bw_latent_prep": [c_void_p, c_int, c_int, c_int, c_void_p, c_float, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                       c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                       c_void_p],
    "bw_headwise_linear": [c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                           c_int, c_void_p],
    "bw_causal_conv": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_longlong, c_void_p, c_void_p,
                       c_void_p, c_int, c_int, c_void_p, c_int, c_void_p],
    "bw_pair_rope_unit": [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int,
                          c_int, c_int, c_int, c_void_p],
    "bw_gate_mul": [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p],
    "bw_rglru_scan": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_longlong,
                      c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "bw_norm_add": [c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_float, c_void_p, c_void_p,
                    c_int, c_float, c_void_p],
    "bw_softcap": [c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "bw_scale_rows": [c_void_p, c_int, c_int, c_int, c_float, c_void_p],
    "bw_moe_route": [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p],
    "bw_moe_route_plan": [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p, c_int, c_void_p, c_void_p,
                          c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "bw_moe_max_tiles": [c_int, c_int],
    "bw_moe_plan": [c_void_p, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p],
    "bw_moe_experts": [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                       c_int, c_int, c_int, c_float, c_float, c_int, c_void_p],
    "bw_moe_combine": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p],
    "bw_shared_key_attention": [c_void_p, c_int, c_void_p, c_void_p, c_int, c_void_p, c_int, c_void_p, c_int, c_int,
                                c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_float, c_int, c_void_p],
}

_fns = {}

# While a chain is open (``chain`` below) the library keeps the decode products that can run as phases of one
# launch back; these entry points may be called meanwhile (they join the chain, launch through the library's own
# path that sends the waiting phases first, or launch nothing).  Every other one is a launch that must come after
# what waits.
_CHAIN_KEEPS = frozenset({
    "bw_gemm_bf16", "bw_gemm_add_bf16", "bw_norm_gemm_bf16", "bw_norm_qkv_rope_bf16",
    "bw_gemm_add_scratch", "bw_norm_gemm_supported", "bw_norm_gemm_wide_supported", "bw_attention_decode_scratch",
    "bw_attention_fold_group_tiles", "bw_gemm_add_bf16_static_max", "bw_moe_max_tiles", "bw_chain_sync_words", "bw_chain_begin",
    "bw_chain_flush", "bw_chain_end",
})
_chain_open = False


def _fn(name: str):
    if _chain_open and name not in _CHAIN_KEEPS:
        _check(_fn("bw_chain_flush")(_stream()), "chain flush")
    f = _fns.get(name)
    if f is None:
        lib = _build.load()
        f = getattr(lib, name)
        f.argtypes = _SIGS[name]
        f.restype = c_int
        _fns[name] = f
    return f


def available() -> bool:
    """True if the library is built or can be built here (no GPU needed to answer)."""
    try:
        _build.load()
        return True
    except _build.KernelLibraryError:
        return False


def _check(code: int, what: str) -> None:
    if code != 0:
        why = _ERRORS.get(code, f"HIP error {code}")
        raise RuntimeError(f"{what}: {why}")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)
_raw_device = getattr(torch._C, "_cuda_getDevice", None)


def _stream() -> int:
    """The current stream's handle (the stream a graph capture has made current, too).  torch's own
    ``current_stream()`` builds a Python object for it at some 8 us a call, which an eager step of a short
    prompt pays 170 times; the raw handle costs a fraction of a microsecond."""
    if _raw_stream is not None and _raw_device is not None:
        return _raw_stream(_raw_device())
    return torch.cuda.current_stream().cuda_stream


def _need(t: torch.Tensor, dtype, what: str) -> None:
    if not t.is_cuda:
        raise ValueError(f"{what} must live on the GPU (there is no CPU path)")
    if t.dtype != dtype:
        raise ValueError(f"{what} must be {dtype}, got {t.dtype}")
    if not t.is_contiguous():
        raise ValueError(f"{what} must be contiguous")


def _need_strided(t: torch.Tensor, dtype, what: str) -> None:
    """As ``_need`` for a view whose rows lie a stride apart (the caller passes the stride on)."""
    if not t.is_cuda:
        raise ValueError(f"{what} must live on the GPU (there is no CPU path)")
    if t.dtype != dtype:
        raise ValueError(f"{what} must be {dtype}, got {t.dtype}")
    if t.dim() != 2 or t.stride(1) != 1:
        raise ValueError(f"{what} must be a matrix whose rows are contiguous")


def _is_bf16(t: torch.Tensor, what: str) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise ValueError(f"{what} must be bfloat16 or float32, got {t.dtype}")


# ------------------------------------------------------------------------------ several products, one launch

CHAIN_SPIN_LIMIT = 200000      # looks at a phase's flag before a wait gives up (some tenths of a second)


def chain_sync_words() -> int:
    return int(_fn("bw_chain_sync_words")())


class chain:
    """``with ops.chain(sync, err):`` the decode products of up to 16 rows asked for inside (RMSNorm + product with SwiGLU,
    with a 32-bit store, or with rotation and cache write; residual adds) do not leave one by one: they wait and
    run as phases of one launch, in the order they were asked for, when anything else is launched through this
    module or the block ends.  A phase asks for its weights while the phase before it still runs, and waits inside
    the kernel only for what that phase writes: the same bits, fewer kernel boundaries.  ``sync``: int32 zeros,
    ``chain_sync_words()`` of them (left zero by every launch); ``err``: an int32 word that gets a bit if a wait
    inside a launch gave up (then the step's results are void and ``sync`` has to be zeroed).  Everything put on the
    stream inside the block must come through this module: a launch from elsewhere would overtake what waits."""

    def __init__(self, sync: torch.Tensor, err: torch.Tensor, spin_limit: int = CHAIN_SPIN_LIMIT):
        _need(sync, torch.int32, "sync")
        _need(err, torch.int32, "err")
        if sync.numel() < chain_sync_words() or err.numel() < 1:
            raise ValueError(f"chain: sync needs {chain_sync_words()} words and err one")
        self.sync, self.err, self.spin_limit = sync, err, int(spin_limit)

    def __enter__(self):
        global _chain_open
        if _chain_open:
            raise RuntimeError("a chain is already open")
        _check(_fn("bw_chain_begin")(self.sync.data_ptr(), self.sync.numel(), self.err.data_ptr(), self.spin_limit), "chain")
        _chain_open = True
        return self

    def __exit__(self, *exc):
        global _chain_open
        _chain_open = False
        _check(_fn("bw_chain_end")(_stream()), "chain")
        return False


# ------------------------------------------------------------------------------ row ops

TOKEN_FROM_FEEDBACK = -2     # a token id that means: take this row's token from ``feedback``


def embed(tokens: torch.Tensor, table: torch.Tensor, out: torch.Tensor, feedback: Optional[torch.Tensor] = None) -> None:
    """out[r, :] = float(table[tokens[r], :]); a negative token gives a zero row, except TOKEN_FROM_FEEDBACK,
    which reads the row's token from ``feedback`` (int32, a row each) if that is given."""
    _need(tokens, torch.int32, "tokens")
    _need(out, torch.float32, "out")
    rows = tokens.numel()
    vocab, width = table.shape
    if not table.is_cuda or not table.is_contiguous():
        raise ValueError("embedding table must be a contiguous GPU tensor")
    if out.shape[0] < rows or out.shape[1] != width:
        raise ValueError(f"embed: out {tuple(out.shape)} does not fit {rows} rows of width {width}")
    if feedback is not None:
        _need(feedback, torch.int32, "feedback")
        if feedback.numel() < rows:
            raise ValueError("embed: feedback is shorter than the rows")
    _check(_fn("bw_embed")(tokens.data_ptr(), None if feedback is None else feedback.data_ptr(), table.data_ptr(),
                           _is_bf16(table, "table"), out.data_ptr(), rows, width, vocab, _stream()), "embed")


def embed_sum(tokens: torch.Tensor, positions: torch.Tensor, table: torch.Tensor, scale: float, out: torch.Tensor,
              pair_table: Optional[torch.Tensor] = None, pair_hash: Tuple[int, int, int] = (0, 0, 0),
              pos_table: Optional[torch.Tensor] = None, row_seq: Optional[torch.Tensor] = None,
              seq_rows: Optional[torch.Tensor] = None, slots: Optional[torch.Tensor] = None,
              state: Optional[torch.Tensor] = None, feedback: Optional[torch.Tensor] = None) -> None:
    """out[r] = table[token] * scale + pair_table[row] + pos_table[position], 32-bit, the two last tables optional.
    ``pair_hash`` = (buckets, mul_prev, mul_cur): row = (token before * mul_prev + token * mul_cur) mod buckets, and row
    ``buckets`` at a request's position 0.  The token before a request's first row of the step is ``state[slot]`` (int32, a
    word a slot), which then takes the request's last token of the step.  Tokens as in ``embed``."""
    _need(tokens, torch.int32, "tokens")
    _need(positions, torch.int32, "positions")
    _need(out, torch.float32, "out")
    rows = tokens.numel()
    vocab, width = table.shape
    tables = [t for t in (table, pair_table, pos_table) if t is not None]
    if any(not t.is_cuda or not t.is_contiguous() or t.dim() != 2 or t.shape[1] != width or t.dtype != table.dtype for t in tables):
        raise ValueError("embed_sum: the tables must be contiguous GPU matrices of one dtype and one width")
    if out.shape[0] < rows or out.shape[1] != width or positions.numel() < rows:
        raise ValueError(f"embed_sum: out {tuple(out.shape)} or the positions do not fit {rows} rows of width {width}")
    buckets, mul_prev, mul_cur = (int(v) for v in pair_hash)
    if pair_table is not None:
        for t, what in ((row_seq, "row_seq"), (seq_rows, "seq_rows"), (slots, "slots"), (state, "state")):
            if t is None:
                raise ValueError(f"embed_sum: a table of token pairs needs {what}")
            _need(t, torch.int32, what)
        if buckets < 1 or pair_table.shape[0] != buckets + 1 or row_seq.numel() < rows:
            raise ValueError("embed_sum: the pair table has one row more than buckets")
    if feedback is not None:
        _need(feedback, torch.int32, "feedback")
        if feedback.numel() < rows:
            raise ValueError("embed_sum: feedback is shorter than the rows")
    ptr = lambda t: 0 if t is None else t.data_ptr()
    _check(_fn("bw_embed_sum")(tokens.data_ptr(), ptr(feedback), positions.data_ptr(), ptr(row_seq), ptr(seq_rows), ptr(slots),
                               ptr(state), table.data_ptr(), ptr(pair_table), ptr(pos_table), _is_bf16(table, "table"),
                               float(scale), buckets, mul_prev, mul_cur,
                               0x7fffffff if pos_table is None else pos_table.shape[0], out.data_ptr(), rows, width, vocab,
                               _stream()), "embed_sum")


def rmsnorm(x: torch.Tensor, weight: torch.Tensor, out: torch.Tensor, rows: int, eps: float) -> None:
    """out[r] = (x[r] * 1/sqrt(mean(x[r]^2) + eps)) * weight; out float32 (reference order of
    operations) or bfloat16 (32-bit arithmetic, one rounding)."""
    _need(x, torch.float32, "x")
    dim = x.shape[-1]
    if weight.numel() != dim or not weight.is_cuda:
        raise ValueError(f"rmsnorm: weight has {weight.numel()} elements, rows are {dim} wide")
    if x.shape[0] < rows or out.shape[0] < rows or out.shape[-1] != dim or not out.is_contiguous() or not out.is_cuda:
        raise ValueError("rmsnorm: out does not fit x")
    _check(_fn("bw_rmsnorm")(x.data_ptr(), weight.data_ptr(), _is_bf16(weight, "weight"), out.data_ptr(),
                             _is_bf16(out, "out"), rows, dim, out.stride(0), float(eps), _stream()), "rmsnorm")


def add_(x: torch.Tensor, y: torch.Tensor, rows: int) -> None:
    _need(x, torch.float32, "x")
    _need(y, torch.float32, "y")
    if x.shape[1:] != y.shape[1:] or x.shape[0] < rows or y.shape[0] < rows:
        raise ValueError("add_: shapes differ")
    _check(_fn("bw_add")(x.data_ptr(), y.data_ptr(), rows * x.stride(0), _stream()), "add")


def add_bias(x: torch.Tensor, bias: torch.Tensor, rows: int) -> None:
    """x[:rows] += bias (32-bit, one addition an element): a projection's bias behind its product."""
    _need(x, torch.float32, "x")
    _need(bias, torch.float32, "bias")
    if bias.dim() != 1 or bias.shape[0] != x.shape[1] or x.shape[0] < rows:
        raise ValueError(f"add_bias: x {tuple(x.shape)} and bias {tuple(bias.shape)} do not match")
    _check(_fn("bw_add_bias")(x.data_ptr(), bias.data_ptr(), rows, x.shape[1], x.stride(0), _stream()), "add_bias")


def convert(src: torch.Tensor, dst: torch.Tensor, rows: int) -> None:
    """dst[:rows] = src[:rows] between float32 and bfloat16 (narrowing rounds to nearest even)."""
    if not (src.is_cuda and dst.is_cuda) or src.dim() != 2 or dst.dim() != 2:
        raise ValueError("convert: two GPU matrices are needed")
    if src.shape[1] != dst.shape[1] or src.shape[0] < rows or dst.shape[0] < rows:
        raise ValueError(f"convert: {tuple(src.shape)} does not fit {tuple(dst.shape)} for {rows} rows")
    if src.stride(1) != 1 or dst.stride(1) != 1:
        raise ValueError("convert: rows must be contiguous")
    _check(_fn("bw_convert")(src.data_ptr(), _is_bf16(src, "src"), dst.data_ptr(), _is_bf16(dst, "dst"), rows, src.shape[1],
                             src.stride(0), dst.stride(0), _stream()), "convert")


def swiglu_f32(gate_up: torch.Tensor, out: torch.Tensor, rows: int) -> None:
    _need(gate_up, torch.float32, "gate_up")
    _need(out, torch.float32, "out")
    inter = out.shape[1]
    if gate_up.shape[1] != 2 * inter or gate_up.shape[0] < rows or out.shape[0] < rows:
        raise ValueError("swiglu: gate_up must be [rows, 2*inter] for out [rows, inter]")
    _check(_fn("bw_swiglu_f32")(gate_up.data_ptr(), out.data_ptr(), rows, inter, _stream()), "swiglu")


def gather_rows(x: torch.Tensor, index: torch.Tensor, out: torch.Tensor, count: int) -> None:
    _need(x, torch.float32, "x")
    _need(index, torch.int32, "index")
    _need(out, torch.float32, "out")
    if out.shape[1] != x.shape[1] or out.shape[0] < count or index.numel() < count:
        raise ValueError("gather_rows: out does not fit")
    _check(_fn("bw_gather_rows_f32")(x.data_ptr(), index.data_ptr(), out.data_ptr(), count, x.shape[1], x.stride(0),
                                     _stream()), "gather_rows")


def rope_kvwrite(qkv: torch.Tensor, q_out: Optional[torch.Tensor], positions: torch.Tensor, row_seq: torch.Tensor,
                 block_table: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, k_cache: torch.Tensor,
                 v_cache: torch.Tensor, rows: int, heads: int, kv_heads: int, head_dim: int, page_size: int,
                 write_cache: bool = True) -> None:
    """Rotate q and k of every row at its position and store k, v in the row's page slot.
    32-bit caches: q, k rotated in place in ``qkv``.  bfloat16 caches: q goes to ``q_out``."""
    _need(qkv, torch.float32, "qkv")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    bf = _is_bf16(k_cache, "k_cache")
    if v_cache.dtype != k_cache.dtype:
        raise ValueError("k and v caches must have one dtype")
    width = (heads + 2 * kv_heads) * head_dim
    if qkv.shape[1] != width or qkv.shape[0] < rows or positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError(f"rope_kvwrite: qkv must be [>= {rows}, {width}]")
    if cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise ValueError("rope_kvwrite: tables must be [positions, head_dim/2]")
    page_elems = kv_heads * page_size * head_dim
    if k_cache.numel() % page_elems or v_cache.numel() != k_cache.numel():
        raise ValueError("rope_kvwrite: cache size is no multiple of a page")
    if bf:
        if q_out is None:
            raise ValueError("rope_kvwrite: bfloat16 needs q_out")
        _need(q_out, torch.bfloat16, "q_out")
        if q_out.shape[1] != heads * head_dim or q_out.shape[0] < rows:
            raise ValueError("rope_kvwrite: q_out must be [rows, heads*head_dim]")
    _check(_fn("bw_rope_kvwrite")(qkv.data_ptr(), q_out.data_ptr() if q_out is not None else 0, positions.data_ptr(),
                                  row_seq.data_ptr(), block_table.data_ptr(), block_table.stride(0), cos.data_ptr(),
                                  sin.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), bf, rows, heads, kv_heads,
                                  head_dim, page_size, int(write_cache), _stream()), "rope_kvwrite")


# ------------------------------------------------------------------------------ matrix products

def gemm_f32(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows: int, accumulate: bool = False) -> None:
    """out[:rows] (+)= x[:rows] @ w.T with one k-ascending fused multiply-add chain per output.  ``x`` and ``out`` may
    be column slices of wider matrices (rows apart by their strides)."""
    if not x.is_cuda or x.dtype != torch.float32 or x.dim() != 2 or x.stride(1) != 1:
        raise ValueError("gemm_f32: x must be a float32 GPU matrix with contiguous rows")
    _need_strided(out, torch.float32, "out")
    if not w.is_cuda or not w.is_contiguous() or w.dim() != 2:
        raise ValueError("gemm_f32: weight must be a contiguous [N, K] GPU tensor")
    N, K = w.shape
    if x.shape[1] != K or out.shape[1] != N or x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError(f"gemm_f32: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not match")
    _check(_fn("bw_gemm_f32")(x.data_ptr(), w.data_ptr(), _is_bf16(w, "weight"), out.data_ptr(), rows, N, K,
                              x.stride(0), out.stride(0), int(accumulate), _stream()), "gemm_f32")


@functools.lru_cache(maxsize=None)
def gemm_add_scratch(rows: int, N: int, K: int) -> Tuple[int, int]:
    """(float32 elements, int32 counters) that a residual add of this shape wants as ``scratch``
    to give every 2048-segment of K workgroups of its own; (0, 0): it would not.  (A function of the
    three sizes alone: asked once for each.)"""
    floats, counters = ctypes.c_longlong(0), ctypes.c_int(0)
    _check(_fn("bw_gemm_add_scratch")(rows, N, K, ctypes.addressof(floats), ctypes.addressof(counters)), "gemm_add_scratch")
    return int(floats.value), int(counters.value)


def gemm_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows: int, epilogue: int,
              scratch: Optional[Tuple[torch.Tensor, torch.Tensor]] = None) -> None:
    """out[:rows] = epilogue(x[:rows] @ w.T) on the matrix cores; see gemm_bf16.hip for the
    arithmetic.  EPI_SWIGLU_BF16 takes the stacked weight [2N, K] (gate rows, then up rows).
    ``scratch`` (EPI_ADD_F32 only): the tensors ``gemm_add_scratch`` asks for (float32, int32
    zeros); the bits do not depend on it.  ``x`` may be a column slice of a wider matrix that starts at a multiple of 8
    elements, and with a 32-bit store ``out`` may be a column slice too."""
    _need_strided(x, torch.bfloat16, "x")
    _need(w, torch.bfloat16, "weight")
    if w.dim() != 2:
        raise ValueError("gemm_bf16: weight must be [N, K]")
    N, K = w.shape
    if epilogue == EPI_SWIGLU_BF16:
        if N % 2:
            raise ValueError("gemm_bf16: SwiGLU needs a stacked weight with an even number of rows")
        N //= 2
    want = torch.bfloat16 if epilogue in (EPI_BF16, EPI_SWIGLU_BF16) else torch.float32
    if epilogue == EPI_F32:
        _need_strided(out, want, "out")
    else:
        _need(out, want, "out")
    if x.shape[1] != K or out.shape[1] != N or x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError(f"gemm_bf16: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not match")
    if K % 8:
        raise ValueError(f"gemm_bf16: inner size {K} must be a multiple of 8 (16-byte operand loads)")
    if scratch is not None and epilogue == EPI_ADD_F32:
        sc_f, sc_c = scratch
        _need(sc_f, torch.float32, "scratch")
        _need(sc_c, torch.int32, "scratch counters")
        _check(_fn("bw_gemm_add_bf16")(x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, N, K, x.stride(0), out.stride(0),
                                       sc_f.data_ptr(), sc_f.numel(), sc_c.data_ptr(), sc_c.numel(), _stream()), "gemm_bf16")
        return
    _check(_fn("bw_gemm_bf16")(x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, N, K, x.stride(0), out.stride(0),
                               epilogue, _stream()), "gemm_bf16")


CLAMPED_GLU_MIN_ROWS = 65      # steps of fewer rows run the clamped unit as a kernel behind the 32-bit product


def gemm_clamped_glu_bf16(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, rows: int, limit: float, alpha: float) -> None:
    """out[:rows, n] = bf16(g sigmoid(alpha g) (u + 1)), g = min(x . w[n], limit), u = clamp(x . w[N + n], -limit, limit):
    the stacked product [2N, K] of a prompt portion (more than 64 rows) with the clamped gated unit in its epilogue; the
    bits of gemm_bf16 with a 32-bit store followed by ``glu``."""
    _need(x, torch.bfloat16, "x")
    _need(w, torch.bfloat16, "weight")
    _need(out, torch.bfloat16, "out")
    if w.dim() != 2 or w.shape[0] % 2:
        raise ValueError("gemm_clamped_glu_bf16: weight must be the stacked [2N, K]")
    N, K = w.shape[0] // 2, w.shape[1]
    if x.shape[1] != K or out.shape[1] != N or x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError(f"gemm_clamped_glu_bf16: x {tuple(x.shape)}, w {tuple(w.shape)}, out {tuple(out.shape)} do not match")
    if rows < CLAMPED_GLU_MIN_ROWS or K % 8 or not limit > 0:
        raise ValueError("gemm_clamped_glu_bf16: more than 64 rows, an inner size in multiples of 8 and a positive limit")
    _check(_fn("bw_gemm_clamped_glu_bf16")(x.data_ptr(), w.data_ptr(), out.data_ptr(), rows, N, K, x.stride(0), out.stride(0),
                                           float(limit), float(alpha), _stream()), "gemm_clamped_glu_bf16")


# ------------------------------------------------------------------------------ decode fusions

_decode_ok = {}


def norm_gemm_supported(rows: int, inner: int) -> bool:
    """Whether the fused RMSNorm + product kernel (rows kept in LDS) takes this many rows of this width."""
    key = (rows, inner)
    if key not in _decode_ok:
        _decode_ok[key] = bool(_fn("bw_norm_gemm_supported")(rows, inner))
    return _decode_ok[key]


def qkv_rope_head_dim_ok(head_dim: int, inner: int) -> bool:
    """Head sizes the fused norm + q|k|v + rotation kernel takes: multiples of 32 (a workgroup
    is a pair of 16-column strips half a head apart) and 16 or 48 (a workgroup is a head); its epilogue
    reuses the LDS that held the rows, so a workgroup's 32-bit products must fit a row of ``inner`` elements."""
    if head_dim % 16 or head_dim < 16 or not (head_dim % 32 == 0 or head_dim <= 64):
        return False
    return (32 if head_dim % 32 == 0 else head_dim) * 4 <= (inner + 8) * 2


def norm_gemm_wide_supported(rows: int, tiles_of: int, columns: int, inner: int) -> bool:
    """Rows wider than a segment of K (2048): up to 8 of them, up to two segments, for products with at least 64
    workgroups of ``columns`` output columns (``tiles_of`` columns in all)."""
    key = (rows, tiles_of, columns, inner)
    if key not in _decode_ok:
        _decode_ok[key] = bool(_fn("bw_norm_gemm_wide_supported")(rows, tiles_of, inner, columns))
    return _decode_ok[key]


def can_fuse_norm(rows: int, weight: torch.Tensor, x: torch.Tensor, columns: int = 64, stacked: int = 1) -> bool:
    """Whether RMSNorm + product can run as one kernel for this step.  ``columns``: output columns a workgroup of the
    kernel for many columns (32 for SwiGLU and for heads in halves, else 64); ``stacked``: weights stacked in ``weight``
    (2 for gate|up)."""
    K = weight.shape[1]
    if not (weight.dtype == torch.bfloat16 and x.dtype == torch.float32 and x.shape[1] == K and x.stride(0) % 4 == 0):
        return False
    return norm_gemm_supported(rows, K) or norm_gemm_wide_supported(rows, weight.shape[0] // stacked, columns, K)


def norm_gemm_bf16(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w: torch.Tensor, out: torch.Tensor,
                   rows: int, epilogue: int) -> None:
    """out[:rows] = epilogue(rmsnorm(x[:rows]) @ w.T) in one kernel; the bits of rmsnorm followed
    by gemm_bf16.  epilogue as for gemm_bf16 (EPI_SWIGLU_BF16 takes the stacked weight [2N, K])."""
    _need(x, torch.float32, "x")
    _need(w, torch.bfloat16, "weight")
    N, K = w.shape
    if epilogue == EPI_SWIGLU_BF16:
        N //= 2
    _need(out, torch.bfloat16 if epilogue in (EPI_BF16, EPI_SWIGLU_BF16) else torch.float32, "out")
    glu = epilogue == EPI_SWIGLU_BF16
    if not can_fuse_norm(rows, w, x, 32 if glu else 64, 2 if glu else 1) or norm_weight.numel() != K or not norm_weight.is_cuda:
        raise ValueError(f"norm_gemm_bf16: {rows} rows of width {x.shape[1]} against weight {tuple(w.shape)} cannot be fused")
    if out.shape[1] != N or out.shape[0] < rows or x.shape[0] < rows:
        raise ValueError("norm_gemm_bf16: out does not fit")
    _check(_fn("bw_norm_gemm_bf16")(x.data_ptr(), x.stride(0), norm_weight.data_ptr(), _is_bf16(norm_weight, "norm weight"),
                                    float(eps), w.data_ptr(), out.data_ptr(), out.stride(0), rows, N, K, epilogue,
                                    _stream()), "norm_gemm_bf16")


def norm_qkv_rope_bf16(x: torch.Tensor, norm_weight: torch.Tensor, eps: float, w_qkv: torch.Tensor, q_out: torch.Tensor,
                       positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor, cos: torch.Tensor,
                       sin: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, rows: int, heads: int,
                       kv_heads: int, head_dim: int, page_size: int, write_cache: bool = True) -> None:
    """RMSNorm, the stacked q|k|v product, rotation and the cache write in one kernel (one
    workgroup per head); the bits of rmsnorm, gemm_bf16 and rope_kvwrite run one after the other."""
    _need(x, torch.float32, "x")
    _need(w_qkv, torch.bfloat16, "qkv weight")
    _need(q_out, torch.bfloat16, "q_out")
    _need(k_cache, torch.bfloat16, "k_cache")
    _need(v_cache, torch.bfloat16, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    N, K = w_qkv.shape
    if N != (heads + 2 * kv_heads) * head_dim or not qkv_rope_head_dim_ok(head_dim, K):
        raise ValueError("norm_qkv_rope_bf16: weight is not [q|k|v] heads of a supported size")
    if not can_fuse_norm(rows, w_qkv, x) or norm_weight.numel() != K:
        raise ValueError("norm_qkv_rope_bf16: this step cannot be fused")
    if q_out.shape[1] != heads * head_dim or q_out.shape[0] < rows or positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("norm_qkv_rope_bf16: buffers too small")
    if cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise ValueError("norm_qkv_rope_bf16: tables must be [positions, head_dim/2]")
    _check(_fn("bw_norm_qkv_rope_bf16")(x.data_ptr(), x.stride(0), norm_weight.data_ptr(),
                                        _is_bf16(norm_weight, "norm weight"), float(eps), w_qkv.data_ptr(),
                                        q_out.data_ptr(), positions.data_ptr(), row_seq.data_ptr(),
                                        block_table.data_ptr(), block_table.stride(0), cos.data_ptr(), sin.data_ptr(),
                                        k_cache.data_ptr(), v_cache.data_ptr(), rows, heads, kv_heads, head_dim, K,
                                        page_size, int(write_cache), _stream()), "norm_qkv_rope_bf16")


# ------------------------------------------------------------------------------ attention

def _sink_ptr(sink: Optional[torch.Tensor], heads: int) -> int:
    """``sink`` [heads] float32: a score per head that joins the softmax's denominator as exp(sink) and has no value
    (the score scale does not apply to it); None: no sink."""
    if sink is None:
        return 0
    _need(sink, torch.float32, "sink")
    if sink.numel() != heads:
        raise ValueError("attention: a sink per head is needed")
    return sink.data_ptr()


def attention_f32(q: torch.Tensor, positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor,
                  k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor, rows: int, heads: int,
                  kv_heads: int, head_dim: int, page_size: int, window: int, scale: float,
                  sink: Optional[torch.Tensor] = None, chunk: int = 0, softcap: float = 0.0) -> None:
    """q: [rows, stride] float32 with head h at columns h*head_dim.. (the stacked q|k|v rows
    serve as they are); caches [pages, kv_heads, page_size, head_dim] float32.  ``chunk`` > 0: a query sees only the keys
    of its own run of ``chunk`` positions counted from position 0 (instead of a window); ``softcap`` > 0: a score s
    becomes softcap * tanh(s / softcap) before the softmax."""
    _need(q, torch.float32, "q")
    _need(out, torch.float32, "out")
    _need(k_cache, torch.float32, "k_cache")
    _need(v_cache, torch.float32, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    if head_dim not in HEAD_DIMS:
        raise ValueError(f"attention: head size {head_dim} is not supported; supported: {HEAD_DIMS}")
    if q.shape[0] < rows or q.shape[1] < heads * head_dim or out.shape[0] < rows or out.shape[1] != heads * head_dim:
        raise ValueError("attention_f32: q or out too small")
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    _check(_fn("bw_attention_f32")(q.data_ptr(), q.stride(0), positions.data_ptr(), row_seq.data_ptr(),
                                   block_table.data_ptr(), block_table.stride(0), k_cache.data_ptr(),
                                   v_cache.data_ptr(), out.data_ptr(), out.stride(0), rows, heads, kv_heads, head_dim,
                                   page_size, int(window), float(scale), _sink_ptr(sink, heads), int(chunk), float(softcap),
                                   _stream()), "attention_f32")


def attention_f32_tiles(q: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor, tiles: torch.Tensor,
                        num_tiles: int, tiled, k_cache: torch.Tensor, v_cache: torch.Tensor, out: torch.Tensor,
                        heads: int, kv_heads: int, head_dim: int, page_size: int, window: int, scale: float,
                        sink: Optional[torch.Tensor] = None, chunk: int = 0, softcap: float = 0.0) -> None:
    """``attention_f32`` over tiles ([tiles, 4] int32 = first row, rows, request, 0; a tile's rows are consecutive
    rows of one request).  ``tiled`` True (1): a workgroup per tile of up to 16 rows, keys and values shared
    through LDS; 2: a wave per tile of up to 32 rows, both products as chains of single-step matrix instructions
    (head sizes up to 128 either way); False: a workgroup per tile's first row.  The bits are those of
    ``attention_f32``."""
    _need(q, torch.float32, "q")
    _need(out, torch.float32, "out")
    _need(k_cache, torch.float32, "k_cache")
    _need(v_cache, torch.float32, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(block_table, torch.int32, "block_table")
    _need(tiles, torch.int32, "tiles")
    if head_dim not in HEAD_DIMS or (tiled and head_dim > 128):
        raise ValueError(f"attention: head size {head_dim} is not supported here")
    if tiles.numel() < 4 * num_tiles or q.shape[1] < heads * head_dim or out.shape[1] != heads * head_dim:
        raise ValueError("attention_f32_tiles: tiles, q or out too small")
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    _check(_fn("bw_attention_f32_tiles")(q.data_ptr(), q.stride(0), positions.data_ptr(), block_table.data_ptr(),
                                         block_table.stride(0), tiles.data_ptr(), int(num_tiles), int(tiled),
                                         k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), out.stride(0), heads,
                                         kv_heads, head_dim, page_size, int(window), float(scale), _sink_ptr(sink, heads),
                                         int(chunk), float(softcap), _stream()),
           "attention_f32_tiles")


def attention_bf16(q: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor,
                   tiles: Optional[torch.Tensor], num_tiles: int, k_cache: torch.Tensor, v_cache: torch.Tensor,
                   out: torch.Tensor, heads: int, kv_heads: int, head_dim: int, page_size: int, window: int,
                   scale: float, decode: bool = False,
                   scratch: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, sink: Optional[torch.Tensor] = None,
                   chunk: int = 0, softcap: float = 0.0) -> None:
    """q, out: [rows, heads*head_dim] bfloat16; k pages [kv_heads, page, hd], v pages
    [kv_heads, hd, page]; tiles int32 [n, 4] = (first row, tokens, sequence, 0).

    k_cache and v_cache are [pages, kv_heads*page_size*head_dim]: page numbers from the table
    are clamped into the pool, so a stale table entry can cost nothing worse than a wasted load.

    ``decode`` False: a workgroup folds all partitions for ``fold_group_tiles(head_dim)`` tiles;
    the tiles of a sequence must come in runs padded to that number (empty tiles allowed).
    ``decode`` True (tiles of one token each; ``tiles`` None means "tile t is row t of sequence
    t"): a workgroup per tile whose waves take one 64-key partition each and fold through LDS
    in partition order.  The bits are the same either way.

    ``scratch`` (decode only): the tensors ``attention_decode_scratch`` asks for, (float32, int32
    zeros).  With them a launch of few tiles is split over several workgroups per tile; without
    them it is not.  The bits are the same again."""
    _need(q, torch.bfloat16, "q")
    _need(out, torch.bfloat16, "out")
    _need(k_cache, torch.bfloat16, "k_cache")
    _need(v_cache, torch.bfloat16, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(block_table, torch.int32, "block_table")
    if tiles is not None:
        _need(tiles, torch.int32, "tiles")
    elif not decode:
        raise ValueError("attention_bf16: implicit tiles are for decoded tokens only")
    if head_dim not in HEAD_DIMS:
        raise ValueError(f"attention: head size {head_dim} is not supported; supported: {HEAD_DIMS}")
    if heads % kv_heads:
        raise ValueError("attention: heads must be a multiple of kv_heads")
    if q.shape[1] != heads * head_dim or out.shape[1] != heads * head_dim or (
            tiles is not None and tiles.numel() < 4 * num_tiles):
        raise ValueError("attention_bf16: q, out or tiles do not fit")
    if tiles is None and (positions.numel() < num_tiles or block_table.shape[0] < num_tiles):
        raise ValueError("attention_bf16: fewer rows or block tables than implicit tiles")
    page_elems = kv_heads * page_size * head_dim
    if k_cache.dim() != 2 or k_cache.shape[1] != page_elems or v_cache.shape != k_cache.shape:
        raise ValueError(f"attention_bf16: caches must be [pages, {page_elems}]")
    sc_f = sc_c = None
    if scratch is not None and decode:
        sc_f, sc_c = scratch
        _need(sc_f, torch.float32, "scratch")
        _need(sc_c, torch.int32, "scratch counters")
    _check(_fn("bw_attention_bf16")(q.data_ptr(), q.stride(0), positions.data_ptr(), block_table.data_ptr(),
                                    block_table.stride(0), tiles.data_ptr() if tiles is not None else 0, num_tiles,
                                    k_cache.data_ptr(), v_cache.data_ptr(), k_cache.shape[0], out.data_ptr(),
                                    out.stride(0), heads, kv_heads, head_dim, page_size, int(window), float(scale), int(decode),
                                    sc_f.data_ptr() if sc_f is not None else 0, sc_f.numel() if sc_f is not None else 0,
                                    sc_c.data_ptr() if sc_c is not None else 0, sc_c.numel() if sc_c is not None else 0,
                                    _sink_ptr(sink, heads), int(chunk), float(softcap), _stream()),
           "attention_bf16")


def attention_decode_scratch(num_tiles: int, heads: int, kv_heads: int, head_dim: int, table_stride: int,
                             page_size: int) -> Tuple[int, int]:
    """(float32 elements, int32 counters) that a decode launch of ``num_tiles`` tiles wants as
    ``scratch`` to split its tiles over workgroups; (0, 0): it would not split."""
    floats, counters = ctypes.c_longlong(0), ctypes.c_int(0)
    _check(_fn("bw_attention_decode_scratch")(num_tiles, heads, kv_heads, head_dim, table_stride, page_size,
                                              ctypes.addressof(floats), ctypes.addressof(counters)),
           "attention_decode_scratch")
    return int(floats.value), int(counters.value)


def qkv_rope_gemm_ok(rows: int, head_dim: int, inner: int, all_heads: int = 0) -> bool:
    """Whether the q|k|v product of normalised rows can take rotation and cache write into its
    epilogue.  Up to 64 rows (a workgroup per 32 or 16 rotary pairs of a head), or a few blocks of 64 rows whose
    workgroups are 512 at most: head sizes in multiples of 64, K in steps of 64, and enough heads (q, k and v
    heads together) for 64 workgroups.  More rows: heads of 64 and one segment of K."""
    tiles = all_heads * (head_dim // 64)
    small = head_dim % 64 == 0 and inner % 64 == 0 and tiles >= 64
    if rows > 64:
        # (a few blocks of 64 rows at once, while their workgroups fit the chip together: any head size the small kernel takes)
        at_once = small and tiles * ((rows + 63) // 64) <= 512
        return at_once or (head_dim == 64 and inner <= 2048 and inner % 8 == 0)
    return small


def gemm_qkv_rope_bf16(x: torch.Tensor, w_qkv: torch.Tensor, q_out: torch.Tensor, positions: torch.Tensor,
                       row_seq: torch.Tensor, block_table: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor,
                       k_cache: torch.Tensor, v_cache: torch.Tensor, rows: int, heads: int, kv_heads: int,
                       head_dim: int, page_size: int, write_cache: bool = True) -> None:
    """The stacked q|k|v product with rotation and cache write in its epilogue (the shapes of
    ``qkv_rope_gemm_ok``); the bits of gemm_bf16 into a 32-bit buffer followed by rope_kvwrite."""
    _need(x, torch.bfloat16, "x")
    _need(w_qkv, torch.bfloat16, "qkv weight")
    _need(q_out, torch.bfloat16, "q_out")
    _need(k_cache, torch.bfloat16, "k_cache")
    _need(v_cache, torch.bfloat16, "v_cache")
    _need(positions, torch.int32, "positions")
    _need(row_seq, torch.int32, "row_seq")
    _need(block_table, torch.int32, "block_table")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    N, K = w_qkv.shape
    if N != (heads + 2 * kv_heads) * head_dim or not qkv_rope_gemm_ok(rows, head_dim, K, heads + 2 * kv_heads):
        raise ValueError("gemm_qkv_rope_bf16: not a [q|k|v] weight, or a shape the rotary epilogue does not take")
    if x.shape[1] != K or x.shape[0] < rows or q_out.shape[1] != heads * head_dim or q_out.shape[0] < rows:
        raise ValueError("gemm_qkv_rope_bf16: buffers do not fit")
    if positions.numel() < rows or row_seq.numel() < rows or cos.shape[1] != head_dim // 2 or sin.shape != cos.shape:
        raise ValueError("gemm_qkv_rope_bf16: positions or rotary tables do not fit")
    _check(_fn("bw_gemm_qkv_rope_bf16")(x.data_ptr(), x.stride(0), w_qkv.data_ptr(), q_out.data_ptr(),
                                        positions.data_ptr(), row_seq.data_ptr(), block_table.data_ptr(),
                                        block_table.stride(0), cos.data_ptr(), sin.data_ptr(), k_cache.data_ptr(),
                                        v_cache.data_ptr(), rows, heads, kv_heads, head_dim, K, page_size,
                                        int(write_cache), _stream()), "gemm_qkv_rope_bf16")


# ------------------------------------------------------------------------------ mixers with a state per request

RECUR_DECAY_PER_CHANNEL, RECUR_SCALAR_GATES, RECUR_BONUS_DECAY, RECUR_FIXED_DECAY = 0, 1, 2, 3
RECUR_MAX_DIM = 256          # key channels of a head that the recurrence keeps in a lane's registers
GATE_SIGMOID, GATE_SILU = 0, 1
ACT_SILU, ACT_GELU_TANH, ACT_CLAMPED_SWISH = 0, 1, 2


def _act_out(t: torch.Tensor, what: str) -> int:
    if not t.is_cuda or not t.is_contiguous():
        raise ValueError(f"{what} must be a contiguous GPU tensor")
    return _is_bf16(t, what)


def norm_shift(x: torch.Tensor, weight: torch.Tensor, mix: torch.Tensor, state: torch.Tensor, positions: torch.Tensor,
               row_seq: torch.Tensor, seq_rows: torch.Tensor, slots: torch.Tensor, out: torch.Tensor, rows: int,
               eps: float) -> None:
    """out[r] = h[r] + (h_prev[r] - h[r]) * mix with h = rmsnorm(x) * weight and h_prev the h of the request's token
    before (from ``state`` [slots, width] for a request's first row of the step, which then receives the h of
    the request's last row).  ``mix`` [width], or [n, width] for n shifted copies side by side in ``out`` [rows, n*width].
    All 32-bit; ``out`` in float32 or bfloat16."""
    _need(x, torch.float32, "x")
    _need(weight, torch.float32, "norm weight")
    _need(mix, torch.float32, "mix")
    _need(state, torch.float32, "state")
    for t, what in ((positions, "positions"), (row_seq, "row_seq"), (seq_rows, "seq_rows"), (slots, "slots")):
        _need(t, torch.int32, what)
    dim = x.shape[1]
    nmix = mix.numel() // max(dim, 1)
    if weight.numel() != dim or nmix < 1 or mix.numel() != nmix * dim or state.dim() != 2 or state.shape[1] < dim:
        raise ValueError("norm_shift: weight, mix or state do not fit the rows' width")
    if x.shape[0] < rows or out.shape[0] < rows or out.shape[1] != nmix * dim or positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("norm_shift: buffers shorter than the rows")
    _check(_fn("bw_norm_shift")(x.data_ptr(), x.stride(0), weight.data_ptr(), mix.data_ptr(), state.data_ptr(), state.stride(0),
                                positions.data_ptr(), row_seq.data_ptr(), seq_rows.data_ptr(), slots.data_ptr(),
                                out.data_ptr(), _act_out(out, "out"), out.stride(0), rows, dim, float(eps), nmix, _stream()),
           "norm_shift")


def linear_recurrence(mode: int, proj: torch.Tensor, q_off: int, k_off: int, v_off: int, gate: Optional[torch.Tensor], gate_off: int,
                      gate2_off: int, bias: torch.Tensor, bias2: Optional[torch.Tensor], param: float, qscale: float,
                      state: torch.Tensor, out: torch.Tensor, seq_rows: torch.Tensor, slots: torch.Tensor,
                      positions: torch.Tensor, nseq: int, heads: int, dim: int, vdim: int, scan=None, kscale: float = 1.0) -> None:
    """The recurrence S <- decay * S + k v^T, o = S^T (q * qscale) per head over every request's rows in order, from and
    to ``state`` [slots, elements].  RECUR_DECAY_PER_CHANNEL: decay = exp(logsigmoid(gate + bias) * param) per key
    channel (``gate`` [rows, >= gate_off + heads*dim]).  RECUR_SCALAR_GATES: capped input and forget gates per head
    (columns gate_off + h and gate2_off + h of ``gate``), a normaliser and a running maximum in the state; param = cap.
    RECUR_BONUS_DECAY: decay = exp(-exp(gate + bias)) per key channel, and the read-out comes before the update:
    o = (S + diag(bias2) k v^T)^T q with the S the token before left (``bias2`` [heads*dim]: the weight of the token's own
    k v^T), then S <- decay * S + k v^T.  RECUR_FIXED_DECAY: one constant decay a head (``bias`` [heads]; ``gate`` None).
    k is multiplied by ``kscale``.  ``state`` may be a column slice of a wider tensor.

    ``scan`` = (chunks [n, 4] int32 = (first row, rows, request, 1 if the request's last chunk), n, spans [k, 3] int32 =
    (request, its first chunk, its chunks), k, local, start): long portions run in three passes over their chunks (each
    chunk from zero, a walk over a request's chunks that gives each its starting state, each chunk from there), with
    ``local`` and ``start`` float32 of n * heads * (dim*vdim + dim + 2) elements each; ``seq_rows`` then carries no rows
    for those requests (nseq may be 0).  The result differs from the one-pass order by the rounding of the walk's sums."""
    _need_strided(proj, torch.float32, "proj")            # (may be a column slice of a wider product)
    if mode != RECUR_FIXED_DECAY:
        _need(gate, torch.float32, "gate")
    _need(bias, torch.float32, "bias")
    _need_strided(state, torch.float32, "state")
    _need(out, torch.float32, "out")
    for t, what in ((positions, "positions"), (seq_rows, "seq_rows"), (slots, "slots")):
        _need(t, torch.int32, what)
    if dim > RECUR_MAX_DIM:
        raise ValueError(f"linear_recurrence: {dim} key channels a head; the kernel keeps up to {RECUR_MAX_DIM}")
    if mode == RECUR_SCALAR_GATES:
        if bias2 is None:
            raise ValueError("linear_recurrence: scalar gates need both biases")
        _need(bias2, torch.float32, "bias2")
        if bias.numel() != heads or bias2.numel() != heads or max(gate_off, gate2_off) + heads > gate.shape[1]:
            raise ValueError("linear_recurrence: gates or biases do not fit the heads")
        need = heads * (dim * vdim + dim + 1)
    elif mode == RECUR_FIXED_DECAY:
        if bias.numel() != heads:
            raise ValueError("linear_recurrence: a constant decay a head is needed")
        need = heads * dim * vdim
    else:
        if mode == RECUR_BONUS_DECAY:
            if bias2 is None:
                raise ValueError("linear_recurrence: the read-out before the update needs the weights of the token's own k v^T")
            _need(bias2, torch.float32, "bias2")
            if bias2.numel() != heads * dim:
                raise ValueError("linear_recurrence: the weights of the token's own k v^T do not fit heads x dim")
        if bias.numel() != heads * dim or gate_off + heads * dim > gate.shape[1]:
            raise ValueError("linear_recurrence: decay logits or bias do not fit heads x dim")
        need = heads * dim * vdim
    if state.dim() != 2 or state.shape[1] < need:
        raise ValueError(f"linear_recurrence: a state slot needs {need} elements")
    if max(q_off, k_off) + heads * dim > proj.shape[1] or v_off + heads * vdim > proj.shape[1] or out.shape[1] != heads * vdim:
        raise ValueError("linear_recurrence: projections or out do not fit")
    if seq_rows.numel() < 2 * nseq or slots.numel() < nseq:
        raise ValueError("linear_recurrence: fewer request records than requests")
    chunks = spans = local = start = None
    nchunks = nspans = 0
    if scan is not None:
        chunks, nchunks, spans, nspans, local, start = scan
        _need(chunks, torch.int32, "chunks")
        _need(spans, torch.int32, "spans")
        _need(local, torch.float32, "scan records")
        _need(start, torch.float32, "scan records")
        if chunks.numel() < 4 * nchunks or spans.numel() < 3 * nspans or start.numel() < local.numel():
            raise ValueError("linear_recurrence: the scan's tables or records do not fit")
    _check(_fn("bw_linear_recurrence")(int(mode), proj.data_ptr(), proj.stride(0), q_off, k_off, v_off,
                                       0 if gate is None else gate.data_ptr(), 0 if gate is None else gate.stride(0),
                                       gate_off, gate2_off, bias.data_ptr(),
                                       0 if bias2 is None else bias2.data_ptr(), float(param), float(qscale), float(kscale), state.data_ptr(),
                                       state.stride(0), out.data_ptr(), out.stride(0), seq_rows.data_ptr(), slots.data_ptr(),
                                       positions.data_ptr(), nseq, heads, dim, vdim,
                                       0 if chunks is None else chunks.data_ptr(), nchunks,
                                       0 if spans is None else spans.data_ptr(), nspans,
                                       0 if local is None else local.data_ptr(), 0 if start is None else start.data_ptr(),
                                       0 if local is None else local.numel(), _stream()), "linear_recurrence")


def rotate_halves_rows(x: torch.Tensor, offsets: Sequence[int], heads: int, dim: int, rot: int, cos: torch.Tensor,
                       sin: torch.Tensor, positions: torch.Tensor, rows: int) -> None:
    """One or two sections of ``x`` (float32 [rows, >= off + heads*dim], a section at each of ``offsets``) turned in place
    by the rows' positions: of every head's first ``rot`` elements, element i is paired with element i + rot/2; the
    tables are [positions, rot/2].  ``x`` may be a column slice of a wider matrix."""
    _need_strided(x, torch.float32, "x")
    _need(positions, torch.int32, "positions")
    if rot == 0 or rows <= 0:
        return
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    offs = [int(o) for o in offsets]
    if not 1 <= len(offs) <= 2 or rot % 2 or rot > dim or cos.shape[1] != rot // 2 or sin.shape != cos.shape:
        raise ValueError("rotate_halves_rows: one or two sections, tables [positions, rot/2], rot even and at most dim")
    if x.shape[0] < rows or positions.numel() < rows or any(o < 0 or o + heads * dim > x.shape[1] for o in offs):
        raise ValueError("rotate_halves_rows: the sections do not fit the rows")
    _check(_fn("bw_rotate_halves_rows")(x.data_ptr(), x.stride(0), rows, heads, dim, rot, len(offs), offs[0], offs[-1], cos.data_ptr(),
                                        sin.data_ptr(), positions.data_ptr(), _stream()), "rotate_halves_rows")


def tanh_rows(x: torch.Tensor, rows: int) -> None:
    """x[:rows] = tanh(x[:rows]) in place; ``x`` float32, a column slice will do."""
    _need_strided(x, torch.float32, "x")
    if x.shape[0] < rows:
        raise ValueError("tanh_rows: fewer rows than asked for")
    _check(_fn("bw_tanh_rows")(x.data_ptr(), x.stride(0), rows, x.shape[1], _stream()), "tanh_rows")


def norm_mean(ys: Sequence[torch.Tensor], weights: Sequence[torch.Tensor], out: torch.Tensor, rows: int, eps: float) -> None:
    """out[r] = mean over b of ys[b][r] / sqrt(mean(ys[b][r]^2) + eps) * weights[b], all 32-bit: up to four matrices of one
    width, each normed row by row with a weight vector of its own."""
    n = len(ys)
    _need(out, torch.float32, "out")
    dim = out.shape[1]
    if not 1 <= n <= 4 or len(weights) != n or out.shape[0] < rows:
        raise ValueError("norm_mean: one to four inputs, a weight vector each")
    for y, w in zip(ys, weights):
        _need_strided(y, torch.float32, "input")
        _need(w, torch.float32, "weight")
        if y.shape[1] != dim or y.shape[0] < rows or w.numel() != dim:
            raise ValueError("norm_mean: inputs and weights must have out's width")
    yp = (c_void_p * n)(*[y.data_ptr() for y in ys])
    wp = (c_void_p * n)(*[w.data_ptr() for w in weights])
    ld = (c_int * n)(*[y.stride(0) for y in ys])
    _check(_fn("bw_norm_mean")(ctypes.cast(yp, c_void_p), ctypes.cast(ld, c_void_p), ctypes.cast(wp, c_void_p), n, out.data_ptr(),
                               out.stride(0), rows, dim, float(eps), _stream()), "norm_mean")


NORM_MEAN_ADD_MAX_WIDTH = 2048     # rows that the fused mean + norm + add keeps in a workgroup's registers


def norm_mean_add(ys: Sequence[torch.Tensor], weights: Sequence[torch.Tensor], eps: float, post_weight: torch.Tensor, post_eps: float,
                  scale: float, x: torch.Tensor, rows: int) -> None:
    """x[:rows] += scale * (z / sqrt(mean(z^2) + post_eps) * post_weight) with z the mean of ``norm_mean``: one launch, the
    bits of ``norm_mean`` followed by ``norm_add``.  Rows of up to NORM_MEAN_ADD_MAX_WIDTH elements."""
    n = len(ys)
    _need(x, torch.float32, "x")
    _need(post_weight, torch.float32, "post weight")
    dim = x.shape[1]
    if not 1 <= n <= 4 or len(weights) != n or x.shape[0] < rows or dim > NORM_MEAN_ADD_MAX_WIDTH or post_weight.numel() != dim:
        raise ValueError("norm_mean_add: one to four inputs, a weight vector each, rows of up to 2,048 elements")
    for y, w in zip(ys, weights):
        _need_strided(y, torch.float32, "input")
        _need(w, torch.float32, "weight")
        if y.shape[1] != dim or y.shape[0] < rows or w.numel() != dim:
            raise ValueError("norm_mean_add: inputs and weights must have x's width")
    yp = (c_void_p * n)(*[y.data_ptr() for y in ys])
    wp = (c_void_p * n)(*[w.data_ptr() for w in weights])
    ld = (c_int * n)(*[y.stride(0) for y in ys])
    _check(_fn("bw_norm_mean_add")(ctypes.cast(yp, c_void_p), ctypes.cast(ld, c_void_p), ctypes.cast(wp, c_void_p), n, float(eps),
                                   post_weight.data_ptr(), float(post_eps), float(scale), x.data_ptr(), x.stride(0), rows, dim,
                                   _stream()), "norm_mean_add")


def head_norm_gate(o: torch.Tensor, weight: torch.Tensor, per_head_weight: bool, g: torch.Tensor, g_off: int, gate: int,
                   out: torch.Tensor, positions: torch.Tensor, rows: int, heads: int, vdim: int, eps: float) -> None:
    """out[r, h] = o[r, h] / rms(o[r, h]) * weight * gate(g[r, g_off + h*vdim ..]); weight [heads*vdim] or [vdim]."""
    _need(o, torch.float32, "o")
    _need(weight, torch.float32, "weight")
    _need_strided(g, torch.float32, "g")
    _need(positions, torch.int32, "positions")
    if weight.numel() != (heads * vdim if per_head_weight else vdim) or o.shape[1] != heads * vdim or out.shape[1] != heads * vdim:
        raise ValueError("head_norm_gate: weight, o or out do not fit heads x vdim")
    if g_off + heads * vdim > g.shape[1] or min(o.shape[0], out.shape[0], g.shape[0], positions.numel()) < rows:
        raise ValueError("head_norm_gate: buffers too small")
    gp = g.data_ptr() + 4 * g_off
    _check(_fn("bw_head_norm_gate")(o.data_ptr(), o.stride(0), weight.data_ptr(), vdim if per_head_weight else 0, gp, g.stride(0),
                                    int(gate), out.data_ptr(), _act_out(out, "out"), out.stride(0), positions.data_ptr(), rows,
                                    heads, vdim, float(eps), _stream()), "head_norm_gate")


def glu(gate_up: torch.Tensor, out: torch.Tensor, rows: int, act: int, limit: float = 0.0, alpha: float = 1.0,
        row_gate: Optional[torch.Tensor] = None) -> None:
    """out = act(gate) * up of the stacked 32-bit product [rows, >= 2*inter] (gate at column 0, up at column inter); out
    float32 or bfloat16 (one rounding).  ACT_CLAMPED_SWISH: g = min(gate, limit), u = clamp(up, -limit, limit),
    out = g sigmoid(alpha g) (u + 1).  ``row_gate`` (a 32-bit column, one number a row): out's row r is multiplied by
    sigmoid(row_gate[r]).  ``gate_up`` may be a column slice of a wider matrix."""
    _need_strided(gate_up, torch.float32, "gate_up")
    inter = out.shape[1]
    if gate_up.shape[1] < 2 * inter or gate_up.shape[0] < rows or out.shape[0] < rows:
        raise ValueError("glu: gate_up must be [rows, 2*inter] for out [rows, inter]")
    rg, ldrg = 0, 0
    if row_gate is not None:
        _need_strided(row_gate, torch.float32, "row_gate")
        if row_gate.dim() != 2 or row_gate.shape[1] != 1 or row_gate.shape[0] < rows:
            raise ValueError("glu: row_gate must be a column [rows, 1]")
        rg, ldrg = row_gate.data_ptr(), row_gate.stride(0)
    _check(_fn("bw_glu")(gate_up.data_ptr(), gate_up.stride(0), out.data_ptr(), _act_out(out, "out"), rows, inter, int(act),
                         float(limit), float(alpha), rg, ldrg, _stream()), "glu")


# ------------------------------------------------------------------------------ attention over a compressed cache

def latent_prep(proj: torch.Tensor, q_off: int, dkv_off: int, norm_w: torch.Tensor, eps: float, cos: torch.Tensor,
                sin: torch.Tensor, positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor,
                cache: torch.Tensor, qa: torch.Tensor, rows: int, heads: int, dim: int, rot: int, rotary: int, rank: int,
                page_size: int, write_cache: bool = True, latent_t: Optional[torch.Tensor] = None) -> None:
    """From the stacked projections: the latent (RMS-normed) and the rotated shared key part into the row's page slot
    ([pages, page_size * (rank + rot)]), and every head's rotated query part into ``qa`` [rows, heads * (rank + rot)]
    behind the place of its latent-space part.  ``latent_t`` [pages, rank * page_size]: the latent once more, transposed
    within its page ([element][slot]), for the matrix-core attention."""
    _need(proj, torch.float32, "proj")
    _need(norm_w, torch.float32, "norm weight")
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    for t, what in ((positions, "positions"), (row_seq, "row_seq"), (block_table, "block_table")):
        _need(t, torch.int32, what)
    width = rank + rot
    if q_off + heads * (dim + rot) > proj.shape[1] or dkv_off + width > proj.shape[1] or norm_w.numel() != rank:
        raise ValueError("latent_prep: projections or norm weight do not fit")
    if rotary % 2 or rotary > rot or (rotary and (cos.shape[1] != rotary // 2 or sin.shape != cos.shape)):
        raise ValueError("latent_prep: rotary tables must be [positions, rotary/2]")
    if cache.dim() != 2 or cache.shape[1] != page_size * width or qa.shape[1] != heads * width:
        raise ValueError("latent_prep: cache pages or qa do not fit")
    if min(proj.shape[0], qa.shape[0], positions.numel(), row_seq.numel()) < rows:
        raise ValueError("latent_prep: buffers shorter than the rows")
    if latent_t is not None and (latent_t.dtype != cache.dtype or latent_t.dim() != 2 or latent_t.shape != (cache.shape[0], page_size * rank)
                                 or not latent_t.is_contiguous()):
        raise ValueError("latent_prep: the transposed latents must be [pages, rank * page_size] of the cache's dtype")
    _check(_fn("bw_latent_prep")(proj.data_ptr(), proj.stride(0), q_off, dkv_off, norm_w.data_ptr(), float(eps), cos.data_ptr(),
                                 sin.data_ptr(), positions.data_ptr(), row_seq.data_ptr(), block_table.data_ptr(),
                                 block_table.stride(0), cache.data_ptr(), 0 if latent_t is None else latent_t.data_ptr(),
                                 _act_out(cache, "cache"), qa.data_ptr(), _act_out(qa, "qa"), qa.stride(0),
                                 rows, heads, dim, rot, rotary, rank, page_size, int(write_cache), _stream()), "latent_prep")


def headwise_linear(x: torch.Tensor, x_off: int, x_head_stride: int, wt: torch.Tensor, out: torch.Tensor, out_off: int,
                    out_head_stride: int, rows: int) -> None:
    """out[r, out_off + h*out_head_stride + o] = sum_i wt[h, i, o] * x[r, x_off + h*x_head_stride + i]: a product per head,
    weights input-major [heads, in, out] (bfloat16 or float32), 32-bit sums."""
    _need(x, torch.float32, "x")
    if wt.dim() != 3 or not wt.is_cuda or not wt.is_contiguous():
        raise ValueError("headwise_linear: weights must be a contiguous [heads, in, out] GPU tensor")
    heads, inn, outn = wt.shape
    if x_off + (heads - 1) * x_head_stride + inn > x.shape[1] or out_off + (heads - 1) * out_head_stride + outn > out.shape[1]:
        raise ValueError("headwise_linear: x or out narrower than the heads need")
    if x.shape[0] < rows or out.shape[0] < rows:
        raise ValueError("headwise_linear: buffers shorter than the rows")
    ob = _act_out(out, "out")
    _check(_fn("bw_headwise_linear")(x.data_ptr() + 4 * x_off, x.stride(0), x_head_stride, wt.data_ptr(), _is_bf16(wt, "weights"),
                                     inn, outn, out.data_ptr() + (2 if ob else 4) * out_off, ob, out.stride(0), out_head_stride,
                                     rows, heads, _stream()), "headwise_linear")


def shared_key_attention(q: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor, tiles: Optional[torch.Tensor],
                         num_tiles: int, cache: torch.Tensor, sink: Optional[torch.Tensor], out: torch.Tensor, heads: int,
                         dk: int, dv: int, page_size: int, window: int, scale: float, heads_per_group: int) -> None:
    """Causal softmax attention of ``heads`` query heads over keys that all heads share: q [rows, heads*dk], cache
    [pages, page_size*dk] (a token's value is the first dv elements of its key vector), out [rows, heads*dv] (32-bit).
    ``sink`` [heads]: a score per head that joins the softmax's denominator and has no value.  tiles [n, 4] = (first
    row, rows, request, 0) with up to 16 / heads_per_group rows each; None: tile t is row t of request t."""
    _need(q, torch.float32, "q")
    _need(out, torch.float32, "out")
    _need(positions, torch.int32, "positions")
    _need(block_table, torch.int32, "block_table")
    if tiles is not None:
        _need(tiles, torch.int32, "tiles")
        if tiles.numel() < 4 * num_tiles:
            raise ValueError("shared_key_attention: fewer tiles than said")
    elif positions.numel() < num_tiles or block_table.shape[0] < num_tiles:
        raise ValueError("shared_key_attention: fewer rows or block tables than implicit tiles")
    if sink is not None:
        _need(sink, torch.float32, "sink")
        if sink.numel() != heads:
            raise ValueError("shared_key_attention: a sink per head is needed")
    if q.shape[1] != heads * dk or out.shape[1] != heads * dv or dv > dk or dv > 512:
        raise ValueError("shared_key_attention: q or out do not fit (values of up to 512 elements)")
    if cache.dim() != 2 or cache.shape[1] != page_size * dk:
        raise ValueError(f"shared_key_attention: cache must be [pages, {page_size * dk}]")
    _check(_fn("bw_shared_key_attention")(q.data_ptr(), q.stride(0), positions.data_ptr(), block_table.data_ptr(),
                                          block_table.stride(0), 0 if tiles is None else tiles.data_ptr(), num_tiles,
                                          cache.data_ptr(), _act_out(cache, "cache"), cache.shape[0],
                                          0 if sink is None else sink.data_ptr(), out.data_ptr(), out.stride(0), heads, dk, dv,
                                          page_size, int(window), float(scale), int(heads_per_group), _stream()),
           "shared_key_attention")


def shared_key_mfma_ok(cache_dtype: torch.dtype, dk: int, dv: int, page_size: int) -> bool:
    """Whether the matrix-core route of the attention over shared keys takes this cache."""
    return cache_dtype == torch.bfloat16 and dk % 8 == 0 and 0 < dv <= min(dk, 512) and page_size >= 4 and page_size % 4 == 0


def shared_key_attention_mfma(q: torch.Tensor, positions: torch.Tensor, block_table: torch.Tensor, tiles: Optional[torch.Tensor],
                              num_tiles: int, cache: torch.Tensor, latent_t: torch.Tensor, sink: Optional[torch.Tensor],
                              out: torch.Tensor, heads: int, dk: int, dv: int, page_size: int, window: int, scale: float,
                              heads_per_group: int, nsplit: int = 1, kchunk: int = 0,
                              partial: Optional[torch.Tensor] = None) -> None:
    """``shared_key_attention`` on the matrix cores for a bfloat16 cache (``shared_key_mfma_ok``): queries and softmax
    weights are rounded to bfloat16 where they enter a product (``q`` arrives as bfloat16), sums are 32-bit.  ``latent_t`` [pages, dv * page_size]: the
    values transposed within their pages.  Tiles hold up to 16 / heads_per_group rows.  nsplit > 1 (tiles of one row,
    heads_per_group 16): wave s of a tile takes keys [s * kchunk, (s+1) * kchunk) and ``partial`` (float32, at least
    tiles * heads * nsplit * (dv + 2)) holds the pieces that a second kernel joins."""
    _need(q, torch.bfloat16, "q")
    _need(out, torch.float32, "out")
    _need(positions, torch.int32, "positions")
    _need(block_table, torch.int32, "block_table")
    _need(cache, torch.bfloat16, "cache")
    _need(latent_t, torch.bfloat16, "latent_t")
    if not shared_key_mfma_ok(cache.dtype, dk, dv, page_size):
        raise ValueError("shared_key_attention_mfma: this cache is not for the matrix-core route")
    if tiles is not None:
        _need(tiles, torch.int32, "tiles")
        if tiles.numel() < 4 * num_tiles:
            raise ValueError("shared_key_attention_mfma: fewer tiles than said")
    elif positions.numel() < num_tiles or block_table.shape[0] < num_tiles:
        raise ValueError("shared_key_attention_mfma: fewer rows or block tables than implicit tiles")
    if sink is not None:
        _need(sink, torch.float32, "sink")
        if sink.numel() != heads:
            raise ValueError("shared_key_attention_mfma: a sink per head is needed")
    if q.shape[1] != heads * dk or out.shape[1] != heads * dv:
        raise ValueError("shared_key_attention_mfma: q or out do not fit")
    if cache.dim() != 2 or cache.shape[1] != page_size * dk or latent_t.shape != (cache.shape[0], page_size * dv):
        raise ValueError("shared_key_attention_mfma: cache or transposed values do not fit")
    if nsplit > 1:
        if partial is None:
            raise ValueError("shared_key_attention_mfma: splits need room for their pieces")
        _need(partial, torch.float32, "partial")
    _check(_fn("bw_shared_key_attention_mfma")(q.data_ptr(), q.stride(0), positions.data_ptr(), block_table.data_ptr(),
                                               block_table.stride(0), 0 if tiles is None else tiles.data_ptr(), num_tiles,
                                               cache.data_ptr(), latent_t.data_ptr(), cache.shape[0],
                                               0 if sink is None else sink.data_ptr(), out.data_ptr(), out.stride(0), heads,
                                               dk, dv, page_size, int(window), float(scale), int(heads_per_group), int(nsplit),
                                               int(kchunk), 0 if partial is None else partial.data_ptr(),
                                               0 if partial is None else partial.numel(), _stream()),
           "shared_key_attention_mfma")


# ------------------------------------------------------------------------------ convolved, gated and recurrent mixers

CONV_MAX_TAPS = 8


def causal_conv(x: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], state: Optional[torch.Tensor],
                seq_rows: torch.Tensor, slots: torch.Tensor, positions: torch.Tensor, nseq: int, max_seq_rows: int,
                out: torch.Tensor, in_bias: Optional[torch.Tensor] = None) -> None:
    """out[t, c] = sum_j weight[c, j] * x[t - taps + 1 + j, c] (+ bias[c]) along every request's rows, the inputs before a
    portion's first row taken from ``state`` [slots, >= (taps - 1) * channels] (a view may start inside a wider slot),
    which then receives the portion's last taps - 1 inputs.  ``x`` [rows, >= channels] float32 (rows apart by its
    stride), ``out`` likewise.  ``max_seq_rows``: the most rows a request brings in this step.  ``in_bias`` [channels]
    float32: added to every input on its way in (a projection's bias; the state then keeps inputs with it)."""
    if x.dtype != torch.float32 or out.dtype != torch.float32 or x.stride(1) != 1 or out.stride(1) != 1 or not (x.is_cuda and out.is_cuda):
        raise ValueError("causal_conv: x and out must be float32 GPU matrices with contiguous rows")
    if weight.dim() != 2 or not weight.is_cuda or not weight.is_contiguous():
        raise ValueError("causal_conv: weight must be a contiguous [channels, taps] GPU tensor")
    channels, taps = weight.shape
    wb = _is_bf16(weight, "weight")
    if taps < 1 or taps > CONV_MAX_TAPS:
        raise ValueError(f"causal_conv: {taps} taps; the kernel takes 1 to {CONV_MAX_TAPS}")
    if x.shape[1] < channels or out.shape[1] < channels:
        raise ValueError("causal_conv: x or out narrower than the channels")
    if bias is not None and (bias.dtype != weight.dtype or bias.numel() != channels or not bias.is_contiguous()):
        raise ValueError("causal_conv: bias must be [channels] of the weight's dtype")
    for t, what in ((seq_rows, "seq_rows"), (slots, "slots"), (positions, "positions")):
        _need(t, torch.int32, what)
    if seq_rows.numel() < 2 * nseq or slots.numel() < nseq:
        raise ValueError("causal_conv: fewer request records than requests")
    sp, sld = 0, 0
    if taps > 1:
        if state is None or state.dtype != torch.float32 or state.dim() != 2 or state.stride(1) != 1 or state.shape[1] < (taps - 1) * channels:
            raise ValueError(f"causal_conv: a state slot needs {(taps - 1) * channels} float32 elements")
        sp, sld = state.data_ptr(), state.stride(0)
    if in_bias is not None:
        _need(in_bias, torch.float32, "in_bias")
        if in_bias.numel() != channels:
            raise ValueError("causal_conv: in_bias must be [channels]")
    _check(_fn("bw_causal_conv")(x.data_ptr(), x.stride(0), 0 if in_bias is None else in_bias.data_ptr(), weight.data_ptr(), 0 if bias is None else bias.data_ptr(), wb, taps,
                                 channels, sp, sld, seq_rows.data_ptr(), slots.data_ptr(), positions.data_ptr(), int(nseq),
                                 int(max_seq_rows), out.data_ptr(), out.stride(0), _stream()), "causal_conv")


def pair_rope_unit(src: torch.Tensor, positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor,
                   cos: torch.Tensor, sin: torch.Tensor, q_out: torch.Tensor, k_cache: Optional[torch.Tensor],
                   v_cache: Optional[torch.Tensor], rows: int, heads: int, kv_heads: int, dim: int, vdim: int, head_size: int,
                   rot: int, page_size: int, unit_norm: bool, eps: float, has_kv: bool, write_cache: bool,
                   halves: bool = False, values_are_keys: bool = False) -> None:
    """``src`` [rows, >= heads*dim (+ kv_heads*(dim+vdim))] float32: query heads, then key heads, then value heads (with
    ``values_are_keys`` no value heads: a value head is its key head as projected, before rotation).  The
    first ``rot`` elements of every query and key head are rotated pair by pair ((2i, 2i+1), or with ``halves``
    (i, i + rot/2), by the angle of table
    column i at the row's position), the head is then divided by its root mean square if ``unit_norm``; queries go to
    ``q_out`` [rows, heads*head_size], keys and values (as they are) into the row's page slot, all padded with zeros
    to ``head_size``.  Page layouts: bfloat16 keys [kv head][slot][element], values [kv head][element][slot]; float32
    both [kv head][slot][element]."""
    if src.dtype != torch.float32 or src.stride(1) != 1 or not src.is_cuda:
        raise ValueError("pair_rope_unit: src must be a float32 GPU matrix with contiguous rows")
    for t, what in ((positions, "positions"), (row_seq, "row_seq"), (block_table, "block_table")):
        _need(t, torch.int32, what)
    _need(cos, torch.float32, "cos table")
    _need(sin, torch.float32, "sin table")
    bf = _act_out(q_out, "q_out")
    need = heads * dim + (kv_heads * (dim + (0 if values_are_keys else vdim)) if has_kv else 0)
    if values_are_keys and vdim != dim:
        raise ValueError("pair_rope_unit: values that are the keys have the keys' size")
    if src.shape[1] < need or src.shape[0] < rows or q_out.shape[0] < rows or q_out.shape[1] != heads * head_size:
        raise ValueError("pair_rope_unit: src or q_out do not fit")
    if positions.numel() < rows or row_seq.numel() < rows:
        raise ValueError("pair_rope_unit: fewer positions than rows")
    if rot % 2 or rot > dim or (rot and (cos.shape[1] != rot // 2 or sin.shape != cos.shape)):
        raise ValueError("pair_rope_unit: rotary tables must be [positions, rot/2]")
    if max(dim, vdim) > head_size or head_size > 256:
        raise ValueError("pair_rope_unit: heads of up to 256 elements, no larger than the cache's head size")
    kp = vp = 0
    if has_kv and write_cache:
        page_elems = kv_heads * page_size * head_size
        for c in (k_cache, v_cache):
            if c is None or c.dtype != q_out.dtype or c.dim() != 2 or c.shape[1] != page_elems or not c.is_contiguous():
                raise ValueError(f"pair_rope_unit: caches must be [pages, {page_elems}] of q_out's dtype")
        kp, vp = k_cache.data_ptr(), v_cache.data_ptr()
    _check(_fn("bw_pair_rope_unit")(src.data_ptr(), src.stride(0), positions.data_ptr(), row_seq.data_ptr(), block_table.data_ptr(),
                                    block_table.stride(0), cos.data_ptr(), sin.data_ptr(), q_out.data_ptr(), kp, vp, bf, rows,
                                    heads, kv_heads, dim, vdim, head_size, rot, page_size, int(unit_norm), float(eps),
                                    int(has_kv), int(write_cache and has_kv), int(halves), int(values_are_keys), _stream()),
           "pair_rope_unit")


def whole_norm_kv(src: torch.Tensor, positions: torch.Tensor, row_seq: torch.Tensor, block_table: torch.Tensor,
                  q_weight: torch.Tensor, k_weight: torch.Tensor, eps: float, q_out: torch.Tensor, k_cache: torch.Tensor,
                  v_cache: torch.Tensor, rows: int, heads: int, kv_heads: int, dim: int, vdim: int, head_size: int,
                  page_size: int, write_cache: bool, v_first: Optional[torch.Tensor] = None,
                  mix: Optional[torch.Tensor] = None, v_keep: Optional[torch.Tensor] = None) -> None:
    """Queries and keys of ``src`` [rows, q | k | v] (32-bit) normed over their whole projection, all heads at once,
    x / sqrt(mean(x^2) + eps) * weight; the queries go to ``q_out`` [rows, heads * head_size] and keys and values into
    the row's place in the paged cache, heads padded with zeros to ``head_size``.  ``v_first`` [rows, kv_heads * vdim]
    (32-bit) with ``mix`` (one 32-bit number on the device): the values are stored as (1 - mix) v + mix v_first.
    ``v_keep``: receives the values as projected."""
    _need(src, torch.float32, "src")
    _need(q_weight, torch.float32, "q_weight")
    _need(k_weight, torch.float32, "k_weight")
    for t, what in ((positions, "positions"), (row_seq, "row_seq"), (block_table, "block_table")):
        _need(t, torch.int32, what)
    is_bf16 = _act_out(q_out, "q_out")
    if k_cache.dtype != q_out.dtype or v_cache.dtype != q_out.dtype:
        raise ValueError("whole_norm_kv: the queries and the cache have one dtype")
    if src.shape[0] < rows or q_out.shape[0] < rows or q_out.shape[1] != heads * head_size:
        raise ValueError("whole_norm_kv: src or q_out do not fit")
    if q_weight.numel() != heads * dim or k_weight.numel() != kv_heads * dim:
        raise ValueError("whole_norm_kv: the norms' weights cover the whole projections")
    if src.shape[1] < heads * dim + (kv_heads * (dim + vdim) if write_cache else 0):
        raise ValueError("whole_norm_kv: src is narrower than the projections")
    page_elems = kv_heads * page_size * head_size
    if k_cache.shape[-1] != page_elems or v_cache.shape[-1] != page_elems:
        raise ValueError("whole_norm_kv: the cache's pages do not fit")
    for t, what in ((v_first, "v_first"), (v_keep, "v_keep")):
        if t is not None:
            _need(t, torch.float32, what)
            if t.shape[0] < rows or t.shape[1] < kv_heads * vdim:
                raise ValueError(f"whole_norm_kv: {what} does not fit")
    if v_first is not None:
        if mix is None:
            raise ValueError("whole_norm_kv: mixing needs its weight")
        _need(mix, torch.float32, "mix")
    ptr = lambda t: 0 if t is None else t.data_ptr()
    ld = lambda t: 0 if t is None else t.stride(0)
    _check(_fn("bw_whole_norm_kv")(src.data_ptr(), src.stride(0), positions.data_ptr(), row_seq.data_ptr(), block_table.data_ptr(),
                                   block_table.stride(0), q_weight.data_ptr(), k_weight.data_ptr(), float(eps), ptr(v_first),
                                   ld(v_first), ptr(mix) if v_first is not None else 0, ptr(v_keep), ld(v_keep), q_out.data_ptr(),
                                   k_cache.data_ptr(), v_cache.data_ptr(), is_bf16, rows, heads, kv_heads, dim, vdim, head_size,
                                   page_size, int(bool(write_cache)), _stream()), "whole_norm_kv")


def gate_mul(av: torch.Tensor, head_size: int, g: torch.Tensor, out: torch.Tensor, rows: int, heads: int, vdim: int,
             per_head: bool = False) -> None:
    """out[r, h*vdim + d] = av[r, h*head_size + d] * sigmoid(g[r, h*vdim + d]), or with ``per_head`` * sigmoid(g[r, h]);
    ``g`` float32 (a column slice will do)."""
    if g.dtype != torch.float32 or g.stride(1) != 1 or g.shape[1] < (heads if per_head else heads * vdim):
        raise ValueError("gate_mul: g must be float32 with contiguous rows of heads*vdim (a gate a head: of heads)")
    if av.shape[1] != heads * head_size or out.shape[1] != heads * vdim or vdim > head_size:
        raise ValueError("gate_mul: av or out do not fit")
    if min(av.shape[0], out.shape[0], g.shape[0]) < rows:
        raise ValueError("gate_mul: buffers shorter than the rows")
    _check(_fn("bw_gate_mul")(av.data_ptr(), _act_out(av, "av"), av.stride(0), head_size, g.data_ptr(), g.stride(0), out.data_ptr(),
                              _act_out(out, "out"), out.stride(0), rows, heads, vdim, int(per_head), _stream()), "gate_mul")


def rglru_scan(y: torch.Tensor, u: torch.Tensor, gates: torch.Tensor, ra_bias: torch.Tensor, ri_bias: torch.Tensor,
               decay: torch.Tensor, state: torch.Tensor, out: torch.Tensor, seq_rows: torch.Tensor, slots: torch.Tensor,
               positions: torch.Tensor, nseq: int, rows: int, channels: int, block: int,
               y_bias: Optional[torch.Tensor] = None) -> None:
    """S_t = a_t S_(t-1) + sqrt(1 - a_t^2) * i_t * u_t per channel along every request's rows, from and to ``state``
    [slots, >= channels]; a_t = exp(decay * r_t), r_t = sigmoid(gate logits + ra_bias), i_t likewise with ri_bias;
    ``gates`` [rows, channels/block * 2*block]: per block its recurrence-gate logits, then its input-gate logits;
    out = S_t * gelu_tanh(y_t).  y, u: float32 with contiguous rows (column slices will do).  Two launches: what a row
    contributes by itself (factor, addend, activation) for all ``rows`` rows at once, written over ``gates`` and ``y``,
    then the walk along each request's rows."""
    for t, what in ((y, "y"), (u, "u"), (gates, "gates"), (state, "state")):
        if t.dtype != torch.float32 or t.dim() != 2 or t.stride(1) != 1 or not t.is_cuda:
            raise ValueError(f"rglru_scan: {what} must be a float32 GPU matrix with contiguous rows")
    for t, what in ((ra_bias, "ra_bias"), (ri_bias, "ri_bias"), (decay, "decay")):
        _need(t, torch.float32, what)
        if t.numel() != channels:
            raise ValueError(f"rglru_scan: {what} needs an element per channel")
    for t, what in ((seq_rows, "seq_rows"), (slots, "slots"), (positions, "positions")):
        _need(t, torch.int32, what)
    if channels % block or min(y.shape[1], u.shape[1], state.shape[1]) < channels or gates.shape[1] < 2 * channels or out.shape[1] != channels:
        raise ValueError("rglru_scan: widths do not fit the channels")
    if seq_rows.numel() < 2 * nseq or slots.numel() < nseq or positions.numel() < rows or min(y.shape[0], u.shape[0], gates.shape[0], out.shape[0]) < rows:
        raise ValueError("rglru_scan: fewer request records than requests, or buffers shorter than the rows")
    if y_bias is not None:
        _need(y_bias, torch.float32, "y_bias")
        if y_bias.numel() != channels:
            raise ValueError("rglru_scan: y_bias needs an element per channel")
    _check(_fn("bw_rglru_scan")(y.data_ptr(), y.stride(0), 0 if y_bias is None else y_bias.data_ptr(), u.data_ptr(), u.stride(0), gates.data_ptr(), gates.stride(0),
                                ra_bias.data_ptr(), ri_bias.data_ptr(), decay.data_ptr(), state.data_ptr(), state.stride(0),
                                out.data_ptr(), _act_out(out, "out"), out.stride(0), seq_rows.data_ptr(), slots.data_ptr(),
                                positions.data_ptr(), int(nseq), int(rows), channels, block, _stream()), "rglru_scan")


def norm_add(y: torch.Tensor, weight: torch.Tensor, x: torch.Tensor, rows: int, eps: float,
             rounded: Optional[torch.Tensor] = None, combine: Optional[Tuple[torch.Tensor, torch.Tensor, int]] = None,
             scale: float = 1.0) -> None:
    """x[:rows] += scale * (y / sqrt(mean(y^2) + eps) * weight), all 32-bit.  ``rounded`` (bfloat16, x's shape): also receives the new
    rows rounded, for products that follow.  ``combine`` = (place, wts, top): row r of the normed operand is
    sum_j wts[r, j] * y[place[r*top + j]] (j ascending, the chain of ``moe_combine``) instead of y[r]."""
    _need(y, torch.float32, "y")
    _need(x, torch.float32, "x")
    dim = x.shape[1]
    if y.shape[1] != dim or weight.numel() != dim or not weight.is_cuda or x.shape[0] < rows or (combine is None and y.shape[0] < rows):
        raise ValueError("norm_add: y, weight and x do not fit")
    place = wts = None
    top = 0
    if combine is not None:
        place, wts, top = combine
        _need(place, torch.int32, "place")
        _need(wts, torch.float32, "wts")
        if place.numel() < rows * top or wts.numel() < rows * top or top < 1:
            raise ValueError("norm_add: the combination's tables are shorter than the rows")
    if rounded is not None:
        _need(rounded, torch.bfloat16, "rounded")
        if rounded.shape[1] != dim or rounded.shape[0] < rows:
            raise ValueError("norm_add: the rounded copy does not fit")
    _check(_fn("bw_norm_add")(y.data_ptr(), y.stride(0), weight.data_ptr(), _is_bf16(weight, "weight"), x.data_ptr(), x.stride(0),
                              0 if rounded is None else rounded.data_ptr(), 0 if rounded is None else rounded.stride(0),
                              rows, dim, float(eps), 0 if place is None else place.data_ptr(), 0 if wts is None else wts.data_ptr(),
                              int(top), float(scale), _stream()), "norm_add")


def softcap(x: torch.Tensor, rows: int, cap: float) -> None:
    """x[:rows] = cap * tanh(x / cap) in place."""
    _need(x, torch.float32, "x")
    if x.shape[0] < rows or not cap > 0:
        raise ValueError("softcap: fewer rows than said, or a cap that is not positive")
    _check(_fn("bw_softcap")(x.data_ptr(), x.stride(0), rows, x.shape[1], float(cap), _stream()), "softcap")


def scale_rows(x: torch.Tensor, rows: int, factor: float) -> None:
    """x[:rows] *= factor in place (32-bit)."""
    _need(x, torch.float32, "x")
    if x.shape[0] < rows:
        raise ValueError("scale_rows: fewer rows than said")
    _check(_fn("bw_scale_rows")(x.data_ptr(), x.stride(0), rows, x.shape[1], float(factor), _stream()), "scale_rows")


# ------------------------------------------------------------------------------ routed experts

def moe_max_tiles(slots: int, experts: int) -> int:
    """The most tiles a plan of this many (row, choice) pairs over this many experts can have."""
    return int(_fn("bw_moe_max_tiles")(int(slots), int(experts)))


SCORE_SOFTMAX, SCORE_SIGMOID = 0, 1


def _route_rule(score: int, correction: Optional[torch.Tensor], group_best: int, experts: int):
    if score not in (SCORE_SOFTMAX, SCORE_SIGMOID) or not 1 <= int(group_best) <= 4:
        raise ValueError("moe_route: scores are a softmax or sigmoids; a group's score sums one to four of its best")
    if correction is not None:
        _need(correction, torch.float32, "correction")
        if correction.numel() != experts:
            raise ValueError("moe_route: a correction per expert is needed")
    return int(score), 0 if correction is None else correction.data_ptr(), int(group_best)


def moe_route(logits: torch.Tensor, rows: int, top: int, groups: int, keep: int, ids: torch.Tensor, wts: torch.Tensor,
              weight_scale: float = 1.0, experts: Optional[int] = None, score: int = SCORE_SOFTMAX,
              correction: Optional[torch.Tensor] = None, group_best: int = 1) -> None:
    """Per row: scores = softmax over the experts' logits (``score`` SCORE_SIGMOID: the sigmoid of each); the ``top`` best
    experts among those of the ``keep`` best of ``groups`` equal groups of neighbours, judged by score + ``correction``
    (a group's score: the sum of its ``group_best`` best); ``ids`` [rows, top] int32 in the order chosen,
    ``wts`` [rows, top] their scores (without the correction)."""
    _need(logits, torch.float32, "logits")
    _need(ids, torch.int32, "ids")
    _need(wts, torch.float32, "wts")
    experts = logits.shape[1] if experts is None else int(experts)      # (the rows may hold more columns behind the experts')
    if logits.shape[0] < rows or logits.shape[1] < experts or ids.numel() < rows * top or wts.numel() < rows * top:
        raise ValueError("moe_route: buffers shorter than the rows")
    if experts % groups or not 1 <= keep <= groups or not 1 <= top <= keep * (experts // groups):
        raise ValueError("moe_route: groups, keep and top do not fit the experts")
    _check(_fn("bw_moe_route")(logits.data_ptr(), logits.stride(0), rows, experts, top, groups, keep, float(weight_scale),
                               *_route_rule(score, correction, group_best, experts), ids.data_ptr(), wts.data_ptr(), _stream()),
           "moe_route")


def moe_plan(ids: torch.Tensor, slots: int, experts: int, sorted_slots: torch.Tensor, place: torch.Tensor, tiles: torch.Tensor,
             meta: torch.Tensor) -> None:
    """The (row, choice) pairs sorted by expert and cut into tiles of one expert each (see moe.hip)."""
    for t, what in ((ids, "ids"), (sorted_slots, "sorted"), (place, "place"), (tiles, "tiles"), (meta, "meta")):
        _need(t, torch.int32, what)
    if min(ids.numel(), sorted_slots.numel(), place.numel()) < slots or tiles.numel() < 4 * moe_max_tiles(slots, experts) or meta.numel() < 1:
        raise ValueError("moe_plan: buffers too small")
    _check(_fn("bw_moe_plan")(ids.data_ptr(), slots, experts, sorted_slots.data_ptr(), place.data_ptr(), tiles.data_ptr(),
                              meta.data_ptr(), _stream()), "moe_plan")


def moe_route_plan(logits: torch.Tensor, rows: int, top: int, groups: int, keep: int, ids: torch.Tensor, wts: torch.Tensor,
                   sorted_slots: torch.Tensor, place: torch.Tensor, tiles: torch.Tensor, meta: torch.Tensor,
                   weight_scale: float = 1.0, experts: Optional[int] = None, score: int = SCORE_SOFTMAX,
                   correction: Optional[torch.Tensor] = None, group_best: int = 1) -> None:
    """``moe_route`` followed by ``moe_plan`` over the rows' choices; steps of up to 16 rows do both in one launch.
    ``weight_scale``: the chosen scores are multiplied by it; ``experts``: the leading columns of ``logits`` that are the
    experts' (all of them by default)."""
    _need(logits, torch.float32, "logits")
    _need(wts, torch.float32, "wts")
    for t, what in ((ids, "ids"), (sorted_slots, "sorted"), (place, "place"), (tiles, "tiles"), (meta, "meta")):
        _need(t, torch.int32, what)
    experts, slots = (logits.shape[1] if experts is None else int(experts)), rows * top
    if logits.shape[0] < rows or logits.shape[1] < experts or min(ids.numel(), wts.numel(), sorted_slots.numel(), place.numel()) < slots:
        raise ValueError("moe_route_plan: buffers shorter than the rows")
    if experts % groups or not 1 <= keep <= groups or not 1 <= top <= keep * (experts // groups):
        raise ValueError("moe_route_plan: groups, keep and top do not fit the experts")
    if tiles.numel() < 4 * moe_max_tiles(slots, experts) or meta.numel() < 1:
        raise ValueError("moe_route_plan: the plan's tables are too small")
    _check(_fn("bw_moe_route_plan")(logits.data_ptr(), logits.stride(0), rows, experts, top, groups, keep, float(weight_scale),
                                    *_route_rule(score, correction, group_best, experts), ids.data_ptr(), wts.data_ptr(),
                                    sorted_slots.data_ptr(), place.data_ptr(), tiles.data_ptr(), meta.data_ptr(), _stream()),
           "moe_route_plan")


def moe_experts(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor, sorted_slots: torch.Tensor, tiles: torch.Tensor,
                meta: torch.Tensor, slots: int, top: int, gate_up: bool, limit: float = 0.0, alpha: float = 0.0,
                round_out: bool = False) -> None:
    """The experts' products over a plan's tiles.  ``gate_up``: x [rows, K] (a slot reads row slot // top), w [experts, 2N, K]
    (gate rows, then up rows), out [slots, N] = the gated activation by sorted place.  Else: x [slots, K] by sorted place,
    w [experts, N, K], out [slots, N] float32.  bfloat16 x runs on the matrix cores (bfloat16 weights, K a multiple of 8);
    float32 x runs 32-bit chains (``round_out``: the activation is rounded to bfloat16 values)."""
    if w.dim() != 3 or not w.is_cuda or not w.is_contiguous():
        raise ValueError("moe_experts: weights must be a contiguous [experts, N, K] GPU tensor")
    experts, N, K = w.shape
    if gate_up:
        N //= 2
    xb, wb = _act_out(x, "x"), _is_bf16(w, "weights")
    if x.shape[1] != K or out.shape[1] != N or out.shape[0] < slots or (not gate_up and x.shape[0] < slots):
        raise ValueError("moe_experts: x, w and out do not fit")
    if xb and (not wb or K % 8):
        raise ValueError("moe_experts: the matrix-core route takes bfloat16 weights and an inner size that is a multiple of 8")
    want = torch.bfloat16 if (xb and gate_up) else torch.float32
    _need(out, want, "out")
    for t, what in ((sorted_slots, "sorted"), (tiles, "tiles"), (meta, "meta")):
        _need(t, torch.int32, what)
    max_tiles = moe_max_tiles(slots, experts)
    if tiles.numel() < 4 * max_tiles or sorted_slots.numel() < slots:
        raise ValueError("moe_experts: the plan's tables are too small")
    _check(_fn("bw_moe_experts")(x.data_ptr(), xb, x.stride(0), x.shape[0], w.data_ptr(), wb, out.data_ptr(), out.stride(0), sorted_slots.data_ptr(),
                                 tiles.data_ptr(), meta.data_ptr(), slots, max_tiles, top, K, N, int(gate_up), float(limit), float(alpha),
                                 int(round_out), _stream()), "moe_experts")


def moe_combine(y: torch.Tensor, place: torch.Tensor, wts: torch.Tensor, top: int, out: torch.Tensor, rows: int,
                accumulate: bool) -> None:
    """out[r] (+)= sum_j wts[r, j] * y[place[r*top + j]], j ascending."""
    _need(y, torch.float32, "y")
    _need(out, torch.float32, "out")
    _need(place, torch.int32, "place")
    _need(wts, torch.float32, "wts")
    if y.shape[1] != out.shape[1] or out.shape[0] < rows or place.numel() < rows * top or wts.numel() < rows * top:
        raise ValueError("moe_combine: buffers do not fit")
    _check(_fn("bw_moe_combine")(y.data_ptr(), y.stride(0), place.data_ptr(), wts.data_ptr(), top, out.data_ptr(), out.stride(0),
                                 rows, out.shape[1], int(accumulate), _stream()), "moe_combine")


# ------------------------------------------------------------------------------ sampling

def sample(logits: torch.Tensor, rows: int, temperature: torch.Tensor, uniform: torch.Tensor,
           out: torch.Tensor) -> None:
    """out[r] = first maximum of row r if temperature[r] <= 0, else the inverse-CDF draw at
    uniform[r] from softmax(logits[r] / temperature[r])."""
    _need(logits, torch.float32, "logits")
    _need(temperature, torch.float32, "temperature")
    _need(uniform, torch.float64, "uniform")
    _need(out, torch.int32, "out")
    if logits.shape[0] < rows or temperature.numel() < rows or uniform.numel() < rows or out.numel() < rows:
        raise ValueError("sample: buffers shorter than the number of rows")
    _check(_fn("bw_sample")(logits.data_ptr(), logits.shape[1], logits.stride(0), rows, temperature.data_ptr(),
                            uniform.data_ptr(), out.data_ptr(), _stream()), "sample")


def fingerprint(logits: torch.Tensor, rows: int, h_in: torch.Tensor, h_out: torch.Tensor) -> None:
    """h_out[r] = the reference's logits hash chained from h_in[r] (int64 bit patterns)."""
    _need(logits, torch.float32, "logits")
    _need(h_in, torch.int64, "h_in")
    _need(h_out, torch.int64, "h_out")
    _check(_fn("bw_fingerprint")(logits.data_ptr(), logits.shape[1], logits.stride(0), rows, h_in.data_ptr(),
                                 h_out.data_ptr(), _stream()), "fingerprint")
