"""The hand-written gfx950 kernels, as functions over torch tensors.

Every function checks on the host that shapes, types and strides are what the
kernel and its launch assume, then launches on torch's current stream.  There is
no fallback: without the compiled library, or on a tensor that is not on the
GPU, these functions raise.
"""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_void_p

import torch

from . import build
from .errors import TensorError

F32, BF16 = 0, 1
_CODES = {torch.float32: F32, torch.bfloat16: BF16}

_lib = None


def _signatures(lib) -> None:
    p, i, f = c_void_p, c_int, c_float
    lib.pl_last_error.restype = ctypes.c_char_p
    lib.pl_abi_version.restype = c_int
    table = {
        "pl_embed": [p, p, i, p, i, i, i, p],
        "pl_embed_fed": [p, p, p, p, i, p, i, i, i, p],
        "pl_add_rmsnorm": [p, p, p, i, f, p, i, p, i, i, i, p],
        "pl_residual_add": [p, p, i, i, i, p],
        "pl_add_bias": [p, p, i, i, i, i, p],
        "pl_qk_norm_rope_kv_write": [p, p, p, i, f, p, p, i, p, p, p, i, i, p, p, i, i, i, i, i, i, i, p],
        "pl_swiglu": [p, p, i, i, i, i, p],
        "pl_gemm_plain": [p, p, p, i, i, i, i, i, i, i, p],
        "pl_paged_attention_plain": [p, i, p, p, p, p, i, i, p, p, i, i, i, i, f, i, i, p, p, p],
        "pl_gemm_heads": [p, p, p, i, i, i, i, i, ctypes.c_long, i, ctypes.c_long, i, i, p],
        "pl_head_prepare": [p, p, i, i, i, f, p, p, p, p, i, i, i, i, f, i, p, p, p, i, i, i, p, p, p, i, i, i, i, i, i, i, p],
        "pl_latent_prepare": [p, i, i, i, p, f, p, p, i, i, p, p, p, i, i, i, p, p, p, i, i, i, i, i, i, i, p],
        "pl_head_gate": [p, i, p, i, i, p, i, i, i, i, p],
        "pl_add_position_rows": [p, p, i, p, i, i, i, p],
        "pl_paged_attention_prefill_tile": [i, i],
        "pl_argmax": [p, p, p, p, i, i, p],
        "pl_sample": [p, p, p, p, p, p, i, i, i, p],
        "pl_gemm_skinny": [p, p, p, p, f, p, i, i, i, i, i, i, i, p],
        "pl_gemm_skinny_strips_apply": [i, i, i],
        "pl_gemm_skinny_hand": [p, p, p, i, i, i, i, i, i, p, i, f, p, p, p, i, p],
        "pl_gemm_skinny_hand_applies": [i, i, i, i, i],
        "pl_gemm_tiled": [p, p, p, i, i, i, i, i, p],
        "pl_gemm_tiled_applies": [i, i, i, i],
        "pl_gemm_stream": [p, p, p, p, i, i, i, i, i, i, i, p],
        "pl_gemm_stream_splits": [i, i, i, i],
        "pl_gemm_finish": [p, p, ctypes.c_longlong, i, i, i, i, i, p],
        "pl_paged_attention_decode": [p, i, p, p, p, p, p, p, i, i, i, p, i, i, p, p, i, i, i, i, f, i, i,
                                      i, p, p, i, f, p, p, i, p, p, p],
        "pl_paged_attention_prefill": [p, i, p, p, p, p, i, i, i, p, i, i, p, p, i, i, i, f, i, i, p, p, i, p, p, p],
        "pl_paged_attention_grouped": [p, i, p, p, p, p, i, i, i, p, i, i, p, p, i, i, i, f, i, i, p, p, i, i, p, p, p],
        "pl_paged_attention_grouped_applies": [i, i, i, i],
        "pl_recurrent_scan": [i, p, i, i, i, i, p, i, i, i, p, p, f, p, ctypes.c_long, i, i, i, p, p, p, p,
                              i, i, i, i, i, i, p],
        "pl_recurrent_chunked": [i, p, i, i, i, i, p, i, i, i, p, p, f, p, ctypes.c_long, i, i, i, p, p, p, p,
                                 i, i, i, i, i, i, p, p, p, p, p, p],
        "pl_recurrent_chunk_tokens": [i],
        "pl_delta_chunked": [p, i, i, i, i, p, i, i, i, p, p, p, ctypes.c_long, p, p, p, p, i, i, i, i, i, i, i,
                             p, p, p, p, p, p],
        "pl_short_conv": [p, i, i, i, p, i, p, ctypes.c_long, i, p, p, p, p, p, i, i, p],
        "pl_conv_history": [p, i, i, i, i, p, ctypes.c_long, i, p, p, p, i, p],
        "pl_gated_group_norm": [p, i, i, i, p, i, f, p, i, i, i, p, i, p],
        "pl_conv_qk_prepare": [p, i, i, p, i, p, ctypes.c_long, i, p, p, f, p, i, p, p, p, p, p, i, i, p, p, p, i,
                               i, i, i, i, i, i, p],
        "pl_rmsnorm_onto": [p, p, p, f, p, i, i, i, p],
        "pl_scale": [p, f, ctypes.c_long, p],
        "pl_to_bf16": [p, p, ctypes.c_long, p],
        "pl_activation": [p, p, i, i, ctypes.c_long, p],
        "pl_weighted_sum": [p, f, p, f, ctypes.c_long, p],
        "pl_hc_step": [p, p, p, p, p, p, f, p, i, p, i, i, i, p],
        "pl_stream_copies": [p, p, i, i, i, p],
        "pl_softcap": [p, f, ctypes.c_long, p],
        "pl_moe_rows": [p, p, p, p, p, p, p, p, p, p, i, i, i, i, i, i, i, i, p, p, i, p],
        "pl_moe_sort": [p, p, p, p, p, p, i, i, i, i, i, i, p, p, p, p],
        "pl_moe_combine": [p, p, p, i, i, i, i, ctypes.c_longlong, p, p, p, i, i, p, p],
        "pl_router_select": [p, i, p, p, i, i, i, i, i, i, f, p, p, p, p, i, i, p],
        "pl_wide_prepare": [p, p, i, i, i, f, p, p, p, i, p, p, p, i, i, i, p, p, p, i, i, i, i, i, i, p],
        "pl_parallel_step": [p, p, p, p, p, p, p, p, f, p, p, i, p, i, i, p],
        "pl_gemm_tiled_grouped": [p, p, p, p, p, ctypes.c_longlong, i, i, i, i, i, i, i, p],
    }
    for name, argtypes in table.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = c_int


def library():
    """The kernel library, compiled at its first use when nothing is built."""
    global _lib
    if _lib is None:
        lib = build.load("hip")
        _signatures(lib)
        _lib = lib
    return _lib


def _check(code: int) -> None:
    if code != 0:
        raise TensorError(library().pl_last_error().decode())


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream() -> int:
    """The handle of torch's current stream on the current device (asked for once a launch: the short way)."""
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _code(t: torch.Tensor, what: str) -> int:
    if t.dtype not in _CODES:
        raise TensorError(f"{what} is {t.dtype}, the kernels take float32 and bfloat16")
    return _CODES[t.dtype]


def _need(t: torch.Tensor, what: str, shape=None, dtype=None) -> torch.Tensor:
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TensorError(f"{what} is not a tensor on the GPU")
    if not t.is_contiguous():
        raise TensorError(f"{what} is not contiguous (strides {t.stride()} for shape {tuple(t.shape)})")
    if shape is not None and tuple(t.shape) != tuple(shape):
        raise TensorError(f"{what} has shape {tuple(t.shape)}, expected {tuple(shape)}")
    if dtype is not None and t.dtype != dtype:
        raise TensorError(f"{what} is {t.dtype}, expected {dtype}")
    return t


def _ptr(t) -> int:
    return 0 if t is None else t.data_ptr()


# ---------------------------------------------------------------------------

def embed(ids: torch.Tensor, table: torch.Tensor, out: torch.Tensor | None = None,
          src: torch.Tensor | None = None, fed: torch.Tensor | None = None) -> torch.Tensor:
    """out[t] = table[ids[t]] as the 32-bit residual stream; a negative id gives zeros.  With ``src`` and
    ``fed`` a row t whose src[t] is not negative takes fed[src[t]] for its id: a token that an earlier
    kernel left on the device.  (The caller answers for src[t] < len(fed).)"""
    n = ids.numel()
    V, H = table.shape
    _need(ids, "token ids", (n,), torch.int32)
    _need(table, "embedding table")
    if (src is None) != (fed is None):
        raise TensorError("rows fed from the device need both their sources and the tokens")
    if src is not None:
        _need(src, "sources of the token ids", (n,), torch.int32)
        _need(fed, "tokens left on the device", None, torch.int32)
    if out is None:
        out = torch.empty((n, H), dtype=torch.float32, device=table.device)
    _need(out, "embedding output", (n, H), torch.float32)
    _check(library().pl_embed_fed(ids.data_ptr(), _ptr(src), _ptr(fed), table.data_ptr(),
                                  _code(table, "embedding table"), out.data_ptr(), n, H, V, _stream()))
    return out


def add_rmsnorm(resid: torch.Tensor, delta, gain: torch.Tensor, eps: float, out: torch.Tensor,
                rows: torch.Tensor | None = None, write_resid: bool = True) -> torch.Tensor:
    """x = resid (+ delta); resid = x when ``write_resid``; out = rmsnorm(x) * gain.
    With ``rows`` the i-th output row is computed from row rows[i] and nothing is written back."""
    n, H = resid.shape
    _need(resid, "residual stream", None, torch.float32)
    n_out = n if rows is None else rows.numel()
    _need(out, "norm output", (n_out, H))
    if delta is not None:
        _need(delta, "residual delta", (n, H), out.dtype)
    _need(gain, "norm gain", (H,))
    if rows is not None:
        _need(rows, "row list", (n_out,), torch.int32)
        write_resid = False
    _check(library().pl_add_rmsnorm(resid.data_ptr(), _ptr(delta), gain.data_ptr(), _code(gain, "norm gain"),
                                    float(eps), out.data_ptr(), _code(out, "norm output"), _ptr(rows),
                                    n_out, H, 1 if write_resid else 0, _stream()))
    return out


def residual_add(resid: torch.Tensor, delta: torch.Tensor) -> torch.Tensor:
    n, H = resid.shape
    _need(resid, "residual stream", None, torch.float32)
    _need(delta, "residual delta", (n, H))
    _check(library().pl_residual_add(resid.data_ptr(), delta.data_ptr(), _code(delta, "residual delta"), n, H, _stream()))
    return resid


def add_bias(y: torch.Tensor, bias: torch.Tensor) -> torch.Tensor:
    """y[r, c] += bias[c], in place."""
    n, N = y.shape
    _need(y, "projection output")
    _need(bias, "bias", (N,))
    _check(library().pl_add_bias(y.data_ptr(), bias.data_ptr(), _code(y, "projection output"), _code(bias, "bias"),
                                 n, N, _stream()))
    return y


def qk_norm_rope_kv_write(qkv: torch.Tensor, q_gain, k_gain, eps: float, cos, sin, rot: int,
                          positions: torch.Tensor, seq_of: torch.Tensor, block_table: torch.Tensor,
                          block_size: int, k_pool: torch.Tensor, v_pool: torch.Tensor,
                          nq: int, nkv: int, d: int, write_kv: bool = True, neighbours: bool = False) -> None:
    """Per-head norm of q and k, rotation of q and k at each token's position, and
    the write of k and v into their pages.  q is rewritten in place inside ``qkv``.
    The rotation turns the pairs (i, i + rot/2), or with ``neighbours`` the pairs (2 i, 2 i + 1)."""
    n = qkv.shape[0]
    _need(qkv, "fused q/k/v projection", (n, (nq + 2 * nkv) * d))
    _need(positions, "positions", (n,), torch.int32)
    _need(seq_of, "request index of each token", (n,), torch.int32)
    _need(block_table, "block table", None, torch.int32)
    if block_table.dim() != 2:
        raise TensorError(f"block table has shape {tuple(block_table.shape)}, expected [requests, pages]")
    for pool, what in ((k_pool, "key pool"), (v_pool, "value pool")):
        _need(pool, what, None, qkv.dtype)
        if pool.dim() != 2 or pool.shape[1] != nkv * d or pool.shape[0] % block_size != 0:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{block_size}, {nkv * d}]")
    if k_pool.shape != v_pool.shape:
        raise TensorError("key and value pools differ in shape")
    if k_pool.shape[0] >= 2 ** 31:
        raise TensorError("a pool of 2^31 slots or more is not addressed by these kernels")
    gain_code = F32
    if q_gain is not None:
        _need(q_gain, "query norm gain", (d,))
        _need(k_gain, "key norm gain", (d,), q_gain.dtype)
        gain_code = _code(q_gain, "query norm gain")
    if cos is not None:
        _need(cos, "cosine table", None, torch.float32)
        _need(sin, "sine table", tuple(cos.shape), torch.float32)
        if cos.dim() != 2 or cos.shape[1] != rot // 2:
            raise TensorError(f"rotary tables have shape {tuple(cos.shape)}, expected [positions, {rot // 2}]")
    _check(library().pl_qk_norm_rope_kv_write(
        qkv.data_ptr(), _ptr(q_gain), _ptr(k_gain), gain_code, float(eps), _ptr(cos), _ptr(sin), rot,
        positions.data_ptr(), seq_of.data_ptr(), block_table.data_ptr(), block_table.shape[1], block_size,
        k_pool.data_ptr(), v_pool.data_ptr(), n, nq, nkv, d, 1 if write_kv else 0,
        _code(qkv, "fused q/k/v projection"), 1 if neighbours else 0, _stream()))


# The activations of a gated feed-forward's gate branch, by the names config.json gives them.
ACTIVATIONS = {"silu": 0, "swish": 0, "gelu_pytorch_tanh": 1, "gelu_tanh": 1, "gelu_new": 1, "gelu": 2}


def activation_code(name: str) -> int:
    if name not in ACTIVATIONS:
        raise TensorError(f"activation {name!r}, the kernels know {', '.join(sorted(ACTIVATIONS))}")
    return ACTIVATIONS[name]


def swiglu(gate_up: torch.Tensor, out: torch.Tensor | None = None, activation: str = "silu") -> torch.Tensor:
    """act(gate) * up on rows laid out [gate | up]; ``act`` is SiLU or a GELU."""
    n, two_i = gate_up.shape
    _need(gate_up, "fused gate/up projection")
    if two_i % 2:
        raise TensorError(f"fused gate/up projection has odd width {two_i}")
    inter = two_i // 2
    if out is None:
        out = torch.empty((n, inter), dtype=gate_up.dtype, device=gate_up.device)
    _need(out, "feed-forward activation", (n, inter), gate_up.dtype)
    _check(library().pl_swiglu(gate_up.data_ptr(), out.data_ptr(), n, inter, _code(gate_up, "gate/up"),
                               activation_code(activation), _stream()))
    return out


def gemm_plain(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor | None = None,
               out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """y = x . w^T with 32-bit multiply-add on the vector units (no matrix-core mode)."""
    n, K = x.shape
    N = w.shape[0]
    _need(x, "matrix product input")
    _need(w, "weight", (N, K), x.dtype)
    out_dtype = out_dtype or x.dtype
    if out is None:
        out = torch.empty((n, N), dtype=out_dtype, device=x.device)
    _need(out, "matrix product output", (n, N), out_dtype)
    if out_dtype not in (x.dtype, torch.float32):
        raise TensorError(f"matrix product output {out_dtype} from input {x.dtype}")
    _check(library().pl_gemm_plain(x.data_ptr(), w.data_ptr(), out.data_ptr(), n, N, K, K, N,
                                   _code(x, "matrix product input"), 1 if out_dtype == torch.float32 else 0, _stream()))
    return out


def _head_numbers(t, what: str, heads: int):
    """A 32-bit number a query head (sinks, slopes), or None."""
    if t is None:
        return None
    return _need(t, what, (heads,), torch.float32)


def paged_attention_plain(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, positions: torch.Tensor,
                          seq_of: torch.Tensor, block_table: torch.Tensor, block_size: int,
                          k_pool: torch.Tensor, v_pool: torch.Tensor, nq: int, nkv: int, d: int,
                          scale: float, window: int = 0, sinks: torch.Tensor | None = None,
                          slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention of every token over the keys 0..position of its request, read
    through the block table.  ``q`` is the fused projection buffer whose rows begin
    with the nq*d query values.  ``slopes`` [nq]: slope_h * (i - j) is taken off the score of key j for
    the query at position i.  ``sinks`` [nq]: exp(sink_h) joins the softmax's denominator, once, unscaled
    and without a value.  Key and value pool may be the same tensor."""
    n = positions.numel()
    _need(q, "query buffer")
    if q.dim() != 2 or q.shape[0] != n or q.shape[1] != q_row_stride or q_row_stride < nq * d:
        raise TensorError(f"query buffer has shape {tuple(q.shape)} for {n} tokens and row stride {q_row_stride}")
    _need(out, "attention output", (n, nq * d), q.dtype)
    _need(positions, "positions", (n,), torch.int32)
    _need(seq_of, "request index of each token", (n,), torch.int32)
    _need(block_table, "block table", None, torch.int32)
    for pool, what in ((k_pool, "key pool"), (v_pool, "value pool")):
        _need(pool, what, None, q.dtype)
        if pool.dim() != 2 or pool.shape[1] != nkv * d or pool.shape[0] % block_size != 0:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{block_size}, {nkv * d}]")
    sinks, slopes = _head_numbers(sinks, "sinks", nq), _head_numbers(slopes, "distance slopes", nq)
    _check(library().pl_paged_attention_plain(
        q.data_ptr(), q_row_stride, out.data_ptr(), positions.data_ptr(), seq_of.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], block_size, k_pool.data_ptr(), v_pool.data_ptr(),
        n, nq, nkv, d, float(scale), int(window or 0), _code(q, "query buffer"), _ptr(sinks), _ptr(slopes), _stream()))
    return out


def argmax(logits: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
    """The index of the largest logit of each row; the first maximum wins."""
    m, V = logits.shape
    _need(logits, "logits", None, torch.float32)
    if out is None:
        out = torch.empty((m,), dtype=torch.int32, device=logits.device)
    _need(out, "chosen tokens", (m,), torch.int32)
    scratch_v = torch.empty((m * 64,), dtype=torch.float32, device=logits.device)
    scratch_i = torch.empty((m * 64,), dtype=torch.int32, device=logits.device)
    _check(library().pl_argmax(logits.data_ptr(), out.data_ptr(), scratch_v.data_ptr(), scratch_i.data_ptr(),
                               m, V, _stream()))
    return out


def sample(logits: torch.Tensor, temperature: torch.Tensor, top_k: torch.Tensor, top_p: torch.Tensor,
           uniform: torch.Tensor, out: torch.Tensor | None = None, out_holds_largest: bool = False) -> torch.Tensor:
    """One token a row: logits / temperature, the k most likely, of those the shortest head
    whose mass reaches top_p, and of that the token on which the mass reaches uniform * total,
    all in the order of falling logit and rising index (reference: crates/pagedllm/src/sampler.rs).
    A row with temperature 0 takes its largest logit.  top_k 0 and top_p 1 cut nothing.
    ``out_holds_largest``: ``out`` comes with what ``argmax`` made of these logits, which saves the kernel
    its first pass over every row."""
    m, V = logits.shape
    _need(logits, "logits", None, torch.float32)
    _need(temperature, "temperatures", (m,), torch.float32)
    _need(top_k, "top_k", (m,), torch.int32)
    _need(top_p, "top_p", (m,), torch.float32)
    _need(uniform, "uniform numbers", (m,), torch.float32)
    if out is None:
        if out_holds_largest:
            raise TensorError("no tokens given that could hold the largest logits' places")
        out = torch.empty((m,), dtype=torch.int32, device=logits.device)
    _need(out, "chosen tokens", (m,), torch.int32)
    _check(library().pl_sample(logits.data_ptr(), temperature.data_ptr(), top_k.data_ptr(), top_p.data_ptr(),
                               uniform.data_ptr(), out.data_ptr(), m, V, 1 if out_holds_largest else 0, _stream()))
    return out


_attention_mode = "kernel"

# A request that brings fewer tokens than this to a step has each of them served
# like a decoded token (one row of queries against its keys); longer portions go
# to the tiled kernel.
SHORT_PORTION = 16
SKINNY_ROWS = 64


def set_attention(mode: str) -> None:
    """``kernel``: the fast bfloat16 kernels where they apply; ``tensor``: the plain
    kernel with 32-bit arithmetic that they are checked against (the reference's
    flag of the same name chooses between its kernel and its tensor path)."""
    global _attention_mode
    if mode not in ("kernel", "tensor"):
        raise TensorError(f"attention {mode!r}, which is neither tensor nor kernel")
    _attention_mode = mode


# What a compute unit takes in from memory (bytes a microsecond), what the merge of the shares costs beside the
# kernel (microseconds), and the compute units: the figures of the estimate below.
DECODE_INTAKE = 22e3
DECODE_MERGE_US = 4.0


def decode_splits(tokens: int, nq: int, nkv: int, max_ctx: int, d: int = 128) -> int:
    """Into how many stretches the context is cut for the single-token kernel, each with at least 128 keys
    (two rounds of loads).

    Up to two query heads a key head the kernel waits for memory, and a compute unit takes in only so much:
    the launch is as long as the keys and values of its busiest compute unit take (workgroups are dealt to
    the compute units in turn), plus the merge's kernel where there are shares; the count with the smallest
    such estimate is taken.  (Measured, 16 query over 8 key heads of 128, one share against the estimate's
    choice: 12 tokens at context 2,048, three shares 32.9 us, eight 28.0; 24 tokens, two 50.1, four 45.4; 48
    tokens at 1,024, one 48.1, two 45.3; 24 tokens at 512, two 20.9, one 18.8.)
    With more query heads a key head a workgroup has more arithmetic a key and the compute units are what
    is short: none when the tokens and heads alone give about two workgroups a compute unit, else up to
    that many (8 tokens at context 2,048 with four heads a key head: eight shares 24.6 us, four 25.9; 32
    tokens, two 61.9, one 68.3; 63 tokens, one 105.7, two 111.2)."""
    g = nq // nkv
    gt = 8 if g >= 8 else (4 if g > 2 else g)
    base = max(tokens * nkv * ((g + gt - 1) // gt), 1)
    most = max(1, min((max_ctx + 127) // 128, 64))
    if g > 2:
        target = 2 * compute_units()
        if base >= target - target // 16:
            return 1
        return max(1, min((target + base - 1) // base, most))
    units = compute_units()
    best, best_us = 1, None
    for splits in range(1, most + 1):
        busiest = -(-base * splits // units)                      # workgroups on one compute unit
        keys = -(-max_ctx // splits)
        us = busiest * keys * (4 * d) / DECODE_INTAKE + (DECODE_MERGE_US if splits > 1 else 0.0)
        if best_us is None or us < best_us - 1e-9:
            best, best_us = splits, us
    return best


def paged_attention_decode(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, positions: torch.Tensor,
                           seq_of: torch.Tensor, block_table: torch.Tensor, block_size: int,
                           k_pool: torch.Tensor, v_pool: torch.Tensor, nq: int, nkv: int, d: int, scale: float,
                           window: int = 0, splits: int = 1, q_len: torch.Tensor | None = None,
                           short_limit: int = 0, fuse: "QkFusion | None" = None, live_seqs: int | None = None,
                           short_rows: int = 0, sinks: torch.Tensor | None = None,
                           slopes: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 attention of single tokens over their requests' pages, split along the context.
    With ``q_len`` the tokens of requests with ``short_limit`` tokens or more are left out; ``short_rows``
    then bounds the tokens that the other requests bring (0: not known) and ``live_seqs`` says how many
    requests, the first ones, bring tokens, so that the launch has workgroups for those tokens only.
    With ``fuse`` the rows of ``q`` are the raw projection [q | k | v]: queries (and, when it says so, each
    token's key) are normalised and rotated inside the kernel, and key and value are written into the pages.
    ``sinks`` and ``slopes``: as in ``paged_attention_plain``."""
    n = positions.numel()
    sinks, slopes = _head_numbers(sinks, "sinks", nq), _head_numbers(slopes, "distance slopes", nq)
    _need(q, "query buffer", None, torch.bfloat16)
    if q.dim() != 2 or q.shape[0] != n or q.shape[1] != q_row_stride or q_row_stride < nq * d:
        raise TensorError(f"query buffer has shape {tuple(q.shape)} for {n} tokens and row stride {q_row_stride}")
    _need(out, "attention output", (n, nq * d), torch.bfloat16)
    _need(positions, "positions", (n,), torch.int32)
    _need(seq_of, "request index of each token", (n,), torch.int32)
    _need(block_table, "block table", None, torch.int32)
    if q_len is not None:
        _need(q_len, "tokens of each request", (block_table.shape[0],), torch.int32)
    for pool, what in ((k_pool, "key pool"), (v_pool, "value pool")):
        _need(pool, what, None, torch.bfloat16)
        if pool.dim() != 2 or pool.shape[1] != nkv * d or pool.shape[0] % block_size != 0:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{block_size}, {nkv * d}]")
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((n * nq * splits * d,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n * nq * splits * 2,), dtype=torch.float32, device=q.device)
    mode, q_gain, k_gain, gain_code, eps, cos, sin, rot = 0, None, None, F32, 0.0, None, None, 0
    if fuse is not None:
        if q_len is not None:
            raise TensorError("the fused norm, rotation and cache write are for steps of one token a request")
        mode = 2 if fuse.write_kv else 1
        q_gain, k_gain, eps, cos, sin, rot = fuse.q_gain, fuse.k_gain, fuse.eps, fuse.cos, fuse.sin, fuse.rot
        if q_gain is not None:
            _need(q_gain, "query norm gain", (d,))
            _need(k_gain, "key norm gain", (d,), q_gain.dtype)
            gain_code = _code(q_gain, "query norm gain")
        if cos is not None:
            _need(cos, "cosine table", None, torch.float32)
            _need(sin, "sine table", tuple(cos.shape), torch.float32)
            if cos.dim() != 2 or cos.shape[1] != rot // 2:
                raise TensorError(f"rotary tables have shape {tuple(cos.shape)}, expected [positions, {rot // 2}]")
        if mode == 2 and q_row_stride != (nq + 2 * nkv) * d:
            raise TensorError(f"rows of {q_row_stride} values are not [q | k | v] of {nq}+2*{nkv} heads of {d}")
    _check(library().pl_paged_attention_decode(
        q.data_ptr(), q_row_stride, out.data_ptr(), _ptr(part_acc), _ptr(part_ml), positions.data_ptr(),
        seq_of.data_ptr(), _ptr(q_len), int(short_limit),
        int(block_table.shape[0] if live_seqs is None else live_seqs), int(short_rows if q_len is not None else 0),
        block_table.data_ptr(), block_table.shape[1], block_size,
        k_pool.data_ptr(), v_pool.data_ptr(), n, nq, nkv, d, float(scale), int(window or 0), int(splits),
        mode, _ptr(q_gain), _ptr(k_gain), gain_code, float(eps), _ptr(cos), _ptr(sin), int(rot), _ptr(sinks),
        _ptr(slopes), _stream()))
    return out


class QkFusion:
    """What turns a raw projection row into queries and keys: the per-head norm's gains and eps, the
    rotation's tables and width, and whether key and value go into the pages."""

    __slots__ = ("q_gain", "k_gain", "eps", "cos", "sin", "rot", "write_kv", "neighbours")

    def __init__(self, q_gain, k_gain, eps: float, cos, sin, rot: int, write_kv: bool, neighbours: bool = False):
        self.q_gain, self.k_gain, self.eps, self.cos, self.sin = q_gain, k_gain, eps, cos, sin
        self.rot, self.write_kv = rot, write_kv
        self.neighbours = neighbours        # the rotation pairs (2 i, 2 i + 1) instead of (i, i + rot/2)


def paged_attention_prefill(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, q_start: torch.Tensor,
                            q_len: torch.Tensor, ctx_len: torch.Tensor, max_q_len: int, block_table: torch.Tensor,
                            block_size: int, k_pool: torch.Tensor, v_pool: torch.Tensor, nq: int, nkv: int, d: int,
                            scale: float, window: int = 0, short_limit: int = 0, max_ctx: int | None = None,
                            splits: int | None = None, live_seqs: int | None = None,
                            sinks: torch.Tensor | None = None, slopes: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 attention of prompt portions on the matrix cores.  Request s brings the rows
    q_start[s] .. q_start[s]+q_len[s]-1 at the positions ctx_len[s]-q_len[s] .. ctx_len[s]-1;
    requests with fewer than ``short_limit`` tokens are skipped.  ``max_ctx`` (the longest context
    of the step) lets the keys of a token tile be dealt to several workgroups where the tiles alone
    would leave compute units idle; ``splits`` sets their number by hand.  ``live_seqs``: only so many
    of the requests, the first ones, bring tokens (the rest is padding and gets no workgroups)."""
    n = q.shape[0]
    S = block_table.shape[0]
    _need(q, "query buffer", None, torch.bfloat16)
    if q.dim() != 2 or q.shape[1] != q_row_stride or q_row_stride < nq * d:
        raise TensorError(f"query buffer has shape {tuple(q.shape)} for row stride {q_row_stride}")
    _need(out, "attention output", (n, nq * d), torch.bfloat16)
    _need(block_table, "block table", None, torch.int32)
    for t, what in ((q_start, "first row of each request"), (q_len, "tokens of each request"),
                    (ctx_len, "context length of each request")):
        _need(t, what, (S,), torch.int32)
    for pool, what in ((k_pool, "key pool"), (v_pool, "value pool")):
        _need(pool, what, None, torch.bfloat16)
        if pool.dim() != 2 or pool.shape[1] != nkv * d or pool.shape[0] % block_size != 0:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{block_size}, {nkv * d}]")
    if not 0 < max_q_len <= n:
        raise TensorError(f"the longest portion is said to have {max_q_len} of the step's {n} tokens")
    live = S if live_seqs is None else int(live_seqs)
    if not 0 < live <= S:
        raise TensorError(f"{live} requests with tokens of {S}")
    if splits is None:
        splits = prefill_splits(live, int(max_q_len), nq, d, int(max_ctx or 0), n, int(short_limit))
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((n * nq * splits * d,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n * nq * splits * 2,), dtype=torch.float32, device=q.device)
    _check(library().pl_paged_attention_prefill(
        q.data_ptr(), q_row_stride, out.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(),
        int(short_limit), live, int(max_q_len), block_table.data_ptr(), block_table.shape[1], block_size,
        k_pool.data_ptr(), v_pool.data_ptr(), nq, nkv, d, float(scale), int(window or 0), int(splits),
        part_acc.data_ptr() if splits > 1 else None, part_ml.data_ptr() if splits > 1 else None, n,
        _ptr(_head_numbers(sinks, "sinks", nq)), _ptr(_head_numbers(slopes, "distance slopes", nq)), _stream()))
    return out


_compute_units = None


def compute_units() -> int:
    global _compute_units
    if _compute_units is None:
        _compute_units = torch.cuda.get_device_properties(torch.cuda.current_device()).multi_processor_count
    return _compute_units


# From this many query heads a key head on, single tokens go to the tiled kernel with a group's heads as
# its rows: the kernel for single tokens multiplies on the vector units, once a query head, and at eight
# heads a key that work, not the memory, bounds it (at four the two are as fast as each other).
GROUPED_FROM = 8


def grouped_applies(nq: int, nkv: int, d: int, block_size: int) -> bool:
    return nq >= GROUPED_FROM * nkv and bool(library().pl_paged_attention_grouped_applies(nq, nkv, d, block_size))


def grouped_splits(tokens: int, nkv: int, max_ctx: int, d: int = 128) -> int:
    """Into how many shares the keys of a token are cut for the grouped kernel: two workgroups a compute
    unit (as many as its LDS holds) if the tokens and key heads alone do not give that many, every share
    two tiles of keys at least.  (Context 4,096 over 8 key heads: 16 tokens take 65 us in four shares and
    67 in two, 8 tokens 39 us in eight shares and 41 in four.)  Heads above 128 leave LDS room for one
    workgroup a compute unit, and that is what their shares fill."""
    base = max(tokens * nkv, 1)
    key_tiles = -(-max(max_ctx, 1) // 64)
    a_unit = 2 if d <= 128 else 1
    return max(1, min(16, key_tiles // 2, -(-a_unit * compute_units() // base)))


def paged_attention_grouped(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, q_start: torch.Tensor,
                            q_len: torch.Tensor, ctx_len: torch.Tensor, max_q_len: int, block_table: torch.Tensor,
                            block_size: int, k_pool: torch.Tensor, v_pool: torch.Tensor, nq: int, nkv: int, d: int,
                            scale: float, window: int = 0, short_limit: int = 0, max_ctx: int | None = None,
                            splits: int | None = None, live_seqs: int | None = None,
                            tokens: int | None = None, sinks: torch.Tensor | None = None,
                            slopes: torch.Tensor | None = None) -> torch.Tensor:
    """bfloat16 attention for single tokens and the tokens of short portions, the query heads of a
    key-head group as the rows of a tile of the tiled kernel.  Arguments as for
    ``paged_attention_prefill``, but requests with ``short_limit`` tokens or more are the ones skipped
    (0: none), and ``max_q_len`` bounds the tokens of those that are served.  ``tokens``: how many
    tokens those requests bring together (for the choice of ``splits``)."""
    n = q.shape[0]
    S = block_table.shape[0]
    _need(q, "query buffer", None, torch.bfloat16)
    if q.dim() != 2 or q.shape[1] != q_row_stride or q_row_stride < nq * d:
        raise TensorError(f"query buffer has shape {tuple(q.shape)} for row stride {q_row_stride}")
    _need(out, "attention output", (n, nq * d), torch.bfloat16)
    _need(block_table, "block table", None, torch.int32)
    for t, what in ((q_start, "first row of each request"), (q_len, "tokens of each request"),
                    (ctx_len, "context length of each request")):
        _need(t, what, (S,), torch.int32)
    for pool, what in ((k_pool, "key pool"), (v_pool, "value pool")):
        _need(pool, what, None, torch.bfloat16)
        if pool.dim() != 2 or pool.shape[1] != nkv * d or pool.shape[0] % block_size != 0:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{block_size}, {nkv * d}]")
    if not 0 < max_q_len <= n:
        raise TensorError(f"the longest portion is said to have {max_q_len} of the step's {n} tokens")
    live = S if live_seqs is None else int(live_seqs)
    if not 0 < live <= S:
        raise TensorError(f"{live} requests with tokens of {S}")
    if splits is None:
        splits = grouped_splits(n if tokens is None else int(tokens), nkv, int(max_ctx or 0), d)
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((n * nq * splits * d,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n * nq * splits * 2,), dtype=torch.float32, device=q.device)
    _check(library().pl_paged_attention_grouped(
        q.data_ptr(), q_row_stride, out.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(),
        int(short_limit), live, int(max_q_len), block_table.data_ptr(), block_table.shape[1], block_size,
        k_pool.data_ptr(), v_pool.data_ptr(), nq, nkv, d, float(scale), int(window or 0), int(splits),
        part_acc.data_ptr() if splits > 1 else None, part_ml.data_ptr() if splits > 1 else None, n, int(tokens or 0),
        _ptr(_head_numbers(sinks, "sinks", nq)), _ptr(_head_numbers(slopes, "distance slopes", nq)), _stream()))
    return out


def prefill_splits(requests: int, max_q_len: int, nq: int, d: int, max_ctx: int, rows: int | None = None,
                   short_limit: int = 0) -> int:
    """Into how many shares the keys of a token tile are cut.  A share more costs a trip of the
    unnormalised outputs through memory (rows * nq * d floats written and read) and one launch;
    it pays where few token tiles stand before a long context, as in a late portion of a long
    prompt.  The shares that make the estimate below smallest are taken: a workgroup spends about
    1.5 us on 64 keys, memory moves about 3 TB/s for this."""
    if max_ctx <= 0:
        return 1
    tile = library().pl_paged_attention_prefill_tile(max_q_len, d)
    base = max(1, -(-max_q_len // tile) * nq * requests)
    key_tiles = -(-max_ctx // 64)
    rows = rows if rows is not None else requests * max_q_len
    # Where the rows cannot fill that many token tiles the kernel deals its workgroups to the tiles there can
    # be; most of those are empty too when the step is one portion beside single tokens, so the portion's
    # own tiles are what is counted.
    served = min(requests, rows // short_limit) if short_limit > 0 else requests
    if (rows + served * (tile - 1)) // tile < -(-max_q_len // tile) * requests:
        base = (rows // tile + 1) * nq
    best, best_cost = 1, None
    for s in (1, 2, 3, 4, 6, 8, 12, 16):
        if s > 1 and key_tiles // s < 4:
            break
        turns = -(-base * s // compute_units())
        cost = turns * -(-key_tiles // s) * 1.5
        if s > 1:
            cost += 3.0 + rows * nq * d * 8.0 * s / 3e6
        if best_cost is None or cost < best_cost:
            best, best_cost = s, cost
    return best


def attention_step(qkv: torch.Tensor, out: torch.Tensor, batch, kv, nq: int, nkv: int, d: int, scale: float,
                   window: int, prepare: QkFusion) -> torch.Tensor:
    """Everything between the fused q/k/v projection and the output projection for the tokens of a step:
    per-head norm and rotation of q and k, the write of k and v into the pages, attention.  A step in
    which every request brings one token (in bfloat16) does all of it in the attention kernel;
    any other step runs the stand-alone kernel for the first three and then attention."""
    if (qkv.dtype == torch.bfloat16 and _attention_mode == "kernel" and batch.max_q_len == 1
            and prepare.rot % 16 == 0 and not prepare.neighbours and not grouped_applies(nq, nkv, d, kv.block_size)):
        splits = decode_splits(batch.num_tokens, nq, nkv, batch.max_ctx_len, d)
        return paged_attention_decode(qkv, qkv.shape[1], out, batch.positions, batch.seq_of, kv.block_table,
                                      kv.block_size, kv.k_pool, kv.v_pool, nq, nkv, d, scale, window, splits,
                                      fuse=prepare)
    qk_norm_rope_kv_write(qkv, prepare.q_gain, prepare.k_gain, prepare.eps, prepare.cos, prepare.sin, prepare.rot,
                          batch.positions, batch.seq_of, kv.block_table, kv.block_size, kv.k_pool, kv.v_pool,
                          nq, nkv, d, write_kv=prepare.write_kv, neighbours=prepare.neighbours)
    return paged_attention(qkv, out, batch, kv, nq, nkv, d, scale, window)


# Up to this many workgroups (requests times query heads) the tiled kernel takes a mixed step's short requests too.
TILED_TAKES_SHORT_WORKGROUPS = 512


def paged_attention(qkv: torch.Tensor, out: torch.Tensor, batch, kv, nq: int, nkv: int, d: int,
                    scale: float, window: int = 0, sinks: torch.Tensor | None = None,
                    slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention for every token of a step.  ``qkv`` rows begin with the rotated queries.
    In bfloat16 the long portions go to the tiled kernel and the tokens of short ones
    (decoded tokens among them) to the kernel for single tokens, or, where many query heads share a key
    head, to the tiled kernel with a group's heads as its rows; all read the same pages."""
    if qkv.dtype != torch.bfloat16 or _attention_mode != "kernel" or d % 16 or d > 256:
        return paged_attention_plain(qkv, qkv.shape[1], out, batch.positions, batch.seq_of, kv.block_table,
                                     kv.block_size, kv.k_pool, kv.v_pool, nq, nkv, d, scale, window,
                                     sinks=sinks, slopes=slopes)
    stride = qkv.shape[1]
    short_tokens = batch.tokens_of_short_requests(SHORT_PORTION)
    if batch.max_q_len >= SHORT_PORTION:
        # A few short requests beside a long portion ride along in the tiled kernel, a token tile each: their
        # workgroups run beside the portion's and finish sooner, which saves the other kernel's launch and
        # its merge.  (Counted by requests, which a step's shape fixes; the tokens of short ones it does not.)
        all_tiled = (short_tokens > 0 and batch.num_seqs * nq <= TILED_TAKES_SHORT_WORKGROUPS
                     and not grouped_applies(nq, nkv, d, kv.block_size))   # (grouped, a token reads its keys once for all its heads)
        paged_attention_prefill(qkv, stride, out, batch.q_start, batch.q_len, batch.ctx_len, batch.max_q_len,
                                kv.block_table, kv.block_size, kv.k_pool, kv.v_pool, nq, nkv, d, scale, window,
                                short_limit=0 if all_tiled else SHORT_PORTION, max_ctx=batch.max_ctx_len,
                                live_seqs=getattr(batch, "live_seqs", None), sinks=sinks, slopes=slopes)
        if short_tokens == 0 or all_tiled:
            return out
    mixed = batch.max_q_len >= SHORT_PORTION
    if grouped_applies(nq, nkv, d, kv.block_size):
        # many query heads a key head: a token's group of heads as the rows of a tile of the tiled kernel
        return paged_attention_grouped(qkv, stride, out, batch.q_start, batch.q_len, batch.ctx_len,
                                       min(batch.max_q_len, SHORT_PORTION - 1), kv.block_table, kv.block_size,
                                       kv.k_pool, kv.v_pool, nq, nkv, d, scale, window,
                                       short_limit=SHORT_PORTION if mixed else 0, max_ctx=batch.max_ctx_len,
                                       live_seqs=getattr(batch, "live_seqs", None), tokens=short_tokens,
                                       sinks=sinks, slopes=slopes)
    splits = decode_splits(short_tokens, nq, nkv, batch.max_ctx_len, d)
    return paged_attention_decode(qkv, stride, out, batch.positions, batch.seq_of, kv.block_table,
                                  kv.block_size, kv.k_pool, kv.v_pool, nq, nkv, d, scale, window, splits,
                                  q_len=batch.q_len if mixed else None, short_limit=SHORT_PORTION if mixed else 0,
                                  live_seqs=getattr(batch, "live_seqs", None), short_rows=short_tokens,
                                  sinks=sinks, slopes=slopes)


class HandedNorm:
    """An RMSNorm handed forward by the product that last added into the stream: that product owns whole
    16-column stripes of the updated stream, so it leaves ``x`` = bfloat16(stream * gain) [n, width] and, for
    every row, the sum of squares over each stripe, ``ssq`` [n, stripes].  The product that stands behind the
    norm then loads ``x`` (half the bytes of the 32-bit stream, nothing to convert or square), adds a row's
    sums in a fixed order and scales its result by 1 / sqrt(sum / width + eps).  ``filled`` says that a
    product has written both."""

    __slots__ = ("gain", "eps", "x", "ssq", "filled")

    def __init__(self, gain: torch.Tensor, eps: float, rows: int, width: int, device):
        self.gain, self.eps = gain, float(eps)
        self.x = torch.empty((rows, width), dtype=torch.bfloat16, device=device)
        self.ssq = torch.empty((rows, (width + 15) // 16), dtype=torch.float32, device=device)
        self.filled = False


# From this many rows on a norm is handed forward.  With fewer the product behind the norm normalises the 32-bit
# stream itself at no cost that shows, and what the adding product does more is not made up for (decode steps of
# the 0.6B shape, handed against not, ms: 1 row 1.103 / 1.080, 4 rows 1.152 / 1.134, 8 rows 1.252 / 1.251, 16 rows
# 1.422 / 1.438, 17 rows 1.547 / 1.721, 32 rows 1.692 / 1.872, 64 rows 2.161 / 2.314).
HAND_FROM_ROWS = 16


def hands_norm_forward(rows: int, columns: int, width: int) -> bool:
    """Whether the product of ``rows`` bfloat16 rows that adds into a stream of ``columns`` hands the next
    norm forward: rows enough that the norm would otherwise be a kernel of its own or a costly first stage,
    against a stream that is not wide (every product behind the norm adds up all of a row's stripes)."""
    return (rows >= HAND_FROM_ROWS and columns <= FUSED_NORM_MAX_WIDTH and skinny_wins(rows, columns, width)
            and bool(library().pl_gemm_skinny_hand_applies(rows, columns, width, 2, 0)))


def takes_handed_norm(rows: int, columns: int, width: int, swiglu: bool = False) -> bool:
    """Whether the product of ``rows`` rows against ``columns`` (outputs) can take a norm handed forward."""
    return (width <= FUSED_NORM_MAX_WIDTH and columns <= FUSED_NORM_MAX_COLUMNS
            and skinny_wins(rows, columns * (2 if swiglu else 1), width)
            and bool(library().pl_gemm_skinny_hand_applies(rows, columns, width, 1 if swiglu else 0, 1)))


def weights_in_strips(w: torch.Tensor) -> torch.Tensor | None:
    """The bfloat16 weights ``w`` [N, K] again, in the order the waves of ``gemm_skinny`` take them: strips of 16
    rows, a strip a run of K/32 tiles of 1 KB, a tile stored as [4 groups of 8 elements][16 rows][8 elements], so
    that a wave's stretch of K of a strip is one contiguous stretch of memory, which the memory serves faster
    than 64 bytes from each of 16 rows that lie K elements apart.  The result has the shape of ``w`` and is
    read by ``gemm_skinny(..., strips=...)`` only.  None where the layout is not defined: rows that are no
    multiple of 16, a K that is no multiple of 32."""
    if w.dim() != 2 or w.dtype != torch.bfloat16 or not w.is_cuda:
        return None
    N, K = w.shape
    if N % 16 or K % 32:
        return None
    return w.view(N // 16, 16, K // 32, 4, 8).permute(0, 2, 3, 1, 4).contiguous().view(N, K)


def strips_apply(rows: int, columns: int, width: int) -> bool:
    """Whether ``gemm_skinny`` of so many rows, with ``columns`` columns of output over an inner width of ``width``,
    reads weights in strips: its kernel for one tile of 16 rows does (up to 16 rows, and beyond where the tiles of
    rows go to workgroups of their own)."""
    return bool(library().pl_gemm_skinny_strips_apply(rows, columns, width))


def gemm_skinny(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, swiglu: bool = False,
                norm_gain: torch.Tensor | None = None, eps: float = 0.0, rows: torch.Tensor | None = None,
                add_into: torch.Tensor | None = None, activation: str = "silu",
                handed: "HandedNorm | None" = None, hand: "HandedNorm | None" = None,
                strips: torch.Tensor | None = None) -> torch.Tensor:
    """y = x . w^T for up to 64 rows on the matrix cores, the bfloat16 weights streamed once.

    ``x`` is bfloat16 [n, K]; or, with ``norm_gain``, the 32-bit residual stream, whose rows
    (``rows[i]`` for output row i when a row list is given) are RMS-normalised on the way in.
    With ``swiglu`` the rows of ``w`` are [gate | up] and y = act(x . gate^T) * (x . up^T), in bfloat16
    (``activation``: silu or a gelu).
    With ``add_into`` (the 32-bit residual stream, [n, N]) the result is added there and that
    tensor is returned.
    ``handed``: a norm that an earlier product left behind; its rows are the input (``x`` is not looked at)
    and its sums of squares scale the result.  ``hand`` (with ``add_into``): the norm that follows the
    stream is left behind in it.
    ``strips``: what ``weights_in_strips`` made of ``w``; read instead of ``w`` where ``strips_apply`` says so."""
    if handed is not None:
        if norm_gain is not None or not handed.filled:
            raise TensorError("a handed norm is the product's input by itself, once a product has written it")
        x = handed.x
    K = x.shape[1]
    if norm_gain is None:
        _need(x, "matrix product input", None, torch.bfloat16)
        n = x.shape[0]
        if rows is not None:
            raise TensorError("a row list goes with a norm")
    else:
        _need(x, "residual stream", None, torch.float32)
        _need(norm_gain, "norm gain", (K,), torch.float32)
        n = x.shape[0] if rows is None else rows.numel()
        if rows is not None:
            _need(rows, "row list", (n,), torch.int32)
    _need(w, "weight", None, torch.bfloat16)
    if x.dim() != 2 or w.dim() != 2 or w.shape[1] != K:
        raise TensorError(f"weight has shape {tuple(w.shape)} for an input of shape {tuple(x.shape)}")
    N_out = w.shape[0] // 2 if swiglu else w.shape[0]
    if swiglu and w.shape[0] % 2:
        raise TensorError(f"fused gate/up weight has an odd number of rows, {w.shape[0]}")
    if add_into is not None:
        if swiglu or norm_gain is not None:
            raise TensorError("a product that adds into the residual stream has a plain input and no activation")
        _need(add_into, "residual stream", (n, N_out), torch.float32)
        out, epilogue, out_f32 = add_into, 2, 1
    else:
        if out_dtype not in (torch.bfloat16, torch.float32) or (swiglu and out_dtype != torch.bfloat16):
            raise TensorError(f"matrix product output {out_dtype}" + (" after the activation" if swiglu else ""))
        out = torch.empty((n, N_out), dtype=out_dtype, device=x.device)
        epilogue, out_f32 = (1 if swiglu else 0), (1 if out_dtype == torch.float32 else 0)
    in_strips = 0
    if strips is not None and library().pl_gemm_skinny_strips_apply(n, N_out, K):
        _need(strips, "weights in strips", tuple(w.shape), torch.bfloat16)
        w, in_strips = strips, 1
    if handed is not None or hand is not None:
        if hand is not None:
            if add_into is None:
                raise TensorError("a norm is handed forward by a product that adds into the stream")
            _need(hand.gain, "gain of the norm handed forward", (N_out,), torch.float32)
            _need(hand.x, "rows of the norm handed forward", (n, N_out), torch.bfloat16)
            _need(hand.ssq, "sums of squares of the norm handed forward", (n, (N_out + 15) // 16), torch.float32)
        if handed is not None:
            _need(handed.ssq, "sums of squares of the handed norm", (n, (K + 15) // 16), torch.float32)
        _check(library().pl_gemm_skinny_hand(
            x.data_ptr(), w.data_ptr(), out.data_ptr(), n, N_out, K, epilogue, out_f32, activation_code(activation),
            _ptr(handed.ssq if handed is not None else None), handed.ssq.shape[1] if handed is not None else 0,
            float(handed.eps if handed is not None else 0.0),
            _ptr(hand.gain if hand is not None else None), _ptr(hand.x if hand is not None else None),
            _ptr(hand.ssq if hand is not None else None), in_strips, _stream()))
        if hand is not None:
            hand.filled = True
        return out
    _check(library().pl_gemm_skinny(
        x.data_ptr(), w.data_ptr(), out.data_ptr(), _ptr(norm_gain), float(eps), _ptr(rows), n, N_out, K,
        epilogue, out_f32, activation_code(activation), in_strips, _stream()))
    return out


# Where the hand-written product beats the library's on this chip (both timed over weights that come from
# memory, not from a cache).  It streams a weight matrix of up to a few tens of megabytes faster than
# the library starts, and fuses what stands before and after the product; a larger matrix the library
# streams at a higher rate, except a very deep one (K several times N), which it cuts badly.  With more
# than 16 rows the rows of x no longer stay in a wave's registers and only a shallow product is worth it.
SKINNY_WEIGHT_BYTES = 48 << 20
SKINNY_DEEP = 4
SKINNY_SHALLOW_K = 2048
SKINNY_ROW_TILES_GRID = 512  # column tiles times row tiles up to which the rows are dealt to workgroups too ...
SKINNY_ROW_TILES_BYTES = 16 << 20   # ... for weights up to this size (4,096 x 4,096 at 32 rows: 19.8 us against the library's 14.0)
SKINNY_F32_FEW_K = 4096     # the widest stream whose projection onto a large vocabulary it wins, up to 16 rows
# Over weights in strips, up to 8 rows and a K that sixteen waves cover in one round of loads, it also wins larger
# matrices (24,576 x 4,096 at 8 rows: 42.6 us against the library's 44 to 46; 10,240 x 5,120: 29.8 against 23.4).
SKINNY_STRIPS_ROWS = 8
SKINNY_STRIPS_K = 4096
SKINNY_STRIPS_BYTES = 256 << 20


def skinny_wins(rows: int, weight_rows: int, width: int, strips: bool = False) -> bool:
    """``strips``: the weights are there in strips as well (``weights_in_strips``)."""
    if not 0 < rows <= SKINNY_ROWS or width % 8 or stream_wins(rows, weight_rows, width):
        return False
    if rows <= 16:
        if (strips and rows <= SKINNY_STRIPS_ROWS and width <= SKINNY_STRIPS_K
                and weight_rows * width * 2 <= SKINNY_STRIPS_BYTES):
            return True
        return weight_rows * width * 2 <= SKINNY_WEIGHT_BYTES or width >= SKINNY_DEEP * weight_rows
    # ... or a narrow output, whose tiles of 16 rows go to workgroups of their own (the kernel for up to 16 rows)
    return width <= SKINNY_SHALLOW_K or ((weight_rows // 16) * -(-rows // 16) <= SKINNY_ROW_TILES_GRID
                                         and weight_rows * width * 2 <= SKINNY_ROW_TILES_BYTES)


def gemm_tiled_applies(rows: int, columns: int, width: int, swiglu: bool = False, add: bool = False) -> bool:
    return bool(library().pl_gemm_tiled_applies(rows, columns, width, 1 if swiglu else (2 if add else 0)))


# The tiled product reads LDS once a matrix instruction (a wave's tile is 64 x 64) and levels off at about
# 0.7 PFLOP/s, below the library's best; what it saves is the trip of gate and up through memory and a
# launch.  That wins for the gated feed-forward of a narrow model in portions of a prompt (512 rows of
# width 1,024: 12.6 us against 20 for product plus activation; 2,048 rows: 38 against 39, no better inside
# a step), and loses from a width of 4,096 on, as do the plain and the adding product at every size measured.
TILED_SWIGLU_MAX_ROWS = 1024
TILED_SWIGLU_MAX_WIDTH = 2048


def tiled_swiglu_wins(rows: int, columns: int, width: int) -> bool:
    return (SKINNY_ROWS < rows <= TILED_SWIGLU_MAX_ROWS and width <= TILED_SWIGLU_MAX_WIDTH
            and gemm_tiled_applies(rows, columns, width, swiglu=True))


def gemm_tiled(x: torch.Tensor, w: torch.Tensor, swiglu: bool = False, add_into: torch.Tensor | None = None,
               activation: str = "silu") -> torch.Tensor:
    """y = x . w^T for many rows of bfloat16 on the matrix cores, 32-bit sums, with SwiGLU (``w`` is
    [gate | up] stacked, silu(gate) * up comes back) or the sum into the 32-bit residual stream
    (``add_into``, which is returned) as the product's last stage."""
    _need(x, "matrix product input", None, torch.bfloat16)
    _need(w, "weight", None, torch.bfloat16)
    if x.dim() != 2 or w.dim() != 2 or w.shape[1] != x.shape[1]:
        raise TensorError(f"weight has shape {tuple(w.shape)} for an input of shape {tuple(x.shape)}")
    M, K = x.shape
    if swiglu and (w.shape[0] % 2 or add_into is not None):
        raise TensorError("the activation needs an even number of weight rows and is not added into the stream")
    N = w.shape[0] // 2 if swiglu else w.shape[0]
    if add_into is not None:
        _need(add_into, "residual stream", (M, N), torch.float32)
        out, epilogue = add_into, 2
    else:
        out, epilogue = torch.empty((M, N), dtype=torch.bfloat16, device=x.device), (1 if swiglu else 0)
    _check(library().pl_gemm_tiled(x.data_ptr(), w.data_ptr(), out.data_ptr(), M, N, K, epilogue,
                                   activation_code(activation), _stream()))
    return out


STREAM_ROWS = 64
# Where the streamed product beats both the library and the skinny kernel (each timed over weights from
# memory, at 8 to 64 rows).  The library cuts a deep product over few columns badly (5,120 x 25,600 at 64
# rows: 158 us against 67 here), and from 17 rows on it is slower over very many columns of a narrow stream
# (the vocabulary of 151,936 over a width of 1,024, 32-bit out, 17 to 64 rows: 74 to 84 us against 62 to
# 77; over widths of 4,096 and 5,120 the two are within a tenth of each other, either way, and the
# library keeps them).  A wide product of moderate depth (51,200 x 5,120) stays the
# library's: its columns give too few workgroups for an even share a compute unit, and cutting K there
# costs more in partial results than it gains.
STREAM_DEEP = 1.5            # K / N from which the product counts as deep, with more than 16 rows
STREAM_VERY_DEEP = 4.0       # the same for up to 16 rows (below it the library is the fastest of the three)
STREAM_WEIGHT_BYTES = 48 << 20
STREAM_MANY_COLUMNS = 131072
STREAM_NARROW_WIDTH = 2048


def stream_wins(rows: int, weight_rows: int, width: int) -> bool:
    if not 0 < rows <= STREAM_ROWS or width % 8 or weight_rows * width * 2 < STREAM_WEIGHT_BYTES:
        return False
    if rows <= 16:
        return width >= STREAM_VERY_DEEP * weight_rows
    return width >= STREAM_DEEP * weight_rows or (weight_rows >= STREAM_MANY_COLUMNS and width <= STREAM_NARROW_WIDTH)


def gemm_stream(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype = torch.bfloat16, swiglu: bool = False,
                add_into: torch.Tensor | None = None, activation: str = "silu",
                splits: int | None = None) -> torch.Tensor:
    """y = x . w^T for up to 64 rows of bfloat16 over a large weight matrix: a workgroup owns 128 rows
    of ``w`` and a stretch of K, its waves take their weights from memory straight into registers, a chunk
    ahead, and share the rows of ``x`` through LDS.  ``swiglu``: ``w`` is [gate | up] stacked and
    act(gate) * up comes back.  ``add_into``: the 32-bit residual stream takes the sum and is returned.
    ``splits``: into how many stretches K is cut between workgroups (chosen here when not given); with
    more than one, a second kernel adds the partial results in a fixed order."""
    _need(x, "matrix product input", None, torch.bfloat16)
    _need(w, "weight", None, torch.bfloat16)
    if x.dim() != 2 or w.dim() != 2 or w.shape[1] != x.shape[1]:
        raise TensorError(f"weight has shape {tuple(w.shape)} for an input of shape {tuple(x.shape)}")
    n, K = x.shape
    if swiglu and (w.shape[0] % 2 or add_into is not None):
        raise TensorError("the activation needs an even number of weight rows and is not added into the stream")
    N_out = w.shape[0] // 2 if swiglu else w.shape[0]
    if add_into is not None:
        _need(add_into, "residual stream", (n, N_out), torch.float32)
        out, epilogue, out_f32 = add_into, 2, 1
    else:
        if out_dtype not in (torch.bfloat16, torch.float32) or (swiglu and out_dtype != torch.bfloat16):
            raise TensorError(f"matrix product output {out_dtype}" + (" after the activation" if swiglu else ""))
        out = torch.empty((n, N_out), dtype=out_dtype, device=x.device)
        epilogue, out_f32 = (1 if swiglu else 0), (1 if out_dtype == torch.float32 else 0)
    lib = library()
    if splits is None:
        splits = lib.pl_gemm_stream_splits(n, N_out, K, 1 if swiglu else 0)
    workspace = torch.empty((splits * n * w.shape[0],), dtype=torch.float32, device=x.device) if splits > 1 else None
    _check(lib.pl_gemm_stream(x.data_ptr(), w.data_ptr(), out.data_ptr(), _ptr(workspace), n, N_out, K, epilogue,
                              out_f32, activation_code(activation), int(splits), _stream()))
    return out


# A deep product of some hundred rows the library runs as one workgroup a tile of the output, each walking
# all of K: with few tiles (a projection back to the width of the model) most of the chip idles.  The same
# product as a batch of stretches of K (strided views of x and w, no copies; 32-bit partial results) fills
# it, and the kernel that ends the streamed product adds the parts in their order and stores them or adds
# them into the stream.  Measured over weights from memory: 4,096 x 12,288 at 576 rows 102 us whole, 62 in
# four stretches (and 6 for the sum); 5,120 x 25,600 at 576 rows 270 against 150 in two, at 1,088 rows 428
# against 237; at 2,048 rows nothing is gained, and neither for small matrices (1,024 x 3,072), where the
# second kernel costs what the stretches save.
SPLIT_DEEP = 2.5             # K / N from which it pays
SPLIT_MAX_ROWS = 1280
SPLIT_WEIGHT_BYTES = 48 << 20


def library_splits(rows: int, weight_rows: int, width: int) -> int:
    """Into how many stretches of K the library's product of this shape is cut (1: not at all)."""
    if (rows <= STREAM_ROWS or rows > SPLIT_MAX_ROWS or width < SPLIT_DEEP * weight_rows
            or weight_rows * width * 2 < SPLIT_WEIGHT_BYTES):
        return 1
    for splits in ((4, 2) if rows <= 640 else (2,)):
        if width % (8 * splits) == 0:
            return splits
    return 1


def gemm_split_library(x: torch.Tensor, w: torch.Tensor, splits: int, out_dtype: torch.dtype = torch.bfloat16,
                       add_into: torch.Tensor | None = None) -> torch.Tensor:
    """y = x . w^T as ``splits`` products over stretches of K, run by the library as one batch, and their sum in
    a fixed order: stored, or added into the 32-bit residual stream ``add_into`` (which is returned)."""
    _need(x, "matrix product input", None, torch.bfloat16)
    _need(w, "weight", None, torch.bfloat16)
    if x.dim() != 2 or w.dim() != 2 or w.shape[1] != x.shape[1]:
        raise TensorError(f"weight has shape {tuple(w.shape)} for an input of shape {tuple(x.shape)}")
    M, K = x.shape
    N = w.shape[0]
    if splits < 2 or K % (8 * splits):
        raise TensorError(f"a width of {K} in {splits} stretches")
    part = K // splits
    partial = torch.bmm(x.view(M, splits, part).transpose(0, 1), w.view(N, splits, part).permute(1, 2, 0),
                        out_dtype=torch.float32)
    if add_into is not None:
        _need(add_into, "residual stream", (M, N), torch.float32)
        out, epilogue, out_f32 = add_into, 2, 1
    else:
        if out_dtype not in (torch.bfloat16, torch.float32):
            raise TensorError(f"matrix product output {out_dtype}")
        out = torch.empty((M, N), dtype=out_dtype, device=x.device)
        epilogue, out_f32 = 0, (1 if out_dtype == torch.float32 else 0)
    _check(library().pl_gemm_finish(partial.data_ptr(), out.data_ptr(), M, N, splits, epilogue, out_f32,
                                    activation_code("silu"), _stream()))
    return out


def skinny_applies(x: torch.Tensor, w: torch.Tensor | None = None, strips: bool = False) -> bool:
    """Whether the product of ``x`` goes to the hand-written kernel: whether it can, and, given the
    weight (and whether it is there in strips as well), whether it is the faster of the two."""
    if x.dtype != torch.bfloat16 or x.shape[0] > SKINNY_ROWS or x.shape[1] % 8:
        return False
    return w is None or skinny_wins(x.shape[0], w.shape[0], x.shape[1], strips)


# A product with more columns than this walks its column tiles in a loop; the norm as its first stage
# then costs the registers that keep enough waves resident, and a norm kernel of its own is cheaper.
FUSED_NORM_MAX_COLUMNS = 32768
# The norm as the product's first stage is done again by every workgroup; beyond this width a norm kernel
# of its own, once, is cheaper.
FUSED_NORM_MAX_WIDTH = 2048


# ... and every workgroup reads the rows of the 32-bit stream, twice the bytes of normalised bfloat16 rows, and
# converts them; beyond this many rows a norm kernel of its own is cheaper (64 rows of width 1,024 against
# 4,096 columns: 12.1 us fused, 11.0 apart; against 6,144 with SwiGLU: 14.3 and 12.6).
FUSED_NORM_MAX_ROWS = 32


def fused_norm_applies(rows_out: int, width: int, weight: torch.Tensor) -> bool:
    """Whether norm and product run as one kernel: few rows of a bfloat16 model, a stream that is not wide."""
    return (weight.dtype == torch.bfloat16 and width <= FUSED_NORM_MAX_WIDTH and rows_out <= FUSED_NORM_MAX_ROWS
            and skinny_wins(rows_out, weight.shape[0], width))


def linear_bf16(x: torch.Tensor, w: torch.Tensor, out_dtype: torch.dtype,
                strips: torch.Tensor | None = None) -> torch.Tensor:
    """y = x . w^T for bfloat16 operands with 32-bit accumulation: few rows stream the
    weights through the hand-written kernel, many rows go to the library's product.
    ``strips``: the weights again as ``weights_in_strips`` lays them out, for the product that reads them so."""
    _need(x, "matrix product input", None, torch.bfloat16)
    _need(w, "weight", None, torch.bfloat16)
    if out_dtype == torch.float32:
        # the projection onto the vocabulary: 32-bit out of the 32-bit sums, from either product
        if stream_wins(x.shape[0], w.shape[0], x.shape[1]):
            return gemm_stream(x, w, torch.float32)
        if skinny_applies(x) and x.shape[1] <= (SKINNY_F32_FEW_K if x.shape[0] <= 16 else SKINNY_SHALLOW_K):
            return gemm_skinny(x, w, torch.float32, strips=strips)
        if x.shape[1] % 8 == 0:
            return torch.mm(x, w.t(), out_dtype=torch.float32)
        return gemm_plain(x, w, out_dtype=torch.float32)
    if skinny_applies(x, w):
        return gemm_skinny(x, w, out_dtype, strips=strips)
    if stream_wins(x.shape[0], w.shape[0], x.shape[1]):
        return gemm_stream(x, w, out_dtype)
    splits = library_splits(x.shape[0], w.shape[0], x.shape[1])
    if splits > 1:
        return gemm_split_library(x, w, splits, out_dtype)
    return torch.mm(x, w.t())


# ---------------------------------------------------------------------------
# Mixers with a carried state, short convolutions, and the layer that normalises a sublayer's output

SCAN_KINDS = {"lightning": 0, "mlstm": 1, "delta": 2}
SCAN_MAX_DIM = 256
# A request that brings at least this many tokens to a step goes through the chunked kernels, where its mixer has
# them (64 tokens at once instead of one after the other); the others, single tokens among them, go token by token.
SCAN_CHUNKED_FROM = 16


def _state_view(state: torch.Tensor, what: str):
    """(tensor, floats between two slots): a [slots, floats] 32-bit state, possibly a run of columns of a wider one."""
    if not isinstance(state, torch.Tensor) or not state.is_cuda or state.dtype != torch.float32 or state.dim() != 2 \
            or (state.shape[1] > 0 and state.stride(1) != 1):
        raise TensorError(f"{what} is not a 32-bit [slots, floats] tensor on the GPU with unit stride along a slot")
    return state, state.stride(0)


def _step_rows(batch, n: int):
    for t, what, count in ((batch.q_start, "first rows", batch.num_seqs), (batch.q_len, "row counts", batch.num_seqs),
                           (batch.state_slots, "state slots", batch.num_seqs), (batch.positions, "positions", n),
                           (batch.seq_of, "request index of each token", n)):
        _need(t, what, (count,), torch.int32)


def scan_state_floats(kind: str, heads: int, dim: int, vdim: int) -> int:
    """32-bit floats a request's state takes: the matrices S [heads, dim, vdim]; for ``mlstm`` also the normaliser n
    and the running maximum m, a copy of each for every tile of 64 columns of vdim (the waves of a head's tiles
    run on their own and keep equal copies): n [heads, tiles, dim], m [heads, tiles]."""
    tiles = (vdim + 63) // 64
    return heads * dim * vdim + (heads * tiles * (dim + 1) if kind == "mlstm" else 0)


def recurrent_scan(kind: str, qkv: torch.Tensor, q_off: int, k_off: int, v_off: int, state: torch.Tensor,
                   batch, heads: int, qk_heads: int, dim: int, vdim: int, *, gates: torch.Tensor | None = None,
                   g1_off: int = 0, g2_off: int = 0, p1: torch.Tensor | None = None, p2: torch.Tensor | None = None,
                   cap: float = 0.0, out: torch.Tensor | None = None, chunked: bool = False) -> torch.Tensor:
    """The read-out [rows, heads * vdim] (32-bit) of a mixer that carries a [dim, vdim] matrix a head from
    token to token, over the tokens of a step, request by request, from and into the requests' state slots.

    ``lightning``: S = decay S + silu(k) silu(v)^T, o = S^T silu(q); ``p1`` = the decays.
    ``mlstm``: log gates i = cap tanh((x1 + b_i)/cap), f = logsigmoid(cap tanh((x2 + b_f)/cap)) from the two
    gate columns a head, a running maximum m, S and a normaliser n; ``p1``, ``p2`` = the biases; the state a
    slot is laid out as ``scan_state_floats`` says.
    ``delta``: ``qkv`` holds convolved and activated rows; q and k become unit vectors, beta = sigmoid(x1),
    decay = exp(-exp(A_log) softplus(x2 + dt_bias)); ``p1`` = A_log, ``p2`` = dt_bias.
    q and k have ``qk_heads`` heads (head h of v reads head h / (heads / qk_heads)).
    ``chunked`` (lightning only with decays above zero): requests that bring ``SCAN_CHUNKED_FROM`` tokens or more
    are computed in chunks of tokens, the same sums in another order."""
    if kind not in SCAN_KINDS:
        raise TensorError(f"a scan of kind {kind!r}, the kernels know {', '.join(SCAN_KINDS)}")
    n = qkv.shape[0]
    _need(qkv, "rows of q, k and v", None, torch.float32)
    if qkv.dim() != 2:
        raise TensorError(f"rows of q, k and v of shape {tuple(qkv.shape)}")
    width = qkv.shape[1]
    if not (0 <= q_off and q_off + qk_heads * dim <= width and 0 <= k_off and k_off + qk_heads * dim <= width
            and 0 <= v_off and v_off + heads * vdim <= width):
        raise TensorError(f"q, k, v at columns {q_off}, {k_off}, {v_off} of rows of {width}")
    if heads < 1 or qk_heads < 1 or heads % qk_heads or not 1 <= dim <= SCAN_MAX_DIM or vdim < 1:
        raise TensorError(f"a scan over {heads} heads ({qk_heads} of q and k) of {dim} by {vdim}")
    state, stride = _state_view(state, "the state")
    tiles = (vdim + 63) // 64
    need = scan_state_floats(kind, heads, dim, vdim)
    if state.shape[1] != need:
        raise TensorError(f"a state of {state.shape[1]} floats a slot, this mixer keeps {need}")
    _step_rows(batch, n)
    if kind != "lightning":
        _need(gates, "rows of the gates", None, torch.float32)
        if gates.dim() != 2 or gates.shape[0] != n or not (0 <= g1_off and g1_off + heads <= gates.shape[1]
                                                         and 0 <= g2_off and g2_off + heads <= gates.shape[1]):
            raise TensorError(f"gates at columns {g1_off}, {g2_off} of rows of shape {tuple(gates.shape)}")
        _need(p2, "second gate constant", (heads,), torch.float32)
    _need(p1, "decays" if kind == "lightning" else "first gate constant", (heads,), torch.float32)
    if out is None:
        out = torch.empty((n, heads * vdim), dtype=torch.float32, device=qkv.device)
    _need(out, "read-out", (n, heads * vdim), torch.float32)
    hdv = heads * dim * vdim
    chunked = bool(chunked) and batch.max_q_len >= SCAN_CHUNKED_FROM
    common = (SCAN_KINDS[kind], qkv.data_ptr(), width, q_off, k_off, v_off, _ptr(gates),
              0 if gates is None else gates.shape[1], g1_off, g2_off, _ptr(p1), _ptr(p2), float(cap),
              state.data_ptr(), stride, 0, hdv, hdv + heads * tiles * dim, out.data_ptr(), batch.q_start.data_ptr(),
              batch.q_len.data_ptr(), batch.state_slots.data_ptr(), batch.num_seqs)
    _check(library().pl_recurrent_scan(*common, heads, qk_heads, dim, vdim, SCAN_CHUNKED_FROM if chunked else 0, _stream()))
    if chunked and kind == "delta":
        tokens = library().pl_recurrent_chunk_tokens(dim)
        chunks = (n // tokens + batch.num_seqs + 1) * heads
        f32 = dict(dtype=torch.float32, device=qkv.device)
        padded = (dim + 3) // 4 * 4
        unit_k, unit_q = torch.empty((chunks, tokens * padded), **f32), torch.empty((chunks, tokens * padded), **f32)
        inverse, masked = torch.empty((chunks, tokens * tokens), **f32), torch.empty((chunks, tokens * tokens), **f32)
        scalars = torch.empty((chunks, 3 * tokens), **f32)
        _check(library().pl_delta_chunked(
            qkv.data_ptr(), width, q_off, k_off, v_off, gates.data_ptr(), gates.shape[1], g1_off, g2_off,
            p1.data_ptr(), p2.data_ptr(), state.data_ptr(), stride, out.data_ptr(), batch.q_start.data_ptr(),
            batch.q_len.data_ptr(), batch.state_slots.data_ptr(), batch.num_seqs, batch.max_q_len, heads, qk_heads, dim,
            vdim, SCAN_CHUNKED_FROM, unit_k.data_ptr(), unit_q.data_ptr(), inverse.data_ptr(), masked.data_ptr(),
            scalars.data_ptr(), _stream()))
    elif chunked:
        chunks = n // library().pl_recurrent_chunk_tokens(dim) + batch.num_seqs + 1
        f32 = dict(dtype=torch.float32, device=qkv.device)
        sums, before = torch.empty((chunks, hdv), **f32), torch.empty((chunks, hdv), **f32)
        k_sums, n_before = (torch.empty((chunks, heads * dim), **f32), torch.empty((chunks, heads * dim), **f32)) \
            if kind == "mlstm" else (None, None)
        scalars = torch.empty((chunks, heads * 4), **f32)
        _check(library().pl_recurrent_chunked(*common, batch.max_q_len, heads, dim, vdim, SCAN_CHUNKED_FROM,
                                              sums.data_ptr(), _ptr(k_sums), before.data_ptr(), _ptr(n_before),
                                              scalars.data_ptr(), _stream()))
    return out


def _conv_args(rows, off, weight, history, batch):
    n = rows.shape[0]
    _need(rows, "projected rows", None, torch.float32)
    _need(weight, "convolution filters", None, torch.float32)
    if rows.dim() != 2 or weight.dim() != 2:
        raise TensorError(f"rows of shape {tuple(rows.shape)}, filters of shape {tuple(weight.shape)}")
    taps, channels = weight.shape
    if not 1 <= taps <= 16 or off < 0 or off + channels > rows.shape[1]:
        raise TensorError(f"{channels} channels of {taps} taps from column {off} of rows of {rows.shape[1]}")
    history, stride = _state_view(history, "the convolution's history")
    if history.shape[1] != (taps - 1) * channels:
        raise TensorError(f"a history of {history.shape[1]} floats a slot for {taps} taps over {channels} channels")
    _step_rows(batch, n)
    return n, channels, taps, history, stride


def short_conv(rows: torch.Tensor, off: int, weight: torch.Tensor, history: torch.Tensor, batch,
               silu: bool = False, out: torch.Tensor | None = None) -> torch.Tensor:
    """y[t, c] = sum_j weight[j, c] * u[t - taps + 1 + j, c] over the columns [off, off + channels) of
    ``rows`` (``weight`` is [taps, channels]: a checkpoint's [channels, taps] transposed, so that neighbouring
    channels' values of a tap are neighbours in memory); the rows before a request's first of this step come from ``history`` [slots, (taps-1) * channels]
    (newest last, zeros at a request's start), which is left as it is: ``conv_history`` moves it afterwards."""
    n, channels, taps, history, stride = _conv_args(rows, off, weight, history, batch)
    if out is None:
        out = torch.empty((n, channels), dtype=torch.float32, device=rows.device)
    _need(out, "convolved rows", (n, channels), torch.float32)
    _check(library().pl_short_conv(rows.data_ptr(), rows.shape[1], off, channels, weight.data_ptr(), taps,
                                   history.data_ptr(), stride, 0, batch.positions.data_ptr(), batch.seq_of.data_ptr(),
                                   batch.q_start.data_ptr(), batch.state_slots.data_ptr(), out.data_ptr(),
                                   1 if silu else 0, n, _stream()))
    return out


def conv_history(rows: torch.Tensor, off: int, weight: torch.Tensor, history: torch.Tensor, batch) -> None:
    """The history becomes the last taps - 1 inputs of every request of the step."""
    n, channels, taps, history, stride = _conv_args(rows, off, weight, history, batch)
    _check(library().pl_conv_history(rows.data_ptr(), rows.shape[1], off, channels, taps, history.data_ptr(), stride, 0,
                                     batch.q_start.data_ptr(), batch.q_len.data_ptr(), batch.state_slots.data_ptr(),
                                     batch.num_seqs, _stream()))


GATES = {None: -1, "sigmoid": 0, "silu": 1}


def gated_group_norm(x: torch.Tensor, group: int, gain: torch.Tensor, eps: float, out_dtype: torch.dtype,
                     gate: torch.Tensor | None = None, gate_off: int = 0, gate_act: str | None = None) -> torch.Tensor:
    """x / sqrt(mean over each run of ``group`` columns of x^2 + eps) * gain * act(gate); ``gain`` has a value a
    column or a value a column of a group; ``gate`` are the columns from ``gate_off`` of 32-bit rows."""
    n, width = x.shape
    _need(x, "read-out", None, torch.float32)
    _need(gain, "gain of the grouped norm", None, torch.float32)
    if group < 1 or width % group or gain.numel() not in (group, width):
        raise TensorError(f"rows of {width} in groups of {group} with {gain.numel()} gains")
    if gate_act not in GATES or (gate_act is None) != (gate is None):
        raise TensorError(f"a gate through {gate_act!r}")
    if gate is not None:
        _need(gate, "rows of the gate", None, torch.float32)
        if gate.dim() != 2 or gate.shape[0] != n or gate_off < 0 or gate_off + width > gate.shape[1]:
            raise TensorError(f"a gate at column {gate_off} of rows of shape {tuple(gate.shape)}")
    out = torch.empty((n, width), dtype=out_dtype, device=x.device)
    _check(library().pl_gated_group_norm(x.data_ptr(), n, width, group, gain.data_ptr(), gain.numel(), float(eps),
                                         _ptr(gate), 0 if gate is None else gate.shape[1], gate_off, GATES[gate_act],
                                         out.data_ptr(), _code(out, "normalised read-out"), _stream()))
    return out


def conv_qk_prepare(rows: torch.Tensor, off: int, weight: torch.Tensor, history: torch.Tensor, q_gain, k_gain,
                    eps: float, freq, rot: int, batch, kv, heads: int, kv_heads: int, dim: int, vdim: int,
                    padded: int, q_out: torch.Tensor) -> torch.Tensor:
    """For an attention layer with short convolutions: convolution of the projected q | k | v columns, norm a
    head of q and k, rotation of the first ``rot`` values of a head by position * freq, q into ``q_out``
    [rows, heads * padded] and k, v into the pages, every head in a row of ``padded`` values."""
    n, channels, taps, history, stride = _conv_args(rows, off, weight, history, batch)
    if channels != heads * dim + kv_heads * dim + kv_heads * vdim:
        raise TensorError(f"{channels} channels for {heads} heads and {kv_heads} key heads of {dim} and {vdim}")
    _need(q_gain, "query norm gain", (dim,), torch.float32)
    _need(k_gain, "key norm gain", (dim,), torch.float32)
    if rot:
        _need(freq, "rotation frequencies", (rot // 2,), torch.float32)
    if rot < 0 or rot % 2 or rot > dim or not max(dim, vdim) <= padded <= 256:
        raise TensorError(f"a rotation over {rot} of {dim} values, heads in rows of {padded}")
    _need(q_out, "query buffer", (n, heads * padded))
    for pool, what in ((kv.k_pool, "key pool"), (kv.v_pool, "value pool")):
        _need(pool, what, None, q_out.dtype)
        if pool.dim() != 2 or pool.shape[1] != kv_heads * padded or pool.shape[0] % kv.block_size:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{kv.block_size}, {kv_heads * padded}]")
    _need(kv.block_table, "block table", None, torch.int32)
    if kv.block_table.dim() != 2 or kv.block_table.shape[0] != batch.num_seqs:
        raise TensorError(f"block table has shape {tuple(kv.block_table.shape)} for {batch.num_seqs} requests")
    _check(library().pl_conv_qk_prepare(
        rows.data_ptr(), rows.shape[1], off, weight.data_ptr(), taps, history.data_ptr(), stride, 0,
        q_gain.data_ptr(), k_gain.data_ptr(), float(eps), _ptr(freq) if rot else 0, rot,
        batch.positions.data_ptr(), batch.seq_of.data_ptr(), batch.q_start.data_ptr(), batch.state_slots.data_ptr(),
        kv.block_table.data_ptr(), kv.block_table.shape[1], kv.block_size, q_out.data_ptr(), kv.k_pool.data_ptr(),
        kv.v_pool.data_ptr(), _code(q_out, "query buffer"), n, heads, kv_heads, dim, vdim, padded, _stream()))
    return q_out


def rmsnorm_onto(resid: torch.Tensor, y: torch.Tensor, gain: torch.Tensor, eps: float,
                 rows_dtype: torch.dtype | None = None):
    """resid += y / sqrt(mean(y^2) + eps) * gain, all 32-bit.  With ``rows_dtype`` the updated rows come back
    in that type as well (what the next part multiplies), otherwise None."""
    n, H = resid.shape
    _need(resid, "residual stream", None, torch.float32)
    _need(y, "sublayer output", (n, H), torch.float32)
    _need(gain, "norm gain", (H,), torch.float32)
    rows = None if rows_dtype is None else torch.empty((n, H), dtype=rows_dtype, device=resid.device)
    _check(library().pl_rmsnorm_onto(resid.data_ptr(), y.data_ptr(), gain.data_ptr(), float(eps), _ptr(rows),
                                     F32 if rows is None else _code(rows, "rows of the stream"), n, H, _stream()))
    return rows


def scale_(x: torch.Tensor, s: float) -> torch.Tensor:
    _need(x, "values to scale", None, torch.float32)
    _check(library().pl_scale(x.data_ptr(), float(s), x.numel(), _stream()))
    return x


def to_bf16(x: torch.Tensor) -> torch.Tensor:
    _need(x, "32-bit rows", None, torch.float32)
    out = torch.empty(x.shape, dtype=torch.bfloat16, device=x.device)
    _check(library().pl_to_bf16(x.data_ptr(), out.data_ptr(), x.numel(), _stream()))
    return out


def activation(x: torch.Tensor, name: str) -> torch.Tensor:
    """act(x) element by element, computed in 32-bit and rounded once."""
    _need(x, "values to activate")
    out = torch.empty_like(x)
    _check(library().pl_activation(x.data_ptr(), out.data_ptr(), _code(x, "values to activate"), activation_code(name),
                                   x.numel(), _stream()))
    return out


def weighted_sum_(x: torch.Tensor, a: float, y: torch.Tensor, b: float) -> torch.Tensor:
    """x = a x + b y, 32-bit."""
    _need(x, "first branch", None, torch.float32)
    _need(y, "second branch", tuple(x.shape), torch.float32)
    _check(library().pl_weighted_sum(x.data_ptr(), float(a), y.data_ptr(), float(b), x.numel(), _stream()))
    return x


# ---- attention layers with sinks, distance penalties, and pages that hold one small vector a token -------------

def gemm_heads(x: torch.Tensor, w: torch.Tensor, out: torch.Tensor) -> torch.Tensor:
    """A product a head: out[t, h, :N] = x[t, h, :K] . w[h]^T, w [heads, N, K].  ``x`` [n, heads, >= K] and ``out``
    [n, heads, >= N] may be views whose rows and heads lie further apart than their own sizes (the last axis
    contiguous); a view's values behind K or N are neither read nor written.  In 32-bit on the vector units
    (sums in ascending k: the true 32-bit path); in bfloat16 the library's batched product on the matrix cores."""
    heads, N, K = w.shape
    _need(w, "weights a head")
    n = x.shape[0]
    if x.dim() != 3 or out.dim() != 3 or x.shape[1] != heads or out.shape[1] != heads or out.shape[0] != n:
        raise TensorError(f"a product a head of {tuple(x.shape)} with {tuple(w.shape)} into {tuple(out.shape)}")
    if x.shape[2] != K or out.shape[2] != N or x.stride(2) != 1 or out.stride(2) != 1:
        raise TensorError(f"a product a head of {tuple(x.shape)} with {tuple(w.shape)} into {tuple(out.shape)}")
    if not x.is_cuda or x.dtype != w.dtype or out.dtype != w.dtype:
        raise TensorError("a product a head needs its operands on the GPU and of one type")
    if n == 0:
        return out
    if w.dtype == torch.bfloat16 and n > GEMM_HEADS_PLAIN_ROWS:
        torch.bmm(x.transpose(0, 1), w.transpose(1, 2), out=out.transpose(0, 1))
        return out
    _check(library().pl_gemm_heads(x.data_ptr(), w.data_ptr(), out.data_ptr(), n, heads, N, K, x.stride(0), x.stride(1),
                                   out.stride(0), out.stride(1), _code(w, "weights a head"), 0, _stream()))
    return out


# Up to this many rows a bfloat16 product a head runs on the vector units (one small launch); above, the library's.
GEMM_HEADS_PLAIN_ROWS = 0


def head_prepare(rows: torch.Tensor, off: int, batch, kv, q_out: torch.Tensor, H: int, G: int, D: int, V: int,
                 padded: int, unit_eps: float | None = None, q_gain=None, k_gain=None, cos=None, sin=None,
                 rot_off: int = 0, rot: int = 0, temperature: tuple | None = None, write_kv: bool = True,
                 bias: torch.Tensor | None = None) -> None:
    """Between an attention layer's projections and the attention kernels: ``rows`` [n, >= off + H D + G D + G V]
    (32-bit) holds q | k | v from column ``off``.  q and k are divided by their root mean square over a head
    (``unit_eps``; times a gain where one is given), ``rot`` values from ``rot_off`` on turn in pairs (2i, 2i + 1)
    by the tables' angles, q is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1) (``temperature`` =
    (coef, every)); q goes to ``q_out`` [n, H * padded], k and v into the pages, every head in ``padded`` values.
    ``bias`` (32-bit, [H D + G D + G V]): the projections' biases, added to q | k | v before anything else."""
    n = rows.shape[0]
    _need(rows, "projected rows", None, torch.float32)
    if rows.dim() != 2:
        raise TensorError(f"projected rows of shape {tuple(rows.shape)}")
    _need(q_out, "query buffer", (n, H * padded))
    for pool, what in ((kv.k_pool, "key pool"), (kv.v_pool, "value pool")):
        _need(pool, what, None, q_out.dtype)
        if pool.dim() != 2 or pool.shape[1] != G * padded or pool.shape[0] % kv.block_size:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{kv.block_size}, {G * padded}]")
    for g, what in ((q_gain, "query gain"), (k_gain, "key gain")):
        if g is not None:
            _need(g, what, (D,), torch.float32)
    table_rows = 0
    if rot:
        _need(cos, "cosine table", None, torch.float32)
        _need(sin, "sine table", tuple(cos.shape), torch.float32)
        if cos.dim() != 2 or cos.shape[1] != rot // 2:
            raise TensorError(f"rotary tables have shape {tuple(cos.shape)}, expected [positions, {rot // 2}]")
        table_rows = cos.shape[0]
    coef, every = temperature if temperature is not None else (0.0, 1)
    if bias is not None:
        _need(bias, "biases of q, k and v", (H * D + G * D + G * V,), torch.float32)
    _check(library().pl_head_prepare(
        rows.data_ptr(), _ptr(bias), rows.shape[1], int(off), 1 if unit_eps is not None else 0, float(unit_eps or 0.0),
        _ptr(q_gain), _ptr(k_gain), _ptr(cos) if rot else 0, _ptr(sin) if rot else 0, int(rot_off), int(rot), table_rows,
        1 if temperature is not None else 0, float(coef), int(every), batch.positions.data_ptr(),
        batch.seq_of.data_ptr(), kv.block_table.data_ptr(), kv.block_table.shape[1], kv.block_size,
        1 if write_kv else 0, q_out.data_ptr(), kv.k_pool.data_ptr(), kv.v_pool.data_ptr(),
        _code(q_out, "query buffer"), n, H, G, D, V, padded, _stream()))


def latent_prepare(rows: torch.Tensor, q_off: int, kv_off: int, gain, eps: float, cos, sin, turned: int, batch, kv,
                   q_plain: torch.Tensor, q_out: torch.Tensor, H: int, D: int, rot: int, R: int, padded: int,
                   write_kv: bool = True) -> None:
    """For a layer whose pages hold one small vector a token.  ``rows`` (32-bit): H query heads of [D | rot] from
    column ``q_off``; the small vector's R values and the rotated key part's ``rot`` from ``kv_off``.  The
    unrotated query parts go head-major into ``q_plain`` [H, n, D]; the rotated parts, turned, into values
    R .. R + rot of every head of ``q_out`` [n, H * padded] with zeros behind them; with ``write_kv`` the
    token's row of the pages becomes [norm(vector) * gain | turned key part | zeros]."""
    n = rows.shape[0]
    _need(rows, "projected rows", None, torch.float32)
    _need(q_out, "query buffer", (n, H * padded))
    _need(q_plain, "unrotated query parts", (H, n, D), q_out.dtype)
    pool = kv.k_pool
    _need(pool, "pages", None, q_out.dtype)
    if pool.dim() != 2 or pool.shape[1] != padded or pool.shape[0] % kv.block_size:
        raise TensorError(f"pages have shape {tuple(pool.shape)}, expected [pages*{kv.block_size}, {padded}]")
    if write_kv:
        _need(gain, "gain of the small vector", (R,), torch.float32)
    table_rows = 0
    if turned and sin is None:
        # no tables: ``cos`` lists the frequencies and the kernel works the angles out (position * frequency in 32-bit)
        _need(cos, "rotation frequencies", (turned // 2,), torch.float32)
    elif turned:
        _need(cos, "cosine table", None, torch.float32)
        _need(sin, "sine table", tuple(cos.shape), torch.float32)
        if cos.dim() != 2 or cos.shape[1] != turned // 2:
            raise TensorError(f"rotary tables have shape {tuple(cos.shape)}, expected [positions, {turned // 2}]")
        table_rows = cos.shape[0]
    _check(library().pl_latent_prepare(
        rows.data_ptr(), rows.shape[1], int(q_off), int(kv_off), _ptr(gain) if write_kv else 0, float(eps),
        _ptr(cos) if turned else 0, _ptr(sin) if turned else 0, int(turned), table_rows, batch.positions.data_ptr(),
        batch.seq_of.data_ptr(), kv.block_table.data_ptr(), kv.block_table.shape[1], kv.block_size,
        1 if write_kv else 0, q_plain.data_ptr(), q_out.data_ptr(), pool.data_ptr(), _code(q_out, "query buffer"),
        n, H, D, rot, R, padded, _stream()))


def head_gate_(x: torch.Tensor, rows: torch.Tensor, off: int, positions, H: int, V: int,
               each_element: bool = False) -> torch.Tensor:
    """x[t, h, :] *= sigmoid(rows[t, off + h]) in place; ``x`` [n, H * V], ``rows`` 32-bit.  ``each_element``:
    a gate an element instead of a head, x[t, e] *= sigmoid(rows[t, off + e])."""
    n = x.shape[0]
    gates = H * V if each_element else H
    _need(x, "read-outs", (n, H * V))
    _need(rows, "gate rows", None, torch.float32)
    if rows.dim() != 2 or rows.shape[0] != n or rows.shape[1] < off + gates:
        raise TensorError(f"gate rows of shape {tuple(rows.shape)} for {n} tokens and {gates} gates from column {off}")
    _check(library().pl_head_gate(x.data_ptr(), _code(x, "read-outs"), rows.data_ptr(), rows.shape[1], int(off),
                                  _ptr(positions), n, H, V, 1 if each_element else 0, _stream()))
    return x


def add_position_rows_(x: torch.Tensor, table: torch.Tensor, positions: torch.Tensor) -> torch.Tensor:
    """x[t] += table[positions[t]] on the 32-bit stream; rows at position -1 stay as they are."""
    n, width = x.shape
    _need(x, "stream", None, torch.float32)
    _need(table, "position table")
    if table.dim() != 2 or table.shape[1] != width:
        raise TensorError(f"a position table of shape {tuple(table.shape)} for a stream of width {width}")
    _need(positions, "positions", (n,), torch.int32)
    _check(library().pl_add_position_rows(x.data_ptr(), table.data_ptr(), _code(table, "position table"),
                                          positions.data_ptr(), n, width, table.shape[0], _stream()))
    return x


def sink_attention(q: torch.Tensor, out: torch.Tensor, batch, kv, nq: int, nkv: int, d: int, scale: float,
                   window: int = 0, sinks: torch.Tensor | None = None, slopes: torch.Tensor | None = None) -> torch.Tensor:
    """Attention for every token of a step with a sink a head in the softmax's denominator and a penalty a
    head on the distance; ``q`` [n, nq * d] holds the prepared queries.  In bfloat16 the matrix-core kernel for
    portions and the kernels for single tokens, for head sizes they take; the plain kernel otherwise."""
    return paged_attention(q, out, batch, kv, nq, nkv, d, scale, window, sinks=sinks, slopes=slopes)


# ---- several copies of the stream; experts chosen by a table over token ids ------------------------------------

HC_MAX_COPIES = 8


def stream_copies(x: torch.Tensor, copies: int) -> torch.Tensor:
    """[n, copies * W]: every row of the 32-bit stream ``x`` [n, W] ``copies`` times, one behind the other."""
    n, W = x.shape
    _need(x, "stream", None, torch.float32)
    out = torch.empty((n, copies * W), dtype=torch.float32, device=x.device)
    _check(library().pl_stream_copies(x.data_ptr(), out.data_ptr(), n, int(copies), W, _stream()))
    return out


def hc_step(streams: torch.Tensor, copies: int, y=None, mix=None, out=None, read=None, gain=None, eps: float = 0.0,
            read_dtype: torch.dtype = torch.float32, rows=None):
    """One pass over the copies of the stream, ``streams`` [n, copies * W] in 32-bit, with either half optional.
    Rebuild (``y`` [n, W] 32-bit, ``mix`` [copies, copies], ``out`` [copies]): copy t becomes
    sum_s mix[s, t] x_s + out[t] y, in place.  Read-out (``read`` [copies]): u = sum_s read[s] x_s of the rebuilt
    copies, normed with ``gain`` (32-bit [W]) and ``eps`` where a gain is given, comes back as [rows, W] in
    ``read_dtype`` (None where nothing is read out).  ``rows``: the rows to read out (then nothing is rebuilt)."""
    n = streams.shape[0]
    _need(streams, "copies of the stream", None, torch.float32)
    if streams.dim() != 2 or streams.shape[1] % copies or not 1 <= copies <= HC_MAX_COPIES:
        raise TensorError(f"{copies} copies of the stream in rows of {tuple(streams.shape)}")
    W = streams.shape[1] // copies
    if y is not None:
        _need(y, "sublayer output", (n, W), torch.float32)
        _need(mix, "weights between the copies", (copies, copies), torch.float32)
        _need(out, "weights of the sublayer output", (copies,), torch.float32)
        if rows is not None:
            raise TensorError("a list of rows and a rebuild of the copies")
    result = None
    count = n
    if read is not None:
        _need(read, "weights of the read-out", (copies,), torch.float32)
        if gain is not None:
            _need(gain, "gain of the read-out's norm", (W,), torch.float32)
        if rows is not None:
            _need(rows, "rows to read out", None, torch.int32)
            count = rows.numel()
        result = torch.empty((count, W), dtype=read_dtype, device=streams.device)
    elif y is None:
        return None
    _check(library().pl_hc_step(streams.data_ptr(), _ptr(y), _ptr(mix), _ptr(out), _ptr(read), _ptr(gain), float(eps),
                                _ptr(result), _CODES[read_dtype], _ptr(rows), count, int(copies), W, _stream()))
    return result


def softcap_(x: torch.Tensor, cap: float) -> torch.Tensor:
    """x <- cap * tanh(x / cap) on 32-bit values, in place."""
    _need(x, "logits", None, torch.float32)
    _check(library().pl_softcap(x.data_ptr(), float(cap), x.numel(), _stream()))
    return x


def _routed(n: int, E: int, choice, weight, identity: int) -> int:
    """Checks a router's choice for ``n`` rows ([n, top] int32, with weights [n, top] 32-bit) and gives ``top``."""
    _need(choice, "chosen experts", None, torch.int32)
    if choice.dim() != 2 or choice.shape[0] != n or not 1 <= choice.shape[1] <= E + identity or identity < 0:
        raise TensorError(f"chosen experts of shape {tuple(choice.shape)} for {n} rows and {E} + {identity} experts")
    _need(weight, "weights of the chosen experts", tuple(choice.shape), torch.float32)
    return choice.shape[1]


def moe_rows(x: torch.Tensor, batch, table, w_gate_up: torch.Tensor, w_down: torch.Tensor,
             activation: str = "silu", choice=None, weight=None, identity: int = 0) -> torch.Tensor:
    """Experts chosen by a table over token ids, a row at a time: 32-bit [n, W], row t the mean over the experts e
    that ``table[id of t]`` names of down_e (act(gate_e x_t) * (up_e x_t)).  ``w_gate_up`` [E, 2 F, W] (an expert's
    gate rows, then its up rows), ``w_down`` [E, W, F], of ``x``'s type; ``table`` [vocabulary, top] int32.  A row's
    id is the batch's, or the one an earlier step left on the device; padding rows give zeros.
    With ``choice`` and ``weight`` ([n, top]; no table) a router has chosen: pair (t, c) runs expert choice[t, c] and
    counts weight[t, c]; a choice of E .. E + ``identity`` - 1 is an identity expert, whose output is the row itself;
    -1 is none."""
    n, W = x.shape
    _need(x, "rows")
    E, F2, _ = w_gate_up.shape
    F = F2 // 2
    _need(w_gate_up, "gate and up weights of the experts", (E, 2 * F, W), x.dtype)
    _need(w_down, "down weights of the experts", (E, W, F), x.dtype)
    if choice is not None:
        vocab, top = 1, _routed(n, E, choice, weight, identity)
    else:
        _need(table, "table of experts", None, torch.int32)
        vocab, top = table.shape
    fed = getattr(batch, "fed_tokens", None)
    src = batch.token_src if fed is not None else None
    h = torch.empty((n, top, F), dtype=x.dtype, device=x.device)
    out = torch.empty((n, W), dtype=torch.float32, device=x.device)
    _check(library().pl_moe_rows(x.data_ptr(), batch.token_ids.data_ptr(), _ptr(src), _ptr(fed),
                                 batch.positions.data_ptr(), _ptr(table), w_gate_up.data_ptr(), w_down.data_ptr(),
                                 h.data_ptr(), out.data_ptr(), _code(x, "rows"), n, W, F, E, top, vocab,
                                 activation_code(activation), _ptr(choice), _ptr(weight), int(identity), _stream()))
    return out


MOE_TILE = 128       # rows of a tile of the grouped product


def moe_grouped_applies(x: torch.Tensor, width: int, ff: int) -> bool:
    """Whether the experts of a step run as grouped products on the matrix cores: bfloat16, an inner width the
    tiles take (a multiple of 32), an expert width that is a multiple of 64."""
    return x.dtype == torch.bfloat16 and width % 32 == 0 and ff % 64 == 0


def moe_down_splits(tiles: int, width: int, ff: int) -> int:
    """Into how many stretches the experts' down product cuts its inner width: with few tiles of rows (decoding) its
    launch is tiles x width / 128 workgroups that each walk the whole expert width, most of the chip idle; stretches
    of at least 8 steps of 32 until the launch has a workgroup a compute unit."""
    groups, splits = tiles * -(-width // 128), 1
    while groups * splits < compute_units() and splits < 8 and ff // 32 // (splits * 2) >= 8:
        splits *= 2
    return splits


def moe_grouped(x: torch.Tensor, batch, table, w_gate_up: torch.Tensor, w_down: torch.Tensor,
                activation: str = "silu", choice=None, weight=None, identity: int = 0) -> torch.Tensor:
    """What ``moe_rows`` computes, with the step's (row, choice) pairs dealt to their experts first: an expert's
    pairs fill tiles of 128 rows, and two grouped products on the matrix cores (gate and up with the activation
    behind them; down with 32-bit sums out) read an expert's weights once a tile.  A last pass adds a row's
    choices in their order, in 32-bit.  Nothing is read back by the host: the tiles are laid out for the most
    a step of so many rows can need."""
    n, W = x.shape
    _need(x, "rows", None, torch.bfloat16)
    E, F2, _ = w_gate_up.shape
    F = F2 // 2
    _need(w_gate_up, "gate and up weights of the experts", (E, 2 * F, W), x.dtype)
    _need(w_down, "down weights of the experts", (E, W, F), x.dtype)
    if choice is not None:
        vocab, top = 1, _routed(n, E, choice, weight, identity)
    else:
        _need(table, "table of experts", None, torch.int32)
        vocab, top = table.shape
    out = torch.empty((n, W), dtype=torch.float32, device=x.device)
    if n == 0:
        return out
    fed = getattr(batch, "fed_tokens", None)
    src = batch.token_src if fed is not None else None
    pairs = n * top
    # every expert that has pairs may leave its last tile part empty
    tiles = -(-pairs // MOE_TILE) + min(E, pairs)
    slots = tiles * MOE_TILE
    lib, stream = library(), _stream()
    ints = torch.empty((slots + pairs + tiles,), dtype=torch.int32, device=x.device)
    gather, slot_of, tile_group = ints[:slots], ints[slots:slots + pairs], ints[slots + pairs:]
    _check(lib.pl_moe_sort(batch.token_ids.data_ptr(), _ptr(src), _ptr(fed), batch.positions.data_ptr(), _ptr(table),
                           _ptr(choice), n, top, E, vocab, MOE_TILE, tiles, gather.data_ptr(), slot_of.data_ptr(),
                           tile_group.data_ptr(), stream))
    hidden = torch.empty((slots, F), dtype=torch.bfloat16, device=x.device)
    _check(lib.pl_gemm_tiled_grouped(x.data_ptr(), w_gate_up.data_ptr(), hidden.data_ptr(), tile_group.data_ptr(),
                                     gather.data_ptr(), 2 * F * W, tiles, n, F, W, 1, activation_code(activation), 1, stream))
    splits = moe_down_splits(tiles, W, F)
    y = torch.empty((splits, slots, W), dtype=torch.float32, device=x.device)
    _check(lib.pl_gemm_tiled_grouped(hidden.data_ptr(), w_down.data_ptr(), y.data_ptr(), tile_group.data_ptr(), 0,
                                     W * F, tiles, slots, W, F, 3, 0, splits, stream))
    _check(lib.pl_moe_combine(y.data_ptr(), slot_of.data_ptr(), out.data_ptr(), n, top, W, splits, slots * W,
                              _ptr(weight), _ptr(choice), x.data_ptr(), _code(x, "rows"), E, batch.positions.data_ptr(), stream))
    return out


# A router's logits are worked out inside the kernel that chooses (one wave a row, the router's matrix from L2) for steps
# of up to this many rows and routers of up to this many weights; beyond, a product of its own (the library's) is faster.
ROUTER_FUSED_ROWS = 128
ROUTER_FUSED_WEIGHTS = 1 << 18


def router_fuses(rows: int, total: int, width: int) -> bool:
    return rows <= ROUTER_FUSED_ROWS and total * width <= ROUTER_FUSED_WEIGHTS and width <= 8192 and total <= 1024


def router_select(logits, correction, positions, top: int, groups: int = 1, kept: int = 1,
                  normalised: bool = True, weight_eps: float = 1e-20, x=None, w=None):
    """A router's choice for every row of its 32-bit ``logits`` [n, outputs]: (chosen [n, top] int32, weights [n, top]
    32-bit).  Scores are the softmax over all outputs; the choice goes by score plus ``correction`` ([outputs] 32-bit, or
    None); outputs form ``groups`` equal groups of neighbours, a group counts by its best choice score, and only members
    of the best ``kept`` groups can be chosen; the ``top`` largest are chosen, the lower index among equals; a chosen
    output weighs its score, divided (``normalised``) by the chosen scores' sum plus ``weight_eps``.  Rows at
    position -1 choose nothing (-1).  With ``logits`` None the kernel works them out itself from the rows ``x`` [n, W]
    and the router's matrix ``w`` [outputs, W] (one type; 32-bit sums)."""
    if logits is not None:
        _need(logits, "router logits", None, torch.float32)
        if logits.dim() != 2:
            raise TensorError(f"router logits of shape {tuple(logits.shape)}")
        n, total = logits.shape
        width, code, device = 0, F32, logits.device
    else:
        _need(x, "rows")
        _need(w, "router matrix", None, x.dtype)
        if x.dim() != 2 or w.dim() != 2 or w.shape[1] != x.shape[1]:
            raise TensorError(f"rows of shape {tuple(x.shape)} for a router of shape {tuple(w.shape)}")
        (n, width), total, code, device = x.shape, w.shape[0], _code(x, "rows"), x.device
    if correction is not None:
        _need(correction, "correction of the choice", (total,), torch.float32)
    if positions is not None:
        _need(positions, "positions", (n,), torch.int32)
    choice = torch.empty((n, top), dtype=torch.int32, device=device)
    weight = torch.empty((n, top), dtype=torch.float32, device=device)
    _check(library().pl_router_select(_ptr(logits), total, _ptr(correction), _ptr(positions), n, total, int(top),
                                      int(groups), int(kept), 1 if normalised else 0, float(weight_eps),
                                      choice.data_ptr(), weight.data_ptr(), _ptr(x) if logits is None else 0,
                                      _ptr(w) if logits is None else 0, int(width), code, _stream()))
    return choice, weight


# ---- values that are the keys, q and k normed over all their heads; sublayers side by side ----------------------

def wide_prepare(rows: torch.Tensor, off: int, batch, kv, q_out: torch.Tensor, H: int, G: int, D: int, padded: int,
                 norm_eps: float | None = None, q_gain=None, k_gain=None, freq=None, rot: int = 0,
                 write_kv: bool = True, bias: torch.Tensor | None = None) -> None:
    """Between an attention layer's projections and the attention kernels, for a layer without a value projection:
    ``rows`` [n, >= off + H D + G D] (32-bit) holds q | k from column ``off``; ``bias`` ([H D + G D] 32-bit) is added
    first.  The values are the keys as they stand then.  q is divided by its root mean square over ALL its H D
    values and k over all its G D (``norm_eps``; times a gain a column, [H D] and [G D]); the first ``rot`` values of every
    head turn in pairs (2i, 2i + 1) by position * ``freq``[i] (32-bit).  q goes to ``q_out`` [n, H * padded], the keys and
    the values into the pages, every head in ``padded`` values with zeros behind its own."""
    n = rows.shape[0]
    _need(rows, "projected rows", None, torch.float32)
    if rows.dim() != 2:
        raise TensorError(f"projected rows of shape {tuple(rows.shape)}")
    _need(q_out, "query buffer", (n, H * padded))
    for pool, what in ((kv.k_pool, "key pool"), (kv.v_pool, "value pool")):
        _need(pool, what, None, q_out.dtype)
        if pool.dim() != 2 or pool.shape[1] != G * padded or pool.shape[0] % kv.block_size:
            raise TensorError(f"{what} has shape {tuple(pool.shape)}, expected [pages*{kv.block_size}, {G * padded}]")
    if q_gain is not None:
        _need(q_gain, "query gain", (H * D,), torch.float32)
    if k_gain is not None:
        _need(k_gain, "key gain", (G * D,), torch.float32)
    if rot:
        _need(freq, "rotation frequencies", (rot // 2,), torch.float32)
    if bias is not None:
        _need(bias, "biases of q and k", (H * D + G * D,), torch.float32)
    _check(library().pl_wide_prepare(
        rows.data_ptr(), _ptr(bias), rows.shape[1], int(off), 1 if norm_eps is not None else 0, float(norm_eps or 0.0),
        _ptr(q_gain), _ptr(k_gain), _ptr(freq) if rot else 0, int(rot), batch.positions.data_ptr(), batch.seq_of.data_ptr(),
        kv.block_table.data_ptr(), kv.block_table.shape[1], kv.block_size, 1 if write_kv else 0, q_out.data_ptr(),
        kv.k_pool.data_ptr(), kv.v_pool.data_ptr(), _code(q_out, "query buffer"), n, H, G, D, padded, _stream()))


def parallel_step(resid: torch.Tensor, a=None, ls1=None, b=None, ls2=None, more=None, gain1=None, gain2=None,
                  eps: float = 0.0, out_dtype: torch.dtype = torch.float32, rows=None):
    """One pass over the rows of the 32-bit stream for a layer whose sublayers stand side by side, either half
    optional.  Sums: resid += ls1 * a + ls2 * b + more (``a``, ``b``, ``more`` [n, W] 32-bit; ``ls1``, ``ls2`` [W] 32-bit
    or None for ones), in place.  Norms of the updated rows: rms-normed rows times ``gain1`` and, where given, times
    ``gain2`` (both [W] 32-bit), in ``out_dtype``; (rows1, rows2), each None where its gain is.  ``rows``: the rows to
    norm (then nothing is summed)."""
    _need(resid, "residual stream", None, torch.float32)
    if resid.dim() != 2:
        raise TensorError(f"a stream of shape {tuple(resid.shape)}")
    n, W = resid.shape
    for t, what in ((a, "first sublayer's output"), (b, "second sublayer's output"), (more, "rows to add")):
        if t is not None:
            _need(t, what, (n, W), torch.float32)
    for t, what in ((ls1, "first layer scale"), (ls2, "second layer scale"), (gain1, "first norm gain"), (gain2, "second norm gain")):
        if t is not None:
            _need(t, what, (W,), torch.float32)
    if (ls1 is not None and a is None) or (ls2 is not None and b is None) or (gain2 is not None and gain1 is None):
        raise TensorError("a layer scale without its sublayer's output, or a second norm without a first")
    count = n
    if rows is not None:
        _need(rows, "rows to norm", None, torch.int32)
        count = rows.numel()
    out1 = torch.empty((count, W), dtype=out_dtype, device=resid.device) if gain1 is not None else None
    out2 = torch.empty((count, W), dtype=out_dtype, device=resid.device) if gain2 is not None else None
    if a is None and b is None and more is None and gain1 is None:
        return None, None
    _check(library().pl_parallel_step(resid.data_ptr(), _ptr(a), _ptr(ls1), _ptr(b), _ptr(ls2), _ptr(more), _ptr(gain1),
                                      _ptr(gain2), float(eps), _ptr(out1), _ptr(out2), _CODES[out_dtype], _ptr(rows),
                                      count, W, _stream()))
    return out1, out2
