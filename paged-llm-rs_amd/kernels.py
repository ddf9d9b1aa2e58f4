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
        "pl_paged_attention_plain": [p, i, p, p, p, p, i, i, p, p, i, i, i, i, f, i, i, p],
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
                                      i, p, p, i, f, p, p, i, p],
        "pl_paged_attention_prefill": [p, i, p, p, p, p, i, i, i, p, i, i, p, p, i, i, i, f, i, i, p, p, i, p],
        "pl_paged_attention_grouped": [p, i, p, p, p, p, i, i, i, p, i, i, p, p, i, i, i, f, i, i, p, p, i, i, p],
        "pl_paged_attention_grouped_applies": [i, i, i, i],
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


def paged_attention_plain(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, positions: torch.Tensor,
                          seq_of: torch.Tensor, block_table: torch.Tensor, block_size: int,
                          k_pool: torch.Tensor, v_pool: torch.Tensor, nq: int, nkv: int, d: int,
                          scale: float, window: int = 0) -> torch.Tensor:
    """Attention of every token over the keys 0..position of its request, read
    through the block table.  ``q`` is the fused projection buffer whose rows begin
    with the nq*d query values."""
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
    _check(library().pl_paged_attention_plain(
        q.data_ptr(), q_row_stride, out.data_ptr(), positions.data_ptr(), seq_of.data_ptr(),
        block_table.data_ptr(), block_table.shape[1], block_size, k_pool.data_ptr(), v_pool.data_ptr(),
        n, nq, nkv, d, float(scale), int(window or 0), _code(q, "query buffer"), _stream()))
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
                           short_rows: int = 0) -> torch.Tensor:
    """bfloat16 attention of single tokens over their requests' pages, split along the context.
    With ``q_len`` the tokens of requests with ``short_limit`` tokens or more are left out; ``short_rows``
    then bounds the tokens that the other requests bring (0: not known) and ``live_seqs`` says how many
    requests, the first ones, bring tokens, so that the launch has workgroups for those tokens only.
    With ``fuse`` the rows of ``q`` are the raw projection [q | k | v]: queries (and, when it says so, each
    token's key) are normalised and rotated inside the kernel, and key and value are written into the pages."""
    n = positions.numel()
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
        mode, _ptr(q_gain), _ptr(k_gain), gain_code, float(eps), _ptr(cos), _ptr(sin), int(rot), _stream()))
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
                            splits: int | None = None, live_seqs: int | None = None) -> torch.Tensor:
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
        part_acc.data_ptr() if splits > 1 else None, part_ml.data_ptr() if splits > 1 else None, n, _stream()))
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


def grouped_splits(tokens: int, nkv: int, max_ctx: int) -> int:
    """Into how many shares the keys of a token are cut for the grouped kernel: two workgroups a compute
    unit (as many as its LDS holds) if the tokens and key heads alone do not give that many, every share
    two tiles of keys at least.  (Context 4,096 over 8 key heads: 16 tokens take 65 us in four shares and
    67 in two, 8 tokens 39 us in eight shares and 41 in four.)"""
    base = max(tokens * nkv, 1)
    key_tiles = -(-max(max_ctx, 1) // 64)
    return max(1, min(16, key_tiles // 2, -(-2 * compute_units() // base)))


def paged_attention_grouped(q: torch.Tensor, q_row_stride: int, out: torch.Tensor, q_start: torch.Tensor,
                            q_len: torch.Tensor, ctx_len: torch.Tensor, max_q_len: int, block_table: torch.Tensor,
                            block_size: int, k_pool: torch.Tensor, v_pool: torch.Tensor, nq: int, nkv: int, d: int,
                            scale: float, window: int = 0, short_limit: int = 0, max_ctx: int | None = None,
                            splits: int | None = None, live_seqs: int | None = None,
                            tokens: int | None = None) -> torch.Tensor:
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
        splits = grouped_splits(n if tokens is None else int(tokens), nkv, int(max_ctx or 0))
    part_acc = part_ml = None
    if splits > 1:
        part_acc = torch.empty((n * nq * splits * d,), dtype=torch.float32, device=q.device)
        part_ml = torch.empty((n * nq * splits * 2,), dtype=torch.float32, device=q.device)
    _check(library().pl_paged_attention_grouped(
        q.data_ptr(), q_row_stride, out.data_ptr(), q_start.data_ptr(), q_len.data_ptr(), ctx_len.data_ptr(),
        int(short_limit), live, int(max_q_len), block_table.data_ptr(), block_table.shape[1], block_size,
        k_pool.data_ptr(), v_pool.data_ptr(), nq, nkv, d, float(scale), int(window or 0), int(splits),
        part_acc.data_ptr() if splits > 1 else None, part_ml.data_ptr() if splits > 1 else None, n, int(tokens or 0), _stream()))
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
                    scale: float, window: int = 0) -> torch.Tensor:
    """Attention for every token of a step.  ``qkv`` rows begin with the rotated queries.
    In bfloat16 the long portions go to the tiled kernel and the tokens of short ones
    (decoded tokens among them) to the kernel for single tokens, or, where many query heads share a key
    head, to the tiled kernel with a group's heads as its rows; all read the same pages."""
    if qkv.dtype != torch.bfloat16 or _attention_mode != "kernel":
        return paged_attention_plain(qkv, qkv.shape[1], out, batch.positions, batch.seq_of, kv.block_table,
                                     kv.block_size, kv.k_pool, kv.v_pool, nq, nkv, d, scale, window)
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
                                live_seqs=getattr(batch, "live_seqs", None))
        if short_tokens == 0 or all_tiled:
            return out
    mixed = batch.max_q_len >= SHORT_PORTION
    if grouped_applies(nq, nkv, d, kv.block_size):
        # many query heads a key head: a token's group of heads as the rows of a tile of the tiled kernel
        return paged_attention_grouped(qkv, stride, out, batch.q_start, batch.q_len, batch.ctx_len,
                                       min(batch.max_q_len, SHORT_PORTION - 1), kv.block_table, kv.block_size,
                                       kv.k_pool, kv.v_pool, nq, nkv, d, scale, window,
                                       short_limit=SHORT_PORTION if mixed else 0, max_ctx=batch.max_ctx_len,
                                       live_seqs=getattr(batch, "live_seqs", None), tokens=short_tokens)
    splits = decode_splits(short_tokens, nq, nkv, batch.max_ctx_len, d)
    return paged_attention_decode(qkv, stride, out, batch.positions, batch.seq_of, kv.block_table,
                                  kv.block_size, kv.k_pool, kv.v_pool, nq, nkv, d, scale, window, splits,
                                  q_len=batch.q_len if mixed else None, short_limit=SHORT_PORTION if mixed else 0,
                                  live_seqs=getattr(batch, "live_seqs", None), short_rows=short_tokens)


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
