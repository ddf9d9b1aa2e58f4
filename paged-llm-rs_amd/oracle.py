"""Plain, sequential C++ versions of what the GPU kernels compute (csrc/host/oracle.cpp), over 32-bit
tensors on the CPU.  The kernel tests hold the kernels against them; nothing on the product path calls
them.  (The reference keeps a scalar oracle beside its attention kernel the same way:
crates/pagedllm/src/kernels/paged_attention.rs:150-210.)"""

from __future__ import annotations

import torch

from . import native


def _f32(t: torch.Tensor) -> torch.Tensor:
    return t.detach().to("cpu", torch.float32).contiguous()


def _i32(t) -> torch.Tensor:
    return torch.as_tensor(t).detach().to("cpu", torch.int32).contiguous()


def rms_norm(x: torch.Tensor, gain: torch.Tensor, eps: float) -> torch.Tensor:
    x, gain = _f32(x), _f32(gain)
    rows, width = x.shape
    out = torch.empty_like(x)
    native.library().plh_oracle_rms_norm(x.data_ptr(), gain.data_ptr(), float(eps), rows, width, out.data_ptr())
    return out


def rotate(x: torch.Tensor, positions, rot: int, theta: float, neighbours: bool = False) -> torch.Tensor:
    """x [rows, heads, d] with the first ``rot`` elements of every head turned by each row's position."""
    out, positions = _f32(x).clone(), _i32(positions)
    rows, heads, d = out.shape
    native.library().plh_oracle_rotate(out.data_ptr(), positions.data_ptr(), rows, heads, d, int(rot), float(theta),
                                       1 if neighbours else 0)
    return out


def product(x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
    x, w = _f32(x), _f32(w)
    out = torch.empty((x.shape[0], w.shape[0]), dtype=torch.float32)
    native.library().plh_oracle_product(x.data_ptr(), w.data_ptr(), x.shape[0], w.shape[0], x.shape[1], out.data_ptr())
    return out


def swiglu(gate_up: torch.Tensor) -> torch.Tensor:
    gate_up = _f32(gate_up)
    rows, inter = gate_up.shape[0], gate_up.shape[1] // 2
    out = torch.empty((rows, inter), dtype=torch.float32)
    native.library().plh_oracle_swiglu(gate_up.data_ptr(), rows, inter, out.data_ptr())
    return out


def paged_attention(q: torch.Tensor, k_pool: torch.Tensor, v_pool: torch.Tensor, block_table, positions, seq_of,
                    nq: int, nkv: int, d: int, block_size: int, scale: float, window: int = 0) -> torch.Tensor:
    """q [rows, nq * d] (or wider rows that begin with the queries), pools [slots, nkv * d]; [rows, nq * d] comes back."""
    q = _f32(q)[:, :nq * d].contiguous()
    k_pool, v_pool = _f32(k_pool), _f32(v_pool)
    block_table, positions, seq_of = _i32(block_table), _i32(positions), _i32(seq_of)
    rows = q.shape[0]
    out = torch.empty((rows, nq * d), dtype=torch.float32)
    native.library().plh_oracle_paged_attention(q.data_ptr(), k_pool.data_ptr(), v_pool.data_ptr(), block_table.data_ptr(),
                                                positions.data_ptr(), seq_of.data_ptr(), rows, nq, nkv, d, block_size,
                                                block_table.shape[1], float(scale), int(window or 0), out.data_ptr())
    return out


def argmax(logits: torch.Tensor) -> torch.Tensor:
    logits = _f32(logits)
    out = torch.empty((logits.shape[0],), dtype=torch.int32)
    native.library().plh_oracle_argmax(logits.data_ptr(), logits.shape[0], logits.shape[1], out.data_ptr())
    return out
