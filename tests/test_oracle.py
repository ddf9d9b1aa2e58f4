"""The plain C++ oracles that stand beside the kernels, pinned on the CPU by library routines and by the
plain implementation's functions (which the reference's fixture pins)."""

from __future__ import annotations

import math

import pytest
import torch

import plain_qwen3 as plain


def rel(a, b):
    a, b = a.double(), b.double()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


def test_norm_product_and_activation_are_the_library_s():
    from paged_llm_rs_amd import oracle

    g = torch.Generator().manual_seed(3)
    x = torch.randn(5, 37, generator=g)
    gain = torch.randn(37, generator=g)
    want = x.double() / (x.double().pow(2).mean(-1, keepdim=True) + 1e-5).sqrt() * gain.double()
    assert rel(oracle.rms_norm(x, gain, 1e-5), want) < 1e-6
    assert rel(oracle.rms_norm(x, gain, 1e-5), plain.rms_norm(x.double(), gain.double(), 1e-5)) < 1e-6
    w = torch.randn(11, 37, generator=g)
    assert rel(oracle.product(x, w), x.double() @ w.double().T) < 1e-6
    gu = torch.randn(4, 26, generator=g)
    assert rel(oracle.swiglu(gu), torch.nn.functional.silu(gu[:, :13].double()) * gu[:, 13:].double()) < 1e-6
    logits = torch.tensor([[1.0, 5.0, 5.0, -2.0], [0.0, 0.0, 0.0, 0.0], [-3.0, -1.0, -2.0, -1.0]])
    assert oracle.argmax(logits).tolist() == [1, 0, 1], "the first largest"


@pytest.mark.parametrize("rot,d", [(8, 8), (6, 10)])
def test_rotation_is_the_plain_implementation_s(rot, d):
    from paged_llm_rs_amd import oracle

    g = torch.Generator().manual_seed(rot)
    x = torch.randn(4, 3, d, generator=g)
    positions = torch.tensor([0, 1, 7, 300])
    want = x.double().clone()
    want[..., :rot] = plain.apply_rope(x.double()[..., :rot], positions, 10000.0)
    assert rel(oracle.rotate(x, positions, rot, 10000.0), want) < 1e-6
    # neighbours: the same rotation of the same pairs after a shuffle of the elements
    order = torch.tensor([i // 2 + (rot // 2) * (i % 2) for i in range(rot)])       # where element i of the neighbour layout stands in the half layout
    shuffled = x.clone()
    shuffled[..., :rot] = x[..., :rot][..., order]
    back = oracle.rotate(shuffled, positions, rot, 10000.0, neighbours=True)
    inverse = torch.argsort(order)
    assert rel(back[..., :rot][..., inverse], want[..., :rot]) < 1e-6
    assert torch.equal(back[..., rot:], x[..., rot:]), "what is not rotated passes through"


@pytest.mark.parametrize("nq,nkv,d,bs,window", [(4, 2, 8, 4, 0), (6, 1, 5, 3, 0), (4, 4, 8, 16, 5)])
def test_attention_over_pages_is_plain_attention(nq, nkv, d, bs, window):
    from paged_llm_rs_amd import oracle

    g = torch.Generator().manual_seed(nq * 10 + bs)
    ctx = [9, 17]
    pages = [math.ceil(c / bs) for c in ctx]
    order = torch.randperm(sum(pages) + 3, generator=g).tolist()
    table = torch.full((2, max(pages)), -1, dtype=torch.int32)
    k_pool = torch.randn((sum(pages) + 3) * bs, nkv * d, generator=g)
    v_pool = torch.randn((sum(pages) + 3) * bs, nkv * d, generator=g)
    at = 0
    for s, count in enumerate(pages):
        for i in range(count):
            table[s, i] = order[at]
            at += 1
    positions, seq_of = [8, 16, 3, -1], [0, 1, 1, 0]
    q = torch.randn(4, nq * d, generator=g)
    got = oracle.paged_attention(q, k_pool, v_pool, table, positions, seq_of, nq, nkv, d, bs, 0.3, window)
    assert bool((got[3] == 0).all()), "a padding row"
    for t in range(3):
        s, p = seq_of[t], positions[t]
        first = max(0, p + 1 - window) if window else 0
        slots = [int(table[s, j // bs]) * bs + j % bs for j in range(first, p + 1)]
        keys, values = k_pool[slots].double().view(-1, nkv, d), v_pool[slots].double().view(-1, nkv, d)
        for h in range(nq):
            kv = h // (nq // nkv)
            scores = (keys[:, kv] @ q[t, h * d:(h + 1) * d].double()) * 0.3
            want = torch.softmax(scores, 0) @ values[:, kv]
            assert rel(got[t, h * d:(h + 1) * d], want) < 1e-6
