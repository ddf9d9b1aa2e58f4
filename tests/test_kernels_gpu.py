"""Each kernel alone against a plain 32-bit (or 64-bit) torch reference of the same
operation, at other sizes than the engine's tiny models use."""

from __future__ import annotations

import math
import random

import pytest
import torch

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def rel(got, want):
    got, want = got.double().cpu(), want.double().cpu()
    assert got.shape == want.shape
    return float((got - want).abs().max() / want.abs().max().clamp_min(1e-30))


def tol(dtype):
    return 2e-6 if dtype == torch.float32 else 1e-2


@pytest.fixture(autouse=True)
def _seed():
    torch.manual_seed(1234)


# --- embedding -------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("V,H", [(331, 100), (1000, 1024), (50, 24)])
def test_embed(dtype, V, H):
    from paged_llm_rs_amd import kernels

    table = torch.randn(V, H, device=DEV).to(dtype)
    ids = torch.tensor([0, V - 1, 7, 7, -1, V // 2], dtype=torch.int32, device=DEV)
    out = kernels.embed(ids, table)
    assert out.dtype == torch.float32
    want = table.float()[ids.clamp_min(0).long()]
    want[4] = 0
    assert torch.equal(out, want)


# --- residual add + norm -----------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,H", [(1, 24), (7, 100), (33, 1024), (5, 5120), (3, 33), (2, 9000), (4, 4096), (2, 8192), (3, 2050), (300, 1024), (257, 100), (513, 4096), (260, 5120)])
def test_add_rmsnorm(dtype, n, H):
    from paged_llm_rs_amd import kernels

    resid = torch.randn(n, H, device=DEV) * 3
    delta = torch.randn(n, H, device=DEV).to(dtype)
    gain = (torch.rand(H, device=DEV) + 0.5).to(dtype)
    eps = 1e-5
    x = resid.double() + delta.double()
    want = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain.double()
    out = torch.empty(n, H, dtype=dtype, device=DEV)
    r = resid.clone()
    kernels.add_rmsnorm(r, delta, gain, eps, out)
    assert rel(out, want) < tol(dtype)
    assert rel(r, x) < 1e-6, "the sum is written back in 32-bit"
    # no delta; gathered rows leave the stream untouched; a 32-bit gain beside 16-bit activations
    r2 = resid.clone()
    rows = torch.tensor([n - 1, 0], dtype=torch.int32, device=DEV)
    out2 = torch.empty(2, H, dtype=dtype, device=DEV)
    kernels.add_rmsnorm(r2, delta, gain.float(), eps, out2, rows=rows)
    assert torch.equal(r2, resid)
    assert rel(out2, want[[n - 1, 0]]) < tol(dtype)
    out3 = torch.empty(n, H, dtype=dtype, device=DEV)
    kernels.add_rmsnorm(resid.clone(), None, gain, eps, out3)
    x0 = resid.double()
    assert rel(out3, x0 / torch.sqrt((x0 * x0).mean(-1, keepdim=True) + eps) * gain.double()) < tol(dtype)


# --- q/k norm, rotation, cache write --------------------------------------------------------------------

def rope_ref(x, pos, theta, rot):
    """x [n, heads, d] float64; rotate the first ``rot`` values of each head, halves paired."""
    half = rot // 2
    inv = torch.tensor([1.0 / theta ** (2.0 * i / rot) for i in range(half)], dtype=torch.float64, device=x.device)
    ang = pos.double()[:, None] * inv[None]
    c, s = ang.cos()[:, None, :], ang.sin()[:, None, :]
    out = x.clone()
    x1, x2 = x[..., :half], x[..., half:rot]
    out[..., :half] = x1 * c - x2 * s
    out[..., half:rot] = x2 * c + x1 * s
    return out


def tables(max_pos, rot, theta):
    half = rot // 2
    inv = torch.tensor([1.0 / theta ** (2.0 * i / rot) for i in range(half)], dtype=torch.float64)
    ang = torch.arange(max_pos, dtype=torch.float64)[:, None] * inv[None]
    return ang.cos().float().to(DEV), ang.sin().float().to(DEV)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,bs,norm", [(4, 2, 16, 4, True), (6, 1, 48, 16, True), (3, 3, 128, 8, False),
                                              (8, 2, 256, 2, True), (5, 5, 80, 16, True), (16, 8, 128, 16, True),
                                              (7, 1, 128, 4, True), (3, 1, 24, 4, True), (2, 2, 10, 8, False)])
def test_qk_norm_rope_kv_write(dtype, nq, nkv, d, bs, norm):
    from paged_llm_rs_amd import kernels

    n, S, pages = 11, 3, 64      # positions up to 31: 16 pages a request at a page size of 2
    theta, eps = 1e4, 1e-5
    qkv = torch.randn(n, (nq + 2 * nkv) * d, device=DEV).to(dtype)
    seq_of = torch.tensor([0, 0, 0, 0, 1, 2, 2, 2, 2, 2, 1], dtype=torch.int32, device=DEV)
    positions = torch.tensor([5, 6, 7, 8, 30, 0, 1, 2, 3, -1, 31], dtype=torch.int32, device=DEV)
    perm = torch.randperm(pages)[: S * 16].reshape(S, 16).to(torch.int32).to(DEV)
    k_pool = torch.zeros(pages * bs, nkv * d, dtype=dtype, device=DEV)
    v_pool = torch.zeros_like(k_pool)
    q_gain = (torch.rand(d, device=DEV) + 0.5).to(dtype) if norm else None
    k_gain = (torch.rand(d, device=DEV) + 0.5).to(dtype) if norm else None
    cos, sin = tables(64, d, theta)
    before = qkv.clone()
    kernels.qk_norm_rope_kv_write(qkv, q_gain, k_gain, eps, cos, sin, d, positions, seq_of, perm, bs, k_pool, v_pool,
                                  nq, nkv, d)
    x = before.double().reshape(n, nq + 2 * nkv, d)
    q, k, v = x[:, :nq], x[:, nq:nq + nkv], x[:, nq + nkv:]
    if norm:
        q = q / torch.sqrt((q * q).mean(-1, keepdim=True) + eps) * q_gain.double()
        k = k / torch.sqrt((k * k).mean(-1, keepdim=True) + eps) * k_gain.double()
    pos = positions.clamp_min(0)
    q, k = rope_ref(q, pos, theta, d), rope_ref(k, pos, theta, d)
    live = positions >= 0
    got_q = qkv.reshape(n, nq + 2 * nkv, d)[:, :nq]
    assert rel(got_q[live], q[live]) < tol(dtype)
    assert torch.equal(got_q[~live], before.reshape(n, -1, d)[:, :nq][~live]), "a padding row is left alone"
    for t in range(n):
        if positions[t] < 0:
            continue
        p = int(positions[t])
        slot = int(perm[int(seq_of[t]), p // bs]) * bs + p % bs
        assert rel(k_pool[slot].reshape(nkv, d), k[t]) < tol(dtype)
        assert torch.equal(v_pool[slot].reshape(nkv, d), before.reshape(n, -1, d)[t, nq + nkv:]), "v is copied as it is"
    written = {int(perm[int(seq_of[t]), int(positions[t]) // bs]) * bs + int(positions[t]) % bs
               for t in range(n) if positions[t] >= 0}
    untouched = torch.ones(pages * bs, dtype=torch.bool)
    untouched[list(written)] = False
    assert not k_pool[untouched.to(DEV)].any() and not v_pool[untouched.to(DEV)].any(), "nothing else was written"
    # without the cache write only q changes
    k2, v2 = torch.zeros_like(k_pool), torch.zeros_like(v_pool)
    again = before.clone()
    kernels.qk_norm_rope_kv_write(again, q_gain, k_gain, eps, cos, sin, d, positions, seq_of, perm, bs, k2, v2,
                                  nq, nkv, d, write_kv=False)
    assert not k2.any() and not v2.any()
    assert torch.equal(again.reshape(n, -1, d)[:, :nq], got_q)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,rot", [(4, 2, 128, 128), (3, 1, 48, 32), (2, 2, 20, 20)])
def test_rotation_of_neighbouring_elements(dtype, nq, nkv, d, rot):
    """The other layout of rotary checkpoints: angle i turns the elements 2 i and 2 i + 1.  Rotating halves after
    gathering the even elements before the odd ones is the same thing, which is how it is checked."""
    from paged_llm_rs_amd import kernels

    n, bs = 5, 4
    qkv = torch.randn(n, (nq + 2 * nkv) * d, device=DEV).to(dtype)
    positions = torch.tensor([0, 3, 9, 14, 15], dtype=torch.int32, device=DEV)
    seq_of = torch.zeros(n, dtype=torch.int32, device=DEV)
    bt = torch.arange(4, dtype=torch.int32, device=DEV).reshape(1, 4)
    kp = torch.zeros(16, nkv * d, dtype=dtype, device=DEV)
    vp = torch.zeros_like(kp)
    gain = (1 + 0.2 * torch.randn(d, device=DEV)).to(dtype)
    cos, sin = tables(16, rot, 1e4)
    before = qkv.clone()
    kernels.qk_norm_rope_kv_write(qkv, gain, gain, 1e-5, cos, sin, rot, positions, seq_of, bt, bs, kp, vp, nq, nkv, d,
                                  neighbours=True)
    x = before.double().reshape(n, nq + 2 * nkv, d)[:, :nq + nkv]
    x = x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * gain.double()
    order = torch.cat([torch.arange(0, rot, 2), torch.arange(1, rot, 2), torch.arange(rot, d)]).to(DEV)
    turned = rope_ref(x[..., order], positions, 1e4, rot)
    want = torch.empty_like(turned)
    want[..., order] = turned
    assert rel(qkv.reshape(n, -1, d)[:, :nq], want[:, :nq]) < tol(dtype)
    for t in range(n):
        assert rel(kp[int(positions[t])].reshape(nkv, d), want[t, nq:]) < tol(dtype)


def test_rotation_of_part_of_a_head_and_refused_sizes():
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.errors import TensorError

    n, nq, nkv, d, rot, bs = 3, 2, 1, 32, 16, 4
    qkv = torch.randn(n, (nq + 2 * nkv) * d, device=DEV)
    positions = torch.tensor([3, 4, 9], dtype=torch.int32, device=DEV)
    seq_of = torch.zeros(n, dtype=torch.int32, device=DEV)
    bt = torch.arange(4, dtype=torch.int32, device=DEV).reshape(1, 4)
    kp = torch.zeros(16, d, device=DEV)
    vp = torch.zeros(16, d, device=DEV)
    cos, sin = tables(16, rot, 1e4)
    before = qkv.clone()
    kernels.qk_norm_rope_kv_write(qkv, None, None, 0.0, cos, sin, rot, positions, seq_of, bt, bs, kp, vp, nq, nkv, d)
    want = rope_ref(before.double().reshape(n, 4, d)[:, :nq], positions, 1e4, rot)
    assert rel(qkv.reshape(n, 4, d)[:, :nq], want) < 2e-6
    assert torch.equal(qkv.reshape(n, 4, d)[:, :nq, rot:], before.reshape(n, 4, d)[:, :nq, rot:])
    with pytest.raises(TensorError, match="between 1 and 256"):
        kernels.qk_norm_rope_kv_write(torch.zeros(1, 4 * 264, device=DEV), None, None, 0.0, None, None, 0,
                                      positions[:1], seq_of[:1], bt, bs, torch.zeros(16, 264, device=DEV),
                                      torch.zeros(16, 264, device=DEV), 2, 1, 264)


# --- feed-forward ------------------------------------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_swiglu(dtype):
    from paged_llm_rs_amd import kernels

    gu = torch.randn(9, 2 * 212, device=DEV).to(dtype)
    want = torch.nn.functional.silu(gu.double()[:, :212]) * gu.double()[:, 212:]
    assert rel(kernels.swiglu(gu), want) < tol(dtype)
    assert float(kernels.swiglu(torch.zeros(1, 8, device=DEV)).abs().max()) == 0.0


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("n,N,K", [(1, 5, 3), (7, 331, 100), (70, 130, 257), (64, 64, 64), (3, 1000, 1024)])
def test_gemm_plain(dtype, n, N, K):
    from paged_llm_rs_amd import kernels

    x = torch.randn(n, K, device=DEV).to(dtype)
    w = torch.randn(N, K, device=DEV).to(dtype)
    want = x.double() @ w.double().T
    assert rel(kernels.gemm_plain(x, w), want) < (2e-6 if dtype == torch.float32 else 6e-3)
    assert rel(kernels.gemm_plain(x, w, out_dtype=torch.float32), want) < 2e-6
    # a row's result does not depend on what else is in the batch: bitwise
    alone = kernels.gemm_plain(x[:1].contiguous(), w, out_dtype=torch.float32)
    assert torch.equal(alone, kernels.gemm_plain(x, w, out_dtype=torch.float32)[:1])


@pytest.mark.parametrize("n", [1, 2, 8, 16, 17, 33, 64])
@pytest.mark.parametrize("N,K", [(16, 32), (331, 104), (4096, 1024), (1024, 3072), (50, 8), (1000, 2056)])
def test_gemm_skinny(n, N, K):
    from paged_llm_rs_amd import kernels

    x = torch.randn(n, K, device=DEV).to(torch.bfloat16)
    w = torch.randn(N, K, device=DEV).to(torch.bfloat16)
    want = x.double() @ w.double().T
    assert rel(kernels.gemm_skinny(x, w, torch.float32), want) < 1e-5, "products of bfloat16 summed in 32-bit"
    assert rel(kernels.gemm_skinny(x, w, torch.bfloat16), want) < 6e-3
    if N % 2 == 0:
        g, u = want[:, :N // 2], want[:, N // 2:]
        act = torch.nn.functional.silu(g) * u
        assert rel(kernels.gemm_skinny(x, w, swiglu=True), act) < 6e-3
    # one-hot rows pick single weights: a wrong operand layout cannot pass this
    eye = torch.zeros(min(n, K), K, device=DEV, dtype=torch.bfloat16)
    idx = torch.randperm(K)[:eye.shape[0]]
    eye[torch.arange(eye.shape[0]), idx] = 1
    assert torch.equal(kernels.gemm_skinny(eye, w, torch.bfloat16), w[:, idx].T.contiguous())


@pytest.mark.parametrize("n", [1, 8, 17, 64])
@pytest.mark.parametrize("N,K", [(48, 104), (4096, 1024), (250, 2056), (64, 3072)])
def test_gemm_skinny_with_the_norm_before_and_the_residual_after(n, N, K):
    """The norm as the product's first stage (statistic from the values the product loads, rows picked
    by a list), SwiGLU or the residual sum as its last."""
    from paged_llm_rs_amd import kernels

    eps = 1e-5
    stream = torch.randn(n + 3, K, device=DEV) * 3.0
    stream[0] *= 50.0                                         # rows of very different size: the statistic is a row's own
    gain = 1 + 0.3 * torch.randn(K, device=DEV)
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)

    def normed(rows):
        x = stream[rows].double()
        return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain.double()

    all_rows = list(range(n))
    want = normed(all_rows) @ w.double().T
    got = kernels.gemm_skinny(stream[:n].contiguous(), w, torch.float32, norm_gain=gain, eps=eps)
    assert rel(got, want) < 6e-3, "bfloat16 inputs, 32-bit sums"
    picked = [(7 * i + 2) % (n + 3) for i in range(n)]
    rows = torch.tensor(picked, dtype=torch.int32, device=DEV)
    got = kernels.gemm_skinny(stream, w, torch.bfloat16, norm_gain=gain, eps=eps, rows=rows)
    assert rel(got, normed(picked) @ w.double().T) < 1e-2
    if N % 2 == 0:
        g, u = want[:, :N // 2], want[:, N // 2:]
        got = kernels.gemm_skinny(stream[:n].contiguous(), w, swiglu=True, norm_gain=gain, eps=eps)
        assert rel(got, torch.nn.functional.silu(g) * u) < 1e-2
    # the residual sum: every element of the stream takes its own column's product, once
    x = torch.randn(n, K, device=DEV).to(torch.bfloat16)
    resid = torch.randn(n, N, device=DEV)
    want = resid.double() + x.double() @ w.double().T
    assert kernels.gemm_skinny(x, w, add_into=resid) is resid
    assert rel(resid, want) < 1e-5


@pytest.mark.parametrize("n", [1, 8, 16, 17, 40, 64])
@pytest.mark.parametrize("N,K", [(16, 32), (48, 96), (4096, 1024), (1024, 3072), (6144, 1024), (2064, 4128), (160, 16384),
                                 (32768 + 32, 512)])
def test_gemm_skinny_over_weights_in_strips(n, N, K):
    """The weights in the order the waves take them (strips of 16 rows, tiles of 1 KB): where the product reads
    them so, every variant gives bit for bit what it gives over the rows: plain, with the norm before, with
    act(gate) * up, added into the stream, with a norm taken and handed forward; one-hot rows pick single
    weights.  Where it does not read them so (tiles of rows that go to other kernels), it reads the rows and says
    so; what the layout is not defined for has none."""
    from paged_llm_rs_amd import kernels

    x = torch.randn(n, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    strips = kernels.weights_in_strips(w)
    assert strips.shape == w.shape and strips.dtype == w.dtype
    assert torch.equal(strips.flatten().sort().values, w.flatten().sort().values), "the same numbers in another order"
    def expected(columns):
        """one tile of rows a workgroup"""
        return n <= 16 or (columns // 16) * -(-n // 16) <= 512

    reads_strips = kernels.strips_apply(n, N, K)
    assert reads_strips == expected(N)
    # with zeros for the rows, the result says which of the two was read
    blind = kernels.gemm_skinny(x, torch.zeros_like(w), torch.float32, strips=strips)
    assert torch.equal(blind, kernels.gemm_skinny(x, w, torch.float32) if reads_strips else torch.zeros_like(blind))
    for out_dtype in (torch.float32, torch.bfloat16):
        assert torch.equal(kernels.gemm_skinny(x, w, out_dtype, strips=strips), kernels.gemm_skinny(x, w, out_dtype))
    a, b = torch.randn(n, N, device=DEV), None
    b = a.clone()
    kernels.gemm_skinny(x, w, add_into=a, strips=strips)
    kernels.gemm_skinny(x, w, add_into=b)
    assert torch.equal(a, b)
    if N % 32 == 0:
        assert kernels.strips_apply(n, N // 2, K) == expected(N // 2)
        for act in ("silu", "gelu_tanh"):
            assert torch.equal(kernels.gemm_skinny(x, w, swiglu=True, activation=act, strips=strips),
                               kernels.gemm_skinny(x, w, swiglu=True, activation=act))
    if K <= 4128:
        stream = torch.randn(n + 2, K, device=DEV) * 2.0
        gain = 1 + 0.3 * torch.randn(K, device=DEV)
        rows = torch.tensor([(5 * i + 1) % (n + 2) for i in range(n)], dtype=torch.int32, device=DEV)
        assert torch.equal(kernels.gemm_skinny(stream, w, norm_gain=gain, eps=1e-6, rows=rows, strips=strips),
                           kernels.gemm_skinny(stream, w, norm_gain=gain, eps=1e-6, rows=rows))
    eye, idx = one_hot_rows(min(n, K), K)
    assert torch.equal(kernels.gemm_skinny(eye, w, strips=strips), w[:, idx].T.contiguous())
    # a norm handed forward by a product over strips, and taken by one
    if kernels.hands_norm_forward(n, N, K) and N <= 2048:
        gain = 1 + 0.3 * torch.randn(N, device=DEV)
        outs = []
        for s in (strips, None):
            hand = kernels.HandedNorm(gain, 1e-6, n, N, DEV)
            resid = torch.ones(n, N, device=DEV)
            kernels.gemm_skinny(x, w, add_into=resid, hand=hand, strips=s)
            outs.append((resid, hand.x.clone(), hand.ssq.clone()))
        assert all(torch.equal(p, q) for p, q in zip(*outs))
        w2 = (torch.randn(64, N, device=DEV) / math.sqrt(N)).bfloat16()
        if kernels.takes_handed_norm(n, 64, N, False):
            assert torch.equal(kernels.gemm_skinny(None, w2, handed=hand, strips=kernels.weights_in_strips(w2)),
                               kernels.gemm_skinny(None, w2, handed=hand))
    assert kernels.weights_in_strips(w[:N - 8]) is None and kernels.weights_in_strips(w[:, :K - 8].contiguous()) is None
    assert kernels.weights_in_strips(w.float()) is None


def one_hot_rows(n, K):
    """Rows that pick single columns of a weight matrix, and the columns they pick."""
    eye = torch.zeros(n, K, device=DEV, dtype=torch.bfloat16)
    idx = torch.randint(0, K, (n,), device=DEV)
    eye[torch.arange(n, device=DEV), idx] = 1
    return eye, idx


@pytest.mark.parametrize("N", [32768, 32784, 151936])
@pytest.mark.parametrize("K", [512, 1024, 4096, 5120])
def test_gemm_skinny_against_more_columns_than_a_launch_has_workgroups(N, K):
    """Beyond 32,768 columns a workgroup walks several tiles of columns and uses its LDS again for each:
    the projection onto a real vocabulary does so in every decode step.  One-hot rows pick single
    weights, so a tile that is dropped, written twice or mixed with its neighbour cannot pass."""
    from paged_llm_rs_amd import kernels

    w = torch.randn(N, K, device=DEV).to(torch.bfloat16)
    w64 = w.double()
    for n in (1, 8, 16, 17, 33, 64):
        x = torch.randn(n, K, device=DEV).to(torch.bfloat16)
        want = x.double() @ w64.T
        assert rel(kernels.gemm_skinny(x, w, torch.float32), want) < 1e-5, f"{n} rows, 32-bit out"
        assert rel(kernels.gemm_skinny(x, w, torch.bfloat16), want) < 6e-3, f"{n} rows, bfloat16 out"
        eye, idx = one_hot_rows(n, K)
        picked = w[:, idx].T.contiguous()
        assert torch.equal(kernels.gemm_skinny(eye, w, torch.bfloat16), picked), f"{n} one-hot rows"
        assert torch.equal(kernels.gemm_skinny(eye, w, torch.float32), picked.float()), f"{n} one-hot rows, 32-bit out"
    # the gated product's tiles are pairs of column tiles: its loop starts at 65,536 rows of w
    if N % 2 == 0:
        for n in (1, 17, 64):
            x = (torch.randn(n, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
            both = x.double() @ w64.T
            act = torch.nn.functional.silu(both[:, :N // 2]) * both[:, N // 2:]
            assert rel(kernels.gemm_skinny(x, w, swiglu=True), act) < 6e-3, f"{n} rows, gated"


@pytest.mark.parametrize("N", [32784, 151936])
@pytest.mark.parametrize("K", [512, 1024, 4096])
def test_gemm_skinny_with_the_norm_before_against_many_columns(N, K):
    """The norm as the first stage of a product that walks its column tiles: the gains and the rows'
    statistics have to outlast every tile (K = 512 is where gains and statistics once shared LDS)."""
    from paged_llm_rs_amd import kernels

    eps = 1e-5
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    w64 = w.double()
    gain = 1 + 0.3 * torch.randn(K, device=DEV)
    for n in (1, 8, 17, 33, 64):
        stream = torch.randn(n + 3, K, device=DEV) * 3.0
        stream[0] *= 50.0
        picked = [(7 * i + 2) % (n + 3) for i in range(n)]
        x = stream[picked].double()
        normed = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * gain.double()
        rows = torch.tensor(picked, dtype=torch.int32, device=DEV)
        got = kernels.gemm_skinny(stream, w, torch.float32, norm_gain=gain, eps=eps, rows=rows)
        # the kernel multiplies bf16(x * gain) and scales afterwards: compare with exactly that, tightly ...
        exact = (x.float() * gain).to(torch.bfloat16).double() @ w64.T / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
        assert rel(got, exact) < 1e-5, f"{n} rows against the kernel's own rounding"
        # ... and with the unrounded norm at bfloat16's precision
        assert rel(got, normed @ w64.T) < 6e-3, f"{n} rows"


@pytest.mark.parametrize("M,K", [(65, 1024), (300, 1024), (2048, 1024), (70, 4096), (300, 5120)])
def test_the_librarys_projection_onto_a_real_vocabulary(M, K):
    """More than 64 rows against 151,936 columns go to the library with 32-bit output
    (``linear_bf16``): compared with 64-bit products, not with the library itself."""
    from paged_llm_rs_amd import kernels

    N = 151936
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).to(torch.bfloat16)
    x = torch.randn(M, K, device=DEV).to(torch.bfloat16)
    got = kernels.linear_bf16(x, w, torch.float32)
    assert got.dtype == torch.float32 and got.shape == (M, N)
    assert rel(got, x.double() @ w.double().T) < 1e-5
    eye, idx = one_hot_rows(M, K)
    assert torch.equal(kernels.linear_bf16(eye, w, torch.float32), w[:, idx].T.float().contiguous())


@pytest.mark.parametrize("n", [1, 8, 16, 17, 33, 48, 64])
@pytest.mark.parametrize("N,K", [(48, 136), (130, 256), (1000, 384), (129, 4096), (514, 2056), (2048, 128), (16, 8)])
@pytest.mark.parametrize("splits", [1, 3, 16])
def test_gemm_stream(n, N, K, splits):
    """The product that streams a large weight matrix, at small and odd sizes (columns that are no multiple
    of a workgroup's 128, a K that is no multiple of a chunk's 128), whole and with K cut between workgroups,
    with each of its last stages, against 64-bit products of the same bfloat16 numbers."""
    from paged_llm_rs_amd import kernels

    x = torch.randn(n, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    want = x.double() @ w.double().T
    assert rel(kernels.gemm_stream(x, w, torch.float32, splits=splits), want) < 1e-5, "products of bfloat16 summed in 32-bit"
    assert rel(kernels.gemm_stream(x, w, splits=splits), want) < 6e-3
    stream = torch.randn(n, N, device=DEV)
    before = stream.clone()
    assert kernels.gemm_stream(x, w, add_into=stream, splits=splits) is stream
    assert rel(stream.double() - before.double(), want) < 1e-5
    if N % 2 == 0:
        act = torch.nn.functional.silu(want[:, :N // 2]) * want[:, N // 2:]
        got = kernels.gemm_stream(x, w, swiglu=True, splits=splits)
        assert got.shape == (n, N // 2) and rel(got, act) < 6e-3
        gelu = torch.nn.functional.gelu(want[:, :N // 2], approximate="tanh") * want[:, N // 2:]
        assert rel(kernels.gemm_stream(x, w, swiglu=True, activation="gelu_tanh", splits=splits), gelu) < 6e-3
    # one-hot rows pick single weights: a wrong operand layout cannot pass this
    eye, idx = one_hot_rows(min(n, K), K)
    assert torch.equal(kernels.gemm_stream(eye, w, splits=splits), w[:, idx].T.contiguous())
    # a row's result does not depend on what else is in the batch, nor a call's on the call before: bitwise
    alone = kernels.gemm_stream(x[:1].contiguous(), w, torch.float32, splits=splits)
    assert torch.equal(alone, kernels.gemm_stream(x, w, torch.float32, splits=splits)[:1])


@pytest.mark.parametrize("n,N,K", [(24, 2048, 8192), (64, 1024, 25600), (40, 151936, 1024), (8, 1024, 8192)])
def test_gemm_stream_at_sizes_where_it_is_chosen(n, N, K):
    """Deep products and the projection onto a large vocabulary, the shapes this kernel is there for: its own
    choice of stretches, against the 32-bit product of the same numbers, eager and replayed from a graph."""
    from paged_llm_rs_amd import kernels

    x = torch.randn(n, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    want = x.float() @ w.float().T
    got = kernels.gemm_stream(x, w, torch.float32)
    assert rel(got, want) < 1e-5
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kernels.gemm_stream(x, w, torch.float32)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = kernels.gemm_stream(x, w, torch.float32)
    for replay in range(3):
        x.copy_(torch.randn(n, K, device=DEV).bfloat16())
        eager = kernels.gemm_stream(x, w, torch.float32).clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {replay} differs from the eager product"


@pytest.mark.parametrize("M,N,K,splits", [(70, 96, 256, 2), (576, 512, 3072, 4), (1000, 130, 1032, 3), (300, 1024, 12288, 4)])
def test_a_deep_product_as_a_batch_of_stretches(M, N, K, splits):
    """The library's product over stretches of K as one batch, and the sum of the 32-bit partial results by the
    kernel that ends the streamed product: stored and added into the stream, eager and replayed from a graph."""
    from paged_llm_rs_amd import kernels

    x = torch.randn(M, K, device=DEV).bfloat16()
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    want = x.double() @ w.double().T
    assert rel(kernels.gemm_split_library(x, w, splits, torch.float32), want) < 1e-5
    assert rel(kernels.gemm_split_library(x, w, splits), want) < 6e-3
    stream = torch.randn(M, N, device=DEV)
    before = stream.clone()
    assert kernels.gemm_split_library(x, w, splits, add_into=stream) is stream
    assert rel(stream.double() - before.double(), want) < 1e-5
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        kernels.gemm_split_library(x, w, splits, torch.float32)
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = kernels.gemm_split_library(x, w, splits, torch.float32)
    other = torch.randn(256, 256, device=DEV)
    for replay in range(3):
        x.copy_(torch.randn(M, K, device=DEV).bfloat16())
        float((other @ other).sum())
        eager = kernels.gemm_split_library(x, w, splits, torch.float32).clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, eager), f"replay {replay} differs from the eager product"
    assert kernels.library_splits(576, 4096, 12288) == 4 and kernels.library_splits(1088, 5120, 25600) == 2
    assert kernels.library_splits(2048, 4096, 12288) == 1 and kernels.library_splits(576, 1024, 3072) == 1
    assert kernels.library_splits(64, 4096, 12288) == 1 and kernels.library_splits(576, 6144, 4096) == 1


def test_gemm_stream_refusals_and_where_it_is_chosen():
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.errors import TensorError

    with pytest.raises(TensorError, match="multiple of 8"):
        kernels.gemm_stream(torch.zeros(2, 100, device=DEV, dtype=torch.bfloat16),
                            torch.zeros(5, 100, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(TensorError, match="64 at most"):
        kernels.gemm_stream(torch.zeros(65, 64, device=DEV, dtype=torch.bfloat16),
                            torch.zeros(5, 64, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(TensorError, match="stretches"):
        kernels.gemm_stream(torch.zeros(4, 64, device=DEV, dtype=torch.bfloat16),
                            torch.zeros(5, 64, device=DEV, dtype=torch.bfloat16), splits=17)
    # a deep product over a large matrix and the vocabulary from 17 rows on are this kernel's; small
    # matrices, wide products of moderate depth and anything beyond 64 rows are not
    assert kernels.stream_wins(64, 5120, 25600) and kernels.stream_wins(8, 5120, 25600)
    assert kernels.stream_wins(32, 151936, 1024) and not kernels.stream_wins(16, 151936, 1024)
    assert not kernels.stream_wins(64, 1024, 3072) and not kernels.stream_wins(64, 51200, 5120)
    assert not kernels.stream_wins(64, 151936, 5120)
    assert not kernels.stream_wins(65, 5120, 25600) and not kernels.stream_wins(8, 4096, 12288)
    assert not kernels.skinny_wins(8, 5120, 25600), "one product, one kernel"


@pytest.mark.parametrize("M", [1, 127, 128, 300, 2048])
@pytest.mark.parametrize("N,K", [(128, 32), (256, 96), (1024, 1024), (384, 2080)])
@pytest.mark.parametrize("kind", ["store", "swiglu", "add"])
def test_gemm_tiled(M, N, K, kind):
    """The product for many rows, with its fused last stages, against 64-bit products of the same bfloat16 numbers."""
    from paged_llm_rs_amd import kernels

    x = (torch.randn(M, K, device=DEV) * 0.5).bfloat16()
    if kind == "swiglu":
        w = (torch.randn(2 * N, K, device=DEV) / math.sqrt(K)).bfloat16()
        both = x.double() @ w.double().t()
        want = torch.nn.functional.silu(both[:, :N]) * both[:, N:]
        got = kernels.gemm_tiled(x, w, swiglu=True)
        assert got.dtype == torch.bfloat16 and got.shape == (M, N)
        assert rel(got, want) < 6e-3
        return
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    want = x.double() @ w.double().t()
    if kind == "store":
        assert rel(kernels.gemm_tiled(x, w), want) < 4e-3      # one rounding to bfloat16
    else:
        stream = torch.randn(M, N, device=DEV)
        before = stream.clone()
        assert kernels.gemm_tiled(x, w, add_into=stream) is stream
        assert rel(stream.double() - before.double(), want) < 1e-5


def test_gemm_tiled_refusals():
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.errors import TensorError

    assert not kernels.gemm_tiled_applies(64, 100, 64) and not kernels.gemm_tiled_applies(64, 128, 40)
    assert kernels.gemm_tiled_applies(64, 192, 64, swiglu=True) and not kernels.gemm_tiled_applies(64, 192, 64)
    x = torch.zeros(4, 40, device=DEV, dtype=torch.bfloat16)
    with pytest.raises(TensorError):
        kernels.gemm_tiled(x, torch.zeros(128, 40, device=DEV, dtype=torch.bfloat16))


@pytest.mark.parametrize("M,N,K,out_dtype", [(576, 6144, 4096, None), (2048, 24576, 4096, None), (2048, 4096, 12288, None),
                                             (40, 151936, 1024, torch.float32), (300, 3001, 2560, torch.float32)])
def test_library_products_in_a_captured_graph_replay_like_the_eager_ones(M, N, K, out_dtype):
    """The library's products stand inside captured steps (large weights, many rows, the projection onto the
    vocabulary).  Some of its kernels clear a workspace first, and a clearing node in a graph is what has
    given wrong replays on this chip: every replay, with eager work and a synchronisation between, has to
    give the bits of the eager product."""
    w = (torch.randn(N, K, device=DEV) / math.sqrt(K)).bfloat16()
    x = torch.randn(M, K, device=DEV).bfloat16()
    other = torch.randn(512, 512, device=DEV)

    def product():
        return torch.mm(x, w.t()) if out_dtype is None else torch.mm(x, w.t(), out_dtype=out_dtype)

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        product()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        y = product()
    for replay in range(4):
        x.copy_(torch.randn(M, K, device=DEV).bfloat16())
        float((other @ other).sum())
        want = product().clone()
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y, want), f"replay {replay} differs from the eager product"


def test_gemm_skinny_refusals():
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.errors import TensorError

    with pytest.raises(TensorError, match="multiple of 8"):
        kernels.gemm_skinny(torch.zeros(2, 100, device=DEV, dtype=torch.bfloat16),
                            torch.zeros(5, 100, device=DEV, dtype=torch.bfloat16))
    with pytest.raises(TensorError, match="up to 64"):
        kernels.gemm_skinny(torch.zeros(65, 64, device=DEV, dtype=torch.bfloat16),
                            torch.zeros(5, 64, device=DEV, dtype=torch.bfloat16))


# --- attention ------------------------------------------------------------------------------------------------

def build_paged(nkv, d, bs, ctx_lens, dtype, seed=0, pages_extra=7):
    """Random keys and values for requests of the given lengths, scattered over shuffled pages."""
    g = torch.Generator().manual_seed(seed)
    S = len(ctx_lens)
    need = [(c + bs - 1) // bs for c in ctx_lens]
    pages = sum(need) + pages_extra
    order = torch.randperm(pages, generator=g).tolist()
    max_blocks = max(need) + 2
    bt = torch.full((S, max_blocks), -1, dtype=torch.int32)
    k_pool = torch.randn(pages * bs, nkv * d, generator=g).to(dtype)
    v_pool = torch.randn(pages * bs, nkv * d, generator=g).to(dtype)
    keys, values = [], []
    at = 0
    used = torch.zeros(pages * bs, dtype=torch.bool)
    for s, c in enumerate(ctx_lens):
        for b in range(need[s]):
            bt[s, b] = order[at]
            at += 1
        slots = [int(bt[s, p // bs]) * bs + p % bs for p in range(c)]
        used[slots] = True
        keys.append(k_pool[slots].reshape(c, nkv, d).double())
        values.append(v_pool[slots].reshape(c, nkv, d).double())
    # Every row that belongs to no request (the rest of a last page, pages that are free) holds what a
    # page's last owner may have left there: infinities, NaNs and the largest finite numbers.
    k_pool[~used] = poison_rows(int((~used).sum()), nkv * d, dtype)
    v_pool[~used] = poison_rows(int((~used).sum()), nkv * d, dtype)
    return bt.to(DEV), k_pool.to(DEV), v_pool.to(DEV), keys, values


def give_back_pages_behind_the_window(bt, k_pool, v_pool, bs, requests, window):
    """What a windowed cache group does: the pages that lie wholly before the window of a request's first
    token of the step are no longer the request's (-1 in its table) and hold anything."""
    if not window:
        return
    for s, (ctx, count) in enumerate(requests):
        first_needed = max(0, ctx - count + 1 - window)
        for b in range(first_needed // bs):
            page = int(bt[s, b])
            for pool in (k_pool, v_pool):
                pool[page * bs:(page + 1) * bs] = poison_rows(bs, pool.shape[1], pool.dtype).to(pool.device)
            bt[s, b] = -1


def same_bits(a, b):
    """Equal bit for bit, NaNs included."""
    as_int = torch.int16 if a.element_size() == 2 else torch.int32
    return a.shape == b.shape and torch.equal(a.view(as_int), b.view(as_int))


def poison_rows(rows, width, dtype):
    pattern = torch.tensor([float("inf"), float("nan"), 3e38, float("-inf")])
    at = (torch.arange(rows)[:, None] + torch.arange(width)[None]) % 4
    return pattern[at].to(dtype)


def attention_ref(q, keys, values, pos, g, scale, window):
    """q [nq, d] float64 at position pos against keys/values [ctx, nkv, d]."""
    out = []
    first = max(0, pos + 1 - window) if window else 0
    for h in range(q.shape[0]):
        k = keys[first:pos + 1, h // g]
        v = values[first:pos + 1, h // g]
        p = torch.softmax(k @ q[h] * scale, dim=0)
        out.append(p @ v)
    return torch.stack(out)


ATTENTION_CASES = [
    # nq, nkv, d, block size, context lengths, window
    (4, 2, 16, 4, [1, 5, 33], 0),
    (6, 1, 32, 8, [70, 9], 0),
    (6, 2, 48, 16, [100, 17, 64], 0),
    (16, 8, 128, 16, [513, 40], 0),
    (8, 1, 64, 16, [200, 129], 0),
    (3, 3, 80, 2, [37, 12], 0),
    (12, 2, 112, 16, [90], 0),
    (32, 2, 128, 16, [300], 0),
    (4, 2, 256, 16, [77, 150], 0),
    (4, 2, 64, 16, [300, 31], 48),
    (2, 2, 16, 4, [50], 7),
    (16, 8, 128, 128, [513, 40], 0),
    (8, 2, 64, 64, [300], 100),
]


@pytest.mark.parametrize("kernel", ["plain-f32", "plain-bf16", "decode-1", "decode-3", "decode-8"])
@pytest.mark.parametrize("nq,nkv,d,bs,ctx_lens,window", ATTENTION_CASES)
def test_paged_attention_of_single_tokens(kernel, nq, nkv, d, bs, ctx_lens, window):
    from paged_llm_rs_amd import kernels

    dtype = torch.float32 if kernel == "plain-f32" else torch.bfloat16
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=d + bs)
    # several tokens a request, at its end and in its middle, plus a padding row
    toks = []
    for s, c in enumerate(ctx_lens):
        for p in sorted({c - 1, c // 2, 0, min(c - 1, bs), max(0, c - 2)}):
            toks.append((s, p))
    n = len(toks) + 1
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    positions = torch.tensor([p for _, p in toks] + [-1], dtype=torch.int32, device=DEV)
    seq_of = torch.tensor([s for s, _ in toks] + [0], dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    if kernel.startswith("plain"):
        kernels.paged_attention_plain(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d, scale, window)
    else:
        kernels.paged_attention_decode(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d, scale,
                                       window, splits=int(kernel.split("-")[1]))
    g = nq // nkv
    for i, (s, p) in enumerate(toks):
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s], values[s], p, g, scale, window)
        err = rel(out[i].reshape(nq, d), want)
        assert err < (2e-6 if dtype == torch.float32 else 1e-2), f"token {i} (request {s}, position {p}): {err:.3e}"
    assert bool((out[-1] == 7.0).all()), "a padding row is not written"


@pytest.mark.parametrize("splits", [1, 2])
@pytest.mark.parametrize("bs,ctx,window", [(1, 2600, 0), (2, 5001, 0), (1, 2600, 2300)])
def test_single_tokens_over_more_pages_than_the_kernel_keeps_at_hand(bs, ctx, window, splits):
    """The single-token kernel copies the page numbers of a workgroup's stretch of keys into LDS, 2,048 of them
    at most; a longer stretch (small pages, one share) looks each page up in the table.  Both ways, beside each
    other in one launch (the second request is short), against 64-bit arithmetic; one key far back carries
    nearly all the weight of the long request's last token, so that a page looked up wrongly shows."""
    from paged_llm_rs_amd import kernels

    nq, nkv, d = 4, 2, 64
    dtype = torch.bfloat16
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, [ctx, 37], dtype, seed=ctx + bs)
    toks = [(0, ctx - 1), (0, ctx // 2), (0, 2047 * bs), (0, 2048 * bs), (1, 36), (1, 0)]
    stride = (nq + 2 * nkv) * d
    q = torch.randn(len(toks), stride, device=DEV).to(dtype)
    target = ctx - 2200                      # (inside the window where there is one)
    slot = int(bt[0, target // bs]) * bs + target % bs
    for kvh in range(nkv):
        k_pool[slot, kvh * d:(kvh + 1) * d] = (q[0, kvh * 2 * d: kvh * 2 * d + d].float() * 4).to(dtype)
        keys[0][target, kvh] = k_pool[slot, kvh * d:(kvh + 1) * d].double().cpu()
    positions = torch.tensor([p for _, p in toks], dtype=torch.int32, device=DEV)
    seq_of = torch.tensor([s for s, _ in toks], dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    out = torch.zeros(len(toks), nq * d, dtype=dtype, device=DEV)
    kernels.paged_attention_decode(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d, scale, window,
                                   splits=splits)
    for i, (s, p) in enumerate(toks):
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s], values[s], p, nq // nkv, scale, window)
        assert rel(out[i].reshape(nq, d), want) < 1e-2, f"token {i} (request {s}, position {p})"
    assert rel(out[0].reshape(nq, d)[0], values[0][target, 0]) < 0.2, "the far key's value is the answer"


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("nq,nkv,d,bs,ctx_lens,window", [(3, 1, 24, 4, [37, 5], 0), (4, 2, 10, 8, [70], 0),
                                                          (2, 2, 100, 16, [130, 20], 33), (5, 5, 1, 2, [9], 0)])
def test_the_plain_attention_kernel_takes_any_head_size(dtype, nq, nkv, d, bs, ctx_lens, window):
    """The plain kernel (the 32-bit path's, and the others' check) has no width it works in units of."""
    from paged_llm_rs_amd import kernels

    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=d)
    toks = [(s, p) for s, c in enumerate(ctx_lens) for p in sorted({c - 1, c // 2, 0})]
    n = len(toks)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    positions = torch.tensor([p for _, p in toks], dtype=torch.int32, device=DEV)
    seq_of = torch.tensor([s for s, _ in toks], dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    kernels.paged_attention_plain(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d, scale, window)
    for i, (s, p) in enumerate(toks):
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s], values[s], p, nq // nkv, scale, window)
        assert rel(out[i].reshape(nq, d), want) < (2e-6 if dtype == torch.float32 else 1e-2), f"token {i}"


@pytest.mark.parametrize("kernel", ["plain", "decode", "grouped-1", "grouped-4"])
def test_a_far_key_among_hundreds_is_found(kernel):
    """Random scores hide a lost key; here one key far back (just across a page edge,
    then just inside a window's edge) carries nearly all the weight, and its value is the answer."""
    from paged_llm_rs_amd import kernels

    nq, nkv, d, bs = 4, 2, 64, 16
    dtype = torch.bfloat16
    for ctx, target, window in [(700, 16, 0), (700, 15, 0), (700, 699, 0), (700, 0, 0), (700, 700 - 100, 100),
                                (700, 700 - 101, 100)]:
        bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, [ctx], dtype, seed=ctx + target)
        stride = (nq + 2 * nkv) * d
        q = torch.randn(1, stride, device=DEV).to(dtype)
        slot = int(bt[0, target // bs]) * bs + target % bs
        for kvh in range(nkv):
            k_pool[slot, kvh * d:(kvh + 1) * d] = (q[0, kvh * 2 * d: kvh * 2 * d + d].float() * 4).to(dtype)
            keys[0][target, kvh] = k_pool[slot, kvh * d:(kvh + 1) * d].double().cpu()
        positions = torch.tensor([ctx - 1], dtype=torch.int32, device=DEV)
        seq_of = torch.zeros(1, dtype=torch.int32, device=DEV)
        out = torch.zeros(1, nq * d, dtype=dtype, device=DEV)
        scale = 1 / math.sqrt(d)
        if kernel == "plain":
            kernels.paged_attention_plain(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d, scale, window)
        elif kernel == "decode":
            kernels.paged_attention_decode(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d,
                                           scale, window, splits=4)
        else:
            one = torch.ones(1, dtype=torch.int32, device=DEV)
            kernels.paged_attention_grouped(q, stride, out, seq_of, one, one * ctx, 1, bt, bs, k_pool, v_pool, nq, nkv, d,
                                            scale, window, splits=int(kernel.split("-")[1]))
        want = attention_ref(q[0, :nq * d].double().cpu().reshape(nq, d), keys[0], values[0], ctx - 1, 2, scale, window)
        assert rel(out[0].reshape(nq, d), want) < 1e-2, (ctx, target, window)
        inside = window == 0 or target > ctx - 1 - window
        hit = rel(out[0].reshape(nq, d)[0], values[0][target, 0]) < 0.2
        assert hit == inside, f"key {target} of {ctx} with window {window}: found {hit}, visible {inside}"


@pytest.mark.parametrize("nq,nkv,d,bs,ctx_lens,window,rot,norm", [
    (16, 8, 128, 16, [513, 40, 1], 0, 128, True), (6, 1, 32, 8, [70, 9], 0, 32, True), (6, 2, 48, 16, [100, 17, 64], 0, 32, False),
    (4, 2, 64, 16, [300, 31], 48, 64, True), (32, 2, 128, 16, [300], 0, 128, True), (3, 3, 80, 2, [37, 12], 0, 0, True),
    (4, 2, 64, 1, [2300, 5], 0, 64, True)])     # (more pages than the kernel copies into LDS: looked up in the table)
@pytest.mark.parametrize("splits", [1, 3])
def test_decode_attention_that_prepares_its_own_queries_and_keys(nq, nkv, d, bs, ctx_lens, window, rot, norm, splits):
    """One token a request: the norm, the rotation and the cache write inside the attention kernel give what
    the stand-alone kernel followed by attention gives, in the output and in the pages."""
    from paged_llm_rs_amd import kernels

    dtype = torch.bfloat16
    bt, k_pool, v_pool, _, _ = build_paged(nkv, d, bs, ctx_lens, dtype, seed=d + bs + rot)
    n = len(ctx_lens) + 1
    stride = (nq + 2 * nkv) * d
    raw = torch.randn(n, stride, device=DEV).to(dtype)
    positions = torch.tensor([c - 1 for c in ctx_lens] + [-1], dtype=torch.int32, device=DEV)
    seq_of = torch.tensor(list(range(len(ctx_lens))) + [0], dtype=torch.int32, device=DEV)
    q_gain = (1 + 0.2 * torch.randn(d, device=DEV)).to(dtype) if norm else None
    k_gain = (1 + 0.2 * torch.randn(d, device=DEV)).to(dtype) if norm else None
    cos = sin = None
    if rot:
        angle = torch.arange(600, dtype=torch.float64)[:, None] * (1.0 / 10000 ** (torch.arange(rot // 2, dtype=torch.float64) * 2 / rot))
        cos, sin = angle.cos().float().to(DEV), angle.sin().float().to(DEV)
    scale = 1 / math.sqrt(d)
    apart, k_a, v_a = raw.clone(), k_pool.clone(), v_pool.clone()
    kernels.qk_norm_rope_kv_write(apart, q_gain, k_gain, 1e-5, cos, sin, rot, positions, seq_of, bt, bs, k_a, v_a, nq, nkv, d)
    want = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    kernels.paged_attention_decode(apart, stride, want, positions, seq_of, bt, bs, k_a, v_a, nq, nkv, d, scale, window, splits)
    got = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    k_b, v_b = k_pool.clone(), v_pool.clone()
    kernels.paged_attention_decode(raw, stride, got, positions, seq_of, bt, bs, k_b, v_b, nq, nkv, d, scale, window, splits,
                                   fuse=kernels.QkFusion(q_gain, k_gain, 1e-5, cos, sin, rot, True))
    assert same_bits(k_a, k_b) and same_bits(v_a, v_b), "the same keys and values in the same places"
    # The outputs are bfloat16 and the probabilities are rounded to bfloat16 before they meet the values; the
    # token's own key enters first and unrounded here, last and rounded there.  One unit in the last place of
    # the largest element (2^-7 of it) is what two such sums may differ by.
    assert rel(got[:-1], want[:-1]) < 8e-3
    assert bool((got[-1] == 7.0).all()), "a padding row is not written"
    # queries only: a layer that reads pages another layer wrote
    again = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    kernels.paged_attention_decode(raw, stride, again, positions, seq_of, bt, bs, k_a, v_a, nq, nkv, d, scale, window, splits,
                                   fuse=kernels.QkFusion(q_gain, k_gain, 1e-5, cos, sin, rot, False))
    assert rel(again[:-1], want[:-1]) < 8e-3


PORTION_CASES = [
    # nq, nkv, d, block size, [(context length after the step, tokens of the step)], window
    (4, 2, 16, 4, [(40, 40), (70, 17), (5, 1)], 0),
    (6, 1, 32, 8, [(200, 130), (9, 9)], 0),
    (6, 2, 48, 16, [(150, 64), (33, 33), (64, 16)], 0),
    (16, 8, 128, 16, [(513, 300), (40, 2), (129, 129)], 0),
    (3, 3, 80, 2, [(97, 65)], 0),
    (4, 2, 112, 16, [(260, 129)], 0),
    (2, 1, 256, 16, [(150, 77)], 0),
    (4, 2, 64, 16, [(300, 140), (31, 31)], 48),
    (2, 2, 16, 4, [(90, 70)], 7),
    (2, 2, 32, 16, [(500, 200)], 64),
    (16, 8, 128, 64, [(513, 300), (129, 129)], 0),
    (8, 2, 64, 256, [(700, 200), (40, 17)], 0),
]


@pytest.mark.parametrize("splits", [1, 3, 16])
@pytest.mark.parametrize("nq,nkv,d,bs,requests,window", PORTION_CASES)
def test_paged_attention_of_portions(nq, nkv, d, bs, requests, window, splits):
    """The tiled kernel takes the requests that bring 16 tokens or more, the single-token kernel
    the others; together they fill every row of the step.  The keys of a token tile may be dealt to
    several workgroups (more of them than there are key tiles, too)."""
    from paged_llm_rs_amd import kernels

    dtype = torch.bfloat16
    ctx_lens = [c for c, _ in requests]
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=d + bs + len(requests))
    give_back_pages_behind_the_window(bt, k_pool, v_pool, bs, requests, window)
    n = sum(c for _, c in requests)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    q_start, q_len, positions, seq_of = [], [], [], []
    for s, (ctx, count) in enumerate(requests):
        q_start.append(len(positions))
        q_len.append(count)
        positions += list(range(ctx - count, ctx))
        seq_of += [s] * count
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    q_start_t, q_len_t, ctx_t = as_i32(q_start), as_i32(q_len), as_i32(ctx_lens)
    scale = 1 / math.sqrt(d)
    out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    limit = kernels.SHORT_PORTION
    kernels.paged_attention_prefill(q, stride, out, q_start_t, q_len_t, ctx_t, max(q_len), bt, bs, k_pool, v_pool,
                                    nq, nkv, d, scale, window, short_limit=limit, splits=splits)
    for s, (ctx, count) in enumerate(requests):
        if count < limit:
            rows = out[q_start[s]:q_start[s] + count]
            assert bool((rows == 7.0).all()), "a short request is left to the other kernel"
    # the launch has workgroups for the tokens of the short requests only when it is told how many there are at most
    few = sum(c for c in q_len if c < limit)
    again = out.clone()
    kernels.paged_attention_decode(q, stride, out, as_i32(positions), as_i32(seq_of), bt, bs, k_pool, v_pool, nq, nkv, d,
                                   scale, window, splits=2, q_len=q_len_t, short_limit=limit)
    kernels.paged_attention_decode(q, stride, again, as_i32(positions), as_i32(seq_of), bt, bs, k_pool, v_pool, nq, nkv, d,
                                   scale, window, splits=2, q_len=q_len_t, short_limit=limit, live_seqs=len(requests),
                                   short_rows=few + 2)
    assert torch.equal(out, again)
    g = nq // nkv
    worst = 0.0
    for i in range(n):
        s, p = seq_of[i], positions[i]
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s], values[s], p, g, scale, window)
        err = rel(out[i].reshape(nq, d), want)
        worst = max(worst, err)
        assert err < 1e-2, f"token {i} (request {s}, position {p}): {err:.3e}"


def test_paged_attention_over_pages_beyond_four_gib_of_a_pool():
    """The byte offset of a page is a 64-bit number: a request whose pages lie behind the first 4 GiB of the
    pools (each 4.5 GiB here, untouched but for those pages) gets what it gets from the same pages at the
    pools' start, from the tiled kernel (a portion of 48 tokens) and from the single-token kernel."""
    from paged_llm_rs_amd import kernels

    dtype = torch.bfloat16
    nq, nkv, d, bs = 4, 2, 128, 16
    requests = [(210, 48), (77, 1)]
    ctx_lens = [c for c, _ in requests]
    bt, k_small, v_small, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=3)
    small_pages = k_small.shape[0] // bs
    page_bytes = bs * nkv * d * 2
    far = (4 << 30) // page_bytes + 11                       # the first page behind 4 GiB, and a few more
    big_pages = far + small_pages
    k_pool = torch.empty(big_pages * bs, nkv * d, dtype=dtype, device=DEV)
    v_pool = torch.empty(big_pages * bs, nkv * d, dtype=dtype, device=DEV)
    k_pool[far * bs:] = k_small
    v_pool[far * bs:] = v_small
    k_pool[:small_pages * bs] = poison_rows(small_pages * bs, nkv * d, dtype).to(DEV)   # what an offset cut to 32 bits would read
    v_pool[:small_pages * bs] = poison_rows(small_pages * bs, nkv * d, dtype).to(DEV)
    bt_far = torch.where(bt >= 0, bt + far, bt)
    n = sum(c for _, c in requests)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    q_start, q_len, positions, seq_of = [], [], [], []
    for s_, (ctx, count) in enumerate(requests):
        q_start.append(len(positions))
        q_len.append(count)
        positions += list(range(ctx - count, ctx))
        seq_of += [s_] * count
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    out = torch.zeros((n, nq * d), dtype=dtype, device=DEV)
    limit = kernels.SHORT_PORTION
    kernels.paged_attention_prefill(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32(ctx_lens), max(q_len), bt_far, bs,
                                    k_pool, v_pool, nq, nkv, d, scale, 0, short_limit=limit, splits=1)
    kernels.paged_attention_decode(q, stride, out, as_i32(positions), as_i32(seq_of), bt_far, bs, k_pool, v_pool, nq, nkv, d,
                                   scale, 0, splits=2, q_len=as_i32(q_len), short_limit=limit)
    g = nq // nkv
    for i in range(n):
        s_, pos = seq_of[i], positions[i]
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s_], values[s_], pos, g, scale, 0)
        err = rel(out[i].reshape(nq, d), want)
        assert err < 1e-2, f"token {i} (request {s_}, position {pos}): {err:.3e}"
    del k_pool, v_pool
    torch.cuda.empty_cache()


GROUPED_CASES = [
    # nq, nkv, d, block size, [(context length after the step, tokens of the step)], window
    (32, 8, 128, 16, [(513, 1), (40, 1), (2100, 1), (1, 1)], 0),
    (16, 4, 64, 8, [(300, 3), (70, 1), (64, 15)], 0),
    (64, 8, 128, 16, [(777, 2)], 0),
    (32, 1, 128, 32, [(200, 1), (65, 4)], 0),
    (8, 2, 64, 16, [(300, 5), (31, 1)], 48),
    (16, 4, 128, 16, [(150, 64), (90, 2), (129, 1)], 0),
    (10, 2, 128, 4, [(97, 1), (130, 2)], 0),
    (32, 4, 128, 64, [(513, 1), (300, 2)], 0),
    (16, 2, 64, 256, [(700, 3)], 100),
    # contexts around the edges of the 64-key tiles, through more tiles than the rings of LDS buffers hold
    (64, 8, 128, 16, [(63, 1), (127, 1), (128, 1), (191, 1), (192, 1), (193, 1), (384, 1), (385, 1), (449, 2)], 0),
]


@pytest.mark.parametrize("splits", [1, 3, 16])
@pytest.mark.parametrize("nq,nkv,d,bs,requests,window", GROUPED_CASES)
def test_paged_attention_with_a_group_of_heads_as_the_rows_of_a_tile(nq, nkv, d, bs, requests, window, splits):
    """Single tokens and short portions through the tiled kernel, the query heads that share a key head as
    its rows; requests of 16 tokens or more are left out and their rows untouched."""
    from paged_llm_rs_amd import kernels

    assert kernels.library().pl_paged_attention_grouped_applies(nq, nkv, d, bs)
    dtype = torch.bfloat16
    ctx_lens = [c for c, _ in requests]
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=nq + bs + len(requests))
    give_back_pages_behind_the_window(bt, k_pool, v_pool, bs, requests, window)
    n = sum(c for _, c in requests)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    q_start, q_len, positions, seq_of = [], [], [], []
    for s, (ctx, count) in enumerate(requests):
        q_start.append(len(positions))
        q_len.append(count)
        positions += list(range(ctx - count, ctx))
        seq_of += [s] * count
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    limit = kernels.SHORT_PORTION
    short = [c for c in q_len if c < limit]
    out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    scale = 1 / math.sqrt(d)
    kernels.paged_attention_grouped(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32(ctx_lens), max(short), bt, bs,
                                    k_pool, v_pool, nq, nkv, d, scale, window, short_limit=limit, splits=splits)
    g = nq // nkv
    for i in range(n):
        s, p = seq_of[i], positions[i]
        if q_len[s] >= limit:
            assert bool((out[i] == 7.0).all()), "a long request is left to the other launch"
            continue
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s], values[s], p, g, scale, window)
        err = rel(out[i].reshape(nq, d), want)
        assert err < 1e-2, f"token {i} (request {s}, position {p}): {err:.3e}"


def test_grouped_attention_refuses_what_it_does_not_serve():
    from paged_llm_rs_amd import kernels

    applies = kernels.library().pl_paged_attention_grouped_applies
    assert not applies(16, 8, 96, 16)      # a head that is neither 64 nor 128
    assert not applies(66, 2, 128, 16)     # more heads a group than a tile has rows
    assert not applies(32, 8, 128, 2)      # pages smaller than one load of a wave
    assert not applies(32, 8, 128, 24)     # no power of two
    assert not kernels.grouped_applies(32, 8, 128, 16)   # four heads a key: the vector kernel is as fast
    assert kernels.grouped_applies(64, 8, 128, 16)


@pytest.mark.parametrize("splits", [1, 4])
@pytest.mark.parametrize("nq,nkv,d,bs,requests,window", PORTION_CASES)
def test_the_tiled_kernel_takes_short_requests_too(nq, nkv, d, bs, requests, window, splits):
    """With no lower limit the tiled kernel serves every request of the step, those of one token as well."""
    from paged_llm_rs_amd import kernels

    dtype = torch.bfloat16
    requests = list(requests) + [(37, 1), (9, 3)]
    ctx_lens = [c for c, _ in requests]
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=d + bs + len(requests))
    give_back_pages_behind_the_window(bt, k_pool, v_pool, bs, requests, window)
    n = sum(c for _, c in requests)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    q_start, q_len, positions, seq_of = [], [], [], []
    for s, (ctx, count) in enumerate(requests):
        q_start.append(len(positions))
        q_len.append(count)
        positions += list(range(ctx - count, ctx))
        seq_of += [s] * count
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
    kernels.paged_attention_prefill(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32(ctx_lens), max(q_len), bt, bs,
                                    k_pool, v_pool, nq, nkv, d, scale, window, short_limit=0, splits=splits)
    g = nq // nkv
    for i in range(n):
        s, p = seq_of[i], positions[i]
        want = attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[s], values[s], p, g, scale, window)
        err = rel(out[i].reshape(nq, d), want)
        assert err < 1e-2, f"token {i} (request {s}, position {p}): {err:.3e}"


@pytest.mark.parametrize("nq,nkv,d,bs", [(4, 2, 64, 16), (16, 2, 128, 16)])
def test_attention_of_a_step_with_more_requests_than_a_wave_has_lanes(nq, nkv, d, bs):
    """150 requests, long portions at the start, in the middle and at the end among single tokens and short
    portions: the kernels count their work through the requests 64 at a time, so the count has to carry over."""
    from paged_llm_rs_amd import kernels

    dtype = torch.bfloat16
    requests = []
    for i in range(150):
        count = {0: 40, 5: 130, 70: 17, 149: 64}.get(i, 3 if i % 11 == 0 else 1)
        requests.append((count + (i * 7) % 90, count))
    ctx_lens = [c for c, _ in requests]
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, ctx_lens, dtype, seed=nq)
    n = sum(c for _, c in requests)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(dtype)
    q_start, q_len, positions, seq_of = [], [], [], []
    for s, (ctx, count) in enumerate(requests):
        q_start.append(len(positions))
        q_len.append(count)
        positions += list(range(ctx - count, ctx))
        seq_of += [s] * count
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    limit = kernels.SHORT_PORTION
    few = sum(c for c in q_len if c < limit)
    g = nq // nkv
    want = [attention_ref(q[i, :nq * d].double().cpu().reshape(nq, d), keys[seq_of[i]], values[seq_of[i]], positions[i], g,
                          scale, 0) for i in range(n)]

    def check(out, rows, what):
        for i in rows:
            err = rel(out[i].reshape(nq, d), want[i])
            assert err < 1e-2, f"{what}: token {i} (request {seq_of[i]}, position {positions[i]}): {err:.3e}"

    long_rows = [i for i in range(n) if q_len[seq_of[i]] >= limit]
    short_rows = [i for i in range(n) if q_len[seq_of[i]] < limit]
    for splits in (1, 3):
        out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
        kernels.paged_attention_prefill(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32(ctx_lens), max(q_len), bt, bs,
                                        k_pool, v_pool, nq, nkv, d, scale, 0, short_limit=limit, splits=splits)
        assert all(bool((out[i] == 7.0).all()) for i in short_rows), "short requests are left to the other kernel"
        check(out, long_rows, f"tiled, {splits} splits")
        kernels.paged_attention_decode(q, stride, out, as_i32(positions), as_i32(seq_of), bt, bs, k_pool, v_pool, nq, nkv, d,
                                       scale, 0, splits=splits, q_len=as_i32(q_len), short_limit=limit, short_rows=few + 5)
        check(out, range(n), f"tiled and single tokens, {splits} splits")
        out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
        kernels.paged_attention_prefill(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32(ctx_lens), max(q_len), bt, bs,
                                        k_pool, v_pool, nq, nkv, d, scale, 0, short_limit=0, splits=splits)
        check(out, range(n), f"tiled for all, {splits} splits")
        if kernels.library().pl_paged_attention_grouped_applies(nq, nkv, d, bs):
            out = torch.full((n, nq * d), 7.0, dtype=dtype, device=DEV)
            kernels.paged_attention_grouped(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32(ctx_lens), limit - 1, bt, bs,
                                            k_pool, v_pool, nq, nkv, d, scale, 0, short_limit=limit, splits=splits)
            check(out, short_rows, f"grouped, {splits} splits")
            assert all(bool((out[i] == 7.0).all()) for i in long_rows)


def test_a_far_key_is_found_from_inside_a_portion():
    """One key carries nearly all the weight of one query in the middle of a long portion: a key of an
    earlier step across a page edge, a key of the same step, the query's own key, and keys at a window's edge."""
    from paged_llm_rs_amd import kernels

    nq, nkv, d, bs = 4, 2, 64, 16
    dtype = torch.bfloat16
    ctx, count = 700, 333
    start = ctx - count
    for query, target, window in [(500, 16, 0), (500, 15, 0), (500, 500, 0), (500, 0, 0), (699, 698, 0),
                                  (start, start - 1, 0), (start + 127, start + 64, 0), (start + 128, start + 127, 0),
                                  (500, 401, 100), (500, 400, 100), (start + 1, start + 1 - 99, 100)]:
        bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, [ctx], dtype, seed=query + target)
        stride = (nq + 2 * nkv) * d
        q = torch.randn(count, stride, device=DEV).to(dtype)
        row = query - start
        slot = int(bt[0, target // bs]) * bs + target % bs
        for kvh in range(nkv):
            k_pool[slot, kvh * d:(kvh + 1) * d] = (q[row, kvh * 2 * d: kvh * 2 * d + d].float() * 4).to(dtype)
            keys[0][target, kvh] = k_pool[slot, kvh * d:(kvh + 1) * d].double().cpu()
        as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
        out = torch.zeros(count, nq * d, dtype=dtype, device=DEV)
        scale = 1 / math.sqrt(d)
        kernels.paged_attention_prefill(q, stride, out, as_i32([0]), as_i32([count]), as_i32([ctx]), count, bt, bs,
                                        k_pool, v_pool, nq, nkv, d, scale, window, short_limit=16)
        want = attention_ref(q[row, :nq * d].double().cpu().reshape(nq, d), keys[0], values[0], query, 2, scale, window)
        assert rel(out[row].reshape(nq, d), want) < 1e-2, (query, target, window)
        inside = target <= query and (window == 0 or target > query - window)
        hit = rel(out[row].reshape(nq, d)[0], values[0][target, 0]) < 0.2
        assert hit == inside, f"key {target} for the query at {query} with window {window}: found {hit}, visible {inside}"


# --- sampling ------------------------------------------------------------------------------------------------------

def test_argmax_first_maximum_wins():
    from paged_llm_rs_amd import kernels

    logits = torch.randn(5, 151936, device=DEV)
    logits[0, 77] = logits[0, 99999] = 50.0
    logits[1, 151935] = 60.0
    logits[2, 0] = 70.0
    logits[3] = -5.0
    got = kernels.argmax(logits).cpu().tolist()
    assert got[:4] == [77, 151935, 0, 0]
    assert got[4] == int(torch.argmax(logits[4]))
    small = torch.tensor([[1.0, 3.0, 3.0, 2.0]], device=DEV)
    assert kernels.argmax(small).item() == 1


def sampling_recipe(x, temperature, top_k, top_p, u, band=1e-5, slack=2e-5):
    """The tokens the recipe allows (reference: crates/pagedllm/src/sampler.rs): scale, order by falling
    logit and rising index, keep k, softmax, keep the head of mass top_p, walk it to u * total.  Logits
    closer than `band` may stand in either order, and sums may differ by `slack` of the total."""
    import numpy as np
    y = (x.astype(np.float32) * np.float32(1.0 / temperature)).astype(np.float64)
    order = np.lexsort((np.arange(y.size), -y))
    if top_k and top_k < y.size:
        order = order[:top_k]
    mass = np.exp(y[order] - y[order[0]])
    if top_p < 1.0:
        running = np.cumsum(mass)
        kept = int(np.searchsorted(running, top_p * running[-1], side="left")) + 1
        order, mass = order[:kept], mass[:kept]
    total = mass.sum()
    point = float(np.float32(u)) * total
    allowed = set()
    ys = y[order]
    for j, token in enumerate(order):
        before = mass[ys > ys[j] + band].sum()          # what surely stands before it
        through = mass[ys >= ys[j] - band].sum()        # what may stand before it, and itself
        if before <= point + slack * total and point - slack * total <= through:
            allowed.add(int(token))
    return allowed, set(int(t) for t in order)


def test_sampling_kernel_follows_the_recipe():
    import numpy as np
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.sampling.sampler import Rng, Sampling, sample_host

    g = torch.Generator().manual_seed(11)
    V = 15193     # not a multiple of the workgroup
    cases = [(0.7, 0, 1.0), (1.0, 50, 1.0), (1.3, 0, 0.9), (0.8, 40, 0.95), (2.0, 5, 0.5), (0.0, 0, 1.0),
             (1.0, V + 5, 1.0), (0.05, 0, 0.3), (5.0, 3000, 0.999)]
    rows, how = [], []
    for rep in range(6):
        for t, k, p in cases:
            rows.append(torch.randn(V, generator=g) * (1.0 + rep))
            how.append((t, k, p, float(torch.rand((), generator=g))))
    logits = torch.stack(rows).to(DEV)
    as_f = lambda col: torch.tensor([h[col] for h in how], dtype=torch.float32, device=DEV)
    got = kernels.sample(logits, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV), as_f(2),
                         as_f(3)).cpu().tolist()
    again = kernels.sample(logits, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV), as_f(2),
                           as_f(3)).cpu().tolist()
    assert got == again, "a row and a number give the same token on every run"
    # with the largest logits' places handed in (as behind a decoding step, whose argmax has run), the same tokens;
    # a place that is none (of a row of NaNs, or nonsense) is not believed
    spoiled = logits.clone()
    spoiled[3] = float("nan")
    hint = kernels.argmax(spoiled)
    want = kernels.sample(spoiled, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV), as_f(2), as_f(3))
    handed = kernels.sample(spoiled, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV), as_f(2),
                            as_f(3), out=hint.clone(), out_holds_largest=True)
    assert torch.equal(handed, want) and want.cpu().tolist()[:3] == got[:3] and int(want[3]) == 0
    nonsense = hint.clone()
    nonsense[5], nonsense[6] = -7, V + 3
    assert torch.equal(kernels.sample(spoiled, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV),
                                      as_f(2), as_f(3), out=nonsense, out_holds_largest=True), want)
    same_as_host = 0
    for row, (t, k, p, u) in enumerate(how):
        x = logits[row].cpu().numpy()
        if t == 0.0:
            assert got[row] == int(np.argmax(x))
            continue
        allowed, kept = sampling_recipe(x, t, k, p, u)
        assert got[row] in kept, f"row {row} {how[row]}: token {got[row]} had been cut"
        assert got[row] in allowed, f"row {row} {how[row]}: token {got[row]}, the recipe allows {sorted(allowed)}"
    # the host sampler and the kernel, fed the same numbers of the same generator
    rng_a, rng_b = Rng(77), Rng(77)
    us = [rng_a.next_f32() if h[0] > 0 else 0.0 for h in how]      # a greedy row draws nothing
    got2 = kernels.sample(logits, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV), as_f(2),
                          torch.tensor(us, dtype=torch.float32, device=DEV)).cpu().tolist()
    for row, (t, k, p, _) in enumerate(how):
        if t == 0.0:
            continue
        host = sample_host(Sampling(t, k or None, p if p < 1.0 else None), logits[row].cpu().numpy(), rng_b)
        same_as_host += int(host == got2[row])
    drawn = sum(1 for h in how if h[0] > 0)
    assert same_as_host >= drawn - 1, f"{same_as_host} of {drawn} tokens are the host sampler's"


def test_sampling_kernel_with_few_candidates_kept():
    """top_k up to 256 takes a way of its own (the kept candidates are gathered and walked by one thread);
    above it, or when more than 256 candidates stand in the k-th one's bin, the general way.  Logits rounded
    to bfloat16 make equal values, so that the index decides who is kept."""
    import numpy as np
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(23)
    V = 151936
    cases = [(1.0, 1, 1.0), (0.6, 20, 0.95), (0.6, 20, 1.0), (1.0, 255, 0.8), (1.0, 256, 0.8), (1.0, 257, 0.8),
             (3.0, 64, 0.99), (0.3, 100, 0.5)]
    rows, how = [], []
    for rep in range(4):
        for t, k, p in cases:
            x = torch.randn(V, generator=g) * (1.0 + rep)
            if rep % 2:
                x = x.bfloat16().float()
            rows.append(x)
            how.append((t, k, p, float(torch.rand((), generator=g))))
    logits = torch.stack(rows).to(DEV)
    as_f = lambda col: torch.tensor([h[col] for h in how], dtype=torch.float32, device=DEV)
    got = kernels.sample(logits, as_f(0), torch.tensor([h[1] for h in how], dtype=torch.int32, device=DEV), as_f(2),
                         as_f(3)).cpu().tolist()
    for row, (t, k, p, u) in enumerate(how):
        allowed, kept = sampling_recipe(logits[row].cpu().numpy(), t, k, p, u)
        assert got[row] in kept, f"row {row} {how[row]}: token {got[row]} had been cut"
        assert got[row] in allowed, f"row {row} {how[row]}: token {got[row]}, the recipe allows {sorted(allowed)}"
    # equal logits: the lowest indices are kept, whether the k-th one's bin holds few candidates or many
    few, many = torch.zeros(200), torch.zeros(5000)
    few[150:] = -3.0
    hand = [(few, 10, 1.0, 0.55, 5), (few, 10, 0.5, 0.99, 4), (few, 160, 1.0, 0.99, 148), (few, 160, 1.0, 0.9995, 158),
            (few, 1, 1.0, 0.99, 0), (many[:200], 10, 1.0, 0.95, 9), (many[:200], 256, 1.0, 0.5025, 100)]
    for x, k, p, u, want in hand:
        one = kernels.sample(x[None].to(DEV), torch.ones(1, device=DEV), torch.tensor([k], dtype=torch.int32, device=DEV),
                             torch.tensor([p], device=DEV), torch.tensor([u], device=DEV)).item()
        assert one == want, (k, p, u, one, want)
    wide = kernels.sample(many[None].to(DEV), torch.ones(1, device=DEV), torch.tensor([10], dtype=torch.int32, device=DEV),
                          torch.ones(1, device=DEV), torch.tensor([0.95], device=DEV)).item()
    assert wide == 9


def test_sampling_kernel_on_rows_made_by_hand():
    from paged_llm_rs_amd import kernels

    V = 1000
    probs = {17: 0.5, 900: 0.25, 3: 0.15, 512: 0.10}
    row = torch.full((V,), -1000.0)
    for token, p in probs.items():
        row[token] = math.log(p)
    flat = torch.zeros(V)             # all equal: the order is that of the indices
    cases = [
        (row, 1.0, 0, 1.0, 0.10, 17), (row, 1.0, 0, 1.0, 0.49, 17), (row, 1.0, 0, 1.0, 0.51, 900),
        (row, 1.0, 0, 1.0, 0.76, 3), (row, 1.0, 0, 1.0, 0.95, 512), (row, 1.0, 0, 1.0, 0.0, 17),
        (row, 1.0, 2, 1.0, 0.70, 900),          # of 0.75 kept: 0.525 > 0.5
        (row, 1.0, 0, 0.6, 0.70, 900),          # 0.5 < 0.6: the second crosses and is kept
        (row, 1.0, 0, 0.45, 0.99, 17),          # the first reaches 0.45 by itself
        (row, 1.0, 3, 0.8, 0.99, 900),          # k keeps three (0.9), p two of them (0.72 of 0.9 is crossed at 0.75)
        (flat, 1.0, 0, 1.0, 0.3705, 370), (flat, 0.5, 10, 1.0, 0.55, 5), (flat, 2.0, 0, 0.25, 0.5, 124),
        (flat, 0.0, 0, 1.0, 0.9, 0),
    ]
    logits = torch.stack([c[0] for c in cases]).to(DEV)
    col = lambda j, dt: torch.tensor([c[j] for c in cases], dtype=dt, device=DEV)
    got = kernels.sample(logits, col(1, torch.float32), col(2, torch.int32), col(3, torch.float32),
                         col(4, torch.float32)).cpu().tolist()
    assert got == [c[5] for c in cases]


# --- every kernel beside its plain C++ oracle ----------------------------------------------------------------

@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_the_kernels_beside_their_plain_cpp_oracles(dtype):
    """The oracles are the sequential C++ functions of csrc/host/oracle.cpp (pinned on the CPU by
    tests/test_oracle.py); each kernel is run on the same numbers, at sizes that are no powers of two."""
    from paged_llm_rs_amd import kernels, oracle

    tol = 2e-5 if dtype == torch.float32 else 1.2e-2
    g = torch.Generator().manual_seed(11)
    rnd = lambda *shape: torch.randn(*shape, generator=g).to(dtype)

    # norm (with the residual sum before it)
    resid, delta, gain = torch.randn(7, 200, generator=g), rnd(7, 200), rnd(200)
    out = torch.empty(7, 200, dtype=dtype, device=DEV)
    stream = resid.to(DEV)
    kernels.add_rmsnorm(stream, delta.to(DEV), gain.to(DEV), 1e-5, out)
    assert rel(out, oracle.rms_norm(resid + delta.float(), gain, 1e-5)) < tol
    assert rel(stream, resid + delta.float()) < 1e-6

    # activation and argmax
    gu = rnd(9, 2 * 77)
    assert rel(kernels.swiglu(gu.to(DEV)), oracle.swiglu(gu)) < tol
    logits = torch.randn(5, 1003, generator=g)
    logits[2, 17] = logits[2, 900] = 50.0
    assert kernels.argmax(logits.to(DEV)).cpu().tolist() == oracle.argmax(logits).tolist()

    # products: the plain one in either dtype, the matrix-core ones in bfloat16
    x, w = rnd(19, 264), (torch.randn(130, 264, generator=g) / 16).to(dtype)
    want = oracle.product(x, w)
    assert rel(kernels.gemm_plain(x.to(DEV), w.to(DEV), out_dtype=torch.float32), want) < 2e-5
    if dtype == torch.bfloat16:
        assert rel(kernels.gemm_skinny(x.to(DEV), w.to(DEV), torch.float32), want) < 2e-5
        assert rel(kernels.gemm_stream(x.to(DEV), w.to(DEV), torch.float32), want) < 2e-5
        xm, wm = rnd(200, 96), (torch.randn(256, 96, generator=g) / 10).to(dtype)
        assert rel(kernels.gemm_tiled(xm.to(DEV), wm.to(DEV)), oracle.product(xm, wm)) < tol

    # q/k norm, rotation (either layout) and the write into the pages
    nq, nkv, d, bs, rot, theta = 6, 2, 48, 4, 32, 10000.0
    ctx = [13, 6]
    bt, k_pool, v_pool, _, _ = build_paged(nkv, d, bs, ctx, dtype, seed=5)
    positions = [12, 5, 4]
    seq_of = [0, 1, 1]
    qkv = rnd(3, (nq + 2 * nkv) * d)
    q_gain, k_gain = 1 + 0.2 * torch.randn(d, generator=g), 1 + 0.2 * torch.randn(d, generator=g)
    as_i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    for neighbours in (False, True):
        angle = torch.arange(64, dtype=torch.float64)[:, None] * theta ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)
        cos, sin = angle.cos().float().to(DEV), angle.sin().float().to(DEV)
        buf, kp, vp = qkv.to(DEV).clone(), k_pool.clone(), v_pool.clone()
        kernels.qk_norm_rope_kv_write(buf, q_gain.to(DEV), k_gain.to(DEV), 1e-6, cos, sin, rot, as_i32(positions), as_i32(seq_of),
                                      bt, bs, kp, vp, nq, nkv, d, neighbours=neighbours)
        heads = qkv.float().view(3, nq + 2 * nkv, d)
        q_want = oracle.rotate(oracle.rms_norm(heads[:, :nq].reshape(-1, d), q_gain, 1e-6).view(3, nq, d), positions, rot, theta, neighbours)
        k_want = oracle.rotate(oracle.rms_norm(heads[:, nq:nq + nkv].reshape(-1, d), k_gain, 1e-6).view(3, nkv, d), positions, rot, theta, neighbours)
        assert rel(buf[:, :nq * d].view(3, nq, d), q_want) < tol
        for t in range(3):
            slot = int(bt[seq_of[t], positions[t] // bs]) * bs + positions[t] % bs
            assert rel(kp[slot].view(nkv, d), k_want[t]) < tol
            assert rel(vp[slot].view(nkv, d), heads[t, nq + nkv:]) < 1e-6

    # attention over the pages: every kernel that serves single tokens and portions
    nq, nkv, d, bs = 8, 2, 64, 16
    ctx = [150, 37, 64]
    bt, k_pool, v_pool, _, _ = build_paged(nkv, d, bs, ctx, dtype, seed=9)
    positions = [149, 36, 63, 20, -1]
    seq_of = [0, 1, 2, 0, 0]
    stride = (nq + 2 * nkv) * d
    q = rnd(5, stride).to(DEV)
    scale = 1 / math.sqrt(d)
    for window in (0, 40):
        want = oracle.paged_attention(q, k_pool, v_pool, bt, positions, seq_of, nq, nkv, d, bs, scale, window)
        out = torch.zeros(5, nq * d, dtype=dtype, device=DEV)
        kernels.paged_attention_plain(q, stride, out, as_i32(positions), as_i32(seq_of), bt, bs, k_pool, v_pool, nq, nkv, d, scale, window)
        assert rel(out[:4], want[:4]) < tol
        if dtype == torch.bfloat16:
            for splits in (1, 3):
                out = torch.zeros(5, nq * d, dtype=dtype, device=DEV)
                kernels.paged_attention_decode(q, stride, out, as_i32(positions), as_i32(seq_of), bt, bs, k_pool, v_pool, nq, nkv, d,
                                               scale, window, splits=splits)
                assert rel(out[:4], want[:4]) < tol, f"single-token kernel, {splits} shares, window {window}"
            # the tiled kernel and its grouped mode take requests, not rows: the last token of each request
            last = [149, 36, 63]
            q3 = q[:3].contiguous()
            want3 = oracle.paged_attention(q3, k_pool, v_pool, bt, last, [0, 1, 2], nq, nkv, d, bs, scale, window)
            one, start, lens = as_i32([1, 1, 1]), as_i32([0, 1, 2]), as_i32(ctx)
            out = torch.zeros(3, nq * d, dtype=dtype, device=DEV)
            kernels.paged_attention_prefill(q3, stride, out, start, one, lens, 1, bt, bs, k_pool, v_pool, nq, nkv, d, scale, window)
            assert rel(out, want3) < tol, f"tiled kernel, window {window}"


@pytest.mark.parametrize("requests,splits,window", [(70, 2, 0), (70, 8, 48), (5, 8, 48), (5, 1, 0), (40, 16, 20)])
def test_the_single_token_kernel_that_prepares_its_keys_beside_the_oracles(requests, splits, window):
    """One token a request through the kernel that also normalises and rotates q and the new k and writes k and v
    into the pages, against the plain C++ oracles of each of those stages: with few workgroups (eight keys a lane
    group in flight) and with many (four), with a window whose newest key is the token's own, with more shares
    than the window has rounds of keys (the trailing ones are empty), and with one key at the window's far edge
    (or the context's first) that carries nearly all the weight, so that a dropped edge cannot hide."""
    from paged_llm_rs_amd import kernels, oracle

    nq, nkv, d, bs, rot, theta, eps = 4, 2, 64, 16, 64, 10000.0, 1e-6
    g = nq // nkv
    gen = torch.Generator().manual_seed(requests * 100 + splits)
    ctx = [200] + [int(c) for c in torch.randint(1, 230, (requests - 1,), generator=gen)]
    bt, k_pool, v_pool, _, _ = build_paged(nkv, d, bs, ctx, torch.bfloat16, seed=requests + splits)
    n = requests + 1                                    # and a padding row
    positions = [c - 1 for c in ctx] + [-1]
    seq_of = list(range(requests)) + [0]
    stride = (nq + 2 * nkv) * d
    qkv = torch.randn(n, stride, generator=gen).to(torch.bfloat16)
    q_gain, k_gain = 1 + 0.2 * torch.randn(d, generator=gen), 1 + 0.2 * torch.randn(d, generator=gen)
    angle = torch.arange(256, dtype=torch.float64)[:, None] * theta ** (-torch.arange(rot // 2, dtype=torch.float64) * 2 / rot)
    cos, sin = angle.cos().float().to(DEV), angle.sin().float().to(DEV)
    # what the stages before attention make of the rows, by their oracles, rounded as the kernel keeps them
    live = list(range(requests))
    heads = qkv[live].float().view(requests, nq + 2 * nkv, d)
    pos_live = positions[:requests]
    q_want = oracle.rotate(oracle.rms_norm(heads[:, :nq].reshape(-1, d), q_gain, eps).view(requests, nq, d), pos_live, rot, theta)
    k_want = oracle.rotate(oracle.rms_norm(heads[:, nq:nq + nkv].reshape(-1, d), k_gain, eps).view(requests, nkv, d), pos_live, rot, theta)
    q_want, k_want = q_want.to(torch.bfloat16), k_want.to(torch.bfloat16)
    # the far key of request 0: the oldest key its token sees answers the first head of every group
    far = max(0, 199 - window + 1) if window else 0
    far_slot = int(bt[0, far // bs]) * bs + far % bs
    for kvh in range(nkv):
        k_pool[far_slot, kvh * d:(kvh + 1) * d] = (q_want[0, kvh * g].float() * 4).to(torch.bfloat16).to(DEV)
    kp, vp = k_pool.cpu().clone(), v_pool.cpu().clone()
    for t in range(requests):
        slot = int(bt[t, pos_live[t] // bs]) * bs + pos_live[t] % bs
        kp[slot] = k_want[t].reshape(-1)
        vp[slot] = heads[t, nq + nkv:].reshape(-1).to(torch.bfloat16)
    scale = 1 / math.sqrt(d)
    want = oracle.paged_attention(q_want.reshape(requests, nq * d), kp, vp, bt, pos_live, live, nq, nkv, d, bs, scale, window)
    as_i32 = lambda v: torch.tensor(v, dtype=torch.int32, device=DEV)
    out = torch.full((n, nq * d), 7.0, dtype=torch.bfloat16, device=DEV)
    fuse = kernels.QkFusion(q_gain.to(DEV), k_gain.to(DEV), eps, cos, sin, rot, True)
    kernels.paged_attention_decode(qkv.to(DEV), stride, out, as_i32(positions), as_i32(seq_of), bt, bs, k_pool, v_pool,
                                   nq, nkv, d, scale, window, splits=splits, fuse=fuse)
    for t in range(requests):
        err = rel(out[t], want[t])
        assert err < 1.2e-2, f"request {t} (context {ctx[t]}), {splits} shares, window {window}: {err:.3e}"
        slot = int(bt[t, pos_live[t] // bs]) * bs + pos_live[t] % bs
        assert rel(k_pool[slot], kp[slot]) < 1e-2 and torch.equal(v_pool[slot].cpu(), vp[slot])
    for kvh in range(nkv):
        found = rel(out[0].view(nq, d)[kvh * g], v_pool[far_slot].view(nkv, d)[kvh])
        assert found < 0.05, f"the key at {far}, the oldest that position 199 sees with window {window}: {found:.3e}"
    assert bool((out[-1] == 7.0).all()), "a padding row is not written"


@pytest.mark.parametrize("n", [1, 8, 16, 17, 33, 40, 64])
@pytest.mark.parametrize("H,deep,N2,swiglu", [(1024, 3072, 4096, False), (1024, 2048, 3072, True), (1000, 264, 130, False),
                                              (2048, 512, 1000, True), (512, 1024, 20000, False), (1000, 264, 4096, False)])
def test_a_norm_handed_forward_from_one_product_to_the_next(n, H, deep, N2, swiglu):
    """The product that adds into the stream leaves the next norm's work behind (the normalised stripe in
    bfloat16, the stripe's sum of squares a row); the product behind that norm takes both.  Each half against
    64-bit arithmetic, and the pair against the product that normalises the 32-bit stream itself."""
    from paged_llm_rs_amd import kernels

    g = torch.Generator().manual_seed(n * 7 + H)
    eps = 1e-6
    stream = torch.randn(n, H, generator=g).to(DEV)
    before = stream.clone()
    part = torch.randn(n, deep, generator=g).bfloat16().to(DEV)
    w_add = (torch.randn(H, deep, generator=g) / math.sqrt(deep)).bfloat16().to(DEV)
    gain = (1 + 0.2 * torch.randn(H, generator=g)).to(DEV)
    w_next = (torch.randn(N2 * (2 if swiglu else 1), H, generator=g) / math.sqrt(H)).bfloat16().to(DEV)
    assert kernels.hands_norm_forward(n, H, deep) == (n >= kernels.HAND_FROM_ROWS)     # (the kernel takes any count)
    hand = kernels.HandedNorm(gain, eps, n, H, DEV)
    hand.x.fill_(7.0)
    hand.ssq.fill_(float("nan"))
    kernels.gemm_skinny(part, w_add, add_into=stream, hand=hand)
    assert hand.filled
    want_stream = before.double() + part.double() @ w_add.double().T
    assert rel(stream, want_stream) < 1e-5
    assert rel(hand.x, stream.double() * gain.double()) < 5e-3               # one rounding to bfloat16
    stripes = torch.nn.functional.pad(stream.double() ** 2, (0, -H % 16)).reshape(n, -1, 16).sum(-1)
    assert hand.ssq.shape == stripes.shape and rel(hand.ssq, stripes) < 1e-5
    # the product behind the norm
    takes = kernels.takes_handed_norm(n, N2, H, swiglu)
    # (beyond 16 rows: the kernel for one tile of rows where the launch stays small, else the kernel whose waves
    # take a tile of rows each, which wants a stream that is a multiple of 512 wide)
    assert takes == (n <= 16 or -(-N2 // 16) * -(-n // 16) <= 512 or H % 512 == 0)
    if not takes:
        with pytest.raises(Exception, match="take no handed norm"):
            kernels.gemm_skinny(None, w_next, swiglu=swiglu, handed=hand)
        return
    got = kernels.gemm_skinny(None, w_next, torch.bfloat16, swiglu=swiglu, handed=hand)
    rinv = 1 / torch.sqrt((stream.double() ** 2).mean(-1, keepdim=True) + eps)
    raw = (hand.x.double() @ w_next.double().T) * rinv
    want = torch.nn.functional.silu(raw[:, :N2]) * raw[:, N2:] if swiglu else raw
    assert rel(got, want) < 1e-2
    if n <= 32 and N2 <= 32768:
        own = kernels.gemm_skinny(stream, w_next, torch.bfloat16, swiglu=swiglu, norm_gain=gain, eps=eps)
        assert rel(got, own.double()) < 1e-2
