"""The three bfloat16 attention kernels at the contexts the benchmark configurations run (4,096 to
16,384 keys), with the share counts the engine's own choice gives and with the extremes, against a
64-bit reference.  (The reference's kernel ends at about 12 k keys, the size of its score buffer:
kernels/paged_attention.rs:626-634; an online softmax over shares of the context has no such end, and
these tests are what says so.)

Random scores over thousands of keys hide a lost key: one key in 16,384 moves the result by under a
percent.  So beside the comparison of every row with the reference, some rows carry a query that one
chosen key answers with nearly all the weight: the first key, the last, keys at both sides of page
edges, of 64- and 128-key tiles and of the edges between shares.  Such a row's output is that key's
value, or the key was lost.
"""

from __future__ import annotations

import math

import pytest
import torch

from test_kernels_gpu import DEV, build_paged, rel

pytestmark = pytest.mark.gpu

BF16 = torch.bfloat16


def reference(q, keys, values, positions, g, scale):
    """q [rows, nq, d] at ``positions`` against keys/values [ctx, nkv, d], in 64-bit on the GPU."""
    q, keys, values = q.double().to(DEV), keys.double().to(DEV), values.double().to(DEV)
    rows, nq, d = q.shape
    ctx = keys.shape[0]
    visible = torch.arange(ctx, device=DEV)[None, :] <= torch.as_tensor(positions, device=DEV)[:, None]
    out = torch.empty(rows, nq, d, dtype=torch.float64, device=DEV)
    for h in range(nq):
        scores = q[:, h] @ keys[:, h // g].T * scale
        scores = scores.masked_fill(~visible, float("-inf"))
        out[:, h] = torch.softmax(scores, dim=-1) @ values[:, h // g]
    return out.cpu()


def plant(q_row, k_pool, keys, bt_row, bs, target, nkv, g, d):
    """Make key ``target`` of the request the one that the first query head of every group of this row finds."""
    slot = int(bt_row[target // bs]) * bs + target % bs
    for kvh in range(nkv):
        k = (q_row[kvh * g * d: kvh * g * d + d].float() * 4).to(BF16)
        k_pool[slot, kvh * d:(kvh + 1) * d] = k
        keys[target, kvh] = k.double().cpu()


def edges(ctx, shares):
    """Keys where one is most easily lost: ends, page and tile edges, and both sides of the edges between
    ``shares`` equal stretches of the context (whatever way a kernel rounds them)."""
    found = {0, 1, 15, 16, 63, 64, 127, 128, ctx - 1, ctx - 2, ctx - 16, ctx - 17, ctx - 64, ctx - 65, ctx // 2}
    for s in shares:
        for i in range(1, s):
            for cut in (ctx * i // s, -(-ctx // s) * i, (-(-ctx // s) + 63) // 64 * 64 * i, (-(-ctx // s) + 127) // 128 * 128 * i):
                found |= {cut - 1, cut}
    return sorted(t for t in found if 0 <= t < ctx)


def spread(targets, count, seed):
    """At most ``count`` of the targets, evenly thinned, the ends kept."""
    if len(targets) <= count:
        return targets
    g = torch.Generator().manual_seed(seed)
    keep = {targets[0], targets[-1]} | {targets[int(i)] for i in torch.randperm(len(targets), generator=g)[:count - 2]}
    return sorted(keep)


@pytest.mark.parametrize("ctx", [4096, 8191, 16384])
@pytest.mark.parametrize("splits", ["chosen", 1, 64])
def test_single_tokens_over_long_contexts(ctx, splits):
    """The kernel for single tokens (16 query heads over 8 key heads of 128, pages of 16): 8 decoded tokens at the
    end of contexts of this length, as the benchmark's batch of 8 has them, and rows whose answer is one key."""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.engine.batch import context_bound

    nq, nkv, d, bs = 16, 8, 128, 16
    g = nq // nkv
    chosen = kernels.decode_splits(8, nq, nkv, context_bound(ctx), d)
    count = chosen if splits == "chosen" else splits
    assert 1 <= chosen <= 64
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, [ctx, ctx - 700], BF16, seed=ctx)
    targets = spread(edges(ctx, {chosen, 64, 16, 3}), 72, seed=ctx)
    # rows: the planted ones (request 0, its last position), then plain decoded tokens of both requests
    rows = [(0, ctx - 1)] * len(targets) + [(0, ctx - 1), (1, ctx - 701), (0, ctx // 3), (1, 17)] * 2 + [(0, -1)]
    n = len(rows)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(BF16)
    for i, t in enumerate(targets):
        q[i] = torch.randn(stride, generator=torch.Generator().manual_seed(1000 + i)).to(BF16).to(DEV)
    # every planted key is large; the row it belongs to is the one it dominates, the others see it as one more key
    for i, t in enumerate(targets):
        plant(q[i], k_pool, keys[0], bt[0].tolist(), bs, t, nkv, g, d)
    positions = torch.tensor([p for _, p in rows], dtype=torch.int32, device=DEV)
    seq_of = torch.tensor([s for s, _ in rows], dtype=torch.int32, device=DEV)
    scale = 1 / math.sqrt(d)
    out = torch.full((n, nq * d), 7.0, dtype=BF16, device=DEV)
    kernels.paged_attention_decode(q, stride, out, positions, seq_of, bt, bs, k_pool, v_pool, nq, nkv, d, scale, 0,
                                   splits=count)
    for s in (0, 1):
        mine = [i for i, (r, p) in enumerate(rows) if r == s and p >= 0]
        want = reference(q[mine, :nq * d].reshape(len(mine), nq, d), keys[s], values[s], [rows[i][1] for i in mine], g, scale)
        for j, i in enumerate(mine):
            err = rel(out[i].reshape(nq, d), want[j])
            assert err < 1e-2, f"row {i} (request {s}, position {rows[i][1]}), {count} shares: {err:.3e}"
    for i, t in enumerate(targets):
        got = out[i].reshape(nq, d)
        for kvh in range(nkv):
            err = rel(got[kvh * g], values[0][t, kvh])
            assert err < 0.05, f"key {t} of {ctx} in {count} shares is not what row {i} found: {err:.3e}"
    assert bool((out[-1] == 7.0).all()), "a padding row is not written"


@pytest.mark.parametrize("ctx", [4096, 8191, 16384])
@pytest.mark.parametrize("splits", ["chosen", 1, 16])
def test_a_group_of_heads_over_long_contexts(ctx, splits):
    """The grouped kernel (64 query heads over 8 key heads of 128, pages of 16, the 32B shape's attention) with
    single tokens at the end of contexts of this length.  Requests share pages here: each is one row of queries
    with a key of its own to find."""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.engine.batch import context_bound

    nq, nkv, d, bs = 64, 8, 128, 16
    g = nq // nkv
    assert kernels.grouped_applies(nq, nkv, d, bs)
    bt1, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, [ctx], BF16, seed=ctx + 1)
    chosen = kernels.grouped_splits(64, nkv, context_bound(ctx))
    few = kernels.grouped_splits(8, nkv, context_bound(ctx))
    count = chosen if splits == "chosen" else splits
    targets = spread(edges(ctx, {chosen, few, 16, 3}), 40, seed=ctx)
    # every planted row is a request of its own over the same pages; then two requests that end earlier, one of
    # them with three tokens
    requests = [(ctx, 1)] * len(targets) + [(ctx - 1, 1), (ctx // 2 + 5, 3), (ctx, 1)]
    S = len(requests)
    bt = bt1.repeat(S, 1).contiguous()
    n = sum(c for _, c in requests)
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(BF16)
    for i, t in enumerate(targets):
        plant(q[i], k_pool, keys[0], bt1[0].tolist(), bs, t, nkv, g, d)
    q_start, q_len, positions = [], [], []
    for c, count_s in requests:
        q_start.append(len(positions))
        q_len.append(count_s)
        positions += list(range(c - count_s, c))
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    out = torch.full((n, nq * d), 7.0, dtype=BF16, device=DEV)
    scale = 1 / math.sqrt(d)
    kernels.paged_attention_grouped(q, stride, out, as_i32(q_start), as_i32(q_len), as_i32([c for c, _ in requests]), 3,
                                    bt, bs, k_pool, v_pool, nq, nkv, d, scale, 0, short_limit=0, splits=count)
    want = reference(q[:, :nq * d].reshape(n, nq, d), keys[0], values[0], positions, g, scale)
    for i in range(n):
        err = rel(out[i].reshape(nq, d), want[i])
        assert err < 1e-2, f"row {i} (position {positions[i]}), {count} shares: {err:.3e}"
    for i, t in enumerate(targets):
        got = out[i].reshape(nq, d)
        for kvh in range(nkv):
            err = rel(got[kvh * g], values[0][t, kvh])
            assert err < 0.05, f"key {t} of {ctx} in {count} shares is not what row {i} found: {err:.3e}"


@pytest.mark.parametrize("behind", [3584, 15872])
@pytest.mark.parametrize("splits", ["chosen", 1, 16])
def test_a_portion_behind_a_long_context(behind, splits):
    """The tiled kernel: a portion of 512 tokens behind this many earlier ones (a late slice of a long prompt),
    beside a short request, with the share count that the engine would choose and with the extremes."""
    from paged_llm_rs_amd import kernels
    from paged_llm_rs_amd.engine.batch import context_bound

    nq, nkv, d, bs, portion = 16, 8, 128, 16, 512
    g = nq // nkv
    ctx = behind + portion
    requests = [(ctx, portion), (300, 40)]
    chosen = kernels.prefill_splits(2, portion, nq, d, context_bound(ctx), portion + 40, 0)
    count = chosen if splits == "chosen" else splits
    bt, k_pool, v_pool, keys, values = build_paged(nkv, d, bs, [c for c, _ in requests], BF16, seed=behind)
    n = portion + 40
    stride = (nq + 2 * nkv) * d
    q = torch.randn(n, stride, device=DEV).to(BF16)
    # one row in eight of the portion has a key to find: far back, at edges, or among the portion's own tokens
    targets = spread(edges(ctx - portion, {chosen, 16, 3, 6}), 56, seed=behind)
    planted = {}
    for j, t in enumerate(targets):
        planted[j * 8 + 3] = t
    first = ctx - portion
    for row, t in ((5, first + 5), (130, first + 129), (257, first + 200), (511, first + 511), (400, first + 402)):
        planted[row] = t                      # the last of these lies after its row: it must not be found
    for row, t in planted.items():
        plant(q[row], k_pool, keys[0], bt[0].tolist(), bs, t, nkv, g, d)
    as_i32 = lambda x: torch.tensor(x, dtype=torch.int32, device=DEV)
    out = torch.full((n, nq * d), 7.0, dtype=BF16, device=DEV)
    scale = 1 / math.sqrt(d)
    kernels.paged_attention_prefill(q, stride, out, as_i32([0, portion]), as_i32([portion, 40]), as_i32([ctx, 300]),
                                    portion, bt, bs, k_pool, v_pool, nq, nkv, d, scale, 0, short_limit=0, splits=count)
    at = 0
    for s, (c, tokens) in enumerate(requests):
        positions = list(range(c - tokens, c))
        want = reference(q[at:at + tokens, :nq * d].reshape(tokens, nq, d), keys[s], values[s], positions, g, scale)
        for i in range(tokens):
            err = rel(out[at + i].reshape(nq, d), want[i])
            assert err < 1e-2, f"request {s}, position {positions[i]}, {count} shares: {err:.3e}"
        at += tokens
    for row, t in planted.items():
        got = out[row].reshape(nq, d)
        visible = t <= first + row
        for kvh in range(nkv):
            hit = rel(got[kvh * g], values[0][t, kvh]) < 0.05
            assert hit == visible, f"key {t} and the row at {first + row}, {count} shares: found {hit}, visible {visible}"
