"""Megozen on the GPU: every mechanism alone against its plain function, then whole models cut into steps in
different ways, then generation through the engine's entry point and scheduler."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

from tests import megozen_helpers as MH
from tests import traces
from tests.plain import megozen_plain as M

pytestmark = pytest.mark.gpu
DEV = "cuda"
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = [torch.float32, torch.bfloat16]


def dev(x, dtype=torch.float32):
    return torch.as_tensor(np.asarray(x)).to(DEV).to(dtype).contiguous()


def rounded(x, dtype):
    return M.bf16_round(x) if dtype == torch.bfloat16 else np.asarray(x, np.float32)


def store_of(dtype):
    return M.bf16_round if dtype == torch.bfloat16 else M.f32


class Harness:
    """Runs one part on a batch of sequences through the engine's own cache manager and batch builder."""

    def __init__(self, specs, dtype, page=8, pages=64, slots=4):
        from sprout_lm_amd.cache import CacheManager
        from sprout_lm_amd.engine.batch import DescriptorStager, Workspace
        self.dtype = dtype
        self.cache = CacheManager(specs, page, pages, slots, prefix_caching=False)
        self.cache.attach_storage(dtype, DEV)
        self.workspace, self.stager = Workspace(DEV), DescriptorStager(DEV)

    def context(self, batch):
        """batch: [(sequence, its next tokens)]"""
        from sprout_lm_amd.engine.batch import StepEntry, build_context
        entries = []
        for seq, tokens in batch:
            assert self.cache.reserve(seq, seq.length + len(tokens))
            entries.append(StepEntry(seq, [int(t) for t in tokens], []))
        ctx = build_context(entries, self.cache, self.stager, self.workspace, self.dtype,
                            1 if self.dtype == torch.float32 else 0)
        return ctx, entries

    def view(self, ctx, slot):
        from sprout_lm_amd.engine.batch import CacheSlotView
        kind, g, index = self.cache.slot_location[slot]
        if kind == "state":
            return CacheSlotView(True, state=self.cache.state_groups[g].data[index])
        group = self.cache.groups[g]
        return CacheSlotView(True, k=group.k[index], v=group.v[index], block_tables=ctx.group_tables[g],
                             slot_mapping=ctx.group_slots[g], page_size=group.page_tokens)

    def commit(self, entries):
        for e in entries:
            self.cache.commit(e.seq, e.seq.length + len(e.tokens))


# ---------------------------------------------------------------------------------------------- mechanisms alone
@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("H", [24, 72, 256, 1000, 4100])
def test_layer_norm(dtype, H):
    """Rows with a mean far from zero (a variance taken as E[x^2] - mean^2 would lose its digits), all rows and
    gathered rows."""
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(H)
    eps = 1e-5
    part = make_part("norm", "layernorm", size=H, eps=eps, tensor="norm1")
    assert list(part.tensors()) == ["norm1"]
    w = rounded(1.0 + 0.2 * rng.standard_normal(H), dtype)
    part.bind({"norm1": dev(w, dtype)})
    x = (rng.standard_normal((9, H)) * rng.uniform(0.01, 3.0, (9, 1)) + rng.uniform(-40.0, 40.0, (9, 1))).astype(np.float32)
    want = M.layer_norm(x, w, eps)
    tol = 3e-5 if dtype == torch.float32 else 2.0 ** -7
    out = torch.empty(9, H, dtype=dtype, device=DEV)
    part.forward(None, dev(x), out)
    assert np.abs(out.float().cpu().numpy() - want).max() <= tol * max(1.0, np.abs(want).max())
    rows = [7, 0, 7, 3]
    picked = torch.empty(4, H, dtype=dtype, device=DEV)
    part.forward(None, dev(x), picked, rows=torch.tensor(rows, dtype=torch.int32, device=DEV))
    assert np.abs(picked.float().cpu().numpy() - want[rows]).max() <= tol * max(1.0, np.abs(want).max())
    # two norms of one input in one pass
    other = make_part("norm", "layernorm", size=H, eps=eps, tensor="norm2")
    w2 = rounded(1.0 + 0.2 * rng.standard_normal(H), dtype)
    other.bind({"norm2": dev(w2, dtype)})
    out2 = torch.empty(9, H, dtype=dtype, device=DEV)
    first = out.clone()
    out.zero_()
    assert part.forward_pair(None, other, dev(x), out, out2)
    assert torch.equal(out, first)
    assert np.abs(out2.float().cpu().numpy() - M.layer_norm(x, w2, eps)).max() <= tol * max(1.0, np.abs(want).max())
    assert not part.forward_pair(None, make_part("norm", "layernorm", size=H, eps=2 * eps), dev(x), out, out2)
    # a constant row has no deviation at all: the result is 0 whatever eps is, not a NaN
    flat = torch.full((1, H), 3.25, device=DEV)
    part.forward(None, flat, out[:1])
    assert float(out[:1].float().abs().max()) == 0.0


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("vocab,buckets,mul_prev,mul_cur", [(150, 97, 31, 5), (40, 1, 0, 0), (300, 64, 3, 1),
                                                          (60000, 1013, 40009, 77003), (90, 7, 0, 3), (90, 11, 5, 0),
                                                          (500, 1013, 2 ** 40 + 7, 2 ** 35 + 1)])
def test_bigram_embedding_across_steps_and_reused_slots(dtype, vocab, buckets, mul_prev, mul_cur):
    """Sequences fed in portions and single tokens beside each other; the token before a portion comes from the
    request's state slot; a slot given back serves the next request, whose first token takes the last row.  The
    largest case overflows 32-bit products."""
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(buckets)
    Hd = 40
    part = make_part("embedding", "bigram_embedding", vocab=vocab, hidden=Hd, buckets=buckets, mul_prev=mul_prev,
                     mul_cur=mul_cur, tensors=("embed", "bigram"))
    shapes = {n: tuple(s.shape) for n, s in part.tensors().items()}
    assert shapes == {"embed": (vocab, Hd), "bigram": (buckets + 1, Hd)}
    table = rounded(rng.standard_normal((vocab, Hd)), dtype)
    pairs = rounded(rng.standard_normal((buckets + 1, Hd)), dtype)
    part.bind({"embed": dev(table, dtype), "bigram": dev(pairs, dtype)})
    harness = Harness([part.cache_spec()], dtype, slots=2)
    w = {"embed": table, "bigram": pairs}
    cfg = {"embedding": {"bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}

    def run(requests, schedule):
        seqs = {r: harness.cache.create() for r in requests}
        fed = {r: 0 for r in requests}
        got = {r: [] for r in requests}
        for step in schedule:
            batch = [(r, requests[r][fed[r]:fed[r] + n]) for r, n in step if fed[r] < len(requests[r])]
            ctx, entries = harness.context([(seqs[r], t) for r, t in batch])
            residual = torch.full((ctx.n_tokens, Hd), 7.0, device=DEV)
            part.forward(ctx, ctx.token_ids, residual, harness.view(ctx, 0))
            out = residual.cpu().numpy()
            harness.commit(entries)
            row = 0
            for r, t in batch:
                got[r].append(out[row:row + len(t)])
                row += len(t)
                fed[r] += len(t)
        for r in requests:
            assert fed[r] == len(requests[r])
            assert np.array_equal(np.concatenate(got[r]), M.embed(w, cfg, requests[r]).astype(np.float32)), r
            seqs[r].release()

    first = {"a": MH.random_tokens(vocab, 23, 1), "b": MH.random_tokens(vocab, 9, 2)}
    run(first, [[("a", 5), ("b", 1)], [("b", 1), ("a", 1)], [("a", 2)], [("b", 4), ("a", 9)], [("a", 1), ("b", 1)],
                [("b", 2), ("a", 5)]])
    # both slots have been used: the next two requests find another request's last token there unless admission clears it
    run({"c": MH.random_tokens(vocab, 6, 3), "d": MH.random_tokens(vocab, 1, 4)}, [[("d", 1), ("c", 2)], [("c", 1)], [("c", 3)]])


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("heads,dim,rot,rot_dims,rank,scaling", [(3, 24, 8, 8, 20, (4.0, 64, 16.0, 2.0)),
                                                                (2, 16, 32, 20, 48, None),
                                                                (5, 0, 16, 16, 16, (40.0, 4096, 32.0, 1.0)),
                                                                (4, 32, 0, 0, 64, None)])
def test_latent_norm_rotation_and_cache_write(dtype, heads, dim, rot, rot_dims, rank, scaling):
    """The kernel between the input projections and attention, at positions up to a million: the latent's RMS norm,
    the turn of neighbouring numbers with blended frequencies and the magnitude factor, numbers behind rot.dims
    passing unchanged, keys and values landing in the slots asked for and nowhere else."""
    from sprout_lm_amd import ops
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(heads * 100 + rot)
    named = dict(zip(("factor", "original", "fast", "slow"), scaling)) if scaling else None
    position = make_part("position", "rotary_interleaved", rotary_dim=rot_dims, theta=5000.0, scaling=named)
    position.prepare(DEV, dtype)
    rot_cfg = {"dims": rot_dims, "base": 5000.0, "scaling": named}
    T, page, pages, eps = 11, 4, 9, 1e-5
    width = rank + rot
    q_off, dkv_off = 3, 3 + heads * (dim + rot) + 2
    stride = dkv_off + width + 5
    proj = rounded(rng.standard_normal((T, stride)) * 2.0, dtype)
    w_norm = rounded(1.0 + 0.3 * rng.standard_normal(rank), dtype)
    positions = np.asarray([0, 1, 2, 3, 63, 64, 65, 4095, 4096, 250000, 1000000], dtype=np.int32)
    slots = rng.permutation(page * pages)[:T].astype(np.int32)
    slots[4] = -1       # a row that writes nothing (a padded row of a recorded step)
    k_pool = torch.full((pages, 1, page, width), 9.0, dtype=dtype, device=DEV)
    v_pool = torch.full((pages, 1, width, page), 9.0, dtype=dtype, device=DEV)
    q_out = torch.full((T, heads * width), 5.0, dtype=dtype, device=DEV)
    ops.latent_prepare(dev(proj, dtype), q_off, heads, dim, rot, dkv_off, rank, dev(w_norm, dtype), eps,
                       dev(positions, torch.int32), position.freq, rot_dims, position.magnitude,
                       dev(slots, torch.int32), k_pool, v_pool, q_out)
    angle = np.float64 if dtype == torch.float32 else np.float32
    c = M.rms_norm(proj[:, dkv_off:dkv_off + rank], w_norm, eps)
    r = M.rotate_interleaved(proj[:, dkv_off + rank:dkv_off + width], positions, rot_cfg, angle) if rot else np.zeros((T, 0))
    tol = 2e-5 if dtype == torch.float32 else 2.0 ** -7
    scale = max(1.0, float(np.abs(proj).max()) * 1.5)
    keys, values = k_pool.float().cpu().numpy().reshape(-1, width), v_pool.float().cpu().numpy()
    written = np.zeros(page * pages, bool)
    for t in range(T):
        if slots[t] < 0:
            continue
        written[slots[t]] = True
        assert np.abs(keys[slots[t], :rank] - c[t]).max() <= tol * scale, f"latent of token {t}"
        assert not rot or np.abs(keys[slots[t], rank:] - r[t]).max() <= tol * scale, f"turned key part of token {t}"
        assert np.abs(values[slots[t] // page, 0, :rank, slots[t] % page] - c[t]).max() <= tol * scale
    assert np.all(keys[~written] == 9.0), "a key was written where no token belongs"
    got = q_out.float().cpu().numpy().reshape(T, heads, width)
    assert np.all(got[:, :, :rank] == 5.0), "the latent part of the queries belongs to the per-head product"
    if rot:
        q = proj[:, q_off:q_off + heads * (dim + rot)].reshape(T, heads, dim + rot)[:, :, dim:]
        want = M.rotate_interleaved(q.transpose(1, 0, 2), positions, rot_cfg, angle).transpose(1, 0, 2)
        assert np.abs(got[:, :, rank:] - want).max() <= tol * scale
        if rot_dims < rot:
            assert np.array_equal(got[:, :, rank + rot_dims:], rounded(q[:, :, rot_dims:], dtype))


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("T,heads,N,K", [(1, 3, 40, 20), (70, 3, 40, 20), (130, 2, 16, 48), (5, 20, 12, 12),
                                         (200, 4, 64, 64), (33, 1, 7, 104), (300, 6, 80, 96), (513, 3, 200, 72)])
@pytest.mark.parametrize("eights", [False, True])
def test_per_head_product_with_and_without_gate(dtype, T, heads, N, K, eights):
    """`eights`: every head's operand starts at a multiple of 8 numbers, which is what the matrix-core kernels take
    (in bfloat16, where K is in eights too); otherwise the float32-arithmetic kernel runs."""
    from sprout_lm_amd import ops
    rng = np.random.default_rng(T + N)
    a_off, out_off, g_off = (8, 2, 1) if eights else (5, 2, 1)
    a_stride, out_stride = (-(-K // 8) * 8 + 8 if eights else K + 3), N + 4
    a = rounded(rng.standard_normal((T, a_off + heads * a_stride + (3 if not eights else 0))), dtype)
    w = rounded(rng.standard_normal((heads, N, K)) * 0.3, dtype)
    gate = rounded(rng.standard_normal((T, g_off + heads + 2)) * 2.0, dtype)
    tol = 3e-5 if dtype == torch.float32 else 2.0 ** -7
    for gated in (False, True):
        out = torch.full((T, out_off + heads * out_stride), 3.0, dtype=dtype, device=DEV)
        ops.head_gemm(dev(a, dtype), a_off, a_stride, dev(w, dtype), out, out_off, out_stride,
                      gate=dev(gate, dtype) if gated else None, gate_offset=g_off)
        got = out.float().cpu().numpy()
        for h in range(heads):
            want = a[:, a_off + h * a_stride:a_off + h * a_stride + K].astype(np.float64) @ w[h].astype(np.float64).T
            if gated:
                want = want / (1.0 + np.exp(-gate[:, g_off + h].astype(np.float64)))[:, None]
            cols = slice(out_off + h * out_stride, out_off + h * out_stride + N)
            assert np.abs(got[:, cols] - want).max() <= tol * max(1.0, np.abs(want).max()), f"head {h} gated={gated}"
            assert np.all(got[:, cols.stop:cols.stop + out_stride - N] == 3.0), "wrote between the heads"


def test_router_choice_ties_and_weights():
    from sprout_lm_amd import ops
    rng = np.random.default_rng(4)
    for T, E, top in ((1, 5, 2), (77, 12, 3), (300, 7, 7), (64, 6, 1), (9, 130, 5)):
        logits = rng.standard_normal((T, E)).astype(np.float32) * 2.0
        logits[0, :] = 0.5                      # all equal: the lowest indices win
        if T > 3 and E > 3:
            logits[3, [1, 3]] = 9.0             # two equal at the top
        ids = torch.empty(T, top, dtype=torch.int32, device=DEV)
        weights = torch.empty(T, top, device=DEV)
        ops.route_topk(dev(logits), ids, weights)
        chosen, want = M.route(logits.astype(np.float64), top)
        assert np.array_equal(ids.cpu().numpy(), chosen)
        assert np.abs(weights.cpu().numpy() - want).max() <= 2e-6
        assert np.allclose(weights.sum(dim=1).cpu().numpy(), 1.0, atol=1e-5)
        # the order in which the grouped products walk the pairs
        pairs = T * top
        row_of_pair = torch.empty(pairs, dtype=torch.int32, device=DEV)
        pair_of_row = torch.empty(pairs, dtype=torch.int32, device=DEV)
        tiles = torch.full((3 * ops.route_max_tiles(pairs, E),), -7, dtype=torch.int32, device=DEV)
        n_tiles = torch.zeros(1, dtype=torch.int32, device=DEV)
        ops.route_sort(ids, E, row_of_pair, pair_of_row, tiles, n_tiles)
        # choice and order in one call, for tiles of either size
        for tile_rows in (16, 64, 128, 256):
            ids2, weights2 = torch.empty_like(ids), torch.empty_like(weights)
            rp2, pr2 = torch.empty_like(row_of_pair), torch.empty_like(pair_of_row)
            tiles2 = torch.full((3 * ops.route_max_tiles(pairs, E, tile_rows),), -7, dtype=torch.int32, device=DEV)
            n2 = torch.zeros(1, dtype=torch.int32, device=DEV)
            ops.route(dev(logits), ids2, weights2, rp2, pr2, tiles2, n2, tile_rows)
            assert torch.equal(ids2, ids) and torch.equal(weights2, weights)
            cut2 = tiles2.cpu().numpy()[:3 * int(n2.item())].reshape(-1, 3)
            assert cut2[:, 2].sum() == pairs and cut2[:, 2].max() <= tile_rows
            assert np.array_equal(chosen.reshape(-1)[pr2.cpu().numpy()], np.repeat(cut2[:, 0], cut2[:, 2]))
        rp, pr, n = row_of_pair.cpu().numpy(), pair_of_row.cpu().numpy(), int(n_tiles.item())
        assert sorted(rp.tolist()) == list(range(pairs)) and np.array_equal(pr[rp], np.arange(pairs))
        by_row = chosen.reshape(-1)[pr]
        assert np.all(np.diff(by_row) >= 0), "rows are not grouped by expert"
        cut = tiles.cpu().numpy()[:3 * n].reshape(n, 3)
        assert n <= ops.route_max_tiles(pairs, E) and cut[:, 2].sum() == pairs and np.all(cut[:, 2] > 0)
        covered = np.zeros(pairs, int)
        for e, first, rows in cut:
            assert rows <= ops.group_tile_rows() and np.all(by_row[first:first + rows] == e)
            covered[first:first + rows] += 1
        assert np.all(covered == 1)


def expert_weights(rng, hidden, inner, experts, shared, dtype, bias=True):
    w = {}
    for e in range(experts):
        w[f"e{e}.gate"] = rounded(rng.standard_normal((inner, hidden)) * 0.2, dtype)
        w[f"e{e}.up"] = rounded(rng.standard_normal((inner, hidden)) * 0.2, dtype)
        w[f"e{e}.down"] = rounded(rng.standard_normal((hidden, inner)) * 0.2, dtype)
    w["router"] = rounded(rng.standard_normal((experts, hidden)) * 0.5, dtype)
    if bias:
        w["router.b"] = rounded(rng.standard_normal(experts) * 0.5, dtype)
    if shared:
        w["shared.gate"] = rounded(rng.standard_normal((shared, hidden)) * 0.2, dtype)
        w["shared.up"] = rounded(rng.standard_normal((shared, hidden)) * 0.2, dtype)
        w["shared.down"] = rounded(rng.standard_normal((hidden, shared)) * 0.2, dtype)
    return w


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("hidden,inner,experts,top,shared", [(40, 48, 5, 2, 24), (64, 24, 4, 4, None), (72, 40, 6, 1, 72),
                                                            (128, 64, 16, 3, 32), (256, 128, 9, 2, 192), (100, 36, 9, 4, 28)])
@pytest.mark.parametrize("T", [1, 7, 150, 1100])
def test_routed_experts_part(dtype, hidden, inner, experts, top, shared, T):
    """The feed-forward alone: one token (most experts get no row), a handful, more than a tile per expert, and enough
    for tiles of 128 rows.  Both
    sides route the same stored input, so a token changes sides only within float32 rounding of the router."""
    from sprout_lm_amd.engine.batch import StepContext, Workspace
    from sprout_lm_amd.parts import make_part
    rng = np.random.default_rng(hidden + T)
    part = make_part("feed_forward", "routed_experts", hidden=hidden, inner=inner, experts=experts, top=top,
                     shared_inner=shared, router_bias=True, activation="silu")
    w = expert_weights(rng, hidden, inner, experts, shared, dtype)
    assert sorted(part.tensors()) == sorted(w)
    part.bind({k: dev(v, dtype) for k, v in w.items()})
    h = rounded(rng.standard_normal((T, hidden)), dtype)
    mlp = {"router": {"experts": experts, "top": top}, "shared": {"ff": shared} if shared else None}
    want, gap = M.moe({"x." + k: v for k, v in w.items()}, "x.", mlp, h.astype(np.float64))
    ctx = StepContext(Workspace(DEV), dtype, 0)
    base = rng.standard_normal((T, hidden)).astype(np.float32)
    residual = dev(base)
    part.forward(ctx, dev(h, dtype), residual)
    got = residual.cpu().numpy() - base
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    sure = gap > 1e-4
    assert sure.sum() >= 0.9 * T
    assert np.abs(got - want)[sure].max() <= tol * max(1.0, np.abs(want).max())


def mixer_weights(rng, hidden, heads, dim, rot, vdim, rank, dtype, spiky=False):
    w = {"q": rng.standard_normal((heads * (dim + rot), hidden)) * 0.2,
         "dkv": rng.standard_normal((rank + rot, hidden)) * 0.2,
         "dkv.norm": 1.0 + 0.2 * rng.standard_normal(rank),
         "uk": rng.standard_normal((heads * dim, rank)) * 0.2,
         "uv": rng.standard_normal((heads * vdim, rank)) * 0.3,
         "g": rng.standard_normal((heads, hidden)) * 0.3,
         "o": rng.standard_normal((hidden, heads * vdim)) * 0.2}
    if spiky:
        # hidden number 0 is a flag that fills latent number 0; hidden number 1 is the same for every token and
        # fills every head's query number 0; U_k carries latent number 0 to key number 0: a flagged key outweighs
        # all others of a window together
        w["dkv"][0, :] = 0.0
        w["dkv"][0, 0] = 4.0
        w["dkv.norm"][0] = 1.0
        for h in range(heads):
            w["q"][h * (dim + rot), :] = 0.0
            w["q"][h * (dim + rot), 1] = 4.0
            w["uk"][h * dim, :] = 0.0
            w["uk"][h * dim, 0] = 1.5
    return {k: rounded(v, dtype) for k, v in w.items()}


LATENT_SHAPES = [  # heads, dim, rot, vdim, rank, window, page
    (3, 24, 8, 40, 20, 37, 8),       # key width 28: the general attention kernels
    (4, 32, 16, 16, 48, 70, 16),     # key width 64: the matrix-core kernels
    (2, 16, 32, 24, 32, 33, 4),
    (20, 8, 4, 12, 12, 16, 8),       # more heads than one group of the attention kernels holds; a window of two pages
    (4, 32, 16, 48, 48, None, 16),   # no window
    (1, 48, 16, 16, 80, 50, 16)]     # one head, key width 96


@pytest.mark.parametrize("dtype", DTYPES)
@pytest.mark.parametrize("shape", LATENT_SHAPES)
@pytest.mark.parametrize("schedule", ["portions", "decoded"])
@pytest.mark.parametrize("spiky", [False, True])
def test_latent_attention_part(dtype, shape, schedule, spiky):
    """The mixer alone on two sequences beside each other, in uneven portions or token by token behind a prompt.

    `spiky`: a few flagged tokens whose keys outweigh everything else in a window, placed so that queries in
    prompts and decoded queries alike have one just inside their window, just outside it, at a page's first and last
    place, and far back: one key too many or too few moves the output by the size of a value."""
    from sprout_lm_amd.parts import make_part
    heads, dim, rot, vdim, rank, window, page = shape
    rng = np.random.default_rng(heads * 10 + rank + (1 if spiky else 0))
    hidden, eps, scale = 40, 1e-5, 0.4
    named = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
    position = make_part("position", "rotary_interleaved", rotary_dim=rot, theta=5000.0, scaling=named)
    part = make_part("mixer", "latent_attention", hidden=hidden, heads=heads, dim=dim, rot_dim=rot, vdim=vdim,
                     kv_rank=rank, scale=scale, eps=eps, position=position, window=window, gated=True)
    w = mixer_weights(rng, hidden, heads, dim, rot, vdim, rank, dtype, spiky)
    assert sorted(part.tensors()) == sorted(w)
    part.bind({k: dev(v, dtype) for k, v in w.items()})
    part.prepare(DEV, dtype)
    # without a window the first sequence is long enough for several chunks of the one-query kernel, with flagged
    # keys hundreds of places back and on both sides of a chunk's border
    lengths = [150 if window else 600, 61]
    hs = [rng.standard_normal((n, hidden)) for n in lengths]
    if spiky:
        reach = window or 100
        far = [] if window else [3, 255, 256, 511, 512]
        for h, flagged in zip(hs, ([0, 2 * page - 1, 2 * page, 149 - reach, 150 - reach, 90] + far, [7, 60 - reach if reach < 60 else 8])):
            h[:, 0], h[:, 1] = 0.0, 1.0
            h[[f for f in flagged if 0 <= f < len(h)], 0] = 8.0
    hs = [rounded(h, dtype) for h in hs]
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "kv_rank": rank, "scale": scale,
         "mask": {"size": window} if window else None, "rot": {"dims": rot, "base": 5000.0, "scaling": named}}
    angle = np.float64 if dtype == torch.float32 else np.float32
    want = [M.latent_attention({"x." + k: v for k, v in w.items()}, "x.", m, h.astype(np.float64), np.arange(len(h)), eps,
                               store_of(dtype), angle) for h in hs]
    harness = Harness([part.cache_spec()], dtype, page=page, pages=-(-lengths[0] // page) + -(-61 // page) + 2)
    seqs = [harness.cache.create() for _ in lengths]
    fed = [0, 0]
    got = [np.zeros((n, hidden), np.float32) for n in lengths]
    if schedule == "portions":
        steps = [(16, 1), (5, 9), (1, 1), (2, 3), (13, 8), (40, 2), (2, 30), (64, 2), (7, 5), (200, 1), (250, 1)]
    else:
        steps = [(lengths[0] - 50, 20)] + [(1, 1)] * 50
    for step in steps:
        index = [i for i in range(2) if fed[i] < lengths[i]]
        if not index:
            break
        counts = [min(step[i], lengths[i] - fed[i]) for i in index]
        ctx, entries = harness.context([(seqs[i], [0] * n) for i, n in zip(index, counts)])
        h = torch.cat([dev(hs[i][fed[i]:fed[i] + n], dtype) for i, n in zip(index, counts)])
        residual = torch.zeros(h.shape[0], hidden, device=DEV)
        part.forward(ctx, h, residual, harness.view(ctx, 0))
        out = residual.cpu().numpy()
        harness.commit(entries)
        row = 0
        for i, n in zip(index, counts):
            got[i][fed[i]:fed[i] + n] = out[row:row + n]
            fed[i] += n
            row += n
    assert fed == lengths
    tol = 3e-5 if dtype == torch.float32 else 3e-2
    for i in range(2):
        err = np.abs(got[i] - want[i]).max(axis=1)
        bound = tol * max(1.0, float(np.abs(want[i]).max()))
        assert err.max() <= bound, f"sequence {i}: position {int(err.argmax())} is off by {err.max():.3e} (bound {bound:.1e})"

# ---------------------------------------------------------------------------------------------- whole models
@pytest.fixture(scope="module")
def folders(tmp_path_factory):
    root = str(tmp_path_factory.mktemp("megozen"))
    return {name: MH.make_folder(root, name) for name in MH.CONFIGS}


def requests_for(name, lengths, seed=100):
    vocab = MH.CONFIGS[name]["vocab"]
    return {f"r{i}": MH.random_tokens(vocab, n, seed + i) for i, n in enumerate(lengths)}


def replay(folder, name, dtype, trace, max_tokens, page=None, slots=4, reused=None):
    """The engine's trace session on a pool of `max_tokens` and `slots` state slots; per step the logits rows."""
    from sprout_lm_amd.engine import ModelRunner
    from sprout_lm_amd.engine.trace import TraceSession
    page = page or MH.PAGE[name]
    runner = ModelRunner.from_folder(folder, dtype, block_size=page, num_blocks=-(-max_tokens // page), max_sequences=slots,
                                     prefix_caching=False)
    session = TraceSession(runner)
    out, owners, slot_users = [], {}, {}
    for record in trace.steps:
        logits = session.run_step(record)
        out.append(None if logits is None or not logits.shape[0] else logits.cpu().numpy().copy())
        for rid, seq in session.live.items():
            users = slot_users.setdefault(seq.state_slot, [])
            if rid not in users:
                users.append(rid)
            for page_id in seq.blocks[0]:
                if page_id >= 0 and rid not in owners.setdefault(page_id, []):
                    owners[page_id].append(rid)
    if reused is not None:
        reused["pages"] = sum(len(r) > 1 for r in owners.values())
        reused["slots"] = sum(len(r) > 1 for r in slot_users.values())
    assert all(free == total for free, total in zip(runner.cache.free_pages(), [g.pool.num_pages for g in runner.cache.groups]))
    assert not session.live
    return out


def check(folder, dtype, requests, trace, results):
    worst = 0.0
    for step, (rows, got) in enumerate(zip(trace.expected, results)):
        if not rows:
            assert got is None
            continue
        assert got.shape[0] == len(rows)
        for i, (rid, pos) in enumerate(rows):
            want = MH.plain_logits(folder, dtype, requests[rid])[pos]
            err = float(np.abs(got[i] - want).max())
            worst = max(worst, err)
            assert err <= MH.tolerance(dtype, want), f"step {step} request {rid} position {pos}: error {err:.3e}"
    return worst


LENGTHS = {"odd": [1, 2, 21, 70, 45, 97], "general": [1, 9, 40, 97, 130, 33, 2, 75], "varied": [48, 150, 65, 90, 33, 3], "many_heads": [5, 17, 70, 64, 40],
           "one_layer": [2, 70, 97, 33, 64, 120], "all_chosen": [9, 40, 97, 33, 110]}
# bfloat16 where rounding cannot flip an expert between the two sides: one layer (both sides route the same stored
# input), or every expert chosen
CASES = [(n, "float32") for n in MH.CONFIGS] + [("one_layer", "bfloat16"), ("all_chosen", "bfloat16")]


@pytest.mark.parametrize("name,dtype", CASES)
@pytest.mark.parametrize("family", ["whole", "tail", "portions", "mixed"])
def test_replay_family(folders, name, dtype, family):
    """Whole prompts; a prompt and its last 48 tokens one by one (windows of 16 to 37 pass over decoded tokens);
    portions down to two tokens; four live requests in a pool and on state slots that hold no more, so that both
    are used again."""
    requests = requests_for(name, LENGTHS[name])
    roomy = 4 * 64 * (1 + max(LENGTHS[name]) // 64)
    if family == "whole":
        trace, pool = traces.whole(requests), roomy
    elif family == "tail":
        trace, pool = traces.tail_decoded(requests, tail=48), roomy
    elif family == "portions":
        trace, pool = traces.portions(requests), roomy
    else:
        trace = traces.mixed(requests, seed=7)
        pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    reused = {}
    results = replay(folders[name], name, dtype, trace, pool, reused=reused)
    if family == "mixed":
        assert reused["pages"] >= 2 and reused["slots"] >= 1, f"nothing was used again: {reused}"
    worst = check(folders[name], dtype, requests, trace, results)
    print(f"{family} {name} {dtype}: {len(trace.steps)} steps, worst error {worst:.3e}")


@pytest.mark.parametrize("name,page", [("general", 12), ("varied", 4), ("one_layer", 6)])
def test_replay_with_other_page_sizes(folders, name, page):
    requests = requests_for(name, LENGTHS[name], seed=300)
    trace = traces.mixed(requests, seed=11)
    pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    results = replay(folders[name], name, "float32", trace, pool, page=page)
    check(folders[name], "float32", requests, trace, results)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_cuts_agree_with_each_other(folders, dtype):
    """Whole, token-by-token and portioned replays give the same logits beyond rounding."""
    name = "all_chosen"
    requests = requests_for(name, [90])
    rows_of = {}
    for family, trace in (("whole", traces.whole(requests)), ("tail", traces.tail_decoded(requests, tail=89)),
                          ("portions", traces.portions(requests))):
        results = replay(folders[name], name, dtype, trace, 256)
        rows_of[family] = {key: got[i] for expect, got in zip(trace.expected, results) for i, key in enumerate(expect)}
    bound = 1e-5 if dtype == "float32" else 3e-2
    for key, row in rows_of["whole"].items():
        for other in ("tail", "portions"):
            if key in rows_of[other]:
                assert np.abs(row - rows_of[other][key]).max() <= bound * max(1.0, np.abs(row).max()), (key, other)


def test_first_tokens_and_long_decoding(folders):
    """Positions 0, 1, 2, ... fed one by one from the very first token, 260 in a row, past every window."""
    from sprout_lm_amd.engine import ModelRunner, StepEntry
    for name, dtype in (("general", "float32"), ("one_layer", "bfloat16")):
        tokens = MH.random_tokens(MH.CONFIGS[name]["vocab"], 260, 9)
        runner = ModelRunner.from_folder(folders[name], dtype, block_size=8, num_blocks=40, max_sequences=2,
                                         prefix_caching=False)
        seq = runner.cache.create()
        want = MH.plain_logits(folders[name], dtype, tokens)
        for p, token in enumerate(tokens):
            assert runner.cache.reserve(seq, p + 1)
            got = runner.step([StepEntry(seq, [token], [0])]).cpu().numpy()[0]
            assert np.abs(got - want[p]).max() <= MH.tolerance(dtype, want[p]), f"{name} {dtype} position {p}"
        seq.release()


def test_trace_run_program(folders, tmp_path):
    """bin/trace_run as a user runs it, on a model it picks by the folder's config.json."""
    name, dtype = "varied", "float32"
    requests = requests_for(name, [33, 70, 20, 64, 45])
    trace = traces.mixed(requests, seed=3)
    pool = sum(sorted(-(-len(t) // 64) * 64 for t in requests.values())[-4:])
    out = tmp_path / "logits"
    proc = subprocess.Popen([sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folders[name],
                             "--dtype", dtype, "--out", str(out), "--max-tokens", str(pool), "--max-sequences", "4"],
                            stdin=subprocess.PIPE, stdout=subprocess.PIPE, text=True, bufsize=1)
    try:
        for record in trace.steps:
            proc.stdin.write(json.dumps(record) + "\n")
            proc.stdin.flush()
            assert proc.stdout.readline().strip() == f"done {record['step']}"
        proc.stdin.close()
        assert proc.wait(timeout=60) == 0
    finally:
        if proc.poll() is None:
            proc.kill()
    vocab = MH.CONFIGS[name]["vocab"]
    results = [np.fromfile(out / f"{r['step']}.f32", dtype="<f4").reshape(len(rows), vocab) if rows else None
               for r, rows in zip(trace.steps, trace.expected)]
    check(folders[name], dtype, requests, trace, results)


# ---------------------------------------------------------------------------------------------- generation
def plain_greedy(folder, dtype, prompt, steps):
    history, out = list(prompt), []
    for _ in range(steps):
        token = int(np.argmax(MH.plain_logits(folder, dtype, history)[-1]))
        history.append(token)
        out.append(token)
    return out


def test_greedy_generation_through_the_entry_point(folders):
    """Prompts of 1 to 70 tokens in portions of 16, 20 greedy tokens each, float32: every token is the plain side's."""
    from sprout_lm_amd.engine import Engine
    for name in ("general", "varied"):
        engine = Engine.from_folder(folders[name], "float32", block_size=MH.PAGE[name], num_blocks=64, max_sequences=4,
                                    max_batch_tokens=48, prefill_chunk_size=16, record_trace=True)
        vocab = MH.CONFIGS[name]["vocab"]
        prompts = [MH.random_tokens(vocab, n, 40 + i) for i, n in enumerate((1, 9, 40, 70))]
        outputs = engine.generate(prompts, max_new_tokens=20, ignore_eos=True)
        for prompt, got in zip(prompts, outputs):
            assert got == plain_greedy(folders[name], "float32", prompt, 20), f"{name}, prompt of {len(prompt)}"
        assert all(free == g.pool.num_pages for free, g in zip(engine.cache.free_pages(), engine.cache.groups))


def test_scheduling_never_changes_generation(folders):
    """Too few pages (preemption, then the prompt and what was generated computed again, from the first token's
    own row of the pair table) and a late arrival give what each request generates alone."""
    from sprout_lm_amd.engine import Engine
    name, dtype = "general", "float32"
    vocab = MH.CONFIGS[name]["vocab"]
    prompts = {"A": MH.random_tokens(vocab, 33, 78), "B": MH.random_tokens(vocab, 29, 79),
               "C": MH.random_tokens(vocab, 40, 80), "D": MH.random_tokens(vocab, 3, 81)}
    want = {k: plain_greedy(folders[name], dtype, p, 14) for k, p in prompts.items()}
    for num_blocks, expect_preemption in ((64, False), (14, True)):
        engine = Engine.from_folder(folders[name], dtype, block_size=8, num_blocks=num_blocks, max_sequences=4,
                                    max_batch_tokens=24, prefill_chunk_size=16, record_trace=True)
        engine.add("A", prompts["A"], 14, ignore_eos=True)
        engine.step(); engine.step(); engine.step()
        for k in "BCD":
            engine.add(k, prompts[k], 14, ignore_eos=True)
        ticks = 0
        while engine.pending:
            ticks += 1
            assert ticks < 2000
            engine.step()
        for k in prompts:
            assert engine.result(k)["output"] == want[k], f"request {k} with {num_blocks} pages"
        assert any(e["type"] == "preempted" for e in engine.trace) == expect_preemption


def test_recorded_steps_equal_eager_steps(folders):
    """Steps replayed from recorded graphs (decoded tokens with the sampler inside; the pair table's previous token
    read from the request's state on the device) give the tokens of eagerly launched steps."""
    from sprout_lm_amd.engine import Engine
    name = "all_chosen"
    vocab = MH.CONFIGS[name]["vocab"]
    prompts = [MH.random_tokens(vocab, n, 60 + i) for i, n in enumerate((7, 21, 3, 40, 12))]

    def run(use_graphs):
        engine = Engine.from_folder(folders[name], "bfloat16", block_size=16, num_blocks=48, max_sequences=4,
                                    max_batch_tokens=32, prefill_chunk_size=16)
        engine.model.use_graphs = use_graphs
        engine.add("r0", prompts[0], 30, ignore_eos=True)
        engine.add("r1", prompts[1], 25, ignore_eos=True)
        steps = 0
        while engine.pending:
            steps += 1
            if steps == 6:
                engine.add("r2", prompts[2], 20, temperature=0.8, seed=5, ignore_eos=True)
            if steps == 15:
                engine.add("r3", prompts[3], 10, ignore_eos=True)
                engine.add("r4", prompts[4], 28, temperature=1.2, seed=9, ignore_eos=True)
            engine.step()
        replays = engine.model._graphs.replays if engine.model._graphs else 0
        return [engine.result(f"r{i}")["output"] for i in range(5)], replays

    eager, none = run(False)
    graphed, replays = run(True)
    assert none == 0 and replays > 40
    assert graphed == eager


def test_command_line_generates(folders):
    done = subprocess.run([sys.executable, "-m", "sprout_lm_amd", "generate", folders["varied"], "--prompt-ids",
                           "3,1,4,1,5,9,2,6", "--dtype", "float32", "--ignore-eos"], cwd=ROOT,
                          env=dict(os.environ, MAX_NEW_TOKENS="6"), capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stderr
    final = json.loads(done.stdout.strip().splitlines()[-1])
    assert final["output"] == plain_greedy(folders["varied"], "float32", [3, 1, 4, 1, 5, 9, 2, 6], 6)
