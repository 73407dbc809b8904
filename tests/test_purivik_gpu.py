"""Purivik on the MI355X: each of its kernels alone against tests/reference_ops.py (float64), then the engine's steps however
a request is cut and batched, captured decode steps and greedy generation against tests/plain_purivik.py."""

import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_purivik
import purivik_configs as pc
import trace_tools as tt
from reference_ops import ReferenceOps

pytestmark = pytest.mark.gpu

DEV = "cuda:0"
BF16_EPS = 2.0 ** -8


@pytest.fixture(scope="module")
def ops():
    from fllm_amd.kernels import Ops
    return Ops()


@pytest.fixture(scope="module")
def ref():
    return ReferenceOps()


def gen(seed):
    g = torch.Generator()
    g.manual_seed(seed)
    return g


def close(got, want, rtol, atol, what=""):
    got, want = got.detach().double().cpu(), want.detach().double().cpu()
    err = (got - want).abs()
    worst = (err - (atol + rtol * want.abs())).max().item()
    assert worst <= 0, f"{what}: max err {err.max().item():.3e} (|want| max {want.abs().max().item():.3e}), over by {worst:.3e}"


# ---------------------------------------------------------------------------------------------
# a branch normed on its way into the stream
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("branch_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("parts,normalize,then", [(1, True, None), (1, True, torch.bfloat16), (3, True, torch.float32), (2, False, None)])
@pytest.mark.parametrize("rows,width", [(1, 64), (7, 203), (33, 1000), (130, 4096)])
def test_a_branch_normed_into_the_stream(ops, ref, rows, width, parts, normalize, then, branch_dtype):
    x = torch.randn(rows, width, generator=gen(1)) * 3
    branch = (torch.randn(rows * parts, width, generator=gen(2)) * 5).to(branch_dtype)
    gain = 0.7 * (1 + 0.3 * torch.randn(width, generator=gen(3)))
    next_w = 1 + 0.3 * torch.randn(width, generator=gen(4))
    eps = 1e-5 if normalize else None
    want = x.double().clone()
    want_next = torch.empty(rows, width, dtype=torch.float64) if then is not None else None
    ref.postnorm_add(want, branch.double(), gain, eps, parts=parts, next_weight=next_w if then is not None else None, next_eps=1e-6,
                     next_out=want_next)
    got = x.clone().to(DEV)
    got_next = torch.empty(rows, width, dtype=then, device=DEV) if then is not None else None
    ops.postnorm_add(got, branch.to(DEV), gain.to(DEV), eps, parts=parts, next_weight=next_w.to(DEV) if then is not None else None,
                     next_eps=1e-6, next_out=got_next)
    close(got, want, 2e-6, 2e-6, "stream")
    if then is not None:
        close(got_next, want_next, 3e-6 if then == torch.float32 else BF16_EPS, 1e-6, "the norm behind the sum")
    # a row's bits do not depend on the rest of the batch
    alone = x[rows - 1:].clone().to(DEV)
    ops.postnorm_add(alone, branch[(rows - 1) * parts:].to(DEV), gain.to(DEV), eps, parts=parts)
    assert torch.equal(alone[0], got[rows - 1])


# ---------------------------------------------------------------------------------------------
# routed experts
# ---------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("rows,width,experts,top", [(1, 64, 5, 2), (9, 68, 7, 7), (40, 320, 12, 1), (200, 1024, 64, 6), (3, 50, 130, 4)])
def test_the_router_picks_the_largest_scores(ops, ref, rows, width, experts, top, dtype):
    h = torch.randn(rows, width, generator=gen(5)).to(dtype)
    w = (torch.randn(experts, width, generator=gen(6)) * 2 * width ** -0.5).to(dtype)
    want_ids, want_w = torch.empty(rows, top, dtype=torch.int32), torch.empty(rows, top, dtype=torch.float32)
    ref.route_topk(h, w, top, want_ids, want_w)
    ids = torch.empty(rows, top, dtype=torch.int32, device=DEV)
    weights = torch.empty(rows, top, dtype=torch.float32, device=DEV)
    ops.route_topk(h.to(DEV), w.to(DEV), top, ids, weights)
    score = torch.sigmoid(h.double() @ w.double().T)
    # where two scores are closer than float32 sums can tell apart either order is right: compare the scores of the picks
    close(weights, torch.gather(score, 1, ids.cpu().long()), 1e-5, 1e-6, "a pick's weight is its own score")
    close(weights, want_w.double(), 1e-5, 1e-6, "the k-th largest score")
    for r in range(rows):
        assert len(set(ids[r].tolist())) == top, "an expert is picked once"
    margin = (want_w[:, :-1] - want_w[:, 1:]).min().item() if top > 1 else 1.0
    if margin > 1e-5:
        assert torch.equal(ids.cpu(), want_ids)


def test_equal_scores_go_to_the_lower_index(ops):
    width, experts = 32, 6
    h = torch.randn(4, width, generator=gen(7))
    row = torch.randn(width, generator=gen(8))
    w = torch.stack([row * 0.1, row, row * 0.5, row, -row, row])          # experts 1, 3 and 5 score alike
    ids = torch.empty(4, 3, dtype=torch.int32, device=DEV)
    weights = torch.empty(4, 3, dtype=torch.float32, device=DEV)
    ops.route_topk(h.to(DEV), w.to(DEV), 3, ids, weights)
    for r in range(4):
        positive = float(h[r] @ row) > 0
        assert ids[r].tolist() == ([1, 3, 5] if positive else [4, 0, 2])


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("limit,alpha,offset", [(0.0, 1.0, 0.0), (1.5, 1.702, 1.0)])
@pytest.mark.parametrize("rows,width,inter,experts,top", [(1, 64, 24, 5, 2), (9, 68, 18, 7, 3), (40, 320, 96, 12, 1), (70, 256, 130, 4, 4)])
def test_the_products_of_the_picked_experts(ops, ref, rows, width, inter, experts, top, limit, alpha, offset, dtype):
    g = gen(9)
    h = torch.randn(rows, width, generator=g).to(dtype)
    w_gate_up = (torch.randn(experts, 2 * inter, width, generator=g) * 2 * width ** -0.5).to(dtype)
    w_down = (torch.randn(experts, width, inter, generator=g) * inter ** -0.5).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(rows)]).to(torch.int32)
    weights = torch.rand(rows, top, generator=g)
    want_act = torch.empty(rows * top, inter, dtype=torch.float64)
    ref.experts_gate_up(h, ids, weights, w_gate_up, want_act, limit, alpha, offset)
    act = torch.empty(rows * top, inter, dtype=dtype, device=DEV)
    ops.experts_gate_up(h.to(DEV), ids.to(DEV), weights.to(DEV), w_gate_up.to(DEV), act, limit, alpha, offset)
    tol = 2e-5 if dtype == torch.float32 else 2 * BF16_EPS
    close(act, want_act, tol, tol, "activations")
    want = torch.empty(rows * top, width, dtype=torch.float64)
    ref.experts_down(act.cpu(), ids, w_down, want)
    out = torch.empty(rows * top, width, dtype=torch.float32, device=DEV)
    ops.experts_down(act, ids.to(DEV), w_down.to(DEV), out)
    close(out, want, 2e-5, 2e-5, "outputs")
    # a pair alone gives the bits it gives in the batch
    one = torch.empty(top, inter, dtype=dtype, device=DEV)
    ops.experts_gate_up(h[rows - 1:].to(DEV), ids[rows - 1:].to(DEV), weights[rows - 1:].to(DEV), w_gate_up.to(DEV), one, limit, alpha, offset)
    assert torch.equal(one, act[(rows - 1) * top:])


@pytest.mark.parametrize("spread", ["random", "one expert", "two experts"])
@pytest.mark.parametrize("limit,alpha,offset", [(0.0, 1.0, 0.0), (1.5, 1.702, 1.0)])
@pytest.mark.parametrize("rows,width,inter,experts,top", [(17, 64, 24, 5, 2), (70, 136, 40, 7, 3), (300, 320, 96, 12, 1), (1000, 256, 136, 40, 4),
                                                           (129, 512, 264, 3, 3)])
def test_experts_grouped_on_the_matrix_cores(ops, ref, rows, width, inter, experts, top, limit, alpha, offset, spread):
    """Prompt portions: the pairs are grouped by expert and multiplied as tiles.  Experts without a row, experts with more
    rows than a tile, tiles that are not full."""
    g = gen(11)
    dtype = torch.bfloat16
    h = torch.randn(rows, width, generator=g).to(dtype)
    w_gate_up = (torch.randn(experts, 2 * inter, width, generator=g) * 2 * width ** -0.5).to(dtype)
    w_down = (torch.randn(experts, width, inter, generator=g) * inter ** -0.5).to(dtype)
    ids = torch.stack([torch.randperm(experts, generator=g)[:top] for _ in range(rows)]).to(torch.int32)
    if spread == "one expert":
        ids[:, 0] = experts - 1
    elif spread == "two experts":
        ids[:, 0] = torch.where(torch.arange(rows) % 5 == 0, 0, 2).to(torch.int32)
    weights = torch.rand(rows, top, generator=g)
    want_act = torch.empty(rows * top, inter, dtype=torch.float64)
    ref.experts_gate_up(h, ids, weights, w_gate_up, want_act, limit, alpha, offset)
    want = torch.empty(rows * top, width, dtype=torch.float64)
    ref.experts_down(want_act.to(dtype), ids, w_down, want)
    out = torch.full((rows * top, width), float("nan"), dtype=torch.float32, device=DEV)
    taken = ops.experts_grouped(h.to(DEV), ids.to(DEV), weights.to(DEV), w_gate_up.to(DEV), w_down.to(DEV), out, limit, alpha, offset)
    assert taken
    close(out, want, 2 * BF16_EPS, 2 * BF16_EPS * want.abs().max().item(), "grouped experts")
    # the plain kernels on the same pairs; and a row's result does not depend on which rows share its tile
    act = torch.empty(rows * top, inter, dtype=dtype, device=DEV)
    ops.experts_gate_up(h.to(DEV), ids.to(DEV), weights.to(DEV), w_gate_up.to(DEV), act, limit, alpha, offset)
    plain = torch.empty(rows * top, width, dtype=torch.float32, device=DEV)
    ops.experts_down(act, ids.to(DEV), w_down.to(DEV), plain)
    close(out, plain.double(), 2 * BF16_EPS, 2 * BF16_EPS * want.abs().max().item(), "grouped against plain kernels")
    keep = torch.randperm(rows, generator=g)[:max(17, rows // 3)].sort()[0]
    part = torch.empty(len(keep) * top, width, dtype=torch.float32, device=DEV)
    assert ops.experts_grouped(h[keep].to(DEV), ids[keep].to(DEV), weights[keep].to(DEV), w_gate_up.to(DEV), w_down.to(DEV), part, limit, alpha, offset)
    # (to the last bits only: few rows cut the down product along K, and the slices are summed in another order)
    close(part.view(len(keep), top, width), out.view(rows, top, width)[keep.to(DEV)].double(), 1e-5, 1e-5 * want.abs().max().item(), "other company")
    few = 1 if top > 1 else 2           # fewer than two pairs an expert: left to the plain kernels
    assert not ops.experts_grouped(h[:few].to(DEV), ids[:few].to(DEV), weights[:few].to(DEV), w_gate_up.to(DEV), w_down.to(DEV), part[:few * top])


# ---------------------------------------------------------------------------------------------
# rotary + store, and the attention, over scattered pages: values of a width of their own, chunks of positions
# ---------------------------------------------------------------------------------------------
class Scene:
    """Requests with `held` tokens in the cache and `new` rows in this step, pages dealt out in a shuffled order, caches
    full of random numbers (so a key that must not be seen is loud, not zero)."""

    def __init__(self, segs, H, G, d, dv, page, rope_dims, seed, dtype, loud=None):
        g = gen(seed)
        self.H, self.G, self.d, self.dv, self.page, self.rope_dims = H, G, d, dv, page, rope_dims
        self.key_chunk = 8 if d % 8 == 0 else 1
        longest = max(h + n for h, n in segs)
        per_seg = -(-longest // page) + 1
        num_pages = per_seg * len(segs) + 3
        self.tables = torch.randperm(num_pages, generator=g)[:per_seg * len(segs)].to(torch.int32).view(len(segs), per_seg).contiguous()
        self.k_pages = torch.randn(num_pages, G, d // self.key_chunk, page, self.key_chunk, generator=g).to(dtype)
        self.v_pages = torch.randn(num_pages, G, dv, page, generator=g).to(dtype)
        pos, seg, start = [], [], [0]
        for s, (held, new) in enumerate(segs):
            pos += list(range(held, held + new))
            seg += [s] * new
            start.append(start[-1] + new)
        self.row_pos = torch.tensor(pos, dtype=torch.int32)
        self.row_seg = torch.tensor(seg, dtype=torch.int32)
        self.seg_start = torch.tensor(start, dtype=torch.int32)
        self.single_from = next((i for i in range(len(segs) + 1) if all(n == 1 for _, n in segs[i:])), len(segs))
        self.qkv = torch.randn(len(pos), (H + G) * d + G * dv, generator=g).to(dtype)
        self.max_pos = longest + 1
        half = rope_dims // 2
        freq = torch.tensor([500.0 ** (-2.0 * i / max(rope_dims, 1)) for i in range(half)], dtype=torch.float64)
        angle = torch.arange(self.max_pos, dtype=torch.float64)[:, None] * freq[None, :]
        self.cos, self.sin = torch.cos(angle).float(), torch.sin(angle).float()
        for s, p, factor in loud or ():     # a cached key that would take all the weight of whoever sees it
            self.k_pages[int(self.tables[s, p // page]), :, :, p % page, :] *= factor

    def tensors(self, device, dtype=None):
        names = ["tables", "k_pages", "v_pages", "row_pos", "row_seg", "seg_start", "qkv", "cos", "sin"]
        out = {n: getattr(self, n).clone().to(device) for n in names}
        if dtype is not None:
            for n in ("k_pages", "v_pages", "qkv"):
                out[n] = out[n].to(dtype)
        return out


def run_attention(o, t, sc, chunk, window, scale, dtype, pairing=0, on_device=True):
    rows = t["qkv"].shape[0]
    H, G, d, dv = sc.H, sc.G, sc.d, sc.dv
    o.rope_kv_store(t["qkv"], t["row_pos"], t["row_seg"], t["tables"], t["cos"], t["sin"], t["k_pages"], t["v_pages"], H, G, d,
                    sc.rope_dims, pairing, sc.page, v_dim=dv, key_chunk=sc.key_chunk)
    out = torch.empty(rows, H * dv, dtype=dtype, device=t["qkv"].device)
    extra = {}
    if on_device:
        need = o.attention_workspace_bytes(rows, H, G, d, sc.max_pos)
        extra = {"single_from": sc.single_from, "workspace": torch.empty(max(need, 1), dtype=torch.uint8, device=t["qkv"].device)}
    o.attention(t["qkv"][:, :H * d], t["k_pages"], t["v_pages"], t["tables"], t["row_pos"], t["row_seg"], t["seg_start"], out, H, G, d,
                sc.page, scale, window, sc.max_pos, v_dim=dv, chunk=chunk, key_chunk=sc.key_chunk, **extra)
    return out


# heads, kv heads, key size, value size, chunk, window, page, rotated lanes
SHAPES = [(4, 2, 32, 16, 24, None, 8, 16), (6, 3, 64, 64, 40, None, 16, 32), (2, 1, 20, 12, None, None, 8, 0),
          (8, 2, 64, 32, 80, None, 16, 32), (3, 1, 24, 40, 7, None, 16, 10), (5, 1, 128, 128, 100, None, 64, 64),
          (8, 8, 128, 128, 33, 50, 16, 128), (8, 2, 64, 64, 16, None, 16, 64), (4, 4, 32, 32, 64, None, 32, 8),
          (16, 4, 128, 64, 200, None, 16, 32), (6, 2, 64, 64, None, None, 8, 16), (3, 3, 72, 72, 30, 19, 16, 24)]
# (held, new) per request: prompts from the first token, portions that begin inside a chunk and cross its edge, single
# rows right before, on and after an edge, two-token portions; the single rows come last, as the step function lays them out
SEGMENTS = [(0, 50), (23, 30), (79, 2), (95, 18), (2, 2), (130, 70), (37, 1), (80, 1), (0, 1), (120, 1), (47, 1), (48, 1), (199, 1)]
# a decode step: one row a request, right before, on and after the edges of chunks, pages and key blocks
SINGLE_ROWS = [(0, 1), (1, 1), (15, 1), (16, 1), (39, 1), (40, 1), (63, 1), (64, 1), (79, 1), (80, 1), (127, 1), (128, 1), (199, 1), (33, 1),
               (6, 1), (7, 1), (99, 1), (100, 1)]


@pytest.mark.parametrize("rows", ["mixed", "single"])
@pytest.mark.parametrize("fast", [True, False])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_attention_over_pages(ops, ref, shape, dtype, fast, rows):
    H, G, d, dv, chunk, window, page, rope_dims = shape
    segments = SINGLE_ROWS if rows == "single" else SEGMENTS
    if dtype == torch.float32 and not fast:
        pytest.skip("float32 has one kernel")
    scale = d ** -0.5 * 1.3
    # loud keys at the edges of what a row may see: the last position of the chunk before its own, and the position after
    # itself (a stale key of a page that was used before)
    loud = []
    for s, (held, new) in enumerate(segments):
        last = held + new - 1
        if chunk and last - last % chunk > 0 and held > 0:
            loud.append((s, min(last - last % chunk, held) - 1, 8.0))
        loud.append((s, last + 1, 8.0))
    sc = Scene(segments, H, G, d, dv, page, rope_dims, seed=H * 100 + d, dtype=dtype, loud=loud)
    want_t = sc.tensors("cpu", torch.float64)
    want = run_attention(ref, want_t, sc, chunk, window, scale, torch.float64, on_device=False)
    ops.set_fast_kernels(fast)
    try:
        got_t = sc.tensors(DEV)
        got = run_attention(ops, got_t, sc, chunk, window, scale, dtype)
        torch.cuda.synchronize()
    finally:
        ops.set_fast_kernels(True)
    assert torch.equal(got_t["v_pages"].cpu().double(), want_t["v_pages"]), "stored values"
    if dtype == torch.float32:
        close(got_t["k_pages"], want_t["k_pages"], 1e-5, 1e-5, "stored keys")
        close(got, want, 5e-4, 5e-4, "attention")
        return
    close(got_t["k_pages"], want_t["k_pages"], BF16_EPS, 1e-3, "stored keys")
    # sharp softmaxes amplify the rounding of the bfloat16 queries and keys, so the kernel is held against the reference run
    # on what the kernel itself stored
    again = torch.empty_like(want)
    ref.attention(got_t["qkv"][:, :H * d].cpu().double(), got_t["k_pages"].cpu().double(), got_t["v_pages"].cpu().double(),
                  want_t["tables"], want_t["row_pos"], want_t["row_seg"], want_t["seg_start"], again, H, G, d, page, scale, window,
                  sc.max_pos, v_dim=dv, chunk=chunk, key_chunk=sc.key_chunk)
    close(got, again, 3 * BF16_EPS, 3e-2, "attention")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("sizes", [(64, 64), (64, 32), (128, 128), (24, 40)])
@pytest.mark.parametrize("held", [340, 2000])
@pytest.mark.parametrize("where", ["first of the chunk", "just outside", "far back", "itself"])
def test_one_key_that_stands_out(ops, where, held, sizes, dtype):
    """One key among hundreds (or thousands) takes nearly all the weight of one head: the output is that key's value when the
    row may see it, and shows no trace of it when the key lies outside the row's chunk.  As a single row (a decode step) and
    as the last row of a portion."""
    d, dv = sizes
    H, G, chunk, page = 4, 2, (100 if held < 1000 else 1500), 16
    lo = held - held % chunk
    target = {"first of the chunk": lo, "just outside": lo - 1, "far back": 5, "itself": held}[where]
    if where == "far back" and held >= 1000:
        target = lo + 3            # far from the row, inside its chunk: a key among a thousand
    for segs in ([(7, 3), (held, 1)], [(held - 20, 21), (7, 1)]):
        sc = Scene(segs, H, G, d, dv, page, 0, seed=9, dtype=dtype)
        s = 1 if segs[0][0] == 7 else 0
        row = int(sc.seg_start[s + 1]) - 1                    # the row at position `held`
        t = sc.tensors(DEV)
        q = (0.05 * torch.randn(t["qkv"].shape[0], H * d, generator=gen(3))).to(dtype).to(DEV)
        direction = torch.randn(d, generator=gen(4))
        direction = direction / direction.norm()
        q[row, d:2 * d] = (direction * 8).to(dtype).to(DEV)      # head 1 reads key/value head 0
        t["k_pages"].mul_(0.05)
        pg, off = int(sc.tables[s, target // page]), target % page
        t["k_pages"][pg, 0, :, off, :] = (direction * 8).view(d // sc.key_chunk, sc.key_chunk).to(dtype).to(DEV)

        def attend(k_pages):
            out = torch.empty(q.shape[0], H * dv, dtype=dtype, device=DEV)
            need = ops.attention_workspace_bytes(q.shape[0], H, G, d, sc.max_pos)
            ops.attention(q, k_pages, t["v_pages"], t["tables"], t["row_pos"], t["row_seg"], t["seg_start"], out, H, G, d, page, 1.0,
                          None, sc.max_pos, v_dim=dv, chunk=chunk, key_chunk=sc.key_chunk, single_from=sc.single_from,
                          workspace=torch.empty(max(need, 1), dtype=torch.uint8, device=DEV))
            return out
        out = attend(t["k_pages"])
        head1 = out[row, dv:2 * dv].float().cpu()
        value = t["v_pages"][pg, 0, :, off].float().cpu()
        if lo <= target <= held:
            close(head1, value, 2 * BF16_EPS, 2e-2, where)
        else:
            assert (head1 - value).abs().max() > 0.3, f"{where}: the key must not be seen"
            quiet = t["k_pages"].clone()
            quiet[pg, 0, :, off, :] = 0
            assert torch.equal(out, attend(quiet)), f"{where}: a key outside the chunk changed the output"


def test_the_matrix_core_attention_takes_chunks_of_positions(ops):
    """bfloat16 with keys and values of 64 or 128 lanes runs the matrix-core kernels, chunks or not: the plain kernel, switched
    on instead, rounds differently somewhere."""
    for segments in (SEGMENTS, SINGLE_ROWS):
        sc = Scene(segments, 8, 2, 64, 64, 16, 32, seed=77, dtype=torch.bfloat16)
        outs = []
        for fast in (True, False):
            ops.set_fast_kernels(fast)
            try:
                outs.append(run_attention(ops, sc.tensors(DEV), sc, 40, None, 0.2, torch.bfloat16).float().cpu())
            finally:
                ops.set_fast_kernels(True)
        assert not torch.equal(outs[0], outs[1])
        close(outs[0], outs[1], 4 * BF16_EPS, 4e-2, "two kernels")


# ---------------------------------------------------------------------------------------------
# the engine
# ---------------------------------------------------------------------------------------------
LENGTHS = {"A": [5, 30, 61, 100, 49], "B": [45, 83, 161, 2, 120], "C": [9, 50, 300, 130], "D": [100, 37, 250, 81, 160], "E": [31, 2, 75, 120], "F": [60, 130, 17],
           "G": [700, 333, 64, 461]}
# about three times the largest error any case here has shown on the MI355X (float32 5.3e-6, bfloat16 2.5e-2).  The float32
# figure is that of the configurations which rotate every lane of a head: the angles are float32 products of a position and
# a frequency, as the design has them, and at positions beyond 100 they differ from the plain implementation's float64
# angles by 1e-5; the error grows with the position and is the same however a request is cut (compared bit for bit below).
TOL = {"float32": 1.5e-5, "bfloat16": 6e-2}


@pytest.fixture(scope="module")
def models(tmp_path_factory):
    """(configuration, precision) -> folder, configuration, requests, plain logits, weights.  float32 runs random routers;
    bfloat16 runs routers whose every pick has a margin (see purivik_configs.weights), since a pick that flips under
    rounding is a large error that says nothing about the kernels."""
    out = {}
    for name, cfg in pc.CONFIGS.items():
        for dtype in ("float32", "bfloat16"):
            tensors = pc.weights(cfg, 30 + ord(name), decided_router=dtype == "bfloat16")
            folder = pc.write_model(str(tmp_path_factory.mktemp(f"purivik_{name}_{dtype}")), cfg, tensors)
            requests = {f"r{i}": pc.random_ids(n, cfg["vocab"], 100 * ord(name) + i) for i, n in enumerate(LENGTHS[name])}
            w64 = pc.to_float64(tensors)
            plain = {rid: plain_purivik.forward(cfg, w64, toks) for rid, toks in requests.items()}
            out[name, dtype] = (folder, cfg, requests, plain, w64)
    return out


def make_runner(folder, dtype, page_size, max_tokens, **kw):
    from fllm_amd.engine import ModelRunner
    return ModelRunner.from_folder(folder, dtype=dtype, page_size=page_size, max_tokens=max_tokens, max_requests=4, **kw)


def check(got, plain, dtype, what):
    for rid, want in plain.items():
        assert rid in got and got[rid].shape == want.shape, f"{what}: request {rid}"
        err = np.abs(got[rid].astype(np.float64) - want)
        scale = np.abs(want).max()
        tt.observe(f"purivik {what.split()[0]} {dtype}", err.max() / scale)
        over = err.max(axis=1) > TOL[dtype] * scale
        assert not over.any(), (f"{what}: request {rid}: max error {err.max():.3e} (limit {TOL[dtype] * scale:.3e}); first "
                                f"position over the limit: {int(np.argmax(over))}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E", "F", "G"])
@pytest.mark.parametrize("family", ["whole", "last40", "portions", "mixed"])
def test_replay(models, tmp_path, name, dtype, family):
    folder, cfg, requests, plain, _ = models[name, dtype]
    refed = [rid for rid, toks in requests.items() if len(toks) >= 60][:1]
    steps = {"whole": tt.whole, "last40": lambda r: tt.last_tokens_one_by_one(r, 40), "portions": tt.portions,
             "mixed": lambda r: tt.mixed(r, seed=5, refeed=refed)}[family](requests)
    steps = tt.number(steps)
    runner = make_runner(folder, dtype, pc.PAGE_SIZES[name], tt.live_tokens_bound(steps))
    handed_out = tt.record_allocations(runner.cache)
    given_up = {}
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path), given_up)
    check(got, plain, dtype, f"{family} {name} {dtype}")
    if family == "mixed" and dtype == "float32":
        for rid, feedings in given_up.items():
            for first in feedings:
                assert np.array_equal(first, got[rid][:len(first)]), f"{rid}: fed again on other pages, other logits"
    runner.cache.check_invariants()
    assert all(pool.available == pool.num_pages for pool in runner.cache.pools), "pages were lost"
    for pages in handed_out:
        assert len(pages) > len(set(pages)), "the trace was meant to use pages again"


@pytest.mark.parametrize("page_size", [4, 32, 64])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_at_other_page_sizes(models, tmp_path, page_size, dtype):
    folder, cfg, requests, plain, _ = models["D", dtype]
    steps = tt.number(tt.mixed(requests, seed=8))
    runner = make_runner(folder, dtype, page_size, tt.live_tokens_bound(steps, round_to=max(64, page_size)))
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, plain, dtype, f"pages-of-{page_size} D {dtype}")


@pytest.mark.parametrize("name", ["A", "D"])
def test_cuts_agree_bit_for_bit_in_float32(models, tmp_path, name):
    folder, cfg, requests, plain, _ = models[name, "float32"]
    results = []
    for i, make in enumerate([tt.whole, tt.portions, lambda r: tt.mixed(r, seed=3)]):
        steps = tt.number(make(requests))
        runner = make_runner(folder, "float32", pc.PAGE_SIZES[name], tt.live_tokens_bound(steps))
        results.append(tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path / str(i))))
    for rid in requests:
        assert np.array_equal(results[0][rid], results[1][rid]), f"whole vs portions differ for {rid}"
        assert np.array_equal(results[0][rid], results[2][rid]), f"whole vs mixed differ for {rid}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["B", "C", "E"])
def test_first_tokens_and_long_decoding(models, tmp_path, name, dtype):
    """Token by token from the very first token, across several chunks of positions (B, E) and with every key seen (C)."""
    folder, cfg, requests, plain, _ = models[name, dtype]
    rid = "r2"
    one = {rid: requests[rid]}
    steps = tt.number(tt.last_tokens_one_by_one(one, tail=len(requests[rid])))
    runner = make_runner(folder, dtype, pc.PAGE_SIZES[name], 320)
    got = tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path))
    check(got, {rid: plain[rid]}, dtype, f"token-by-token {name} {dtype}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "C", "D"])      # C: two decode rows are six pairs over three experts, grouped inside the graph
def test_decode_graphs_and_eager_steps_agree(models, tmp_path, name, dtype):
    folder, cfg, requests, plain, _ = models[name, dtype]
    steps = tt.number(tt.last_tokens_one_by_one(requests) + tt.mixed(requests, seed=21, decode_tail=40))
    results = []
    for i, use_graphs in enumerate((True, False)):
        runner = make_runner(folder, dtype, pc.PAGE_SIZES[name], tt.live_tokens_bound(steps), use_graphs=use_graphs)
        results.append(tt.run_in_process(runner, steps, cfg["vocab"], str(tmp_path / str(i))))
        assert (runner.graph_replays > 30) == use_graphs
    for rid, want in plain.items():
        a, b = results[0][rid].astype(np.float64), results[1][rid].astype(np.float64)
        if dtype == "float32":
            assert np.array_equal(a, b), f"{rid}: graph and eager steps differ in float32"
        else:
            assert np.abs(a - b).max() <= TOL[dtype] * np.abs(want).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_trace_run_program(models, tmp_path, dtype):
    folder, cfg, requests, plain, _ = models["D", dtype]
    steps = tt.number(tt.mixed(requests, seed=9))
    got = tt.run_subprocess(folder, dtype, steps, cfg["vocab"], str(tmp_path), tt.live_tokens_bound(steps))
    check(got, plain, dtype, f"trace_run D {dtype}")


def test_the_residual_stream_after_every_layer_run(models):
    folder, cfg, requests, plain, w64 = models["D", "float32"]
    runner = make_runner(folder, "float32", 16, 320)
    from fllm_amd.engine import StepEntry
    seen = []
    for block in runner.model.blocks:
        def wrapped(ctx, x, binding, _inner=block.forward):
            _inner(ctx, x, binding)
            seen.append(x.clone().cpu().numpy())
        block.forward = wrapped
    toks = requests["r0"]
    runner.step([StepEntry("a", toks, [])])
    want = []
    plain_purivik.forward(cfg, w64, toks, want)
    assert len(seen) == len(want) == 5
    for got, ref_x in zip(seen, want):
        assert np.abs(got - ref_x).max() <= 1e-5 * np.abs(ref_x).max()


def test_decode_steps_take_the_fused_forms(models, monkeypatch):
    """A bfloat16 decode step reads the stream through a layer's first norm inside the q/k/v product's kernel (with rotary
    and the cache store), also where values are narrower than keys (the heads are widened with zero lanes), and the sum of
    the mixer's branch carries the norm before a routed feed-forward: no norm kernel of its own runs but the model's last."""
    from fllm_amd.engine import StepEntry
    from fllm_amd.kernels import Ops
    folder, cfg, requests, _, _ = models["D", "bfloat16"]
    runner = make_runner(folder, "bfloat16", 16, 256, use_graphs=False)
    calls = []
    for name in ("rmsnorm", "norm_qkv_rope_store", "rope_kv_store", "postnorm_add", "route_topk"):
        inner = getattr(Ops, name)
        monkeypatch.setattr(Ops, name, lambda self, *a, _n=name, _i=inner, **k: (calls.append(_n), _i(self, *a, **k))[1])
    toks = requests["r0"]
    runner.step([StepEntry("a", toks[:40], [])])
    calls.clear()
    runner.step([StepEntry("a", toks[40:41], [0])])
    assert calls.count("norm_qkv_rope_store") == 5 and calls.count("rope_kv_store") == 0       # five layer runs
    assert calls.count("rmsnorm") == 1                       # the model's last norm
    assert calls.count("postnorm_add") == 10 and calls.count("route_topk") == 4
    assert runner.model.blocks[1].mixer.v_dim == 64 and runner.model.bindings[1].v_pages.shape[-2] == 64      # 32 in the file
    plain = make_runner(folder, "float32", 16, 256)
    assert plain.model.blocks[1].mixer.v_dim == 32           # float32 runs the plain kernels on the widths of the file


@pytest.mark.parametrize("name", ["A", "D", "E"])
def test_greedy_generation_through_the_scheduler(models, name):
    from fllm_amd import Engine, SamplingParams
    folder, cfg, _, _, w64 = models[name, "float32"]
    prompts = [pc.random_ids(n, cfg["vocab"], 20 + n) for n in (3, 26, 41, 90)]
    want = [plain_purivik.greedy(cfg, w64, p, 12) for p in prompts]
    for opts in (dict(num_blocks=64), dict(num_blocks=14, max_batched_tokens=16)):
        engine = Engine(folder, dtype="float32", ctx=256, max_seqs=3, block_size=pc.PAGE_SIZES[name],
                        **{"max_batched_tokens": 64, **opts})
        assert engine.generate(prompts, SamplingParams(max_tokens=12)) == want
        engine.runner.cache.check_invariants()
    folder, cfg, _, _, w64 = models[name, "bfloat16"]
    engine = Engine(folder, dtype="bfloat16", ctx=256, max_seqs=4, block_size=pc.PAGE_SIZES[name])
    out = engine.generate(prompts, SamplingParams(max_tokens=12))
    assert [len(o) for o in out] == [12] * 4
    # bfloat16 picks the same token wherever the plain logits leave a clear margin: the first token of every prompt
    for p, o in zip(prompts, out):
        logits = plain_purivik.forward(cfg, w64, p)[-1]
        top = np.sort(logits)[-2:]
        if top[1] - top[0] > 0.1 * np.abs(logits).max():
            assert o[0] == int(np.argmax(logits))


def test_the_command_line_generates_and_samples(models):
    """`python -m fllm_amd run` on a Purivik folder: greedy tokens are the plain implementation's, and the sampling options
    (temperature, top-k, top-p, penalties, several answers, log-probabilities, the prefix cache) run."""
    folder, cfg, _, _, w64 = models["D", "float32"]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    prompt = pc.random_ids(30, cfg["vocab"], 4)
    cmd = [sys.executable, "-m", "fllm_amd", "run", folder, "--prompt-ids", ",".join(map(str, prompt)), "--max-tokens", "8",
           "--dtype", "float32", "--ctx", "256", "--kv-blocks", "16", "--max-seqs", "2"]
    proc = subprocess.run(cmd, cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    record = json.loads(proc.stdout.strip().splitlines()[0])
    assert record["finish_reason"] == "length" and record["token_ids"] == plain_purivik.greedy(cfg, w64, prompt, 8)
    flags = ["--temperature", "0.8", "--top-k", "20", "--top-p", "0.9", "--seed", "3", "--repeat-penalty", "1.3", "--n", "2",
             "--logprobs", "2", "--prefix-cache", "--dtype", "bfloat16"]
    proc = subprocess.run(cmd + flags, cwd=root, capture_output=True, text=True, timeout=110)
    assert proc.returncode == 0, proc.stderr[-2000:]
    records = [json.loads(line) for line in proc.stdout.strip().splitlines()]
    assert len(records) == 2 and all(len(r["token_ids"]) == 8 for r in records)
