"""Lelutar on the GPU: each new kernel (and each kernel that took a new option) against its plain reference; sinks in every
attention kernel; the whole model in float32 and bfloat16 through replay (every way of cutting, pages and slots used
again), with a key far back behind split keys, in long decoding, in batches against each request alone, through the
entry point with captured decode steps, and through the replay program itself."""
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

import plain_lelutar as plain
import replay_cases as rc
from lelutar_cases import CONFIGS, PAGE_SIZE, prompts, random_weights, write_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.engine.batch import Workspace
from velox_amd.engine.replay import Replayer
from velox_amd.parts.base import SumOf

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOL = {"float32": dict(rtol=2e-4, atol=3e-5), "bfloat16": dict(rtol=6e-2, atol=6e-2)}
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from velox_amd.kernels import load_ops

    return load_ops("cuda")


def close(got, want, dtype, scale=1.0):
    tol = TOL[dtype]
    torch.testing.assert_close(got.float().cpu(), want.float().cpu(), rtol=tol["rtol"], atol=tol["atol"] * scale)


# ----------------------------------------------------------------------------------------------------
# kernels alone
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("buckets,mul_prev,mul_cur,width", [(31, 7, 3, 72), (1, 5, 5, 6), (257, 2000000011, 1999999973, 321), (65521, (1 << 40) + 3, (1 << 33) + 5, 8)])
def test_pair_table_embedding_with_its_state(ops, dtype, buckets, mul_prev, mul_cur, width):
    """Steps of portions and single tokens of three sequences: rows and the state after every step equal the reference's."""
    ref, dt = TorchOps(), DTYPES[dtype]
    vocab = 90
    table, pairs = torch.randn(vocab, width).to(dt).cuda(), torch.randn(buckets + 1, width).to(dt).cuda()
    states = [torch.full((5, 1), 17, dtype=torch.int32).cuda() for _ in range(2)]
    sequences = {rid: tokens for rid, tokens in prompts(vocab, [40, 9, 300], seed=2).items()}
    slot_of, done = {"r0": 3, "r1": 0, "r2": 1}, {"r0": 0, "r1": 0, "r2": 0}
    for step in ([("r0", 7)], [("r0", 1), ("r1", 2), ("r2", 280)], [("r1", 1), ("r0", 1), ("r2", 1)], [("r2", 19), ("r0", 31), ("r1", 6)]):
        ids, positions, cu, slots = [], [], [0], []
        for rid, n in step:
            ids += sequences[rid][done[rid]:done[rid] + n]
            positions += list(range(done[rid], done[rid] + n))
            cu.append(len(ids))
            slots.append(slot_of[rid])
            done[rid] += n
        args = [torch.tensor(v, dtype=torch.int32).cuda() for v in (positions, cu, slots)]
        ids = torch.tensor(ids, dtype=torch.int32).cuda()
        got = ops.embed_bigram(ids, table, pairs, 1.5, buckets, mul_prev, mul_cur, *args, states[0], max(n for _, n in step))
        want = ref.embed_bigram(ids, table, pairs, 1.5, buckets, mul_prev, mul_cur, *args, states[1], max(n for _, n in step))
        torch.testing.assert_close(got, want, rtol=1e-6, atol=1e-6)
        assert torch.equal(states[0], states[1]) and int(states[0][2, 0]) == 17  # (a slot nobody holds is left alone)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden", [72, 321, 1280])
def test_norm_without_statistics(ops, dtype, hidden):
    ref, dt = TorchOps(), DTYPES[dtype]
    weight, bias, alpha = (1 + 0.1 * torch.randn(hidden)).cuda(), (0.2 * torch.randn(hidden)).cuda(), torch.tensor(0.6).cuda()
    residual = (torch.randn(9, hidden) * 2).cuda()
    deltas = [None, torch.randn(9, hidden).to(dt).cuda()]
    if hidden % 4 == 0:  # (partial sums are what products of such widths leave)
        deltas += [torch.randn(3, 9, hidden).cuda(), SumOf(torch.randn(2, 9, hidden).cuda(), torch.randn(9, hidden).to(dt).cuda())]
    for delta in deltas:
        mine, theirs = residual.clone(), residual.clone()
        got = ops.add_dynamic_tanh(mine, delta, weight, bias, alpha, dt)
        want = ref.add_dynamic_tanh(theirs, delta, weight, bias, alpha, dt)
        torch.testing.assert_close(mine, theirs, rtol=1e-6, atol=1e-6)
        close(got, want, dtype, scale=0.3)
        rows = torch.tensor([8, 0, 4], dtype=torch.int32).cuda()
        kept = mine.clone()
        close(ops.add_dynamic_tanh(mine, delta, weight, bias, alpha, dt, rows=rows), ref.add_dynamic_tanh(theirs, delta, weight, bias, alpha, dt, rows=rows), dtype, scale=0.3)
        assert torch.equal(mine, kept)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_squared_rectifier_and_scaled_logits(ops, dtype):
    ref, dt = TorchOps(), DTYPES[dtype]
    for shape in ((7, 96), (5, 37), (300, 1408)):
        x = (torch.randn(shape) * 3).to(dt).cuda()
        assert torch.equal(ops.activation(x, "relu2"), ref.activation(x, "relu2"))
        weight = (torch.randn(48, shape[1]) / math.sqrt(shape[1])).to(dt).cuda()
        close(ops.linear_act(x, weight, dt, "relu2"), ref.linear_act(x, weight, dt, "relu2"), dtype, scale=3.0)
    logits = torch.randn(5, 1000).cuda()
    want = logits * 1.7
    assert ops.scale_(logits, 1.7) is logits and torch.equal(logits, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,half,tokens", [(4, 2, 16, 24, 4, 11), (8, 2, 64, 96, 24, 300), (3, 3, 10, 14, 3, 5), (1, 1, 8, 8, 0, 7)])
def test_rotation_of_neighbouring_pairs_with_padded_cache_write(ops, dtype, heads, kv_heads, dim, vdim, half, tokens):
    ref, dt = TorchOps(), DTYPES[dtype]
    cached = (max(dim, vdim) + 15) // 16 * 16
    page, pages = 4, (tokens + 3) // 4 + 3
    qkv = torch.randn(tokens, heads * dim + kv_heads * (dim + vdim)).to(dt).cuda()
    positions = torch.randint(0, 64, (tokens,), dtype=torch.int32).cuda()
    cos = sin = None
    if half:
        angles = torch.rand(64, half) * 6.0
        cos, sin = (angles.cos() * 1.07).cuda(), (angles.sin() * 1.07).cuda()
    slots = torch.randperm((pages - 1) * page)[:tokens].to(torch.int32).cuda() + page
    caches = [[torch.full((pages, kv_heads, page, cached), 9.0, dtype=dt).cuda(), torch.full((pages, kv_heads, cached, page), 9.0, dtype=dt).cuda()] for _ in range(2)]
    got = ops.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, cached, positions, cos, sin, slots, *caches[0], page, interleaved=True)
    want = ref.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, cached, positions, cos, sin, slots, *caches[1], page, interleaved=True)
    close(got, want, dtype)
    for mine, theirs in zip(caches[0], caches[1]):
        close(mine, theirs, dtype)
    if half:  # (the two layouts differ: the option is read)
        other = ref.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, cached, positions, cos, sin, slots, *[c.clone() for c in caches[1]], page, write_kv=False)
        assert not torch.allclose(other.float(), want.float(), atol=0.1)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,dim,rot,rank,q_rank,half", [(5, 32, 16, 112, 72, 8), (3, 8, 0, 20, 12, 0), (2, 16, 8, 24, 20, 4), (5, 6, 0, 18, 14, 0), (1, 12, 12, 12, 12, 6)])
def test_cache_write_with_the_queries_latent_and_the_queries_rotation(ops, dtype, heads, dim, rot, rank, q_rank, half):
    """The two calls a layer with a query latent makes: the cache write that also norms the queries' latent, and the
    rotation of queries that come from a tensor of their own."""
    ref, dt = TorchOps(), DTYPES[dtype]
    cached = (rank + rot + 15) // 16 * 16
    tokens, page, pages = 11, 4, 9
    width = q_rank + heads + rank + rot
    projected = torch.randn(tokens, width).to(dt).cuda()
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 8, 9, 10, 63], dtype=torch.int32).cuda()
    cos = sin = None
    if half:
        angles = torch.rand(64, half) * 6.0
        cos, sin = (angles.cos() * 1.07).cuda(), (angles.sin() * 1.07).cuda()
    weight, q_weight = (1 + 0.2 * torch.randn(rank)).cuda(), (1 + 0.2 * torch.randn(q_rank)).cuda()
    slots = torch.randperm(pages * page)[:tokens].to(torch.int32).cuda() + page
    caches = [[torch.full((pages + 1, 1, page, cached), 9.0, dtype=dt).cuda(), torch.full((pages + 1, 1, cached, page), 9.0, dtype=dt).cuda()] for _ in range(2)]
    got = ops.latent_write(projected, rot, rank, cached, q_rank + heads, positions, cos, sin, True, weight, 1e-5, slots, *caches[0], page, q_latent=(0, q_rank, q_weight))
    want = ref.latent_write(projected, rot, rank, cached, q_rank + heads, positions, cos, sin, True, weight, 1e-5, slots, *caches[1], page, q_latent=(0, q_rank, q_weight))
    close(got, want, dtype, scale=3.0)
    for mine, theirs in zip(caches[0], caches[1]):
        close(mine, theirs, dtype, scale=3.0)
    assert torch.equal(caches[0][0][:, 0].transpose(1, 2), caches[0][1][:, 0])
    queries = torch.randn(tokens, heads * (dim + rot)).to(dt).cuda()
    got = ops.latent_rotate_write(queries, heads, dim, rot, rank, cached, -1, positions, cos, sin, True, None, 1e-5, None, None, None, page)
    want = ref.latent_rotate_write(queries, heads, dim, rot, rank, cached, -1, positions, cos, sin, True, None, 1e-5, None, None, None, page)
    close(got.view(tokens, heads, cached)[..., rank:], want.view(tokens, heads, cached)[..., rank:], dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows,groups,n,k", [(70, 4, 64, 32), (5, 3, 40, 12), (130, 2, 24, 96), (1, 5, 7, 9), (16, 16, 128, 192)])
def test_a_gate_per_head_on_the_per_head_products(ops, dtype, rows, groups, n, k):
    ref, dt = TorchOps(), DTYPES[dtype]
    x_stride, out_stride = k + 8, n
    x = torch.randn(rows, groups * x_stride).to(dt).cuda()
    maps = (torch.randn(groups, n, k) / math.sqrt(k)).to(dt).cuda()
    gate = (torch.randn(rows, 16 + groups) * 2).to(dt).cuda()
    outs = [torch.full((rows, groups * out_stride), 5.0, dtype=dt).cuda() for _ in range(2)]
    ops.head_linear(x, x_stride, 0, maps, outs[0], out_stride, 0, gate=gate, gate_offset=16, gate_per_head=True)
    ref.head_linear(x, x_stride, 0, maps, outs[1], out_stride, 0, gate=gate, gate_offset=16, gate_per_head=True)
    close(outs[0], outs[1], dtype)


@pytest.mark.parametrize("experts,top,groups", [(12, 3, (4, 2)), (6, 2, (3, 2)), (9, 2, (3, 1)), (4, 1, (4, 1)), (8, 8, None), (10, 4, (1, 1)), (64, 6, (8, 3)),
                                                (256, 8, (8, 4)), (130, 5, (2, 1))])
def test_router_choice_among_the_best_groups(ops, experts, top, groups):
    ref = TorchOps()
    for tokens in (1, 33, 200):
        logits = (torch.randn(tokens, experts) * 2).cuda()
        correction = (-0.6 + 0.4 * torch.randn(experts)).cuda()
        choice, weight = ops.route_top(logits, top, "sigmoid", True, correction=correction, groups=groups, norm_floor=1e-20)
        want_choice, want_weight = ref.route_top(logits, top, "sigmoid", True, correction=correction, groups=groups, norm_floor=1e-20)
        assert torch.equal(choice, want_choice)  # (random logits do not tie; both give the choices in descending order)
        torch.testing.assert_close(weight, want_weight, rtol=1e-5, atol=1e-6)
        index, weights = plain.choose_experts(logits.cpu(), correction.cpu(), {"experts": experts, "top": top, **({"groups": {"count": groups[0], "keep": groups[1]}} if groups else {})})
        assert torch.equal(choice.cpu().long().sort(-1).values, index.sort(-1).values)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tokens,hidden,inter,experts,top", [(70, 64, 32, 4, 2), (9, 88, 20, 6, 3), (300, 96, 40, 8, 1), (1, 256, 64, 12, 4), (150, 72, 130, 3, 2),
                                                            (700, 136, 72, 2, 2), (900, 192, 160, 3, 1), (8, 128, 96, 12, 4)])
def test_experts_without_a_gate_branch_against_the_plain_loop(ops, dtype, tokens, hidden, inter, experts, top):
    ref, dt = TorchOps(), DTYPES[dtype]
    x = torch.randn(tokens, hidden).to(dt).cuda()
    up = (torch.randn(experts * inter, hidden) / math.sqrt(hidden)).to(dt).cuda()
    down = (torch.randn(experts * hidden, inter) / math.sqrt(inter)).to(dt).cuda()
    logits = (torch.randn(tokens, experts) * 2).cuda()
    logits[: tokens // 2, 1] += 6.0  # many rows of one expert: more than one tile
    choice, weight = ops.route_top(logits, top, "sigmoid", True)
    got = ops.routed_experts(x, choice, weight, up, down, experts, False, None, dt, Workspace(torch.device("cuda")), ungated="relu2")
    want = ref.routed_experts(x, choice, weight, up, down, experts, False, None, dt, ungated="relu2")
    close(got, want, dtype, scale=2.0)
    if dtype == "float32":
        for t in (0, tokens - 1):  # a token's result does not depend on which tokens share its experts
            alone = ops.routed_experts(x[t:t + 1].contiguous(), choice[t:t + 1].contiguous(), weight[t:t + 1].contiguous(), up, down, experts, False, None, dt, None,
                                       ungated="relu2")
            assert torch.equal(alone[0], got[t])


def _paged_case(nh, nkv, d, q_lens, kv_lens, page, dt, seed=0):
    g = torch.Generator().manual_seed(seed)
    need = [(n + page - 1) // page for n in kv_lens]
    pages = sum(need) + 1
    k_cache = torch.randn(pages, nkv, page, d, generator=g).to(dt).cuda()
    v_cache = torch.randn(pages, nkv, d, page, generator=g).to(dt).cuda()
    tables = torch.zeros(len(kv_lens), max(need), dtype=torch.int32)
    perm = torch.randperm(pages - 1, generator=g) + 1
    at = 0
    for b, n in enumerate(need):
        tables[b, :n] = perm[at:at + n]
        at += n
    cu = torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32).cuda()
    q = (torch.randn(sum(q_lens), nh * d, generator=g) * 0.5).to(dt).cuda()
    return q, k_cache, v_cache, tables.cuda(), cu, torch.tensor(kv_lens, dtype=torch.int32).cuda()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,d,q_lens,kv_lens", [
    (5, 1, 80, [1, 1, 1], [70, 1, 300]),                 # single tokens, one workgroup per sequence
    (7, 1, 96, [1, 1], [5000, 2300]),                    # single tokens behind keys that are split over workgroups and merged
    (4, 2, 64, [9, 30, 2], [9, 155, 40]),                # short portions: the staged kernel
    (8, 2, 64, [600, 500], [600, 1500]),                 # long portions of 64 channels (bfloat16: tiles loaded straight into LDS)
    (16, 1, 128, [300], [4500]),                         # a portion behind keys that are split
    (5, 1, 80, [1, 1, 40, 7], [800, 3, 100, 7]),         # single tokens before portions: two launches
    (3, 1, 272, [1, 9, 30], [70, 9, 155]),               # beyond the tiled kernels
])
def test_a_sink_in_every_attention_kernel(ops, dtype, nh, nkv, d, q_lens, kv_lens):
    """Sinks of both signs, one so large that it takes nearly all of a head's weight: every kernel and the merge of split
    keys add exp(sink) to the denominator once."""
    ref, dt = TorchOps(), DTYPES[dtype]
    page = 16
    q, k_cache, v_cache, tables, cu, lens = _paged_case(nh, nkv, d, q_lens, kv_lens, page, dt)
    sinks = (torch.randn(nh) * 2).cuda()
    sinks[0] = 9.0
    prefix = next((i for i, n in enumerate(q_lens) if n != 1), len(q_lens))
    args = (q, nh, nkv, d, k_cache, v_cache, page, tables, cu, lens, max(q_lens), max(kv_lens), 1.0 / math.sqrt(d), None, max(q_lens) == 1, Workspace(torch.device("cuda")))
    got = ops.paged_attention(*args, decode_prefix=prefix, sinks=sinks)
    want = ref.paged_attention(*args, sinks=sinks)
    close(got, want, dtype)
    without = ref.paged_attention(*args)
    assert float((want.float() - without.float()).abs().max()) > 0.2 * float(without.float().abs().max())  # (the sinks matter)
    close(ops.paged_attention(*args, decode_prefix=prefix), without, dtype)  # (and without them nothing changed)


# ----------------------------------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------------------------------
def rows_close(got, want, dtype, label):
    if dtype == "float32":
        torch.testing.assert_close(got, want, msg=lambda m: f"{label}: {m}", **TOL[dtype])
    else:
        # bfloat16: rounding may send a token to another expert where two scores are close; such rows are few
        err = (got - want).abs().amax(-1) / want.abs().amax(-1).clamp(min=1.0)
        assert float((err < 0.08).float().mean()) >= 0.9, f"{label}: {err}"


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_all_ways_of_cutting_on_the_gpu(tmp_path, name, dtype):
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2, dtype=dtype)
    config, weights = plain.read_folder(folder)
    requests = prompts(config["vocab"], [141, 1, 37, 98, 2, 64, 75], seed=11)
    expected = {rid: plain.forward(config, weights, tokens) for rid, tokens in requests.items()}
    page = PAGE_SIZE[name]
    results = {}
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)), ("portions", rc.changing_portions(requests)),
                         ("mixed", rc.mixed(requests, seed=5)), ("recompute", rc.mixed(requests, seed=8, preempt=("r0", "r3", "r6")))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page, max_live=4)
        outputs = rc.run_trace(replayer, trace)
        results[label] = rc.collect(trace, outputs, requests)
        for rid in requests:
            rows_close(results[label][rid], expected[rid], dtype, f"{name} {label} {rid}")
        if label in ("mixed", "recompute"):
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
    if dtype == "float32":
        for label in ("tail", "portions", "mixed", "recompute"):  # the ways of cutting agree with each other at least as closely
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], rtol=1e-4, atol=3e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("far_at,length", [(3, 1100), (0, 200), (15, 200), (16, 200), (17, 200), (64, 200)])
def test_a_key_far_back_behind_split_keys_or_at_a_page_border(tmp_path, dtype, far_at, length):
    """One early token is made loud; 1,100 tokens on, where single tokens read their keys in splits that a kernel merges
    (sinks included), or from a page's first or last place (pages of 16 tokens), the logits still depend on it and equal
    the plain model's, from a portion and from single tokens, written by one step and read by later ones."""
    config = CONFIGS["C"]
    weights = random_weights(config, 9)
    tokens = [t if t != 159 else 158 for t in prompts(config["vocab"], [length], seed=5)["r0"]]
    tokens[far_at] = 159
    weights["embed"][159] *= 4.0
    folder = write_folder(tmp_path / "far", config, seed=9, dtype=dtype, weights=weights)
    config, weights = plain.read_folder(folder)
    right = plain.forward(config, weights, tokens)
    other = list(tokens)
    other[far_at] = 5
    moved = (right[-30:] - plain.forward(config, weights, other)[-30:]).abs().amax(-1)
    assert float(moved.median()) > 0.05
    requests = {"r0": tokens}
    cuts = (500, 2, 300, 3, 250, 1, 2, 38, 1, 1, 1, 1) if length > 1000 else (far_at + 1, 2, 100, 1, 3, 33, 2)
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests, tail=40)), ("portions", rc.changing_portions(requests, sizes=cuts))):
        replayer = Replayer(folder, dtype, length + 16, block_size=16, max_live=2)
        got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
        rows_close(got["r0"][-150:], right[-150:], dtype, f"far {label}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_a_batch_against_each_request_alone(tmp_path, dtype):
    """A prompt of a few tokens, then 200 tokens one by one across many page borders; then four requests of unequal
    length decoded together, whose logits equal those of each request decoded alone."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=4, dtype=dtype)
    config, weights = plain.read_folder(folder)
    tokens = prompts(config["vocab"], [205], seed=12)["r0"]
    want = plain.forward(config, weights, tokens)
    replayer = Replayer(folder, dtype, 4 * 224, block_size=16, max_live=4)
    rows = [replayer.step({"step": 0, "entries": [{"id": "x", "tokens": tokens[:5], "want": [0, 4]}], "end": []})]
    for i in range(5, 205):
        rows.append(replayer.step({"step": i, "entries": [{"id": "x", "tokens": [tokens[i]], "want": [0]}], "end": ["x"] if i == 204 else []}))
    rows_close(torch.from_numpy(np.concatenate(rows)), want[[0] + list(range(4, 205))], dtype, "long decoding")
    texts = prompts(config["vocab"], [70, 9, 33, 120], seed=13)
    alone = {}
    for rid, text in texts.items():
        head = len(text) - 6
        replayer.step({"step": 0, "entries": [{"id": rid, "tokens": text[:head], "want": []}], "end": []})
        alone[rid] = [replayer.step({"step": 1, "entries": [{"id": rid, "tokens": [t], "want": [0]}], "end": []}) for t in text[head:]]
        replayer.step({"step": 2, "entries": [], "end": [rid]})
    replayer.step({"step": 0, "entries": [{"id": rid, "tokens": text[:len(text) - 6], "want": []} for rid, text in texts.items()], "end": []})
    for k in range(6):
        out = replayer.step({"step": 1 + k, "entries": [{"id": rid, "tokens": [text[len(text) - 6 + k]], "want": [0]} for rid, text in texts.items()], "end": []})
        for row, rid in zip(out, texts):
            np.testing.assert_allclose(row, alone[rid][k][0], rtol=1e-4 if dtype == "float32" else 3e-2, atol=1e-5 if dtype == "float32" else 3e-2)


def test_captured_steps_equal_eager_ones(tmp_path):
    """Single tokens replayed from captured HIP graphs (padded rows, the state slot of the padding) against the same steps
    launched one kernel at a time, several replays with other work between them."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=4, dtype="bfloat16")
    texts = prompts(CONFIGS["C"]["vocab"], [40, 9, 33], seed=13)
    outputs = []
    for graphs in (False, True):
        replayer = Replayer(folder, "bfloat16", 4 * 64, block_size=16, max_live=4, enable_graphs=graphs)
        assert replayer.runner.uses_graphs == graphs
        rows = []
        replayer.step({"step": 0, "entries": [{"id": rid, "tokens": text[:-5], "want": []} for rid, text in texts.items()], "end": []})
        for k in range(5):
            rows.append(replayer.step({"step": 1 + k, "entries": [{"id": rid, "tokens": [text[len(text) - 5 + k]], "want": [0]} for rid, text in texts.items()], "end": []}))
            replayer.step({"step": 10 + k, "entries": [{"id": "other", "tokens": [3, 4, 5][: 1 + k % 3], "want": []}], "end": ["other"]})
        outputs.append(np.concatenate(rows))
        if graphs:
            assert replayer.runner.num_graph_replays == 5
    np.testing.assert_allclose(outputs[1], outputs[0], rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(tmp_path, ops, graphs):
    """Scheduler, step function, captured decode steps (``graphs``) and sampler around the model, in float32: greedy tokens
    equal the plain model's, also when the pool is so small that requests wait for pages or are preempted."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=6)
    config, weights = plain.read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 40], seed=7).values())
    steps = 12

    def plain_greedy(prompt):
        tokens = list(prompt)
        for _ in range(steps):
            tokens.append(int(plain.forward(config, weights, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    want = [plain_greedy(p) for p in texts]
    for pages in (64, 7):
        engine = Engine.from_pretrained(EngineConfig(model=folder, dtype="float32", device="cuda", max_model_len=96, max_num_seqs=4, max_num_batched_tokens=32,
                                                     max_prefill_chunk_size=11, block_size=16, num_gpu_blocks=pages, enable_cuda_graphs=graphs, seed=0), ops=ops)
        assert engine.runner.uses_graphs == graphs and engine.cache.prefix is None
        requests = [Request(f"r{i}", p, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True)) for i, p in enumerate(texts)]
        engine.generate(requests)
        assert [r.output_token_ids for r in requests] == want
        assert engine.cache.num_used_pages() == 0
        if graphs:
            assert engine.runner.num_graph_replays > 0


def test_the_replay_program_itself(tmp_path):
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=9, dtype="bfloat16")
    config, weights = plain.read_folder(folder)
    tokens = prompts(config["vocab"], [30], seed=1)["r0"]
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": tokens[:17], "want": [0, 16]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": tokens[17:19], "want": []}], "end": []},
             {"step": 2, "entries": [{"id": "a", "tokens": tokens[19:], "want": [10]}], "end": ["a"]}]
    for dtype in ("float32", "bfloat16"):
        out = tmp_path / f"out_{dtype}"
        done = subprocess.run([os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", str(out), "--max-tokens", "64"],
                              input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=600)
        assert done.returncode == 0, done.stderr[-2000:]
        assert [line for line in done.stdout.splitlines() if line.startswith("done")] == ["done 0", "done 1", "done 2"]
        assert not (out / "1.f32").exists()
        got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)])
        want = plain.forward(config, weights, tokens)[[0, 16, 29]].numpy()
        np.testing.assert_allclose(got, want, **(dict(rtol=2e-4, atol=3e-5) if dtype == "float32" else dict(rtol=8e-2, atol=8e-2)))
