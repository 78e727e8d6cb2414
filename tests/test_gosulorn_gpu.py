"""Gosulorn on the GPU: each new kernel against its plain reference in both dtypes (odd sizes, sequences of unequal
length in slots out of order, single decoded tokens); the attention of the parallel mixer alone with one input row
made to stand out just inside and just outside the window, at page borders and behind thousands of keys; the
recurrences over long portions; the whole model in float32 and bfloat16 through replay (every way of cutting, pages and
slots used again), far memory, long decoding, batches against each request alone, the entry point with captured decode
steps, and the replay program itself."""
import json
import os
import subprocess

import numpy as np
import pytest
import torch

import plain_gosulorn as plain
import replay_cases as rc
from gosulorn_cases import CONFIGS, PAGE_SIZE, attention, delta, layer, parallel, prompts, random_weights, read_folder, write_folder
from helpers import Harness
from test_gosulorn_cpu import _long_memory
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.engine.batch import StepEntry
from velox_amd.engine.replay import Replayer

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}
REL = {"float32": 2e-5, "bfloat16": 1.6e-2}  # of the largest entry: one rounding of the output in bfloat16


@pytest.fixture(scope="module")
def ops():
    from velox_amd.kernels import load_ops

    return load_ops("cuda")


@pytest.fixture(scope="module")
def ref():
    return TorchOps()


def rnd(g, *shape, dtype=torch.float32, scale=1.0):
    return (torch.randn(*shape, generator=g) * scale).to(dtype).cuda()


def near(got, want, rel, msg=""):
    size = max(float(want.float().abs().max()), 1e-6)
    err = float((got.float() - want.float()).abs().max())
    assert err <= rel * size, f"{msg}: error {err:.3e} beside entries up to {size:.3e}"


def logits_of(config, weights, tokens):
    return plain.forward(config, weights, tokens).float()


def close(got, want, dtype, msg=None):
    size = max(1.0, float(want.abs().max()))
    if dtype == "float32":
        torch.testing.assert_close(got, want, msg=msg, rtol=2e-4, atol=3e-5 * size)
    else:
        torch.testing.assert_close(got, want, msg=msg, rtol=6e-2, atol=6e-2 * size)


def row_errors(got, want):
    """Largest error of each row, as a share of the largest logit of the request."""
    return (got - want).abs().amax(-1) / want.abs().amax().clamp(min=1.0)


def rms(errors):
    errors = torch.cat([e.reshape(-1) for e in errors]) if isinstance(errors, (list, tuple)) else errors
    return float(errors.square().mean().sqrt())


def rounding_noise(folder, trace, requests, expected, page):
    """What bfloat16 alone costs with these (sharp) weights: the row errors of the same steps run on the CPU through the
    kernels' plain references, which round where the kernels round.  The yardstick of every bfloat16 comparison below:
    the kernels may err as much as rounding does, not more."""
    replayer = Replayer(folder, "bfloat16", rc.tokens_needed(trace, page), block_size=page, max_live=4, device="cpu", ops=TorchOps())
    got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
    return rms([row_errors(got[rid], expected[rid]) for rid in requests])


# sequences of 1, 2, 20 and 14 rows in slots 2, 0, 3 and 1 of five
LENS, SLOTS, ROWS = [1, 2, 20, 14], [2, 0, 3, 1], 37


def ragged():
    cu = torch.tensor([0, 1, 3, 23, 37], dtype=torch.int32).cuda()
    return cu, torch.tensor(SLOTS, dtype=torch.int32).cuda()


# ----------------------------------------------------------------------------------------------------
# kernels alone
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden,streams", [(96, 4), (70, 1), (2048, 3), (321, 8)])
def test_stream_update_and_norm(ops, ref, dtype, hidden, streams):
    g, dt = torch.Generator().manual_seed(hidden + streams), DTYPES[dtype]
    res = rnd(g, ROWS, streams * hidden)
    terms = (rnd(g, ROWS, hidden, dtype=dt), rnd(g, ROWS, hidden, dtype=dt))
    mix, ow, iw, w = rnd(g, streams, streams), rnd(g, streams), rnd(g, streams), rnd(g, hidden)
    picked = torch.tensor([3, 0, 36], dtype=torch.int32).cuda()
    for center in (True, False):
        for rows in (None, picked):
            for nt in (0, 1, 2):
                a_res, b_res = res.clone(), res.clone()
                a = ops.stream_norm(a_res, terms[:nt], (0.8, 1.1)[:nt], mix, ow, iw, w, 1e-6, streams, center, dt, rows=rows)
                b = ref.stream_norm(b_res, terms[:nt], (0.8, 1.1)[:nt], mix, ow, iw, w, 1e-6, streams, center, dt, rows=rows)
                near(a, b, REL[dtype], f"center={center} rows={rows is not None} terms={nt}")
                near(a_res, b_res, 2e-6, "the streams themselves")  # float32 in both run dtypes
    a_res, b_res = res.clone(), res.clone()  # no weights on the streams: the plain residual sum
    near(ops.stream_norm(a_res, terms[:1], (1.0,), None, None, None, w, 1e-6, streams, True, dt),
         ref.stream_norm(b_res, terms[:1], (1.0,), None, None, None, w, 1e-6, streams, True, dt), REL[dtype], "unweighted")
    near(a_res, b_res, 2e-6, "unweighted streams")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_copies_and_gated_activation(ops, ref, dtype):
    g, dt = torch.Generator().manual_seed(3), DTYPES[dtype]
    ids = torch.tensor([1, 5, 2, 6, 0], dtype=torch.int32).cuda()
    table = rnd(g, 7, 90, dtype=dt)
    for copies in (1, 3):
        assert torch.equal(ops.embed(ids, table, copies=copies), ref.embed(ids, table, copies=copies))
    for inter in (50, 384, 4100):
        gate_up = rnd(g, ROWS, 2 * inter, dtype=dt, scale=2.0)
        for act in ("silu", "gelu_tanh"):
            near(ops.gated_act_mul(gate_up, act), ref.gated_act_mul(gate_up, act), REL[dtype], f"{act} {inter}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("activation", ["silu", "gelu_tanh"])
@pytest.mark.parametrize("rows", [1, 5, 16, 17, 40, 300])
def test_gate_up_product_with_its_activation(ops, ref, dtype, activation, rows):
    """``act(x Wgate^T) * (x Wup^T)``: one kernel for a decode step's few bfloat16 rows, the product and the activation's kernel
    otherwise; both against the plain formula on the float32 sums."""
    g, dt = torch.Generator().manual_seed(rows), DTYPES[dtype]
    inter, width = 176, 192
    x, w = rnd(g, rows, width, dtype=dt), rnd(g, 2 * inter, width, dtype=dt, scale=0.15)
    sums = x.double() @ w.double().t()
    gate, up = sums[:, :inter], sums[:, inter:]
    if activation == "silu":
        want = gate * torch.sigmoid(gate) * up
    else:
        want = 0.5 * gate * (1.0 + torch.tanh(0.7978845608028654 * (gate + 0.044715 * gate ** 3))) * up
    near(ops.linear_gated_act(x, w, dt, activation), want.float(), REL[dtype], f"{activation} {rows} rows")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows", [1, 8, 33, 200, 2048])
def test_products_with_a_bias_at_every_number_of_rows(ops, ref, dtype, rows):
    """The attention's projections carry biases: a few rows take the skinny kernels, many rows the matrix library (bfloat16)
    or exact multiply-adds (float32); the bias is added to the float32 sums before the one rounding in all of them."""
    g, dt = torch.Generator().manual_seed(rows), DTYPES[dtype]
    x, w = rnd(g, rows, 256, dtype=dt), rnd(g, 96, 256, dtype=dt, scale=0.1)
    bias = rnd(g, 96, dtype=torch.bfloat16).float()  # (as a checkpoint in bfloat16 gives it)
    want = (x.double() @ w.double().t() + bias.double()).float()
    near(ops.linear(x, w, bias, dt), want, REL[dtype], "with bias")
    near(ops.linear(x, w, None, dt), want - bias, REL[dtype], "without")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("taps", [1, 2, 3, 4, 7])
def test_short_convolution_with_its_last_inputs(ops, ref, dtype, taps):
    g, dt = torch.Generator().manual_seed(taps), DTYPES[dtype]
    cu, slots = ragged()
    channels, extra = 70, 9  # (the convolved columns are the first of a wider row)
    x, w = rnd(g, ROWS, channels + extra, dtype=dt), rnd(g, channels, taps)
    tail = rnd(g, 5, taps - 1, channels, dtype=dt) if taps > 1 else None
    for act in ("none", "silu"):
        for update in (True, False):
            ta, tb = (tail.clone(), tail.clone()) if tail is not None else (None, None)
            a = ops.short_conv(x, channels, w, ta, slots, cu, 20, activation=act, update_state=update)
            b = ref.short_conv(x, channels, w, tb, slots, cu, 20, activation=act, update_state=update)
            near(a, b, REL[dtype], f"{act} update={update}")
            if tail is not None:
                assert torch.equal(ta, tb)
                assert update or torch.equal(ta, tail)
    cu1, x1 = torch.arange(5, dtype=torch.int32).cuda(), x[:4].contiguous()  # four sequences of one decoded token
    ta, tb = (tail.clone(), tail.clone()) if tail is not None else (None, None)
    near(ops.short_conv(x1, channels, w, ta, slots, cu1, 1, activation="silu"), ref.short_conv(x1, channels, w, tb, slots, cu1, 1, activation="silu"), REL[dtype], "decode")
    if tail is not None:
        assert torch.equal(ta, tb)
    # a portion of 100 tokens (several chunks of the kernel) equals the same tokens cut at 16, 17 and 18
    cu_long = torch.tensor([0, 100], dtype=torch.int32).cuda()
    slot = torch.tensor([4], dtype=torch.int32).cuda()
    xl = rnd(g, 100, channels, dtype=dt)
    ta = tail.clone() if tail is not None else None
    whole = ops.short_conv(xl, channels, w, ta, slot, cu_long, 100, activation="silu")
    tb, parts, at = tail.clone() if tail is not None else None, [], 0
    for n in (16, 1, 1, 82):
        parts.append(ops.short_conv(xl[at:at + n].contiguous(), channels, w, tb, slot, torch.tensor([0, n], dtype=torch.int32).cuda(), n, activation="silu"))
        at += n
    assert torch.equal(torch.cat(parts), whole)
    if tail is not None:
        assert torch.equal(ta, tb)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,padded,half", [(4, 2, 24, 40, 48, 4), (3, 1, 16, 16, 16, 8), (8, 4, 64, 128, 128, 8), (2, 2, 10, 6, 16, 5)])
def test_partial_rotation_and_padded_cache_write(ops, ref, dtype, heads, kv_heads, dim, vdim, padded, half):
    g, dt, page = torch.Generator().manual_seed(dim), DTYPES[dtype], 16
    qkv = rnd(g, ROWS, heads * dim + kv_heads * (dim + vdim), dtype=dt)
    pos = torch.randint(0, 200, (ROWS,), generator=g).int().cuda()
    cos, sin = rnd(g, 200, half), rnd(g, 200, half)
    slot_map = torch.randperm(5 * page, generator=g)[:ROWS].int().cuda()
    ka, va = torch.zeros(5, kv_heads, page, padded, dtype=dt).cuda(), torch.zeros(5, kv_heads, padded, page, dtype=dt).cuda()
    kb, vb = ka.clone(), va.clone()
    near(ops.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, padded, pos, cos, sin, slot_map, ka, va, page),
         ref.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, padded, pos, cos, sin, slot_map, kb, vb, page), REL[dtype], "q")
    near(ka, kb, REL[dtype], "k")
    assert torch.equal(va, vb)
    a = ops.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, padded, pos, None, None, slot_map, ka, va, page)  # no rotation at all
    assert torch.equal(a, ref.rotate_pad_write(qkv, heads, kv_heads, dim, vdim, padded, pos, None, None, slot_map, kb, vb, page))
    assert torch.equal(ka, kb)


RECURRENCES = [(6, 6, 32, 64, True, True), (4, 2, 32, 32, False, True), (2, 2, 32, 32, True, False), (3, 1, 20, 10, True, True), (2, 1, 72, 24, False, True),
               (1, 1, 128, 128, True, True), (5, 5, 7, 3, False, False), (2, 1, 256, 64, True, True)]


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,per_channel,delta_rule", RECURRENCES)
def test_recurrence_prepare_scan_and_head_norm(ops, ref, dtype, heads, kv_heads, dim, vdim, per_channel, delta_rule):
    g, dt = torch.Generator().manual_seed(heads * dim + vdim), DTYPES[dtype]
    cu, slots = ragged()
    qs, vs = kv_heads * dim, heads * vdim
    cols = heads * dim if per_channel else heads
    main = rnd(g, ROWS, 2 * qs + vs + heads + 5, dtype=dt)
    low = rnd(g, ROWS, cols + vs)
    rate, bias = rnd(g, heads).abs() + 0.1, rnd(g, cols)
    sign = 1.0 if delta_rule else -1.0
    for unit in (True, False):
        a = ops.recurrence_prepare(main, 0, qs, kv_heads, dim, unit, dim ** -0.5, low, 0, heads, cols, rate, bias, sign, main if delta_rule else None, 2 * qs + vs)
        b = ref.recurrence_prepare(main, 0, qs, kv_heads, dim, unit, dim ** -0.5, low, 0, heads, cols, rate, bias, sign, main if delta_rule else None, 2 * qs + vs)
        for name, x, y in zip(("qk", "decay", "beta"), a, b):
            assert (x is None) == (y is None)
            if x is not None:
                assert x.dtype == torch.float32
                near(x, y, 2e-5, f"{name} unit={unit}")
    qk, decay, beta = b  # unit vectors off: keys of any length, the delta rule then over- and undershoots
    qk = qk * 0.3
    sa = rnd(g, 5, heads, dim, vdim)
    sb, before = sa.clone(), sa.clone()
    a = ops.linear_scan(qk, main, 2 * qs, decay, beta, sa, slots, cu, 20, heads, kv_heads, dim, vdim, delta_rule)
    b = ref.linear_scan(qk, main, 2 * qs, decay, beta, sb, slots, cu, 20, heads, kv_heads, dim, vdim, delta_rule)
    near(a, b, 3e-5, "read-out")
    near(sa, sb, 3e-5, "state")
    assert torch.equal(sa[4], before[4])  # a slot that no sequence of the step uses
    weight = rnd(g, vdim)
    for kind in ("silu", "sigmoid"):
        near(ops.gated_head_norm(b, weight, 1e-6, low, cols, kind, heads, vdim, dt), ref.gated_head_norm(b, weight, 1e-6, low, cols, kind, heads, vdim, dt), REL[dtype], kind)


@pytest.mark.parametrize("heads,kv_heads,dim,vdim,per_channel,delta_rule", [(4, 2, 64, 64, True, True), (2, 2, 128, 128, False, True), (3, 3, 32, 48, True, False), (2, 1, 256, 20, True, True),
                                                                            (1, 1, 128, 9, True, False), (2, 2, 72, 40, False, True), (1, 1, 512, 16, True, True)])
def test_a_long_portion_equals_its_pieces_and_its_first_token_is_kept(ops, ref, heads, kv_heads, dim, vdim, per_channel, delta_rule):
    """600 tokens in one step, in pieces (one of a single token, one of two) and against the plain loop; with decays
    close to 1 the first token's write still decides the last read-out."""
    g = torch.Generator().manual_seed(dim)
    n, qs, vs = 600, kv_heads * dim, heads * vdim
    cols = heads * dim if per_channel else heads
    qk = torch.nn.functional.normalize(rnd(g, n, kv_heads, 2, dim), dim=-1)
    qk[:, :, 0] *= dim ** -0.5
    values = rnd(g, n, vs)
    values[0] *= 30.0
    decay = 1.0 - 2e-4 * torch.rand(n, cols, generator=g).cuda()
    beta = torch.sigmoid(rnd(g, n, heads)) if delta_rule else None
    slot = torch.tensor([1], dtype=torch.int32).cuda()

    def run(operations, cuts, v):
        state, outs, at = torch.zeros(2, heads, dim, vdim).cuda(), [], 0
        for c in cuts:
            cu = torch.tensor([0, c], dtype=torch.int32).cuda()
            outs.append(operations.linear_scan(qk[at:at + c].clone(), v[at:at + c].clone(), 0, decay[at:at + c].clone(),
                                               None if beta is None else beta[at:at + c].clone(), state, slot, cu, c, heads, kv_heads, dim, vdim, delta_rule))
            at += c
        return torch.cat(outs), state

    whole, state = run(ops, (n,), values)
    pieces, state_pieces = run(ops, (1, 2, 300, 17, 280), values)
    if dim % 64 == 0:  # (long portions of such heads run a kernel of their own, which sums in another order than single tokens do)
        near(pieces, whole, 1e-5, "pieces")
        near(state_pieces, state, 1e-5, "state of the pieces")
        again, state_again = run(ops, (n,), values)
        assert torch.equal(whole, again) and torch.equal(state, state_again)
    else:  # the order of every sum is fixed by the sizes alone
        assert torch.equal(whole, pieces) and torch.equal(state, state_pieces)
    want, want_state = run(ref, (n,), values)
    near(whole, want, 5e-5, "read-out")
    near(state, want_state, 5e-5, "state")
    without = values.clone()
    without[0] = 0.0
    assert float((run(ref, (n,), without)[0][-50:] - want[-50:]).abs().max()) > 0.05 * float(want[-50:].abs().max())


# ----------------------------------------------------------------------------------------------------
# the attention with a window: one input row stands out, the rows around the window's edge see it or not
# ----------------------------------------------------------------------------------------------------
def _windowed(window, conv, page, dim=64, vdim=32, heads=4, kv_heads=2):
    left = attention(heads, kv_heads, dim, vdim, 0.25, window=window, conv=conv, rot=(dim // 2, 10000.0, 4.0))
    config = {"architecture": "Gosulorn", "vocab": 50, "width": 96, "norm": {"eps": 1e-5}, "streams": 2,
              "layers": [layer("parallel", parallel(left, delta(2, 2, 32, 32, conv=2, rank=4, gate_rank=4), 1.0, 0.5), None)]}
    return config, page


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window,conv,page,loud,length,cuts", [
    (24, 1, 16, 7, 60, (60,)), (24, 3, 16, 15, 60, (29, 2, 1, 1, 27)), (24, 3, 16, 16, 60, (16,) + (1,) * 44), (16, 2, 16, 0, 40, (15, 1, 1, 23)),
    (300, 1, 16, 5, 700, (700,)), (300, 4, 16, 100, 420, (398, 2) + (1,) * 20), (1000, 2, 64, 31, 2200, (1029, 1, 1, 1, 1168)), (33, 1, 8, 40, 90, (64, 9, 17))])
def test_a_row_that_stands_out_is_seen_inside_the_window_only(tmp_path, ops, dtype, window, conv, page, loud, length, cuts):
    """Row ``loud`` of the input is eight times as large as the others: its key and value (and, through the convolution, those of the
    next ``conv - 1`` rows) dominate wherever the window still holds them.  Queries ``window - 1`` and ``window`` rows on lie
    just inside and just outside; they fall into prompts' portions, onto page borders or into single decoded tokens as
    ``cuts`` says."""
    config, page = _windowed(window, conv, page)
    weights = random_weights(config, seed=window + conv)
    folder = write_folder(tmp_path / "w", config, seed=0, dtype=dtype, weights=weights)
    config, tensors = read_folder(folder)
    dt = DTYPES[dtype]
    harness = Harness(folder, ops, dt, "cuda", page, (length + page - 1) // page + 2, max_num_seqs=2, max_num_tokens=max(cuts))
    g = torch.Generator().manual_seed(loud)
    quiet = torch.randn(length, config["width"], generator=g).to(dt)
    c = config["layers"][0]["mixer"]["left"]
    unseen = plain.window_attention(quiet.double(), tensors, "l0.mix.left.", c).float()
    edge = loud + window - 1 + (conv - 1)  # the last row whose window still holds a key that the loud row reached
    best = None
    candidates = [8.0 * quiet[loud].float(), -8.0 * quiet[loud].float()] + [8.0 * torch.randn(config["width"], generator=g) for _ in range(10)]
    for row in candidates:  # (among peaked weights a loud key wins only where its score's sign is right: take the row that shows most)
        x = quiet.clone()
        x[loud] = row.to(dt)
        want = plain.window_attention(x.double(), tensors, "l0.mix.left.", c).float()
        shows = float((want[min(edge, length - 1)] - unseen[min(edge, length - 1)]).abs().max())
        if best is None or shows > best[0]:
            best = (shows, x, want)
    shows, x, want = best
    if edge + 1 < length:
        assert shows > 0.05 * float(want[edge].abs().max())                                      # inside: it shows
        torch.testing.assert_close(want[edge + 1:], unseen[edge + 1:], rtol=1e-6, atol=1e-6)   # outside: it is gone
    seq = harness.cache.new_sequence()
    attention_part = harness.model.blocks[0].mixer.mixers[0]
    rows, at = [], 0
    for n in cuts:
        assert harness.cache.append(seq, at, n)
        ctx = harness.runner.builder.build([StepEntry(seq, [0] * n, at, [])], ops, dt, harness.runner.workspace)
        y = attention_part.forward(x[at:at + n].cuda().contiguous(), ctx, ctx.cache_view(0).views[0], True)
        rows.append(y.float().cpu())
        at += n
        harness.cache.release_behind_window(seq, at)
    got = torch.cat(rows)
    size = float(want.abs().max())
    if dtype == "float32":
        torch.testing.assert_close(got, want, rtol=2e-4, atol=3e-5 * size)
    else:  # peaked weights: a rounded score moves a row's weights; most rows are close, the edge rows among them
        err = (got - want).abs().amax(-1) / size
        assert float((err < 0.05).float().mean()) >= 0.9 and float(err.median()) < 0.02, err
        if edge + 1 < length:
            assert float(err[edge - 1:edge + 2].max()) < 0.08
    assert harness.cache.num_used_pages() <= (window + page - 1) // page + 1  # pages behind the window went back


# ----------------------------------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_all_ways_of_cutting_on_the_gpu(tmp_path, name, dtype):
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2, dtype=dtype)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [141, 1, 37, 98, 2, 64, 75], seed=11)
    expected = {rid: logits_of(config, weights, tokens) for rid, tokens in requests.items()}
    page = PAGE_SIZE[name]
    results = {}
    noise = rounding_noise(folder, rc.whole(requests), requests, expected, page) if dtype == "bfloat16" else None
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)), ("portions", rc.changing_portions(requests)),
                         ("mixed", rc.mixed(requests, seed=5)), ("recompute", rc.mixed(requests, seed=8, preempt=("r0", "r3", "r6")))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page, max_live=4)
        outputs = rc.run_trace(replayer, trace)
        results[label] = rc.collect(trace, outputs, requests)
        if dtype == "float32":
            for rid in requests:
                close(results[label][rid], expected[rid], dtype, msg=lambda m: f"{name} {label} {rid}: {m}")
        else:
            errors = rms([row_errors(results[label][rid], expected[rid]) for rid in requests])
            assert errors <= 1.5 * noise, f"{name} {label}: errors of {errors:.4f} where rounding alone makes {noise:.4f}"
        if label in ("mixed", "recompute") and replayer.cache.groups:
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
    if dtype == "float32":
        for label in ("tail", "portions", "mixed", "recompute"):  # the ways of cutting agree with each other at least as closely
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], rtol=1e-4, atol=3e-5 * max(1.0, float(expected[rid].abs().max())))


@pytest.mark.parametrize("name,cuts", [("E", (700,)), ("E", (3, 1, 690, 2, 1, 1, 1, 1)), ("C", (16, 15, 1, 400, 2) + (1,) * 10), ("A", (4, 4, 248) + (1,) * 4)])
def test_what_the_first_tokens_wrote_is_read_far_later_on_the_gpu(tmp_path, name, cuts):
    config = CONFIGS[name]
    weights = _long_memory(config, random_weights(config, 4))
    folder = write_folder(tmp_path / name, config, seed=4, weights=weights)
    config, tensors = read_folder(folder)
    n = sum(cuts)
    base = prompts(config["vocab"], [n], seed=9)["r0"]
    other = [(base[0] + 1) % config["vocab"]] + base[1:]
    want = {rid: logits_of(config, tensors, toks)[-4:] for rid, toks in (("base", base), ("other", other))}
    assert float((want["base"] - want["other"]).abs().max()) > 0.02
    page = PAGE_SIZE[name]
    for rid, toks in (("base", base), ("other", other)):
        replayer = Replayer(folder, "float32", (n + page - 1) // page * page, block_size=page, max_live=2)
        at, rows = 0, []
        for i, c in enumerate(cuts):
            out = replayer.step({"step": i, "entries": [{"id": rid, "tokens": toks[at:at + c], "want": list(range(max(0, c - 4), c))}], "end": [rid] if at + c == n else []})
            rows.append(torch.from_numpy(out))
            at += c
        close(torch.cat(rows)[-4:], want[rid], "float32", msg=lambda m: f"{name} {cuts} {rid}: {m}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_a_batch_against_each_request_alone(tmp_path, dtype):
    """A prompt of a few tokens, then 200 tokens one by one: the window passes over decoded tokens only, pages behind it go
    back, the states are carried 200 times; then four requests of unequal length decoded together, whose logits equal
    those of each request decoded alone, in slots that the long one and each other have used."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=4, dtype=dtype)
    config, weights = read_folder(folder)
    tokens = prompts(config["vocab"], [205], seed=12)["r0"]
    want = logits_of(config, weights, tokens)[[0] + list(range(4, 205))]

    def decode_long(replayer):
        rows = [replayer.step({"step": 0, "entries": [{"id": "x", "tokens": tokens[:5], "want": [0, 4]}], "end": []})]
        most = 0
        for i in range(5, 205):
            rows.append(replayer.step({"step": i, "entries": [{"id": "x", "tokens": [tokens[i]], "want": [0]}], "end": ["x"] if i == 204 else []}))
            most = max(most, replayer.cache.num_used_pages())
        assert most <= 3  # a window of 24 tokens over pages of 16
        return torch.from_numpy(np.concatenate(rows))

    replayer = Replayer(folder, dtype, 4 * 128, block_size=16, max_live=4)
    got = decode_long(replayer)
    noise = None
    if dtype == "float32":
        close(got, want, dtype)
    else:  # (as much error as the plain operations make on the same steps in bfloat16, not more)
        noise = rms(row_errors(decode_long(Replayer(folder, dtype, 4 * 128, block_size=16, max_live=4, device="cpu", ops=TorchOps())), want))
        assert rms(row_errors(got, want)) <= 1.5 * noise
    texts = prompts(config["vocab"], [70, 9, 33, 120], seed=13)
    alone = {}
    for rid, text in texts.items():
        head = len(text) - 6
        replayer.step({"step": 0, "entries": [{"id": rid, "tokens": text[:head], "want": []}], "end": []})
        alone[rid] = [replayer.step({"step": 1, "entries": [{"id": rid, "tokens": [t], "want": [0]}], "end": []}) for t in text[head:]]
        replayer.step({"step": 2, "entries": [], "end": [rid]})
    replayer.step({"step": 0, "entries": [{"id": rid, "tokens": text[:len(text) - 6], "want": []} for rid, text in texts.items()], "end": []})
    apart = []
    for k in range(6):
        out = replayer.step({"step": 1 + k, "entries": [{"id": rid, "tokens": [text[len(text) - 6 + k]], "want": [0]} for rid, text in texts.items()], "end": []})
        for row, rid in zip(out, texts):
            if dtype == "float32":
                np.testing.assert_allclose(row, alone[rid][k][0], rtol=1e-4, atol=1e-4)
            apart.append(row_errors(torch.from_numpy(row)[None], torch.from_numpy(alone[rid][k])))
    if dtype == "bfloat16":  # other kernels multiply a batch's rows than a single row's: two roundings of the same thing
        assert rms(apart) <= 2.0 * noise


@pytest.mark.parametrize("graphs", [False, True])
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_entry_point(tmp_path, ops, name, graphs):
    """Scheduler, step function, captured decode steps (``graphs``) and sampler around the model, in float32: greedy tokens
    equal the plain model's, also when the pool is so small that requests wait for pages or are preempted, and with
    fewer state slots than requests."""
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=6)
    config, weights = read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 40], seed=7).values())
    steps = 12

    def plain_greedy(prompt):
        tokens = list(prompt)
        for _ in range(steps):
            tokens.append(int(plain.forward(config, weights, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    want = [plain_greedy(p) for p in texts]
    page = PAGE_SIZE[name]
    for pages, seqs in ((64, 4), (2 * (64 // page) + 3, 4), (64, 2)):
        engine = Engine.from_pretrained(EngineConfig(model=folder, dtype="float32", device="cuda", max_model_len=96, max_num_seqs=seqs, max_num_batched_tokens=32,
                                                     max_prefill_chunk_size=11, block_size=page, num_gpu_blocks=pages, enable_cuda_graphs=graphs, seed=0), ops=ops)
        assert engine.runner.uses_graphs == graphs and engine.cache.prefix is None
        requests = [Request(f"r{i}", p, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True)) for i, p in enumerate(texts)]
        engine.generate(requests)
        assert [r.output_token_ids for r in requests] == want, f"pages={pages} seqs={seqs}"
        assert engine.cache.num_used_pages() == 0
        if graphs:
            assert engine.runner.num_graph_replays > 0


def test_captured_decode_steps_in_bfloat16_agree_with_eager_ones(tmp_path, ops):
    """Replays of captured steps against the same steps run eagerly, several times over, with other work between."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=3, dtype="bfloat16")
    tokens = prompts(CONFIGS["C"]["vocab"], [60], seed=2)["r0"]
    outs = {}
    for graphs in (False, True):
        replayer = Replayer(folder, "bfloat16", 256, block_size=16, max_live=4, enable_graphs=graphs)
        assert replayer.runner.uses_graphs == graphs
        replayer.step({"step": 0, "entries": [{"id": "a", "tokens": tokens[:40], "want": []}], "end": []})
        outs[graphs] = [replayer.step({"step": i, "entries": [{"id": "a", "tokens": [tokens[i]], "want": [0]}], "end": []}) for i in range(40, 60)]
        assert not graphs or replayer.runner.num_graph_replays == 20
    for eager, replayed in zip(outs[False], outs[True]):
        np.testing.assert_allclose(replayed, eager, rtol=1e-5, atol=1e-5)


def test_the_replay_program_itself(tmp_path):
    folder = write_folder(tmp_path / "B", CONFIGS["B"], seed=9, dtype="bfloat16")
    config, weights = read_folder(folder)
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
        got = torch.from_numpy(np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)]))
        close(got, logits_of(config, weights, tokens)[[0, 16, 29]], dtype)
