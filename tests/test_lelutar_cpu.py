"""Lelutar on a CPU: the kernels' plain references stand in for the kernels; the configuration reader, the parts,
the loader, the cache manager, the step function, replay, the scheduler and the entry point are the product's.
The yardstick is ``plain_lelutar`` (whole sequences, no cache)."""
import copy
import math

import pytest
import torch

import plain_lelutar as plain
import replay_cases as rc
from lelutar_cases import CONFIGS, PAGE_SIZE, prompts, random_weights, tensor_shapes, write_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.config.model_config import ConfigError
from velox_amd.config.registry import config_from_dict
from velox_amd.engine.batch import StepEntry
from velox_amd.engine.engine import build_model
from velox_amd.engine.replay import Replayer
from velox_amd.parts import make_part
from velox_amd.weights import WeightsError, bind_from_checkpoint

TOL = dict(rtol=2e-4, atol=3e-5)


def test_configuration_is_read_layer_by_layer_and_refused_where_it_cannot_run():
    config = config_from_dict(CONFIGS["A"])
    assert config.architecture == "Lelutar" and config.width == 64 and len(config.layers) == 6 and config.bigram == (31, 7, 3)
    model = build_model(config, torch.float32, "cpu", max_position=64)
    assert [e.layer for e in model.schedule] == [0, 1, 2, 0, 2, 0] and len(model.blocks) == 3  # three layers own tensors
    assert sorted(model.positions) == ["rotation0", "rotation1"]
    needs = model.cache_needs()
    assert len(needs) == 7 and all(n is not None for n in needs)  # every run has a cache of its own; the last entry is the embedding's state
    assert needs[0].tensors[0][1] == (2, -1, 32) and needs[1].tensors[0][1] == (1, -1, 32) and needs[2].tensors[0][1] == (1, -1, 32)
    assert needs[6].tensors[0][0] == "previous_token"
    assert type(model.blocks[2].feed_forward).__name__ == "NoFeedForward" and model.blocks[1].feed_forward.groups == (3, 2)
    assert model.blocks[1].mixer.rot_dim == 0 and model.blocks[2].mixer.rot_dim == 8 and model.blocks[1].mixer.gate_per_head
    assert model.head.scale == 1.5 and model.embedding.scale == 1.75
    # a layer may name a layer that itself runs another's weights, or one that comes later: the owner is found either way
    chained = copy.deepcopy(CONFIGS["A"])
    chained["layers"][5]["weights_of"] = 3
    chained["layers"][2], chained["layers"][4] = chained["layers"][4], chained["layers"][2]
    chained["layers"][2]["weights_of"] = 4
    assert [e.layer for e in build_model(config_from_dict(chained), torch.float32, "cpu", max_position=64).schedule] == [0, 1, 2, 0, 2, 0]
    plain_embedding = build_model(config_from_dict(CONFIGS["B"]), torch.float32, "cpu", max_position=32)
    assert type(plain_embedding.embedding).__name__ == "TableEmbedding" and len(plain_embedding.cache_needs()) == 4 and plain_embedding.head.scale == 1.0
    for change, message in (
        (lambda c: c["layers"][3].update(weights_of=1), "type"),
        (lambda c: c["layers"][3].update(weights_of=3), "weights_of"),
        (lambda c: (c["layers"][0].update(weights_of=3), c["layers"][3].update(weights_of=0)), "weights_of"),
        (lambda c: c["layers"][0].update(type="other"), "type"),
        (lambda c: c["layers"][0]["mlp"].update(kind="other"), "kind"),
        (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
        (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=4), "groups"),
        (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(keep=1, count=6), "groups"),
        (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18), "dims"),
        (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "kv_heads"),
        (lambda c: c["layers"][2]["mixer"].pop("rot"), "rot"),
        (lambda c: c["embedding"]["bigram"].update(buckets=0), "buckets"),
        (lambda c: c.pop("width"), "width"),
    ):
        broken = copy.deepcopy(CONFIGS["A"])
        change(broken)
        with pytest.raises(ConfigError, match=message):
            config_from_dict(broken)


def test_every_tensor_is_named_and_shaped_as_the_design_says(tmp_path):
    for name in ("A", "B", "D"):
        folder = write_folder(tmp_path / name, CONFIGS[name], seed=1)
        model = build_model(config_from_dict(CONFIGS[name]), torch.float32, "cpu", max_position=32)
        count = bind_from_checkpoint(model, folder, torch.float32, "cpu")
        assert count == sum(math.prod(s) for s in tensor_shapes(CONFIGS[name]).values())
    weights = random_weights(CONFIGS["A"], 1)
    weights["l3.norm1"] = torch.zeros(64)  # a layer that runs another's weights has no tensors
    del weights["l1.mix.sink"]
    folder = write_folder(tmp_path / "broken", CONFIGS["A"], seed=1, weights=weights)
    model = build_model(config_from_dict(CONFIGS["A"]), torch.float32, "cpu", max_position=32)
    with pytest.raises(WeightsError) as caught:
        bind_from_checkpoint(model, folder, torch.float32, "cpu")
    assert caught.value.unexpected == ["l3.norm1"] and caught.value.missing == ["l1.mix.sink"]


# ----------------------------------------------------------------------------------------------------
# each mechanism alone
# ----------------------------------------------------------------------------------------------------
class _Ctx:
    ops = TorchOps()
    dtype = torch.float32


def test_the_norm_without_statistics():
    norm = make_part("norm", "dynamic_tanh", prefix="n", hidden_size=10, weight_name="", bias_name=".b", alpha_name=".alpha")
    assert {p.sources[0]: p.shape for p in norm.params().values()} == {"": (10,), ".b": (10,), ".alpha": ()}
    norm.weight, norm.bias, norm.alpha = torch.randn(10), torch.randn(10), torch.tensor(0.7)
    w = {"n": norm.weight, "n.b": norm.bias, "n.alpha": norm.alpha}
    residual, delta = torch.randn(5, 10) * 3, torch.randn(5, 10)
    summed = residual + delta
    got = norm.forward(residual, delta, _Ctx)
    torch.testing.assert_close(residual, summed)  # (the residual has taken the delta in)
    torch.testing.assert_close(got, plain.dynamic_tanh(summed, w, "n"))
    rows = torch.tensor([4, 1], dtype=torch.int32)
    kept = residual.clone()
    torch.testing.assert_close(norm.forward(residual, delta, _Ctx, rows=rows), plain.dynamic_tanh((kept + delta)[rows.long()], w, "n"))
    assert torch.equal(residual, kept)
    partial = torch.randn(3, 5, 10)
    torch.testing.assert_close(norm.forward(residual, partial, _Ctx), plain.dynamic_tanh(kept + partial.sum(0), w, "n"))


@pytest.mark.parametrize("buckets,mul_prev,mul_cur", [(31, 7, 3), (1, 5, 5), (257, 2000000011, 1999999973)])
def test_the_pair_table_sees_the_token_before_a_portion(buckets, mul_prev, mul_cur):
    """Two sequences in portions, the second admitted later into a slot that was used before: every row equals the plain
    embedding of the whole sequence."""
    vocab, width = 50, 6
    config = {"embedding": {"scale": 2.0, "bigram": {"buckets": buckets, "mul_prev": mul_prev, "mul_cur": mul_cur}}}
    w = {"embed": torch.randn(vocab, width), "bigram": torch.randn(buckets + 1, width)}
    part = make_part("embedding", "bigram_table", name="embed", vocab_size=vocab, hidden_size=width, scale=2.0, buckets=buckets, mul_prev=mul_prev, mul_cur=mul_cur)
    part.table, part.bigram = w["embed"], w["bigram"]
    sequences = prompts(vocab, [9, 7], seed=1)
    want = {rid: plain.embed(config, w, tokens) for rid, tokens in sequences.items()}
    state = torch.full((3, 1), 41, dtype=torch.int32)  # (whatever an earlier request left behind)

    class Cache:
        tensors = {"previous_token": state}

    done = {"r0": 0, "r1": 0}
    for step in ([("r0", 4)], [("r0", 1), ("r1", 2)], [("r1", 1), ("r0", 2)], [("r0", 2), ("r1", 4)]):
        ids, positions, cu, slots = [], [], [0], []
        for rid, n in step:
            ids += sequences[rid][done[rid]:done[rid] + n]
            positions += list(range(done[rid], done[rid] + n))
            cu.append(len(ids))
            slots.append(2 if rid == "r0" else 0)

        class Ctx(_Ctx):
            pass

        Ctx.positions, Ctx.cu_q, Ctx.slots = (torch.tensor(v, dtype=torch.int32) for v in (positions, cu, slots))
        Ctx.max_q_len = max(n for _, n in step)
        got = part.forward(torch.tensor(ids, dtype=torch.int32), Ctx, cache=Cache)
        at = 0
        for rid, n in step:
            torch.testing.assert_close(got[at:at + n], want[rid][done[rid]:done[rid] + n])
            at, done[rid] = at + n, done[rid] + n


@pytest.mark.parametrize("experts,top,groups", [(12, 3, (4, 2)), (6, 2, (3, 2)), (9, 2, (3, 1)), (4, 1, (4, 1)), (8, 8, None), (10, 4, (1, 1)), (64, 6, (8, 3))])
def test_the_choice_among_the_best_groups(experts, top, groups):
    """The reference of the router's kernel against the plain function; corrections make choice scores negative, so a
    masked expert must count as minus infinity, not 0."""
    logits = torch.randn(40, experts) * 2
    correction = -0.6 + 0.4 * torch.randn(experts)
    router = {"experts": experts, "top": top}
    if groups:
        router["groups"] = {"count": groups[0], "keep": groups[1]}
    index, weights = plain.choose_experts(logits, correction, router)
    choice, weight = TorchOps().route_top(logits, top, "sigmoid", True, correction=correction, groups=groups, norm_floor=1e-20)
    assert torch.equal(choice.long().sort(-1).values, index.sort(-1).values)
    torch.testing.assert_close(weight.gather(1, choice.long().argsort(-1)), weights.gather(1, index.argsort(-1)))
    torch.testing.assert_close(weight.sum(-1), torch.ones(40))
    if groups and groups[1] < groups[0]:
        assert bool(((torch.sigmoid(logits) + correction) < 0).any())
        per = experts // groups[0]
        assert all(len({int(e) // per for e in row}) <= groups[1] for row in choice)
        free = TorchOps().route_top(logits, top, "sigmoid", True, correction=correction)[0]
        assert per == 1 or not torch.equal(free.sort(-1).values, choice.sort(-1).values)  # (the groups decide something)


def test_layer_outputs_one_by_one(tmp_path):
    """The residual stream after every layer run, from the framework's blocks run one at a time, against the plain model's:
    each kind of mixer and of feed-forward, and the layers that run another's weights."""
    from helpers import Harness

    for name in ("A", "D"):
        folder = write_folder(tmp_path / name, CONFIGS[name], seed=5)
        config, weights = plain.read_folder(folder)
        tokens = prompts(config["vocab"], [23], seed=8)["r0"]
        want = []
        plain.forward(config, weights, tokens, layer_outputs=want)
        harness = Harness(folder, TorchOps(), torch.float32, "cpu", 4, 16, max_num_seqs=2, max_num_tokens=64)
        seq = harness.cache.new_sequence()
        assert harness.cache.append(seq, 0, len(tokens))
        ctx = harness.runner.builder.build([StepEntry(seq, tokens, 0, [])], harness.runner.ops, torch.float32, harness.runner.workspace)
        model = harness.model
        residual = model.embed(ctx.token_ids, ctx)
        torch.testing.assert_close(residual, plain.embed(config, weights, tokens), **TOL)
        pending = None
        for index in range(len(model.schedule)):
            pending = model.run_schedule(residual, pending, ctx, first=index, last=index + 1)
            summed = pending.float().sum(0) if pending.dim() == 3 else pending.float()
            torch.testing.assert_close(residual + summed, want[index], msg=lambda m: f"{name} after layer {index}: {m}", **TOL)


# ----------------------------------------------------------------------------------------------------
# the whole model through the step function
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_all_ways_of_cutting_agree_with_the_plain_model(tmp_path, name):
    """Whole prompts; the last tokens one by one; portions of 1 to 16 tokens (many of two); up to four requests mixed in
    a pool so small that pages and slots are used again; requests that are ended half way and recomputed."""
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2)
    config, weights = plain.read_folder(folder)
    requests = prompts(config["vocab"], [41, 1, 17, 58, 9, 33, 2], seed=3)
    expected = {rid: plain.forward(config, weights, tokens) for rid, tokens in requests.items()}
    assert all(float(e.abs().max()) > 1.0 for e in expected.values())  # logits of order one and more: the tolerances bite
    page = PAGE_SIZE[name]
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests, tail=20)),
                         ("portions", rc.changing_portions(requests)), ("mixed", rc.mixed(requests, seed=5)),
                         ("recompute", rc.mixed(requests, seed=6, preempt=("r0", "r3")))):
        replayer = Replayer(folder, "float32", rc.tokens_needed(trace, page), block_size=page, device="cpu", ops=TorchOps(), max_live=4)
        outputs = rc.run_trace(replayer, trace)
        got = rc.collect(trace, outputs, requests)
        for rid in requests:
            torch.testing.assert_close(got[rid], expected[rid], msg=lambda m: f"{name} {label} {rid}: {m}", **TOL)
        if label in ("mixed", "recompute"):
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages


def test_a_mechanism_left_out_would_show(tmp_path):
    """The weights are sharp enough that the tests above can fail: dropping the first key of a sequence, the sink, the
    gate, the stretch, the groups, the correction, the pair table or the logits' scale moves the logits far beyond the
    tolerance."""
    config = CONFIGS["A"]
    weights = random_weights(config, 2)
    tokens = prompts(config["vocab"], [40], seed=4)["r0"]
    right = plain.forward(config, weights, tokens)
    shifted = plain.forward(config, weights, tokens[1:])
    assert float((right[-1] - shifted[-1]).abs().max()) > 0.05

    def changed(edit_config=None, edit_weights=None):
        other, theirs = copy.deepcopy(config), {k: v.clone() for k, v in weights.items()}
        if edit_config:
            edit_config(other)
        if edit_weights:
            edit_weights(theirs)
        return float((right - plain.forward(other, theirs, tokens)).abs().max())

    assert changed(edit_weights=lambda w: w["l1.mix.sink"].fill_(-30.0)) > 0.05  # (no sink)
    assert changed(edit_weights=lambda w: w["l2.mix.sink"].fill_(-30.0)) > 0.05
    assert changed(edit_weights=lambda w: w["l1.mix.g"].zero_()) > 0.05  # (a gate of one half everywhere)
    assert changed(lambda c: c["layers"][0]["mixer"]["rot"].pop("scaling")) > 0.05
    assert changed(lambda c: c["layers"][2]["mixer"]["rot"].pop("scaling")) > 0.05
    assert changed(lambda c: c["layers"][1]["mlp"]["router"].pop("groups")) > 0.05
    assert changed(edit_weights=lambda w: w["l1.mlp.correction"].zero_()) > 0.05
    assert changed(lambda c: c["embedding"].pop("bigram")) > 0.05
    assert changed(lambda c: c["embedding"]["bigram"].update(mul_prev=8)) > 0.05
    assert changed(lambda c: c.update(logit_scale=1.0)) > 0.05
    assert changed(lambda c: c["layers"][3].pop("weights_of"), lambda w: w.update({k.replace("l0.", "l3."): v + 0.05 for k, v in list(w.items()) if k.startswith("l0.")})) > 0.05


@pytest.mark.parametrize("far_at,length", [(3, 300), (0, 90), (4, 90), (7, 90), (8, 90), (16, 90)])
def test_a_key_far_back_is_found_from_a_portion_and_from_a_single_token(tmp_path, far_at, length):
    """One early token is made to stand out (its embedding is loud, so its keys are), hundreds of tokens and many pages
    back, or at a page's first or last place (pages of 4 tokens): the late logits depend on it, and the framework finds
    it from a portion and from single tokens alike, written by one step and read by later ones."""
    config = copy.deepcopy(CONFIGS["A"])
    weights = random_weights(config, 9)
    tokens = [t if t != 96 else 95 for t in prompts(config["vocab"], [length], seed=5)["r0"]]
    tokens[far_at] = 96  # token 96 occurs once
    weights["embed"][96] *= 4.0
    right = plain.forward(config, weights, tokens)
    other = list(tokens)
    other[far_at] = 5
    moved = (right[-40:] - plain.forward(config, weights, other)[-40:]).abs().amax(-1)
    assert float(moved.min()) > 0.02  # (every late position feels the early token)
    folder = write_folder(tmp_path / "far", config, seed=9, weights=weights)
    requests = {"r0": tokens}
    cuts = (64, 2, 100, 3, 50, 1, 2, 38, 1) if length == 300 else (far_at + 1, 2, 30, 1, 3, 17, 2)
    for trace in (rc.whole(requests), rc.tail_one_by_one(requests, tail=45), rc.changing_portions(requests, sizes=cuts)):
        replayer = Replayer(folder, "float32", length + 4, block_size=4, device="cpu", ops=TorchOps(), max_live=2)
        got = rc.collect(trace, rc.run_trace(replayer, trace), requests)
        torch.testing.assert_close(got["r0"], right, **TOL)


def test_a_slot_that_is_used_again_starts_clean(tmp_path):
    """The previous token of a finished request stays in its slot's row; the next request in that slot must not see it,
    and a request that is fed again from its first token must not see its own."""
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=2)
    config, weights = plain.read_folder(folder)
    requests = prompts(config["vocab"], [12, 9, 15], seed=11)
    expected = {rid: plain.forward(config, weights, tokens) for rid, tokens in requests.items()}
    replayer = Replayer(folder, "float32", 64, block_size=4, device="cpu", ops=TorchOps(), max_live=1)  # one slot for all
    for rid, tokens in requests.items():
        first = replayer.step({"step": 0, "entries": [{"id": rid, "tokens": tokens[:5], "want": [0, 4]}], "end": []})
        rest = replayer.step({"step": 1, "entries": [{"id": rid, "tokens": tokens[5:], "want": list(range(len(tokens) - 5))}], "end": [rid]})
        torch.testing.assert_close(torch.from_numpy(first), expected[rid][[0, 4]], **TOL)
        torch.testing.assert_close(torch.from_numpy(rest), expected[rid][5:], **TOL)


def engine_for(folder, page, **overrides):
    options = dict(model=folder, dtype="float32", device="cpu", max_model_len=96, max_num_seqs=4, max_num_batched_tokens=32,
                   max_prefill_chunk_size=7, block_size=page, num_gpu_blocks=64, enable_cuda_graphs=False, seed=0)
    options.update(overrides)
    return Engine.from_pretrained(EngineConfig(**options), ops=TorchOps())


def plain_greedy(config, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(plain.forward(config, weights, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_entry_point_with_preemption(tmp_path):
    """The scheduler, the step function and the sampler around the model: greedy tokens equal the plain model's, together
    and alone, also when the pool is so small that requests are preempted and recomputed.  The prefix cache switches
    itself off (the embedding keeps a state per request)."""
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=2)
    config, weights = plain.read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 26], seed=7).values())
    want = [plain_greedy(config, weights, p, 10) for p in texts]

    def requests(prefix):
        return [Request(f"{prefix}{i}", p, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)) for i, p in enumerate(texts)]

    engine = engine_for(folder, 4)
    assert engine.cache.prefix is None and engine.max_model_len == 96
    assert [r.output_token_ids for r in engine.generate(requests("a"))] == want
    assert [r.output_token_ids for r in engine.generate(requests("again"))] == want
    alone = engine.generate([Request("alone", texts[1], SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))])[0]
    assert alone.output_token_ids == want[1]
    tight = engine_for(folder, 4, num_gpu_blocks=17)
    assert [r.output_token_ids for r in tight.generate(requests("t"))] == want and tight.scheduler.num_preemptions > 0
    assert tight.cache.num_used_pages() == 0
    tight.cache.assert_consistent([])
