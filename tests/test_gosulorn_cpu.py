"""Gosulorn on a CPU: the kernels' plain references stand in for the kernels; the configuration reader, the parts,
the loader, the cache manager with its state slots, the step function, replay, the scheduler and the entry point are the
product's.  The yardstick is ``plain_gosulorn`` (whole sequences, no cache, float64)."""
import copy
import math

import pytest
import torch

import plain_gosulorn as plain
import replay_cases as rc
from gosulorn_cases import CONFIGS, PAGE_SIZE, prompts, random_weights, read_folder, tensor_shapes, write_folder
from helpers import Harness
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.config.model_config import ConfigError
from velox_amd.config.registry import config_from_dict, load_config
from velox_amd.engine.batch import StepEntry
from velox_amd.engine.engine import build_model
from velox_amd.engine.replay import Replayer
from velox_amd.parts.base import ScaledSum, StreamUpdate
from velox_amd.weights import WeightsError, bind_from_checkpoint

TOL = dict(rtol=2e-4, atol=3e-5)


def close(got, want, msg=None):
    """Logits of a float32 run against the float64 yardstick: errors are relative to the size of the logits."""
    torch.testing.assert_close(got, want, msg=msg, rtol=2e-4, atol=3e-5 * max(1.0, float(want.abs().max())))


def logits_of(config, weights, tokens):
    return plain.forward(config, weights, tokens).float()


# ----------------------------------------------------------------------------------------------------------------------
# configuration and tensors
# ----------------------------------------------------------------------------------------------------------------------
def test_configuration_is_read_layer_by_layer_and_refused_where_it_cannot_run(tmp_path):
    config = config_from_dict(CONFIGS["A"])
    assert config.architecture == "Gosulorn" and config.width == 64 and config.streams == 3 and len(config.layers) == 5
    model = build_model(config, torch.float32, "cpu", max_position=64)
    assert len(model.blocks) == 3 and [e.layer for e in model.schedule] == [0, 1, 2, 0, 1]  # two layers run an earlier one's weights
    assert [type(b).__name__ for b in model.blocks] == ["HyperConnectionBlock"] * 3 and model.spec.residual_streams == 3
    pair = model.blocks[0].mixer
    left, right = pair.mixers
    assert pair.scales == (0.7, 1.3) and type(left).__name__ == "ConvAttentionMixer" and type(right).__name__ == "LinearRecurrenceMixer"
    assert (left.num_heads, left.num_kv_heads, left.dim, left.vdim, left.cached_dim, left.window, left.conv_taps, left.scale) == (4, 2, 16, 8, 16, 6, 3, 0.5)
    assert left.position.rotary_dim == 8 and left.position.scaling_factor == 2.0 and left.position.theta == 100.0
    assert (right.rule, right.decay, right.gate, right.unit_qk, right.conv_taps, right.decay_rank, right.gate_rank) == ("delta", "channel", "sigmoid_low_rank", True, 2, 5, 3)
    gla, delta = model.blocks[1].mixer, model.blocks[2].mixer
    assert (gla.rule, gla.decay, gla.gate, gla.unit_qk, gla.tau, gla.conv_taps) == ("additive", "sigmoid_channel", "silu", False, 4.0, 0)
    assert (delta.rule, delta.decay, delta.gate, delta.unit_qk, delta.num_kv_heads, delta.conv_taps) == ("delta", "head", "silu", True, 2, 4)
    assert type(model.blocks[1].feed_forward).__name__ == "NoFeedForward" and model.blocks[0].feed_forward.activation == "gelu_tanh"
    needs = model.cache_needs()
    assert len(needs) == 5 and all(n is not None for n in needs)  # every run of a layer has a cache and a state of its own
    pages, tail = needs[0].parts[0].parts
    assert pages.window == 6 and tail.tensors[0][1] == (2, 4 * 16 + 2 * 16 + 2 * 8) and needs[3] == needs[0]
    assert needs[1].tensors == (("state", (2, 12, 20), torch.float32),) and needs[2].tensors[1][1] == (3, 2 * 16 + 2 * 16 + 4 * 8)
    plain_residual = build_model(config_from_dict(CONFIGS["B"]), torch.float32, "cpu", max_position=32)
    assert plain_residual.spec.residual_streams == 1 and not plain_residual.blocks[0].learned and plain_residual.blocks[0].params() == {}
    assert plain_residual.blocks[1].mixer.mixers[0].window is None and plain_residual.blocks[1].mixer.mixers[0].conv_taps == 0
    for change, message in (
        (lambda c: c["layers"][0].update(type="other"), "type"),
        (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
        (lambda c: c["layers"][0]["mixer"]["left"].update(heads=5), "multiple"),
        (lambda c: c["layers"][0]["mixer"]["left"]["mask"].update(size=0), "mask.size"),
        (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=18), "rot"),
        (lambda c: c["layers"][0]["mixer"]["left"].pop("scale"), "scale"),
        (lambda c: c["layers"][1]["mixer"].update(tau=0.0), "tau"),
        (lambda c: c["layers"][3].update(weights_of=4), "weights_of"),
        (lambda c: c["layers"][4].update(weights_of=3), "weights_of"),
        (lambda c: c["layers"][4].update(weights_of=2), "type"),
        (lambda c: c.pop("width"), "width"),
    ):
        broken = copy.deepcopy(CONFIGS["A"])
        change(broken)
        with pytest.raises(ConfigError, match=message):
            config_from_dict(broken)
    # the inner sizes of the low-rank maps are sizes that only tensors give: a folder's reader takes them from there
    stripped = copy.deepcopy(CONFIGS["A"])
    stripped["layers"][1]["mixer"].pop("a1_rank")
    with pytest.raises(ConfigError, match="a1"):
        config_from_dict(stripped)
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=1)
    loaded = load_config(folder)
    assert "a1_rank" not in loaded.raw["layers"][1]["mixer"] and "tensor_shapes" not in loaded.to_json_dict()
    assert build_model(loaded, torch.float32, "cpu", max_position=32).blocks[0].mixer.mixers[1].gate_rank == 3


def test_every_tensor_is_named_and_shaped_as_the_design_says(tmp_path):
    for name in ("A", "B", "C", "D", "E"):
        folder = write_folder(tmp_path / name, CONFIGS[name], seed=1)
        model = build_model(load_config(folder), torch.float32, "cpu", max_position=32)
        count = bind_from_checkpoint(model, folder, torch.float32, "cpu")
        assert count == sum(math.prod(s) for s in tensor_shapes(CONFIGS[name]).values()), name
    weights = random_weights(CONFIGS["A"], 1)
    weights["l1.norm2"] = torch.ones(64)  # a layer without a feed-forward has no second norm
    del weights["l2.mix.dt_bias"]
    folder = write_folder(tmp_path / "broken", CONFIGS["A"], seed=1, weights=weights)
    model = build_model(load_config(folder), torch.float32, "cpu", max_position=32)
    with pytest.raises(WeightsError) as caught:
        bind_from_checkpoint(model, folder, torch.float32, "cpu")
    assert caught.value.unexpected == ["l1.norm2"] and caught.value.missing == ["l2.mix.dt_bias"]


# ----------------------------------------------------------------------------------------------------------------------
# each mechanism alone: the framework's part, fed through the step's context and the cache manager, against the plain function
# ----------------------------------------------------------------------------------------------------------------------
def _harness(tmp_path, name, seed=2, **kw):
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=seed)
    config, weights = read_folder(folder)
    return Harness(folder, TorchOps(), torch.float32, "cpu", PAGE_SIZE[name], 64, max_num_seqs=3, max_num_tokens=128, **kw), config, weights


def _mixer_in_portions(harness, entry, x, cuts):
    """Runs schedule entry ``entry``'s mixer alone on rows ``x`` of one sequence, cut into portions."""
    seq = harness.cache.new_sequence()
    block = harness.model.blocks[harness.model.schedule[entry].layer]
    out, at = [], 0
    for n in cuts:
        assert harness.cache.append(seq, at, n)
        ctx = harness.runner.builder.build([StepEntry(seq, [0] * n, at, [])], harness.runner.ops, torch.float32, harness.runner.workspace)
        y = block.mixer.forward(x[at:at + n].contiguous(), ctx, ctx.cache_view(entry), True)
        if isinstance(y, ScaledSum):
            y = sum(s * t for s, t in zip(y.scales, y.terms))
        out.append(y)
        at += n
        harness.cache.release_behind_window(seq, at)
    harness.cache.free_sequence(seq)
    return torch.cat(out)


@pytest.mark.parametrize("name,entry", [("A", 0), ("A", 1), ("A", 2), ("B", 0), ("B", 1), ("B", 2), ("D", 0), ("D", 1), ("D", 2)])
def test_each_mixer_alone_whole_and_in_portions(tmp_path, name, entry):
    harness, config, weights = _harness(tmp_path, name)
    layer = config["layers"][entry]
    x = torch.randn(29, config["width"])
    want = plain.mixer(layer["type"], x.double(), weights, f"l{entry}.mix.", layer["mixer"], config["norm"]["eps"]).float()
    assert float(want.abs().max()) > 0.1
    for cuts in ((29,), (1,) * 29, (5, 2, 1, 9, 2, 10), (2, 27)):
        got = _mixer_in_portions(harness, entry, x, cuts)
        torch.testing.assert_close(got, want, msg=lambda m: f"{name} layer {entry} cut {cuts}: {m}", **TOL)


def test_the_parts_of_the_parallel_mixer_one_by_one(tmp_path):
    """The attention on the left and the recurrence on the right, each against its plain function (the pair's weighted sum
    could hide a fault of one in the other's size)."""
    harness, config, weights = _harness(tmp_path, "A")
    x = torch.randn(23, 64)
    seq = harness.cache.new_sequence()
    assert harness.cache.append(seq, 0, 23)
    ctx = harness.runner.builder.build([StepEntry(seq, [0] * 23, 0, [])], harness.runner.ops, torch.float32, harness.runner.workspace)
    y = harness.model.blocks[0].mixer.forward(x, ctx, ctx.cache_view(0), True)
    c = config["layers"][0]["mixer"]
    torch.testing.assert_close(y.terms[0], plain.window_attention(x.double(), weights, "l0.mix.left.", c["left"]).float(), **TOL)
    torch.testing.assert_close(y.terms[1], plain.channel_delta_mixer(x.double(), weights, "l0.mix.right.", c["right"], 1e-5).float(), **TOL)


@pytest.mark.parametrize("streams,center", [(3, True), (1, True), (4, False)])
def test_streams_are_mixed_from_to_and_the_norm_reads_their_weighted_sum(streams, center):
    from velox_amd.parts import make_part

    class Ctx:
        ops = TorchOps()
        dtype = torch.float32

    norm = make_part("norm", "stream_norm", prefix="n", hidden_size=10, eps=1e-5, weight_name="", streams=streams, center=center)
    norm.weight = 1.0 + 0.2 * torch.randn(10)
    x = torch.randn(7, streams, 10)
    y, mix, out, win = torch.randn(7, 10), torch.randn(streams, streams), torch.randn(streams), torch.randn(streams)
    residual = x.reshape(7, streams * 10).clone()
    got = norm.forward_streams(residual, StreamUpdate(y, mix, out), win, Ctx)
    new = [sum(mix[s, t] * x[:, s] for s in range(streams)) + out[t] * y for t in range(streams)]  # [from, to]
    u = sum(win[t] * new[t] for t in range(streams)).double()
    want = plain.layer_norm(u, norm.weight.double(), 1e-5) if center else plain.rms_norm(u, 1e-5) * norm.weight.double()
    torch.testing.assert_close(got, want.float(), **TOL)
    torch.testing.assert_close(residual.view(7, streams, 10), torch.stack(new, 1), **TOL)
    if streams > 1:
        wrong = sum(win[t] * (sum(mix[t, s] * x[:, s] for s in range(streams)) + out[t] * y) for t in range(streams)).double()
        assert float((plain.layer_norm(wrong, norm.weight.double(), 1e-5) - plain.layer_norm(u, norm.weight.double(), 1e-5)).abs().max()) > 0.1


def test_layer_outputs_one_by_one(tmp_path):
    """The sum of the streams after every layer run, from the framework's blocks run one at a time, against the plain model's."""
    harness, config, weights = _harness(tmp_path, "A", seed=5)
    tokens = prompts(config["vocab"], [23], seed=8)["r0"]
    want = []
    plain.forward(config, weights, tokens, want)
    seq = harness.cache.new_sequence()
    assert harness.cache.append(seq, 0, len(tokens))
    ctx = harness.runner.builder.build([StepEntry(seq, tokens, 0, [])], harness.runner.ops, torch.float32, harness.runner.workspace)
    model = harness.model
    residual = model.embed(ctx.token_ids, ctx)
    assert residual.shape == (23, 3 * 64)
    pending = None
    for index in range(len(model.schedule)):
        pending = model.run_schedule(residual, pending, ctx, first=index, last=index + 1)
        # what the layer's last sub-layer produced is still pending: the norm that reads the streams next works it in
        scratch = residual.clone()
        model.final_norm.forward(scratch, pending, ctx)
        torch.testing.assert_close(scratch.view(23, 3, 64).sum(1), want[index].float(), msg=lambda m: f"after layer run {index}: {m}",
                                   rtol=2e-4, atol=3e-5 * max(1.0, float(want[index].abs().max())))


# ----------------------------------------------------------------------------------------------------------------------
# whole models: every way of cutting, batches, pages and slots that are used again
# ----------------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("name", ["A", "B", "D", "E"])
def test_all_ways_of_cutting_agree_with_the_plain_model(tmp_path, name):
    """Whole prompts; the last tokens one by one (more of them than any window or convolution reaches back); portions of 1 to
    16 tokens (many of two); up to four requests mixed in a pool so small that pages are used again, with seven requests on
    four state slots; requests that are ended half way and recomputed in slots that others have used since."""
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [41, 1, 17, 58, 9, 33, 2], seed=3)
    expected = {rid: logits_of(config, weights, tokens) for rid, tokens in requests.items()}
    assert all(float(e.abs().max()) > 1.0 for e in expected.values())  # logits of order one and more: the tolerances bite
    page = PAGE_SIZE[name]
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests, tail=30)),
                         ("portions", rc.changing_portions(requests)), ("mixed", rc.mixed(requests, seed=5)),
                         ("recompute", rc.mixed(requests, seed=6, preempt=("r0", "r3")))):
        replayer = Replayer(folder, "float32", rc.tokens_needed(trace, page), block_size=page, device="cpu", ops=TorchOps(), max_live=4)
        outputs = rc.run_trace(replayer, trace)
        got = rc.collect(trace, outputs, requests)
        for rid in requests:
            close(got[rid], expected[rid], msg=lambda m: f"{name} {label} {rid}: {m}")
        if label in ("mixed", "recompute") and replayer.cache.groups:
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages


def test_a_left_out_mechanism_would_show():
    """The weights are sharp enough that the tests above can fail: each mechanism, taken out or moved by one, changes the
    logits far beyond the tolerance."""
    config = CONFIGS["A"]
    weights = {k: v.double() for k, v in random_weights(config, 2).items()}
    tokens = prompts(config["vocab"], [40], seed=4)["r0"]
    right = plain.forward(config, weights, tokens)

    def moved(change_config=None, change_weights=None):
        c, w = copy.deepcopy(config), dict(weights)
        if change_config:
            change_config(c)
        if change_weights:
            change_weights(w)
        return float((right - plain.forward(c, w, tokens))[-8:].abs().max())

    def flipped(name):
        return lambda w: w.update({name: w[name].flip(-1) if w[name].dim() > 1 else w[name].flip(0)})

    left = lambda c: c["layers"][0]["mixer"]["left"]  # noqa: E731
    assert moved(lambda c: left(c)["mask"].update(size=7)) > 0.05 and moved(lambda c: left(c)["mask"].update(size=5)) > 0.05
    assert moved(lambda c: left(c).pop("mask")) > 0.05
    assert moved(lambda c: left(c)["rot"].pop("scaling")) > 0.05 and moved(lambda c: left(c)["rot"].update(dims=6)) > 0.05
    assert moved(lambda c: left(c).update(scale=0.4)) > 0.05
    assert moved(change_weights=flipped("l0.mix.left.k.conv")) > 0.05 and moved(change_weights=flipped("l0.mix.right.v.conv")) > 0.05
    assert moved(change_weights=lambda w: w.update({"l0.mix.left.q.b": torch.zeros(64, dtype=torch.float64)})) > 0.05
    assert moved(lambda c: c["layers"][0]["mixer"].update(left_scale=1.3, right_scale=0.7)) > 0.05
    assert moved(change_weights=lambda w: w.update({"l0.mix.right.dt_bias": w["l0.mix.right.dt_bias"].view(4, 8).t().reshape(-1)})) > 0.05  # heads x dim, not dim x heads
    assert moved(lambda c: c["layers"][1]["mixer"].update(tau=1.0)) > 0.05
    assert moved(change_weights=lambda w: w.update({"l2.mix.A_log": w["l2.mix.A_log"] + 2.0})) > 0.05
    assert moved(change_weights=lambda w: w.update({"l2.mix.b": -w["l2.mix.b"]})) > 0.05
    assert moved(change_weights=lambda w: w.update({"l0.hc1.mix": w["l0.hc1.mix"].t()})) > 0.05
    assert moved(change_weights=lambda w: w.update({"l2.hc2.in": torch.full((3,), 1 / 3, dtype=torch.float64)})) > 0.05
    assert moved(lambda c: c.pop("streams")) > 0.05
    assert moved(lambda c: c["layers"][3].pop("weights_of"), lambda w: w.update({k.replace("l0.", "l3.", 1): v.flip(0) for k, v in w.items() if k.startswith("l0.")})) > 0.05
    shifted = plain.forward(config, weights, tokens[1:])  # one token less: states, windows and positions all differ
    assert float((right[-1] - shifted[-1]).abs().max()) > 0.05


def _long_memory(config, weights):
    """Decays close to 1 in every recurrent mixer: what the first tokens wrote still decides the read-out hundreds of tokens on."""
    out = dict(weights)
    for name in weights:
        if name.endswith("A_log"):
            out[name] = torch.full_like(weights[name], math.log(2e-4))
        elif name.endswith(".a2.b"):
            out[name] = torch.full_like(weights[name], 9.0)
        elif name.endswith(".a2") and name.replace(".a2", ".a2.b") in weights:
            out[name] = 0.05 * weights[name]
    return out


@pytest.mark.parametrize("name,cuts", [("E", (260,)), ("E", (3, 1, 252, 2, 1, 1)), ("E", (4, 4, 248) + (1,) * 4), ("A", (16, 15, 1, 96, 2) + (1,) * 10)])
def test_what_the_first_tokens_wrote_is_read_far_later(tmp_path, name, cuts):
    """A state that is dropped, zeroed or not carried over a portion's or a page's border loses the first tokens: two
    prompts that differ in their first token only give different logits at their end, and the framework agrees with the
    plain model on both, however the prompt is cut (first portions that end inside the first page, at its border, behind it)."""
    config = CONFIGS[name]
    weights = _long_memory(config, random_weights(config, 4))
    folder = write_folder(tmp_path / name, config, seed=4, weights=weights)
    config, tensors = read_folder(folder)
    n = sum(cuts)
    base = prompts(config["vocab"], [n], seed=9)["r0"]
    other = [(base[0] + 1) % config["vocab"]] + base[1:]
    want = {rid: logits_of(config, tensors, toks)[-4:] for rid, toks in (("base", base), ("other", other))}
    assert float((want["base"] - want["other"]).abs().max()) > 0.05  # the far token shows
    page = PAGE_SIZE[name]
    for rid, toks in (("base", base), ("other", other)):
        replayer = Replayer(folder, "float32", (n + page - 1) // page * page, block_size=page, device="cpu", ops=TorchOps(), max_live=2)
        at, rows = 0, []
        for i, c in enumerate(cuts):
            out = replayer.step({"step": i, "entries": [{"id": rid, "tokens": toks[at:at + c], "want": list(range(c))}], "end": [rid] if at + c == n else []})
            rows.append(torch.from_numpy(out))
            at += c
        close(torch.cat(rows)[-4:], want[rid], msg=lambda m: f"{name} {cuts} {rid}: {m}")


def test_a_slot_that_is_used_again_starts_from_nothing(tmp_path):
    """One state slot: every request starts in the slot the one before it left, and must not see what it wrote there
    (state, the convolutions' last inputs); a request that comes again gives the same logits again."""
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=2)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [19, 3, 1, 26], seed=11)
    replayer = Replayer(folder, "float32", 32, block_size=4, device="cpu", ops=TorchOps(), max_live=1)
    for turn in range(2):
        for rid, toks in requests.items():
            half = max(1, len(toks) // 2)
            first = replayer.step({"step": 0, "entries": [{"id": rid, "tokens": toks[:half], "want": list(range(half))}], "end": [] if half < len(toks) else [rid]})
            rows = [torch.from_numpy(first)]
            if half < len(toks):
                rows.append(torch.from_numpy(replayer.step({"step": 1, "entries": [{"id": rid, "tokens": toks[half:], "want": list(range(len(toks) - half))}], "end": [rid]})))
            close(torch.cat(rows), logits_of(config, weights, toks), msg=lambda m: f"turn {turn} {rid}: {m}")
            assert replayer.cache.state.num_free == 1 and replayer.cache.num_used_pages() == 0


def test_long_decoding_past_every_window(tmp_path):
    """A short prompt and then 150 tokens one by one: the window passes over decoded tokens only, pages behind it go back
    to the pool (which is smaller than the sequence), the states are carried 150 times."""
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=6)
    config, weights = read_folder(folder)
    toks = prompts(config["vocab"], [153], seed=12)["r0"]
    want = logits_of(config, weights, toks)
    replayer = Replayer(folder, "float32", 160, block_size=4, device="cpu", ops=TorchOps(), max_live=1)
    rows = [torch.from_numpy(replayer.step({"step": 0, "entries": [{"id": "a", "tokens": toks[:3], "want": [0, 1, 2]}], "end": []}))]
    most = 0
    for i in range(3, 153):
        rows.append(torch.from_numpy(replayer.step({"step": i, "entries": [{"id": "a", "tokens": [toks[i]], "want": [0]}], "end": ["a"] if i == 152 else []})))
        most = max(most, replayer.cache.num_used_pages())
    close(torch.cat(rows), want)
    assert most <= 4  # a window of 6 tokens over pages of 4: the rest has been given back


# ----------------------------------------------------------------------------------------------------------------------
# the entry point
# ----------------------------------------------------------------------------------------------------------------------
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


@pytest.mark.parametrize("name", ["A", "E"])
def test_greedy_generation_through_the_entry_point_with_preemption(tmp_path, name):
    """The scheduler, the step function and the sampler around the model: greedy tokens equal the plain model's, together
    and alone, in portions of seven tokens, also when the pool is so small that requests are preempted and computed
    again.  Prefixes are not shared: a state of fixed size stands for tokens that a sharer would skip."""
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2)
    config, weights = read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 26], seed=7).values())
    want = [plain_greedy(config, weights, p, 10) for p in texts]

    def requests(prefix):
        return [Request(f"{prefix}{i}", p, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)) for i, p in enumerate(texts)]

    engine = engine_for(folder, 4)
    assert engine.cache.prefix is None
    assert [r.output_token_ids for r in engine.generate(requests("a"))] == want
    assert [r.output_token_ids for r in engine.generate(requests("again"))] == want  # in slots and pages that the first ones used
    alone = engine.generate([Request("alone", texts[1], SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))])[0]
    assert alone.output_token_ids == want[1]
    two_slots = engine_for(folder, 4, max_num_seqs=2)
    assert [r.output_token_ids for r in two_slots.generate(requests("s"))] == want
    if name == "A":
        tight = engine_for(folder, 4, num_gpu_blocks=11)
        assert [r.output_token_ids for r in tight.generate(requests("t"))] == want
        assert tight.cache.num_used_pages() == 0
        tight.cache.assert_consistent([])
