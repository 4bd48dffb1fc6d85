"""Dipisun on a CPU: the kernels' plain references stand in for the kernels; the configuration reader, the parts,
the loader, the cache manager, the step function, replay, the scheduler and the entry point are the product's.
The yardstick is ``plain_dipisun`` (whole sequences, no cache)."""
import copy
import math

import pytest
import torch

import replay_cases as rc
from dipisun_cases import CONFIGS, PAGE_SIZE, prompts, random_weights, tensor_shapes, write_folder
from plain_dipisun import dipisun_forward, distance_bucket, read_folder, sinusoid
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.config.model_config import ConfigError
from velox_amd.config.registry import config_from_dict, load_config
from velox_amd.engine.engine import build_model
from velox_amd.engine.replay import Replayer
from velox_amd.parts import make_part
from velox_amd.parts.base import ResidualCopy
from velox_amd.parts.normed_attention import bias_by_distance
from velox_amd.weights import WeightsError, bind_from_checkpoint

TOL = dict(rtol=2e-4, atol=2e-5)


def test_configuration_is_read_layer_by_layer_and_refused_where_it_cannot_run(tmp_path):
    config = config_from_dict(CONFIGS["A"])
    assert config.architecture == "Dipisun" and config.width == 64 and len(config.layers) == 4 and config.residual_mult == 0.7
    model = build_model(config, torch.float32, "cpu", max_position=64)
    assert [type(b).__name__ for b in model.blocks] == ["OutputNormBlock"] * 4 and model.blocks[2].residual_mult == 0.7
    mixers = [b.mixer for b in model.blocks]
    assert [m.qk_norm for m in mixers] == ["per_head", "whole", "per_head", "whole"]
    assert [m.value_mix for m in mixers] == [None, "first", "blend", "blend"]  # the layer before the first blending one takes no part
    assert [m.cached_dim for m in mixers] == [16, 32, 32, 32] and mixers[1].q_temp == (0.4, 8) and mixers[3].q_temp is None
    assert mixers[1].distance_bias == (8, 24.0) and mixers[0].distance_bias is None
    needs = model.cache_needs()
    assert needs[0].tensors[0][1] == (2, -1, 16) and needs[1].tensors[1][1] == (1, 32, -1) and all(n.window is None for n in needs)
    assert type(model.blocks[1].feed_forward).__name__ == "NoFeedForward" and len(model.blocks[1].children()) == 2
    ff = model.blocks[3].feed_forward
    assert (ff.num_experts, ff.identity_experts, ff.top, ff.score, ff.renormalize, ff.scale_input) == (5, 2, 3, "softmax", False, False)
    assert ff.unit == (1.702, 0.75, 1.0) and model.spec.embedding_position == "sinusoid"
    for change, message in (
        (lambda c: c["layers"][0].update(type="other"), "type"),
        (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
        (lambda c: c["layers"][3]["mlp"]["router"].update(top=8), "top"),
        (lambda c: c["layers"][2]["mixer"].update(vdim=12), "one size"),
        (lambda c: c["layers"][0]["mixer"].update(heads=5), "multiple"),
        (lambda c: c["layers"][1]["mixer"].pop("bias_max"), "bias_max"),
        (lambda c: c["layers"][1]["mixer"]["q_temp"].update(every=0), "every"),
        (lambda c: c.pop("width"), "width"),
    ):
        broken = copy.deepcopy(CONFIGS["A"])
        change(broken)
        with pytest.raises(ConfigError, match=message):
            config_from_dict(broken)
    # the rows of a bias table are a size that only the tensor gives: a folder's reader takes it from there
    stripped = copy.deepcopy(CONFIGS["A"])
    stripped["layers"][1]["mixer"].pop("bias_buckets")
    with pytest.raises(ConfigError, match="bias_buckets"):
        build_model(config_from_dict(stripped), torch.float32, "cpu")
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=1)
    loaded = load_config(folder)
    assert "bias_buckets" not in loaded.raw["layers"][1]["mixer"] and "tensor_shapes" not in loaded.to_json_dict()
    assert build_model(loaded, torch.float32, "cpu").blocks[3].mixer.distance_bias == (6, 10.0)


def test_every_tensor_is_named_and_shaped_as_the_design_says(tmp_path):
    for name in ("A", "B", "D"):
        folder = write_folder(tmp_path / name, CONFIGS[name], seed=1)
        model = build_model(load_config(folder), torch.float32, "cpu", max_position=32)
        count = bind_from_checkpoint(model, folder, torch.float32, "cpu")
        assert count == sum(math.prod(s) for s in tensor_shapes(CONFIGS[name]).values())
    weights = random_weights(CONFIGS["A"], 1)
    weights["l1.norm2"] = torch.ones(64)  # a layer without a feed-forward has no second norm
    del weights["l3.mlp.correction"]
    folder = write_folder(tmp_path / "broken", CONFIGS["A"], seed=1, weights=weights)
    model = build_model(load_config(folder), torch.float32, "cpu", max_position=32)
    with pytest.raises(WeightsError) as caught:
        bind_from_checkpoint(model, folder, torch.float32, "cpu")
    assert caught.value.unexpected == ["l1.norm2"] and caught.value.missing == ["l3.mlp.correction"]


@pytest.mark.parametrize("buckets,far", [(8, 24), (6, 10), (7, 33.5), (2, 3), (32, 1000), (16, 16 * 16), (5, 2.5)])
def test_bias_by_distance_puts_every_distance_in_its_bucket(buckets, far):
    rel = torch.randn(buckets, 3)
    table = bias_by_distance(rel, far)
    assert table.shape[0] == 3 and table.dtype == torch.float32
    last = table.shape[1] - 1
    assert distance_bucket(last, buckets, far) == buckets - 1 and (last == 0 or distance_bucket(last - 1, buckets, far) < buckets - 1)
    for n in list(range(last + 1)) + [last + 1, last + 7, 5 * last + 100, 10 ** 6]:
        assert torch.equal(table[:, min(n, last)], rel[distance_bucket(n, buckets, far)]), n
    # the reference of the attention kernel reads the same column for every farther key
    assert [distance_bucket(n, buckets, far) for n in range(buckets // 2)] == list(range(buckets // 2))


@pytest.mark.parametrize("width", [64, 7, 130])
def test_sinusoid_of_the_part_and_of_the_plain_function(width):
    part = make_part("position", "sinusoidal", width=width, base=10000.0)
    part.finalize(torch.device("cpu"), torch.float32)

    class Ctx:
        ops = TorchOps()
        positions = torch.tensor([0, 1, 2, 63, 64, 1000, 99999], dtype=torch.int32)

    got = part.on_embeddings(torch.zeros(7, width), Ctx)
    want = sinusoid(Ctx.positions.long(), width, torch.float64)
    torch.testing.assert_close(got.double(), want, rtol=0, atol=1e-6)
    assert float(got[0, 0]) == 0.0 and float(got[0, 1 % width]) == (1.0 if width > 1 else 0.0)  # sine in even entries, cosine in odd ones


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_all_ways_of_cutting_agree_with_the_plain_model(tmp_path, name):
    """Whole prompts; the last tokens one by one; portions of 1 to 16 tokens (many of two); up to four requests mixed in
    a pool so small that pages and slots are used again; requests that are ended half way and recomputed."""
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [41, 1, 17, 58, 9, 33, 2], seed=3)
    expected = {rid: dipisun_forward(config, weights, tokens, torch.float64).float() for rid, tokens in requests.items()}
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


def test_a_left_out_mechanism_would_show():
    """The weights are sharp enough that the tests above can fail: each mechanism, taken out or moved by one, changes the
    logits far beyond the tolerance."""
    config = CONFIGS["A"]
    weights = random_weights(config, 2)
    tokens = prompts(config["vocab"], [40], seed=4)["r0"]
    right = dipisun_forward(config, weights, tokens)

    def moved(change_config=None, change_weights=None):
        c, w = copy.deepcopy(config), dict(weights)
        if change_config:
            change_config(c)
        if change_weights:
            change_weights(w)
        return float((right - dipisun_forward(c, w, tokens)).abs().max())

    shifted = dipisun_forward(config, weights, tokens[1:])  # one key less and every position off by one
    assert float((right[-1] - shifted[-1]).abs().max()) > 0.05
    assert moved(lambda c: c["layers"][1]["mixer"].pop("q_temp")) > 0.05
    assert moved(lambda c: c["layers"][1]["mixer"].update(bias_max=12)) > 0.05
    assert moved(change_weights=lambda w: w.update({"l3.mix.rel": torch.zeros_like(w["l3.mix.rel"])})) > 0.05
    assert moved(lambda c: c["layers"][2]["mixer"].pop("v_mix")) > 0.05
    assert moved(change_weights=lambda w: w.update({"l3.mix.vmix": torch.tensor(0.0)})) > 0.05
    assert moved(change_weights=lambda w: w.update({"l3.mlp.correction": torch.zeros(7)})) > 0.05
    assert moved(lambda c: c["layers"][3]["mlp"]["router"].update(experts=7, identity=0), lambda w: w.update(
        {f"l3.mlp.e{e}.{n}": torch.zeros_like(w[f"l3.mlp.e0.{n}"]) for e in (5, 6) for n in ("gate", "up", "down")})) > 0.05  # identity experts hand their input on
    assert moved(lambda c: c["layers"][0]["mlp"]["expert"].update(limit=50.0)) > 0.05
    assert moved(lambda c: c.update(residual_mult=0.8)) > 0.05
    assert moved(lambda c: c["layers"][0]["mixer"].update(scale=0.5)) > 0.05


def engine_for(folder, page, **overrides):
    options = dict(model=folder, dtype="float32", device="cpu", max_model_len=96, max_num_seqs=4, max_num_batched_tokens=32,
                   max_prefill_chunk_size=7, block_size=page, num_gpu_blocks=64, enable_cuda_graphs=False, seed=0)
    options.update(overrides)
    return Engine.from_pretrained(EngineConfig(**options), ops=TorchOps())


def plain_greedy(config, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(dipisun_forward(config, weights, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_entry_point_with_preemption(tmp_path):
    """The scheduler, the step function, the sampler and the prefix cache (which this design may use: every layer keeps
    every token, and a token's blended values depend on nothing but the tokens before it) around the model: greedy tokens
    equal the plain model's, together and alone, also when the pool is so small that requests are preempted."""
    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=2)
    config, weights = read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 26], seed=7).values())
    want = [plain_greedy(config, weights, p, 10) for p in texts]

    def requests(prefix):
        return [Request(f"{prefix}{i}", p, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True)) for i, p in enumerate(texts)]

    engine = engine_for(folder, 4)
    assert engine.cache.prefix is not None and engine.max_model_len == 96
    assert [r.output_token_ids for r in engine.generate(requests("a"))] == want
    assert [r.output_token_ids for r in engine.generate(requests("again"))] == want  # now behind the published pages of the first time
    alone = engine.generate([Request("alone", texts[1], SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))])[0]
    assert alone.output_token_ids == want[1]
    tight = engine_for(folder, 4, num_gpu_blocks=17, enable_prefix_caching=False)
    assert [r.output_token_ids for r in tight.generate(requests("t"))] == want and tight.scheduler.num_preemptions > 0
    assert tight.cache.num_used_pages() == 0
    tight.cache.assert_consistent([])


def test_layer_outputs_one_by_one(tmp_path):
    """The residual stream after every layer, from the framework's blocks run one at a time, against the plain model's."""
    from helpers import Harness
    from velox_amd.engine.batch import StepEntry

    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=5)
    config, weights = read_folder(folder)
    tokens = prompts(config["vocab"], [23], seed=8)["r0"]
    _, want = dipisun_forward(config, weights, tokens, keep_layers=True)
    harness = Harness(folder, TorchOps(), torch.float32, "cpu", 4, 32, max_num_seqs=2, max_num_tokens=64)
    seq = harness.cache.new_sequence()
    assert harness.cache.append(seq, 0, len(tokens))
    ctx = harness.runner.builder.build([StepEntry(seq, tokens, 0, [])], harness.runner.ops, torch.float32, harness.runner.workspace)
    model = harness.model
    residual = model.embed(ctx.token_ids, ctx)
    pending = None
    for index in range(len(model.schedule)):
        pending = model.run_schedule(residual, pending, ctx, first=index, last=index + 1)
        assert isinstance(pending, ResidualCopy) and pending.copy is residual  # nothing is left to add; float32 needs no copy
        torch.testing.assert_close(residual, want[index], msg=lambda m: f"after layer {index}: {m}", **TOL)
