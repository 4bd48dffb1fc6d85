"""Tiverax on a CPU: the kernels' plain references stand in for the kernels; the configuration reader, the parts,
the loader, the cache manager, the step function, replay, the scheduler and the entry point are the product's.
The yardstick is ``plain_tiverax`` (whole sequences, no cache)."""
import copy
import math

import pytest
import torch

import replay_cases as rc
from plain_tiverax import read_folder, rotate_pairs, stretched_frequencies, tiverax_logits
from tiverax_cases import CONFIGS, PAGE_SIZE, layer, mixer, dense, prompts, random_weights, tensor_shapes, write_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.config.model_config import ConfigError
from velox_amd.config.registry import config_from_dict
from velox_amd.engine.engine import build_model
from velox_amd.engine.replay import Replayer
from velox_amd.parts import make_part
from velox_amd.weights import WeightsError, bind_from_checkpoint

TOL = dict(rtol=2e-4, atol=2e-5)


def test_configuration_is_read_layer_by_layer_and_refused_where_it_cannot_run():
    config = config_from_dict(CONFIGS["A"])
    assert config.architecture == "Tiverax" and config.width == 64 and len(config.layers) == 5
    model = build_model(config, torch.float32, "cpu", max_position=64)
    assert [(e.layer, e.cache_from) for e in model.schedule] == [(0, None), (1, 0), (2, None), (3, 2), (4, 0)]
    assert sorted(model.positions) == ["rotation0", "rotation1"]  # layers with the same rotation share its tables
    needs = model.cache_needs()
    assert [n is None for n in needs] == [False, True, False, True, True]
    assert needs[0].tensors[0][1] == (1, -1, 32) and needs[2].tensors[0][1] == (1, -1, 64)  # 28 and 56 cached channels, padded
    assert type(model.blocks[2].feed_forward).__name__ == "NoFeedForward" and model.blocks[1].feed_forward.shared is not None
    assert model.blocks[3].feed_forward.shared is None and model.blocks[1].feed_forward.top == 2
    for change, message in (
        (lambda c: c["layers"][1]["mixer"].update(kv_from=1), "kv_from"),
        (lambda c: c["layers"][1]["mixer"].update(kv_from=2), "kv_from"),
        (lambda c: c["layers"][1]["mixer"].update(kv_rank=24), "kv_rank"),
        (lambda c: c["layers"][1]["mixer"]["rot"].update(base=7.0), "rotation"),
        (lambda c: c["layers"][0].update(type="other"), "type"),
        (lambda c: c["layers"][0]["mlp"].update(kind="other"), "kind"),
        (lambda c: c["layers"][1]["mlp"]["router"].update(top=9), "top"),
        (lambda c: c["layers"][2]["mixer"]["rot"].update(dims=18), "dims"),
        (lambda c: c.pop("width"), "width"),
    ):
        broken = copy.deepcopy(CONFIGS["A"])
        change(broken)
        with pytest.raises(ConfigError, match=message):
            config_from_dict(broken)


def test_every_tensor_is_named_and_shaped_as_the_design_says(tmp_path):
    for name in ("A", "B"):
        folder = write_folder(tmp_path / name, CONFIGS[name], seed=1)
        model = build_model(config_from_dict(CONFIGS[name]), torch.float32, "cpu", max_position=32)
        count = bind_from_checkpoint(model, folder, torch.float32, "cpu")
        assert count == sum(math.prod(s) for s in tensor_shapes(CONFIGS[name]).values())
    weights = random_weights(CONFIGS["B"], 1)
    weights["l1.mix.dkv"] = torch.zeros(16, 88)  # a borrower has no down-projection
    del weights["l0.mlp.shared.up"]
    folder = write_folder(tmp_path / "broken", CONFIGS["B"], seed=1, weights=weights)
    model = build_model(config_from_dict(CONFIGS["B"]), torch.float32, "cpu", max_position=32)
    with pytest.raises(WeightsError) as caught:
        bind_from_checkpoint(model, folder, torch.float32, "cpu")
    assert caught.value.unexpected == ["l1.mix.dkv"] and caught.value.missing == ["l0.mlp.shared.up"]


@pytest.mark.parametrize("dims,base,stretch", [(8, 10000.0, (4.0, 24, 8.0, 1.0)), (24, 2e5, (3.0, 512, 16.0, 2.0)), (12, 500.0, None), (2, 10.0, (8.0, 4, 2.0, 0.5))])
def test_rotation_tables_hold_the_stretched_frequencies_and_the_magnitude(dims, base, stretch):
    part = make_part("position", "rotary", rotary_dim=dims, theta=base, max_position=300, layout="interleaved", stretch=stretch)
    part.finalize(torch.device("cpu"), torch.float32)
    cos, sin = part.rotary_tables()
    scaling = dict(zip(("factor", "original", "fast", "slow"), stretch)) if stretch else None
    freqs, magnitude = stretched_frequencies(dims, base, scaling, torch.float64)
    angles = torch.arange(300, dtype=torch.float64)[:, None] * freqs[None, :]
    assert cos.shape == (300, dims // 2) and part.layout == "interleaved"
    # (float32 angles of up to 300 radians carry an error of about 2e-5)
    torch.testing.assert_close(cos.double(), angles.cos() * magnitude, rtol=0, atol=6e-5)
    torch.testing.assert_close(sin.double(), angles.sin() * magnitude, rtol=0, atol=6e-5)
    if stretch:
        plain, one = stretched_frequencies(dims, base, None, torch.float64)
        assert one == 1.0 and magnitude == pytest.approx(0.1 * math.log(stretch[0]) + 1.0)
        assert bool((freqs <= plain * (1 + 1e-12)).all()) and bool((freqs >= plain / stretch[0] * (1 - 1e-12)).all())
    # the reference of the rotation kernel pairs (2i, 2i + 1) as the plain function does, and passes what lies beyond
    x = torch.randn(5, 3, dims + 4)
    positions = torch.tensor([0, 1, 7, 150, 299])
    got = TorchOps._rotate(x, cos[positions], sin[positions], True)
    want = rotate_pairs(x.double(), positions, freqs, magnitude, dims)
    torch.testing.assert_close(got.double(), want, rtol=0, atol=2e-4)
    assert torch.equal(got[..., dims:], x[..., dims:])


@pytest.mark.parametrize("name", ["A", "B", "D", "E"])
def test_all_ways_of_cutting_agree_with_the_plain_model(tmp_path, name):
    """Whole prompts; the last tokens one by one; portions of 1 to 16 tokens (many of two); up to four requests mixed in
    a pool so small that pages and slots are used again; requests that are ended half way and recomputed."""
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [41, 1, 17, 58, 9, 33, 2], seed=3)
    expected = {rid: tiverax_logits(config, weights, tokens) for rid, tokens in requests.items()}
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


def test_a_lost_or_misplaced_key_would_show(tmp_path):
    """The weights are sharp enough that the tests above can fail: dropping the first key of a sequence, or the stretch of
    the rotation, or the weight on an expert's input, moves the logits far beyond the tolerance."""
    config = CONFIGS["A"]
    weights = random_weights(config, 2)
    tokens = prompts(config["vocab"], [40], seed=4)["r0"]
    right = tiverax_logits(config, weights, tokens)
    shifted = tiverax_logits(config, weights, tokens[1:])  # the same tokens without the first: one key less, positions off by one
    assert float((right[-1] - shifted[-1]).abs().max()) > 0.05
    unstretched = copy.deepcopy(config)
    for entry in unstretched["layers"]:
        entry["mixer"]["rot"].pop("scaling", None)
    assert float((right - tiverax_logits(unstretched, weights, tokens)).abs().max()) > 0.05
    other_top = copy.deepcopy(config)
    other_top["layers"][1]["mlp"]["router"]["top"] = 1
    assert float((right - tiverax_logits(other_top, weights, tokens)).abs().max()) > 0.05


def engine_for(folder, page, **overrides):
    options = dict(model=folder, dtype="float32", device="cpu", max_model_len=96, max_num_seqs=4, max_num_batched_tokens=32,
                   max_prefill_chunk_size=7, block_size=page, num_gpu_blocks=64, enable_cuda_graphs=False, seed=0)
    options.update(overrides)
    return Engine.from_pretrained(EngineConfig(**options), ops=TorchOps())


def plain_greedy(config, weights, prompt, n):
    tokens = list(prompt)
    for _ in range(n):
        tokens.append(int(tiverax_logits(config, weights, tokens)[-1].argmax()))
    return tokens[len(prompt):]


def test_greedy_generation_through_the_entry_point_with_preemption(tmp_path):
    """The scheduler, the step function, the sampler and the prefix cache (which this design may use: every layer keeps
    every token) around the model: greedy tokens equal the plain model's, together and alone, also when the pool is so
    small that requests are preempted and recomputed."""
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

    folder = write_folder(tmp_path / "A", CONFIGS["A"], seed=5)
    config, weights = read_folder(folder)
    tokens = prompts(config["vocab"], [23], seed=8)["r0"]
    want = []
    tiverax_logits(config, weights, tokens, residuals=want)
    harness = Harness(folder, TorchOps(), torch.float32, "cpu", 4, 16, max_num_seqs=2, max_num_tokens=64)
    seq = harness.cache.new_sequence()
    assert harness.cache.append(seq, 0, len(tokens))
    from velox_amd.engine.batch import StepEntry

    ctx = harness.runner.builder.build([StepEntry(seq, tokens, 0, [])], harness.runner.ops, torch.float32, harness.runner.workspace)
    model = harness.model
    residual = model.embed(ctx.token_ids, ctx)
    pending = None
    for index in range(len(model.schedule)):
        pending = model.run_schedule(residual, pending, ctx, first=index, last=index + 1)
        first, second = (pending.first, pending.second) if hasattr(pending, "second") else (pending, 0.0)
        torch.testing.assert_close(residual + (first + second), want[index], msg=lambda m: f"after layer {index}: {m}", **TOL)
