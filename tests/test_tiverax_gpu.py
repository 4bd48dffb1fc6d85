"""Tiverax on the GPU: each new kernel against its plain reference; the latent-attention mixer alone with keys made to
stand out far back and at page borders, in portions and in single decoded tokens; the whole model in float32 and
bfloat16 through replay (every way of cutting, pages and slots used again), in long decoding, in batches against
each request alone, through the entry point with captured decode steps, and through the replay program itself."""
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

import replay_cases as rc
from plain_tiverax import latent_and_shared_key, latent_attention, read_folder, routed_experts, stretched_frequencies, tiverax_logits
from tiverax_cases import CONFIGS, PAGE_SIZE, mixer as mixer_config, moe, prompts, random_weights, write_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.cache import CacheManager
from velox_amd.engine.batch import BatchBuilder, StepEntry, Workspace
from velox_amd.engine.replay import Replayer
from velox_amd.parts import make_part
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
def test_embedding_scale_and_two_term_delta(ops, dtype):
    ref, dt = TorchOps(), DTYPES[dtype]
    table = torch.randn(50, 72).to(dt).cuda()
    ids = torch.tensor([3, 49, 0, 3], dtype=torch.int32).cuda()
    assert torch.equal(ops.embed(ids, table, scale=2.5), ref.embed(ids, table, scale=2.5)) and torch.equal(ops.embed(ids, table), table[ids.long()].float())
    for hidden in (72, 321):  # (rows kept in registers, and the plain loop for a width that is no multiple of 4)
        weight = (1 + 0.1 * torch.randn(hidden)).cuda()
        residual = torch.randn(9, hidden).cuda()
        # a tensor, or partial sums (which only products of widths that are multiples of 4 leave)
        for first in (torch.randn(9, hidden).to(dt).cuda(), torch.randn(3, 9, hidden).cuda())[: 2 if hidden % 4 == 0 else 1]:
            second = torch.randn(9, hidden).to(dt).cuda()
            mine, theirs = residual.clone(), residual.clone()
            got = ops.add_rmsnorm(mine, SumOf(first, second), weight, 1e-5, dt)
            want = ref.add_rmsnorm(theirs, SumOf(first, second), weight, 1e-5, dt)
            torch.testing.assert_close(mine, theirs, rtol=1e-6, atol=1e-6)
            close(got, want, dtype)
            rows = torch.tensor([8, 0, 4], dtype=torch.int32).cuda()
            kept = mine.clone()
            close(ops.add_rmsnorm_rows(mine, SumOf(first, second), rows, weight, 1e-5, dt), ref.add_rmsnorm_rows(theirs, SumOf(first, second), rows, weight, 1e-5, dt), dtype)
            assert torch.equal(mine, kept)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,dim,rot,rank,half,interleaved,own", [(6, 48, 16, 96, 8, True, True), (3, 12, 16, 40, 6, True, True), (2, 16, 8, 20, 4, False, True),
                                                                    (5, 8, 6, 9, 3, True, False), (1, 4, 2, 3, 0, True, True)])
def test_rotation_latent_norm_and_cache_write(ops, dtype, heads, dim, rot, rank, half, interleaved, own):
    ref, dt = TorchOps(), DTYPES[dtype]
    cached = (rank + rot + 15) // 16 * 16
    tokens, page, pages = 11, 4, 9
    gate = 7
    width = heads * (dim + rot) + gate + (rank + rot if own else 0)
    projected = torch.randn(tokens, width).to(dt).cuda()
    positions = torch.tensor([0, 1, 2, 3, 40, 41, 7, 8, 9, 10, 63], dtype=torch.int32).cuda()
    cos = sin = None
    if half:
        angles = torch.rand(64, half) * 6.0
        cos, sin = (angles.cos() * 1.07).cuda(), (angles.sin() * 1.07).cuda()
    weight = (1 + 0.2 * torch.randn(rank)).cuda()
    slots = torch.randperm(pages * page)[:tokens].to(torch.int32).cuda() + page  # (never the null page)
    caches = [[torch.full((pages + 1, 1, page, cached), 9.0, dtype=dt).cuda(), torch.full((pages + 1, 1, cached, page), 9.0, dtype=dt).cuda()] for _ in range(2)]
    down = heads * (dim + rot) + gate if own else -1
    got = ops.latent_rotate_write(projected, heads, dim, rot, rank, cached, down, positions, cos, sin, interleaved, weight, 1e-5, slots, *caches[0], page)
    want = ref.latent_rotate_write(projected, heads, dim, rot, rank, cached, down, positions, cos, sin, interleaved, weight, 1e-5, slots, *caches[1], page)
    tail = got.view(tokens, heads, cached)[..., rank:]
    close(tail, want.view(tokens, heads, cached)[..., rank:], dtype)
    assert bool((tail[..., rot:] == 0).all())
    for mine, theirs in zip(caches[0], caches[1]):
        close(mine, theirs, dtype, scale=3.0)
    if own:  # keys and transposed values hold the same vectors; untouched places keep what they held
        assert torch.equal(caches[0][0][:, 0].transpose(1, 2), caches[0][1][:, 0]) and int((caches[0][0] == 9.0).sum()) == (pages + 1) * page * cached - tokens * cached
    else:
        assert bool((caches[0][0] == 9.0).all()) and bool((caches[0][1] == 9.0).all())


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("rows,groups,n,k,gated", [(70, 4, 64, 32, False), (5, 3, 40, 12, False), (130, 2, 24, 96, True), (1, 5, 7, 9, True), (16, 16, 128, 192, True)])
def test_per_head_products(ops, dtype, rows, groups, n, k, gated):
    ref, dt = TorchOps(), DTYPES[dtype]
    x_stride, x_offset, out_stride, out_offset = k + 5, 3, n + 8, 4
    x = torch.randn(rows, groups * x_stride + 3).to(dt).cuda()
    maps = (torch.randn(groups, n, k) / math.sqrt(k)).to(dt).cuda()
    gate = torch.randn(rows, 11 + groups * n).to(dt).cuda() if gated else None
    outs = [torch.full((rows, groups * out_stride + 4), 5.0, dtype=dt).cuda() for _ in range(2)]
    ops.head_linear(x, x_stride, x_offset, maps, outs[0], out_stride, out_offset, gate=gate, gate_offset=11)
    ref.head_linear(x, x_stride, x_offset, maps, outs[1], out_stride, out_offset, gate=gate, gate_offset=11)
    close(outs[0], outs[1], dtype)
    assert int((outs[0] == 5.0).sum()) >= rows * (groups * (out_stride - n) + 4)  # the columns between the heads are left alone


@pytest.mark.parametrize("score,renormalize", [("sigmoid", False), ("sigmoid", True), ("softmax", False), ("softmax", True)])
def test_router_scores_and_choices(ops, score, renormalize):
    ref = TorchOps()
    for tokens, experts, top in ((33, 8, 1), (200, 5, 3), (1, 64, 8), (7, 3, 3)):
        logits = (torch.randn(tokens, experts) * 3).cuda()
        choice, weight = ops.route_top(logits, top, score, renormalize)
        want_choice, want_weight = ref.route_top(logits, top, score, renormalize)
        assert torch.equal(choice, want_choice)  # (random logits do not tie)
        torch.testing.assert_close(weight, want_weight, rtol=1e-5, atol=1e-6)
    tied = torch.zeros(2, 6).cuda()
    assert ops.route_top(tied, 2, score, renormalize)[0].tolist() == [[0, 1], [0, 1]]  # ties go to the lower index


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tokens,hidden,inter,experts,top,scale_input,with_shared", [(70, 64, 32, 4, 2, True, True), (9, 88, 20, 6, 3, True, False), (300, 96, 40, 8, 1, False, True),
                                                                                   (1, 256, 64, 12, 1, True, True), (150, 72, 130, 3, 2, False, False),
                                                                                   (700, 136, 72, 2, 2, True, True), (900, 192, 80, 3, 1, False, False)])
def test_routed_experts_against_the_plain_loop(ops, dtype, tokens, hidden, inter, experts, top, scale_input, with_shared):
    ref, dt = TorchOps(), DTYPES[dtype]
    x = torch.randn(tokens, hidden).to(dt).cuda()
    gate_up = (torch.randn(experts * 2 * inter, hidden) / math.sqrt(hidden)).to(dt).cuda()
    down = (torch.randn(experts * hidden, inter) / math.sqrt(inter)).to(dt).cuda()
    logits = (torch.randn(tokens, experts) * 2).cuda()
    logits[: tokens // 2, 1] += 6.0  # many rows of one expert: more than one tile
    choice, weight = ops.route_top(logits, top)
    shared = torch.randn(tokens, hidden).to(dt).cuda() if with_shared else None
    got = ops.routed_experts(x, choice, weight, gate_up, down, experts, scale_input, shared, dt, Workspace(torch.device("cuda")))
    want = ref.routed_experts(x, choice, weight, gate_up, down, experts, scale_input, shared, dt)
    close(got, want, dtype, scale=2.0)
    if dtype == "float32":
        # a token's result does not depend on which tokens share its experts: each row alone gives the same numbers
        for t in (0, tokens - 1):
            alone = ops.routed_experts(x[t:t + 1].contiguous(), choice[t:t + 1].contiguous(), weight[t:t + 1].contiguous(), gate_up, down, experts, scale_input,
                                       shared[t:t + 1].contiguous() if with_shared else None, dt, None)
            assert torch.equal(alone[0], got[t])


def test_routed_experts_part_against_the_design(ops):
    """The part with this design's options (sigmoid scores, not renormalised, on the expert's input, a shared expert) against
    the plain function, with two experts per token."""
    hidden, mlp = 64, moe(5, 2, 24, shared=40)
    part = make_part("feed_forward", "routed_experts", prefix="f.", hidden_size=hidden, intermediate_size=24, num_experts=5, top=2, shared_intermediate_size=40,
                     expert_names=("e{e}.gate", "e{e}.up", "e{e}.down"), router_name="router", shared_names=("gate", "up", "down"))
    g = torch.Generator().manual_seed(3)
    w = {}
    for owner in (part, part.shared):
        for attr, param in owner.params().items():
            pieces = []
            for name, shape in zip(param.sources, param.source_shapes):
                w[owner.prefix + name] = torch.randn(shape, generator=g) * ((3.0 if name == "router" else 1.0) / math.sqrt(shape[1]))
                pieces.append(w[owner.prefix + name])
            setattr(owner, attr, torch.cat(pieces).cuda())
    x = torch.randn(37, hidden, generator=g)

    class Ctx:
        dtype, workspace = torch.float32, Workspace(torch.device("cuda"))

    Ctx.ops = ops
    got = part.forward(x.cuda(), Ctx)
    torch.testing.assert_close(got.cpu(), routed_experts(x, w, "f.", mlp), rtol=2e-4, atol=2e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,d,window", [(4, 1, 272, None), (6, 2, 336, None), (2, 2, 1024, 37)])
def test_attention_for_head_sizes_beyond_the_tiled_kernels(ops, dtype, nh, nkv, d, window):
    """Head sizes above 256 go to the plain kernel: portions behind a context, single tokens and a first token in one step."""
    ref, dt = TorchOps(), DTYPES[dtype]
    page, pages = 8, 40
    k_cache = torch.randn(pages, nkv, page, d).to(dt).cuda()
    v_cache = torch.randn(pages, nkv, d, page).to(dt).cuda()
    q_lens, kv_lens = [1, 1, 9, 1, 30], [70, 1, 9, 300, 155]  # (a decoded token behind 299 keys: two rounds of 256 keys)
    tables = torch.zeros(5, 38, dtype=torch.int32)
    perm = torch.randperm(pages - 1) + 1
    tables[0, :9], tables[1, :1], tables[2, :2], tables[4, :20] = perm[:9], perm[9:10], perm[10:12], perm[12:32]
    tables[3, :38] = torch.cat([perm[32:], perm[:31]])  # (this one shares pages with the others: only read here)
    cu = torch.tensor([0, 1, 2, 11, 12, 42], dtype=torch.int32).cuda()
    q = (torch.randn(42, nh * d) * 0.5).to(dt).cuda()
    args = (q, nh, nkv, d, k_cache, v_cache, page, tables.cuda(), cu, torch.tensor(kv_lens, dtype=torch.int32).cuda(), 30, 300, 1.0 / math.sqrt(d), window, False, None)
    got, want = ops.paged_attention(*args), ref.paged_attention(*args)
    close(got, want, dtype)


# ----------------------------------------------------------------------------------------------------
# the mixer alone: one key made to stand out
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("far_at,length,cuts", [(0, 150, (150,)), (3, 150, (100, 2, 47, 1)), (15, 140, (16, 123, 1)), (16, 140, (17, 120, 1, 1, 1)),
                                               (17, 33, (16, 16, 1)), (63, 200, (64, 64, 64, 8)), (64, 129, (65, 63, 1))])
def test_a_key_far_back_or_at_a_page_border_takes_the_attention(ops, far_at, length, cuts):
    """The input at ``far_at`` is made so that its cached vector lines up with what the LAST token asks for (through the
    pseudo-inverse of the down-projection), with a score far above all others: the last token's output is then that key's
    value.  Pages hold 16 tokens, so positions 15, 16, 17, 63 and 64 sit at page borders; the prompt is cut into portions and
    single tokens so that the key is written by one step and read by a later one."""
    hidden, m = 96, mixer_config(3, 16, 8, 12, 24, 0.5, dims=8, base=100.0)
    rope = make_part("position", "rotary", rotary_dim=8, theta=100.0, max_position=256, layout="interleaved")
    rope.finalize(torch.device("cuda"), torch.float32)
    part = make_part("mixer", "latent_attention", prefix="m.", hidden_size=hidden, num_heads=3, dim=16, rot_dim=8, vdim=12, kv_rank=24, scale=0.5, norm_eps=1e-5,
                     position=rope, names=(("q", "q"), ("down", "dkv"), ("down_norm", "dkv.norm"), ("up_k", "uk"), ("up_v", "uv"), ("gate", "g"), ("out", "o")))
    g = torch.Generator().manual_seed(far_at)
    w = {}
    for attr, param in part.params().items():
        pieces = []
        for name, shape in zip(param.sources, param.source_shapes):
            w["m." + name] = 1 + 0.1 * torch.randn(shape, generator=g) if len(shape) == 1 else torch.randn(shape, generator=g) / math.sqrt(shape[1])
            pieces.append(w["m." + name])
        setattr(part, attr, torch.cat(pieces).cuda())
    part.finalize(torch.device("cuda"), torch.float32)
    ops.attention_library(part.cached_dim)
    x = torch.randn(length, hidden, generator=g) * 0.3
    x[-1] *= 5.0  # (a loud query)
    # what head 0 of the last token asks the latent for: U_0^T a_0; a latent along it (before the norm's weight) answers loudest
    q_last = (w["m.q"] @ x[-1]).view(3, 24)[0, :16]
    wanted = (w["m.uk"].view(3, 16, 24)[0].T @ q_last) / w["m.dkv.norm"]
    x[far_at] = torch.linalg.pinv(w["m.dkv"][:24]) @ (wanted / wanted.norm() * 40.0)
    positions = torch.arange(length)
    freqs, magnitude = stretched_frequencies(8, 100.0, None, torch.float32)
    c, shared = latent_and_shared_key(x, w, "m.", m, 1e-5, positions, freqs, magnitude)
    want = latent_attention(x, w, "m.", m, c, shared, positions, freqs, magnitude)
    scores = ((w["m.uk"].view(3, 16, 24)[0].T @ q_last) @ c.T) * 0.5
    assert int(scores.argmax()) == far_at and float(torch.softmax(scores, 0)[far_at]) > 0.8  # the made key does stand out
    cache = CacheManager([part.cache_need()], 16, 20, 2, torch.float32, "cuda")
    builder, workspace = BatchBuilder(cache, "cuda", 256, 2), Workspace(torch.device("cuda"))
    seq, done, got = cache.new_sequence(), 0, []
    assert sum(cuts) == length
    for n in cuts:
        assert cache.append(seq, done, n)
        ctx = builder.build([StepEntry(seq, [0] * n, done)], ops, torch.float32, workspace)
        out = part.forward(x[done:done + n].cuda(), ctx, ctx.cache_view(0), True)
        got.append((out.sum(0) if out.dim() == 3 else out).cpu())
        done += n
    torch.testing.assert_close(torch.cat(got), want, rtol=2e-4, atol=2e-5)


# ----------------------------------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D", "E"])
def test_all_ways_of_cutting_on_the_gpu(tmp_path, name, dtype):
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2, dtype=dtype)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [141, 1, 37, 98, 2, 64, 75], seed=11)
    expected = {rid: tiverax_logits(config, weights, tokens) for rid, tokens in requests.items()}
    page = PAGE_SIZE[name]
    results = {}
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)), ("portions", rc.changing_portions(requests)),
                         ("mixed", rc.mixed(requests, seed=5)), ("recompute", rc.mixed(requests, seed=8, preempt=("r0", "r3", "r6")))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page, max_live=4)
        outputs = rc.run_trace(replayer, trace)
        results[label] = rc.collect(trace, outputs, requests)
        for rid in requests:
            got, want = results[label][rid], expected[rid]
            if dtype == "float32":
                torch.testing.assert_close(got, want, msg=lambda m: f"{name} {label} {rid}: {m}", **TOL[dtype])
            else:
                # bfloat16: rounding may send a token to another expert where two scores are close; such rows are few
                err = (got - want).abs().amax(-1) / want.abs().amax(-1).clamp(min=1.0)
                assert float((err < 0.08).float().mean()) >= 0.9, f"{name} {label} {rid}: {err}"
        if label in ("mixed", "recompute"):
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
    if dtype == "float32":
        for label in ("tail", "portions", "mixed", "recompute"):  # the ways of cutting agree with each other at least as closely
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], rtol=1e-4, atol=3e-5)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_a_batch_against_each_request_alone(tmp_path, dtype):
    """A prompt of a few tokens, then 200 tokens one by one across many page borders; then four requests of unequal
    length decoded together, whose logits equal those of each request decoded alone."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=4, dtype=dtype)
    config, weights = read_folder(folder)
    tokens = prompts(config["vocab"], [205], seed=12)["r0"]
    want = tiverax_logits(config, weights, tokens)
    replayer = Replayer(folder, dtype, 4 * 224, block_size=16, max_live=4)
    rows = [replayer.step({"step": 0, "entries": [{"id": "x", "tokens": tokens[:5], "want": [0, 4]}], "end": []})]
    for i in range(5, 205):
        rows.append(replayer.step({"step": i, "entries": [{"id": "x", "tokens": [tokens[i]], "want": [0]}], "end": ["x"] if i == 204 else []}))
    got = torch.from_numpy(np.concatenate(rows))
    if dtype == "float32":
        torch.testing.assert_close(got, want[[0] + list(range(4, 205))], **TOL[dtype])
    else:
        err = (got - want[[0] + list(range(4, 205))]).abs().amax(-1) / want.abs().amax()
        assert float((err < 0.08).float().mean()) >= 0.9
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


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(tmp_path, ops, graphs):
    """Scheduler, step function, captured decode steps (``graphs``) and sampler around the model, in float32: greedy tokens
    equal the plain model's, also when the pool is so small that requests wait for pages or are preempted (that preemption itself
    leaves the tokens alone is pinned on the CPU, where the pool's size is chosen so that it happens)."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=6)
    config, weights = read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 40], seed=7).values())
    steps = 12

    def plain_greedy(prompt):
        tokens = list(prompt)
        for _ in range(steps):
            tokens.append(int(tiverax_logits(config, weights, tokens)[-1].argmax()))
        return tokens[len(prompt):]

    want = [plain_greedy(p) for p in texts]
    for pages in (64, 7):
        engine = Engine.from_pretrained(EngineConfig(model=folder, dtype="float32", device="cuda", max_model_len=96, max_num_seqs=4, max_num_batched_tokens=32,
                                                     max_prefill_chunk_size=11, block_size=16, num_gpu_blocks=pages, enable_cuda_graphs=graphs, seed=0,
                                                     enable_prefix_caching=False), ops=ops)
        assert engine.runner.uses_graphs == graphs
        requests = [Request(f"r{i}", p, SamplingParams(temperature=0.0, max_tokens=steps, ignore_eos=True)) for i, p in enumerate(texts)]
        engine.generate(requests)
        assert [r.output_token_ids for r in requests] == want
        assert engine.cache.num_used_pages() == 0
        if graphs:
            assert engine.runner.num_graph_replays > 0


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
        got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)])
        want = tiverax_logits(config, weights, tokens)[[0, 16, 29]].numpy()
        np.testing.assert_allclose(got, want, **(dict(rtol=2e-4, atol=3e-5) if dtype == "float32" else dict(rtol=6e-2, atol=6e-2)))
