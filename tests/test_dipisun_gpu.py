"""Dipisun on the GPU: each new kernel against its plain reference; the attention mixer alone with one key made to
stand out far back, at page borders and at the edges of the bias table, in portions and in single decoded tokens,
also behind thousands of keys where the kernels split the keys; the whole model in float32 and bfloat16 through
replay (every way of cutting, pages and slots used again), in long decoding, in batches against each request alone,
through the entry point with captured decode steps, and through the replay program itself."""
import json
import math
import os
import subprocess

import numpy as np
import pytest
import torch

import replay_cases as rc
from dipisun_cases import CONFIGS, PAGE_SIZE, prompts, write_folder
from plain_dipisun import dipisun_forward, distance_bucket, read_folder
from torch_ops import TorchOps
from velox_amd import Engine, EngineConfig, Request, SamplingParams
from velox_amd.cache import CacheManager
from velox_amd.engine.batch import BatchBuilder, StepEntry, Workspace
from velox_amd.engine.replay import Replayer
from velox_amd.parts import make_part
from velox_amd.parts.base import OutputNormSink, ResidualCopy
from velox_amd.parts.normed_attention import bias_by_distance

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
@pytest.mark.parametrize("width", [64, 250, 7, 4096])
def test_sinusoid_added_to_the_embeddings(ops, width):
    positions = torch.tensor([0, 1, 5, 63, 64, 4097, 131071], dtype=torch.int32).cuda()
    freq = torch.tensor([10000.0 ** (-2.0 * i / width) for i in range((width + 1) // 2)], dtype=torch.float64).cuda()
    start = torch.randn(7, width).cuda()
    got = ops.add_sinusoid(start.clone(), positions, freq)
    angle = positions.double()[:, None] * freq[None, :]
    want = start.double()
    want[:, 0::2] += torch.sin(angle)[:, : (width + 1) // 2]
    want[:, 1::2] += torch.cos(angle)[:, : width // 2]
    torch.testing.assert_close(got.double(), want, rtol=0, atol=1e-6)  # (also at position 131,071: the angle is reduced in float64)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tokens,hidden", [(9, 72), (3, 321), (70, 2048), (2, 5000)])
def test_output_norm_and_the_copy_of_the_residual(ops, dtype, tokens, hidden):
    ref, dt = TorchOps(), DTYPES[dtype]
    weight = (1 + 0.1 * torch.randn(hidden)).cuda()
    residual = torch.randn(tokens, hidden).cuda()
    for delta in (torch.randn(tokens, hidden).mul(3.0).to(dt).cuda(), torch.randn(3, tokens, hidden).cuda()):
        mine, theirs = residual.clone(), residual.clone()
        got = ops.norm_add(mine, delta, weight, 1e-5, 0.7, dt)
        want = ref.norm_add(theirs, delta, weight, 1e-5, 0.7, dt)
        torch.testing.assert_close(mine, theirs, rtol=1e-5, atol=1e-5)
        assert got.dtype == dt and (got is mine) == (dtype == "float32")
        close(got, want, dtype, scale=0.5)
        assert dtype == "float32" or torch.equal(got, mine.to(dt))  # the copy is the residual rounded once
    for delta in (None, torch.randn(tokens, hidden).to(dt).cuda()):
        mine, theirs = residual.clone(), residual.clone()
        got, want = ops.add_cast(mine, delta, dt), ref.add_cast(theirs, delta, dt)
        assert torch.equal(mine, theirs) and torch.equal(got, want)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("heads,kv_heads,dim,vdim,whole,temp,blend", [(4, 2, 16, 8, False, None, False), (4, 1, 12, 20, True, (0.4, 8), True), (8, 4, 64, 48, False, None, True),
                                                                       (3, 3, 10, 6, True, (1.1, 1), False), (16, 4, 128, 128, True, (0.5, 256), True), (1, 1, 40, 72, False, (2.0, 3), True)])
def test_qk_norm_temperature_blend_and_cache_write(ops, dtype, heads, kv_heads, dim, vdim, whole, temp, blend):
    ref, dt = TorchOps(), DTYPES[dtype]
    tokens, page, pages = 37, 8, 12
    cached = (max(dim, vdim) + 15) // 16 * 16
    width = (heads + kv_heads) * dim + kv_heads * vdim
    qkv = torch.randn(tokens, width).mul(2.0).to(dt).cuda()
    q_norm = (1.5 + 0.3 * torch.randn(heads * dim if whole else dim)).cuda()
    k_norm = (1.5 + 0.3 * torch.randn(kv_heads * dim if whole else dim)).cuda()
    positions = torch.randint(0, 3000, (tokens,), dtype=torch.int32).cuda()
    slots = torch.randperm(page * pages)[:tokens].to(torch.int32).cuda()
    first = (torch.randn(tokens, 11 + kv_heads * vdim).to(dt).cuda(), 11) if blend else None
    lam = torch.tensor(0.37).cuda() if blend else None
    caches = [[torch.full((pages, kv_heads, page, cached), 7.0, dtype=dt).cuda(), torch.full((pages, kv_heads, cached, page), 7.0, dtype=dt).cuda()] for _ in range(2)]
    got = ops.qk_norm_write(qkv, heads, kv_heads, dim, vdim, cached, q_norm, k_norm, whole, 1e-5, temp, positions, first, lam, slots, caches[0][0], caches[0][1], page)
    want = ref.qk_norm_write(qkv, heads, kv_heads, dim, vdim, cached, q_norm, k_norm, whole, 1e-5, temp, positions, first, lam, slots, caches[1][0], caches[1][1], page)
    close(got, want, dtype, scale=4.0)
    assert float(got.view(tokens, heads, cached)[:, :, dim:].abs().max() if cached > dim else 0.0) == 0.0  # padding channels are zeros
    for mine, theirs in zip(caches[0], caches[1]):
        close(mine, theirs, dtype, scale=4.0)  # (slots that were not written still hold the 7s on both sides)
    again = ops.qk_norm_write(qkv, heads, kv_heads, dim, vdim, cached, q_norm, k_norm, whole, 1e-5, temp, positions, first, lam, slots, None, None, page, write_kv=False)
    assert torch.equal(again, got)


@pytest.mark.parametrize("score", ["softmax", "sigmoid"])
def test_router_choice_with_a_correction(ops, score):
    ref = TorchOps()
    for tokens, experts, top in ((50, 13, 3), (7, 5, 5), (300, 70, 4), (1, 2, 1)):
        logits = torch.randn(tokens, experts).mul(2.0).cuda()
        correction = torch.randn(experts).mul(0.3).cuda()
        choice, weight = ops.route_top(logits, top, score, False, correction=correction)
        want_choice, want_weight = ref.route_top(logits, top, score, False, correction=correction)
        assert torch.equal(choice.cpu(), want_choice.cpu())
        torch.testing.assert_close(weight, want_weight, rtol=1e-5, atol=1e-7)
        plain_choice, _ = ops.route_top(logits, top, score, False)
        assert tokens < 50 or not torch.equal(plain_choice, choice)  # the correction does change choices
        scores = torch.softmax(logits, -1) if score == "softmax" else torch.sigmoid(logits)
        torch.testing.assert_close(weight, scores.gather(-1, choice.long()), rtol=1e-5, atol=1e-7)  # weights are the scores without it


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("tokens,hidden,inter,experts,identity,top,limit", [(70, 64, 32, 4, 2, 3, 1.0), (9, 86, 22, 6, 1, 3, 0.5), (300, 96, 40, 8, 0, 2, 1.5), (1, 128, 64, 3, 3, 2, 2.0),
                                                                            (700, 192, 48, 10, 2, 3, 1.25), (16, 64, 8, 1, 1, 2, 0.75)])
def test_clamped_units_and_identity_experts_against_the_plain_loop(ops, dtype, tokens, hidden, inter, experts, identity, top, limit):
    ref, dt = TorchOps(), DTYPES[dtype]
    x = torch.randn(tokens, hidden).to(dt).cuda()
    gate_up = torch.randn(experts * 2 * inter, hidden).mul(2.0 / math.sqrt(hidden)).to(dt).cuda()
    down = torch.randn(experts * hidden, inter).div(math.sqrt(inter)).to(dt).cuda()
    logits = torch.randn(tokens, experts + identity).cuda()
    choice, weight = ref.route_top(logits, top, "softmax", False, correction=torch.randn(experts + identity).mul(0.2).cuda())
    assert identity == 0 or tokens < 9 or bool((choice >= experts).any())
    unit = (1.702, limit, 1.0)
    got = ops.routed_experts(x, choice, weight, gate_up, down, experts, False, None, dt, None, unit=unit, identity_experts=identity)
    want = ref.routed_experts(x, choice, weight, gate_up, down, experts, False, None, dt, None, unit=unit, identity_experts=identity)
    close(got, want, dtype, scale=0.5)
    # the same with the last kernel norming the sum and adding it to a residual
    norm_weight = (1 + 0.1 * torch.randn(hidden)).cuda()
    mine, theirs = torch.randn(tokens, hidden).cuda(), None
    theirs = mine.clone()
    fused = ops.routed_experts(x, choice, weight, gate_up, down, experts, False, None, dt, None, unit=unit, identity_experts=identity,
                               output_norm=OutputNormSink(mine, norm_weight, 1e-5, 0.7))
    plain = ref.routed_experts(x, choice, weight, gate_up, down, experts, False, None, dt, None, unit=unit, identity_experts=identity,
                               output_norm=OutputNormSink(theirs, norm_weight, 1e-5, 0.7))
    assert isinstance(fused, ResidualCopy) and fused.copy.dtype == dt and (fused.copy is mine) == (dtype == "float32")
    close(mine, theirs, dtype, scale=0.5)
    close(fused.copy, plain.copy, dtype, scale=0.5)
    unclamped = ref.routed_experts(x, choice, weight, gate_up, down, experts, False, None, dt, None, unit=(1.702, 1e9, 1.0), identity_experts=identity)
    assert tokens < 9 or float((unclamped.float() - want.float()).abs().max()) > 0.05  # the clamps are reached


def paged(keys, values, page, pages, dt, seed=0):
    """Keys [n, kv_heads, d] and values [n, kv_heads, d] of one sequence scattered over pages in a shuffled order."""
    n, kv_heads, d = keys.shape
    need = (n + page - 1) // page
    g = torch.Generator().manual_seed(seed)
    table = (torch.randperm(pages - 1, generator=g)[:need] + 1).to(torch.int32)
    k_cache = torch.zeros(pages, kv_heads, page, d, dtype=dt)
    v_cache = torch.zeros(pages, kv_heads, d, page, dtype=dt)
    index = torch.arange(n)
    k_cache[table.long()[index // page], :, index % page, :] = keys.to(dt)
    v_cache[table.long()[index // page], :, :, index % page] = values.to(dt)
    return k_cache.cuda(), v_cache.cuda(), table


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,d,buckets,far", [(4, 2, 48, 14, 200), (8, 2, 64, 8, 24), (3, 1, 32, 7, 33.5), (16, 4, 128, 32, 3000), (2, 2, 16, 2, 3), (32, 2, 64, 12, 100), (2, 1, 272, 10, 50)])
def test_attention_with_a_bias_by_distance(ops, dtype, nh, nkv, d, buckets, far):
    """Sequences of unequal length in one step: whole prompts, portions behind keys that earlier steps wrote, single tokens.
    (A head of 272 channels is beyond the tiled kernels: the plain kernel takes the bias too.)"""
    ref, dt = TorchOps(), DTYPES[dtype]
    page, pages = 16, 64
    bias = bias_by_distance(torch.randn(buckets, nh).mul(1.5), far).cuda()
    kv_lens, q_lens = [300, 1, 130, 77, 260], [1, 1, 130, 9, 30]
    k_cache = torch.randn(pages, nkv, page, d).to(dt).cuda()
    v_cache = torch.randn(pages, nkv, d, page).to(dt).cuda()
    tables = torch.zeros(5, 20, dtype=torch.int32)
    perm = torch.randperm(pages - 1) + 1
    tables[0, :19], tables[1, :1], tables[2, :9], tables[3, :5] = perm[:19], perm[19:20], perm[20:29], perm[29:34]
    tables[4, :17] = perm[34:51]
    cu = torch.tensor([0, 1, 2, 132, 141, 171], dtype=torch.int32).cuda()
    q = (torch.randn(171, nh * d) * 0.5).to(dt).cuda()
    args = (q, nh, nkv, d, k_cache, v_cache, page, tables.cuda(), cu, torch.tensor(kv_lens, dtype=torch.int32).cuda(), 130, 300, 1.0 / math.sqrt(d), None, False, None)
    got, want = ops.paged_attention(*args, decode_prefix=2, distance_bias=bias), ref.paged_attention(*args, distance_bias=bias)
    close(got, want, dtype)
    without = ref.paged_attention(*args)
    assert float((without.float() - want.float()).abs().max()) > 0.1  # the bias does matter
    # single tokens only: the streaming kernel
    lens = torch.tensor([300, 1, 130, 77, 260], dtype=torch.int32).cuda()
    cu1 = torch.arange(6, dtype=torch.int32).cuda()
    args = (q[:5].contiguous(), nh, nkv, d, k_cache, v_cache, page, tables.cuda(), cu1, lens, 1, 300, 1.0 / math.sqrt(d), None, True, Workspace(torch.device("cuda")))
    close(ops.paged_attention(*args, distance_bias=bias), ref.paged_attention(*args, distance_bias=bias), dtype)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("far_at,length,cuts", [(0, 150, (150,)), (3, 150, (100, 2, 47, 1)), (15, 140, (16, 123, 1)), (16, 140, (17, 120, 1, 1, 1)),
                                               (63, 200, (64, 64, 64, 8)), (64, 129, (65, 63, 1)), (0, 5000, (4990, 9, 1)), (4100, 6000, (4096, 1900, 2, 1, 1))])
def test_a_key_far_back_or_at_a_page_border_takes_the_attention(ops, dtype, far_at, length, cuts):
    """The key at ``far_at`` is made to line up with the LAST query, with a score far above all others although its
    bucket's bias is the lowest of the table: the last token's output is then that key's value.  Pages hold 16 tokens, so
    15, 16, 63 and 64 sit at page borders; behind thousands of keys the kernels split the keys over workgroups.  The
    sequence is cut so that the key is written by one step and read by a later one."""
    dt = DTYPES[dtype]
    nh, nkv, d, buckets, far = 4, 2, 48, 14, 200
    g = torch.Generator().manual_seed(far_at + length)
    rel = torch.randn(buckets, nh, generator=g)
    rel[distance_bucket(length - 1 - far_at, buckets, far)] = -3.0
    bias = bias_by_distance(rel, far)
    q = torch.randn(length, nh, d, generator=g).mul(0.3).to(dt).float()
    k = torch.randn(length, nkv, d, generator=g).mul(0.3).to(dt).float()
    v = torch.randn(length, nkv, d, generator=g).to(dt).float()
    k[far_at] = q[-1].view(nkv, nh // nkv, d)[:, 0] * 40.0  # what the first head of every group asks for at the end
    k[far_at] = k[far_at].to(dt).float()
    rows = [length - 1] + list(range(0, length, max(1, length // 40)))
    want = torch.zeros(len(rows), nh * d)
    for at, i in enumerate(rows):  # (row by row: a whole matrix of 6,000 x 6,000 biases per head is not needed)
        behind = (i - torch.arange(i + 1)).clamp(max=bias.shape[1] - 1)
        for h in range(nh):
            scores = (k[: i + 1, h // (nh // nkv)] @ q[i, h]) * 0.2 + bias[h][behind]
            want[at, h * d:(h + 1) * d] = torch.softmax(scores, 0) @ v[: i + 1, h // (nh // nkv)]
            if i == length - 1 and h % (nh // nkv) == 0:
                assert int(scores.argmax()) == far_at and float(torch.softmax(scores, 0)[far_at]) > 0.9
    page, pages = 16, (length + 15) // 16 + 2
    cache = CacheManager([make_part("mixer", "normed_attention", prefix="m.", hidden_size=64, num_heads=nh, num_kv_heads=nkv, dim=d, vdim=d, scale=0.2,
                                    norm_eps=1e-5, distance_bias=(buckets, far)).cache_need()], page, pages, 2, dt, "cuda")
    builder, workspace = BatchBuilder(cache, "cuda", 8192, 2), Workspace(torch.device("cuda"))
    seq, done, got = cache.new_sequence(), 0, []
    assert sum(cuts) == length
    for n in cuts:
        assert cache.append(seq, done, n)
        ctx = builder.build([StepEntry(seq, [0] * n, done)], ops, dt, workspace)
        view = ctx.cache_view(0)
        slots = view.batch.slot_mapping.long()
        view.tensors["k"][slots // page, :, slots % page, :] = k[done:done + n].to(dt).cuda()
        view.tensors["v"][slots // page, :, :, slots % page] = v[done:done + n].to(dt).cuda()
        out = ops.paged_attention(q[done:done + n].reshape(n, nh * d).to(dt).cuda(), nh, nkv, d, view.tensors["k"], view.tensors["v"], page, view.batch.block_tables,
                                  ctx.cu_q, view.batch.kv_lens, n, done + n, 0.2, None, n == 1, workspace, distance_bias=bias.cuda())
        got.append(out.float().cpu())
        done += n
    got = torch.cat(got)[rows]
    torch.testing.assert_close(got, want, **(dict(rtol=2e-4, atol=3e-5) if dtype == "float32" else dict(rtol=3e-2, atol=3e-2)))
    assert float((got[0].view(nh, d)[0] - v[far_at, 0]).abs().max()) < (0.2 if dtype == "float32" else 0.25)  # the far key's value, nearly alone


# ----------------------------------------------------------------------------------------------------
# the whole model
# ----------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", ["A", "B", "C", "D"])
def test_all_ways_of_cutting_on_the_gpu(tmp_path, name, dtype):
    folder = write_folder(tmp_path / name, CONFIGS[name], seed=2, dtype=dtype)
    config, weights = read_folder(folder)
    requests = prompts(config["vocab"], [141, 1, 37, 98, 2, 64, 75], seed=11)
    expected = {rid: dipisun_forward(config, weights, tokens, torch.float64).float() for rid, tokens in requests.items()}
    page = PAGE_SIZE[name]
    results = {}
    for label, trace in (("whole", rc.whole(requests)), ("tail", rc.tail_one_by_one(requests)), ("portions", rc.changing_portions(requests)),
                         ("mixed", rc.mixed(requests, seed=5)), ("recompute", rc.mixed(requests, seed=8, preempt=("r0", "r3", "r6")))):
        replayer = Replayer(folder, dtype, rc.tokens_needed(trace, page), block_size=page, max_live=4)
        outputs = rc.run_trace(replayer, trace)
        results[label] = rc.collect(trace, outputs, requests)
        for rid in requests:
            got, want = results[label][rid], expected[rid]
            size = float(want.abs().max())
            if dtype == "float32":
                torch.testing.assert_close(got, want, msg=lambda m: f"{name} {label} {rid}: {m}", rtol=2e-4, atol=3e-5 * size)
            else:
                # bfloat16: rounding may send a token to another expert where two scores are close (the tests' routers and
                # corrections are sharp, so that float32 shows every fault; bfloat16 then flips some choices): most rows are
                # close, the typical row is very close
                err = (got - want).abs().amax(-1) / want.abs().amax(-1).clamp(min=1.0)
                assert float((err < 0.08).float().mean()) >= 0.8 and (len(err) < 8 or float(err.median()) < 0.04), f"{name} {label} {rid}: {err}"
        if label in ("mixed", "recompute"):
            assert sum((len(t) + page - 1) // page for t in requests.values()) > replayer.cache.num_total_pages
    if dtype == "float32":
        for label in ("tail", "portions", "mixed", "recompute"):  # the ways of cutting agree with each other at least as closely
            for rid in requests:
                torch.testing.assert_close(results[label][rid], results["whole"][rid], rtol=1e-4, atol=3e-5 * float(expected[rid].abs().max()))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_long_decoding_and_a_batch_against_each_request_alone(tmp_path, dtype):
    """A prompt of a few tokens, then 200 tokens one by one across many page borders, the edge of the bias table and several
    steps of the temperature; then four requests of unequal length decoded together, whose logits equal those of each
    request decoded alone."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=4, dtype=dtype)
    config, weights = read_folder(folder)
    tokens = prompts(config["vocab"], [205], seed=12)["r0"]
    want = dipisun_forward(config, weights, tokens, torch.float64).float()
    replayer = Replayer(folder, dtype, 4 * 224, block_size=16, max_live=4)
    rows = [replayer.step({"step": 0, "entries": [{"id": "x", "tokens": tokens[:5], "want": [0, 4]}], "end": []})]
    for i in range(5, 205):
        rows.append(replayer.step({"step": i, "entries": [{"id": "x", "tokens": [tokens[i]], "want": [0]}], "end": ["x"] if i == 204 else []}))
    got = torch.from_numpy(np.concatenate(rows))
    if dtype == "float32":
        torch.testing.assert_close(got, want[[0] + list(range(4, 205))], rtol=2e-4, atol=3e-5 * float(want.abs().max()))
    else:
        err = (got - want[[0] + list(range(4, 205))]).abs().amax(-1) / want.abs().amax()
        assert float((err < 0.08).float().mean()) >= 0.8 and float(err.median()) < 0.04
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
            np.testing.assert_allclose(row, alone[rid][k][0], rtol=1e-4 if dtype == "float32" else 3e-2, atol=1e-4 if dtype == "float32" else 5e-2)


@pytest.mark.parametrize("graphs", [False, True])
def test_greedy_generation_through_the_entry_point(tmp_path, ops, graphs):
    """Scheduler, step function, captured decode steps (``graphs``) and sampler around the model, in float32: greedy tokens
    equal the plain model's, also when the pool is so small that requests wait for pages or are preempted."""
    folder = write_folder(tmp_path / "C", CONFIGS["C"], seed=6)
    config, weights = read_folder(folder)
    texts = list(prompts(config["vocab"], [5, 19, 13, 40], seed=7).values())
    steps = 12

    def plain_greedy(prompt):
        tokens = list(prompt)
        for _ in range(steps):
            tokens.append(int(dipisun_forward(config, weights, tokens)[-1].argmax()))
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
        got = np.concatenate([np.fromfile(out / "0.f32", dtype="<f4").reshape(2, -1), np.fromfile(out / "2.f32", dtype="<f4").reshape(1, -1)])
        want = dipisun_forward(config, weights, tokens, torch.float64)[[0, 16, 29]].float().numpy()
        size = float(np.abs(want).max())
        np.testing.assert_allclose(got, want, **(dict(rtol=2e-4, atol=3e-5 * size) if dtype == "float32" else dict(rtol=6e-2, atol=6e-2 * size)))
