"""The Kodisun architecture through the engine against tests/plain_kodisun.py: each mechanism
alone, whole prompts against token-by-token decoding, portions down to two tokens, mixed batches
with pages that are used again, windows' edges, and greedy generation through the engine. The
configurations are made here; their sizes differ from layer to layer and avoid values that hide a
fault (equal key and value sizes, a rotation over the whole rotated part, one pass)."""

import copy
import json
import math
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import plain_kodisun as plain
from helpers import max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions, trace_tail_decoded, trace_whole
from qwen3_from_scratch_amd.config import load_model_config
from qwen3_from_scratch_amd.config.kodisun_config import KodisunConfig
from qwen3_from_scratch_amd.config.model_config import ConfigError
from qwen3_from_scratch_amd.engine import StepEntry, SyncEngine, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _mixer(heads, dim, rot_dim, vdim, q_rank, kv_rank, window, dims=None, base=10000.0, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "scale": 1.0 / math.sqrt(dim + rot_dim), "rot": {"dims": dims or rot_dim, "base": base}}
    if window:
        m["mask"] = {"size": window}
    if scaling:
        m["rot"]["scaling"] = scaling
    return m


def _mlp(experts, top, ff, shared):
    f = {"kind": "moe", "router": {"experts": experts, "top": top}, "expert": {"ff": ff}}
    if shared:
        f["shared"] = {"ff": shared}
    return f


YARN = {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}
# layers of different sizes, one before the loop and one behind it, three passes, a layer without
# a window, a layer without a feed-forward, one without a shared expert, a rotation over part of
# the rotated numbers, and one expert per token in one layer
LOOPED = {
    "architecture": "Kodisun", "vocab": 131, "width": 48, "norm": {"eps": 1e-5},
    "loop": {"start": 1, "stop": 3, "times": 3},
    "layers": [
        {"type": "latent_attention", "mixer": _mixer(3, 16, 8, 24, 20, 40, 19, scaling=YARN), "mlp": _mlp(5, 2, 24, 40)},
        {"type": "latent_attention", "mixer": _mixer(5, 8, 12, 16, 28, 24, 0, dims=8, base=500.0), "mlp": _mlp(6, 1, 36, 0)},
        {"type": "latent_attention", "mixer": _mixer(2, 24, 4, 8, 12, 36, 33, scaling=YARN), "mlp": None},
        {"type": "latent_attention", "mixer": _mixer(4, 12, 16, 20, 32, 28, 7), "mlp": _mlp(4, 4, 20, 16)},
    ]}
# no loop at all; a window of one token (a query sees itself only) beside a window that is never full
PLAIN = {
    "architecture": "Kodisun", "vocab": 97, "width": 64, "norm": {"eps": 1e-6},
    "layers": [
        {"type": "latent_attention", "mixer": _mixer(2, 32, 32, 48, 24, 64, 1), "mlp": _mlp(7, 3, 32, 48)},
        {"type": "latent_attention", "mixer": _mixer(6, 16, 16, 32, 40, 48, 500, scaling=YARN), "mlp": _mlp(3, 2, 64, 32)},
    ]}
# sizes in steps that the matrix-core kernels take, the loop from the first layer on
WIDE = {
    "architecture": "Kodisun", "vocab": 257, "width": 128, "norm": {"eps": 1e-5},
    "loop": {"start": 0, "stop": 2, "times": 2},
    "layers": [
        {"type": "latent_attention", "mixer": _mixer(4, 32, 32, 64, 64, 96, 45, scaling=YARN), "mlp": _mlp(8, 2, 64, 96)},
        {"type": "latent_attention", "mixer": _mixer(8, 64, 32, 32, 96, 128, 70), "mlp": _mlp(4, 3, 128, 64)},
        {"type": "latent_attention", "mixer": _mixer(4, 32, 64, 64, 32, 64, 0), "mlp": None},
    ]}
# sizes that no vector access and no matrix instruction takes: everything goes through the general kernels;
# one head, one expert, a loop of one pass over the only two layers
ODD = {
    "architecture": "Kodisun", "vocab": 53, "width": 40, "norm": {"eps": 1e-5},
    "loop": {"start": 0, "stop": 2, "times": 1},
    "layers": [
        {"type": "latent_attention", "mixer": _mixer(3, 10, 6, 14, 12, 20, 5, dims=4), "mlp": _mlp(3, 2, 18, 10)},
        {"type": "latent_attention", "mixer": _mixer(1, 6, 2, 3, 5, 7, 0), "mlp": _mlp(1, 1, 9, 0)},
    ]}
CONFIGS = {"looped": LOOPED, "plain": PLAIN, "wide": WIDE, "odd": ODD}


def _write(folder, data, seed=5, std=0.2, peak=None):
    write_random_model(str(folder), KodisunConfig.from_dict(data), seed=seed, std=std, norm_jitter=0.3)
    if peak:                              # larger query latents: every softmax then stands on a few keys
        path = os.path.join(str(folder), "model.safetensors")
        tensors = load_file(path)
        for key in tensors:
            if key.endswith("dq.norm"):
                tensors[key] = (tensors[key].float() * peak).to(tensors[key].dtype)
        save_file(tensors, path, metadata={"format": "pt"})
    return str(folder)


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folder(request, tmp_path_factory):
    return _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], peak=3.0)


def _every_expert(data):
    """The configuration with every expert chosen for every token. In bfloat16 a router's score
    moves by a few thousandths, and with random weights some token in a hundred then changes an
    expert, which no bound on rounding covers; the choice itself is float32 in both precisions and
    is tested there and on the router kernel. With all experts chosen the weights still matter."""
    data = copy.deepcopy(data)
    for layer in data["layers"]:
        if layer["mlp"]:
            layer["mlp"]["router"]["top"] = layer["mlp"]["router"]["experts"]
    return data


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folders(request, tmp_path_factory):
    """{dtype: folder}: the configuration as it is for float32, with every expert chosen for bfloat16."""
    return {"float32": _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], peak=3.0),
            "bfloat16": _write(tmp_path_factory.mktemp(request.param + "_all"), _every_expert(CONFIGS[request.param]))}


def _truth(folder, requests, dtype=torch.float64):
    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    w = {k: v.to(dtype) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}
    return config, w, {rid: plain.logits_of_sequence(config, w, toks) for rid, toks in requests.items()}


def _requests(folder, lengths=(70, 9, 41, 130, 25, 2, 1)):
    vocab = load_model_config(folder).vocab
    return {"k%d" % i: random_tokens(n, vocab, 160 + i) for i, n in enumerate(lengths)}


def _off(got, want, dtype):
    """The worst row: its difference (mean taken off, root mean square) over the spread of the
    true row, in units of what the dtype may be off by. With these weights (no peaked queries in
    bfloat16) the rounding of bfloat16 alone, at the places where the engine rounds, comes to a
    third of its unit; float32 to a fifth of its own."""
    worst = 0.0
    for rid, logits in want.items():
        for p in range(logits.shape[0]):
            d = got[(rid, p)].double() - logits[p].double()
            err = float((d - d.mean()).pow(2).mean().sqrt() / logits[p].double().std())
            worst = max(worst, err / (5e-5 if dtype == "float32" else 5e-2))
    return worst


# ---- configuration and weights ----

def test_config_is_read_by_its_own_keys_and_written_back(folder):
    config = load_model_config(folder)
    assert isinstance(config, KodisunConfig) and config.architecture == "Kodisun"
    with open(os.path.join(folder, "config.json")) as fh:
        raw = json.load(fh)
    assert config.to_dict() == raw and len(config.layers) == len(raw["layers"])
    for layer, entry in zip(config.layers, raw["layers"]):
        assert layer.mixer.window == (entry["mixer"].get("mask") or {}).get("size", 0)
        assert (layer.mlp is None) == (entry["mlp"] is None)
    names = set(load_file(os.path.join(folder, "model.safetensors")))
    assert {"embed", "head", "final.norm", "l0.norm1", "l0.norm1b", "l0.mix.dq.norm", "l0.mix.uk"} <= names
    assert ("loop.step" in names) == ("loop" in raw)
    for i, entry in enumerate(raw["layers"]):
        assert ("l%d.norm2b" % i in names) == (entry["mlp"] is not None)
        assert ("l%d.mlp.shared.up" % i in names) == bool(entry["mlp"] and entry["mlp"].get("shared"))


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="other"), "type"),
    (lambda c: c["layers"][0]["mixer"].pop("kv_rank"), "kv_rank"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=99), "top"),
    (lambda c: c.update(loop={"start": 2, "stop": 9, "times": 2}), "loop"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "even"),
    (lambda c: c.pop("width"), "width"),
])
def test_config_errors_name_the_key(change, word):
    data = copy.deepcopy(LOOPED)
    change(data)
    with pytest.raises(ConfigError, match=word):
        KodisunConfig.from_dict(data)


def test_run_order_and_cache_planes(cpu_ops, tmp_path):
    """The loop's layers appear once per pass, each appearance with a cache plane of its own;
    planes of equal needs share a group, a window makes a group of its own."""
    folder = _write(tmp_path / "m", LOOPED)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=256, max_requests=4)
    order = [(s.layer, s.enters) for s in runner.model.spec.order]
    assert order == [(0, None), (1, 0), (2, None), (1, 1), (2, None), (1, 2), (2, None), (3, None)]
    assert [(s.layer, s.enters) for s in runner.model.spec.order] == [
        (i, t) for i, t in plain.run_order(LOOPED)]
    assert len(runner.model.plane_needs) == 8 and len(set(runner.model.plane_of_step)) == 8
    groups = {(g.tensors[0].shape, g.window): len(g.planes) for g in runner.manager.groups}
    assert groups == {((48,), 19): 1, ((36,), 0): 3, ((40,), 33): 3, ((44,), 7): 1}


# ---- each mechanism alone, on the host twins and against the plain functions ----

def test_rotation_frequencies_with_and_without_blending():
    from qwen3_from_scratch_amd.parts.position import RotaryPairs
    from qwen3_from_scratch_amd.parts.base import Precision

    for rot in ({"dims": 12, "base": 500.0}, {"dims": 24, "base": 30000.0, "scaling": YARN},
                {"dims": 8, "base": 10000.0, "scaling": {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}}):
        scaling = rot.get("scaling")
        part = RotaryPairs("", Precision(torch.float32), "cpu", rot["dims"], rot["base"],
                           tuple(scaling[k] for k in ("factor", "original", "fast", "slow")) if scaling else None)
        part.load(None)
        freqs, factor = plain.rotation_frequencies(rot)
        assert torch.allclose(part.frequencies()[0].double(), torch.tensor(freqs, dtype=torch.float64), rtol=1e-7)
        assert abs(part.frequencies()[1] - factor) < 1e-12
    # the blend really changes the slow pairs and leaves the fastest alone
    blended, factor = plain.rotation_frequencies({"dims": 24, "base": 30000.0, "scaling": YARN})
    straight, _ = plain.rotation_frequencies({"dims": 24, "base": 30000.0})
    assert blended[0] == straight[0] and abs(blended[-1] - straight[-1] / 4.0) < 1e-15 and factor > 1.0


def test_router_twin_and_plain_agree(cpu_ops):
    g = torch.Generator().manual_seed(1)
    h, router = torch.randn(50, 24, generator=g), torch.randn(7, 24, generator=g)
    chosen, weights = cpu_ops.moe_route(h, router, 3)
    s = torch.softmax(h.double() @ router.double().T, dim=-1)
    best, at = torch.topk(s, 3, dim=-1)
    assert torch.equal(chosen.long(), at) and torch.allclose(weights.double(), best / best.sum(-1, keepdim=True), atol=1e-6)


def test_logits_on_the_host_under_every_cutting(cpu_ops, folder):
    requests = _requests(folder)
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype="float32", device="cpu", page_size=8,
                             max_tokens=max_live_tokens(steps, page=8), max_requests=4)
        assert _off(run_trace(runner, steps), want, "float32") <= 1.0, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


def test_layer_streams_on_the_host(cpu_ops, tmp_path):
    """The residual stream behind every run of a layer, what it still lacks included."""
    folder = _write(tmp_path / "m", LOOPED)
    tokens = random_tokens(37, LOOPED["vocab"], 4)
    config, w, _ = _truth(folder, {})
    streams = []
    plain.logits_of_sequence(config, w, tokens, streams)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=64, max_requests=1)
    seen = []

    def observe(i, x, pending):
        d = pending.values.double()
        d = d / torch.sqrt((d * d).mean(-1, keepdim=True) + pending.eps) * pending.weight.double()
        seen.append(x.double() + d)

    runner.model.observer = observe
    runner.step([StepEntry("r", tokens, [])])
    assert len(seen) == len(streams) == 8
    for got, want in zip(seen, streams):
        assert float((got - want).abs().max()) <= 2e-5 * float(want.abs().max())


def test_greedy_generation_through_the_engine_on_the_host(cpu_ops, folder):
    requests = _requests(folder)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=256, block_size=8, num_blocks=60,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [toks[:n] for toks, n in zip(requests.values(), (30, 9, 41, 2))]
    got = engine.generate_ids(prompts, max_new_tokens=5, temperature=0.0, ignore_eos=True)
    for prompt, new in zip(prompts, got):
        seq = list(prompt)
        for _ in range(5):
            seq.append(int(torch.argmax(plain.logits_of_sequence(config, w, seq)[-1])))
        assert new == seq[len(prompt):]
    assert engine.runner.manager.num_free() == 60


# ---- kernels against their twins ----

def _both(fn_name, *args, **kwargs):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    return getattr(ops, fn_name)(*args, **kwargs), getattr(torch_ops, fn_name)(*args, **kwargs)


def _rand(shape, seed, dtype, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(shape, generator=g) * scale).to(dtype).cuda()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H", [(5, 48), (130, 260), (3, 1031)])
def test_addend_norm_kernel(dtype, T, H):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    w, dw = _rand((H,), 1, torch.bfloat16) + 1, _rand((H,), 2, torch.bfloat16) + 1
    delta, bias = _rand((T, H), 3, dtype, 3.0), _rand((H,), 4, torch.float32)
    rows = torch.tensor([T - 1, 0], dtype=torch.int32).cuda()
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for kw in (dict(delta=delta, delta_weight=dw, delta_eps=1e-5, bias=bias), dict(delta=delta, delta_weight=dw),
               dict(bias=bias), dict(delta=delta), dict(delta=delta, delta_weight=dw, delta_eps=1e-6, rows=rows)):
        x1 = _rand((T, H), 5, torch.float32, 2.0)
        x2 = x1.clone()
        a = ops.rmsnorm_addend(x1, w, 1e-5, dtype, **kw)
        b = torch_ops.rmsnorm_addend(x2, w, 1e-5, dtype, **kw)
        assert torch.allclose(x1, x2, atol=1e-5, rtol=1e-5) and float((a.float() - b.float()).abs().max()) <= tol * 4
        if "rows" in kw:
            assert torch.equal(x1, _rand((T, H), 5, torch.float32, 2.0))      # a selection leaves the stream alone
    x1 = _rand((T, H), 5, torch.float32)
    x2 = x1.clone()
    assert ops.rmsnorm_addend(x1, None, 0.0, dtype, delta=delta, delta_weight=dw, delta_eps=1e-5) is None
    torch_ops.rmsnorm_addend(x2, None, 0.0, dtype, delta=delta, delta_weight=dw, delta_eps=1e-5)
    assert torch.allclose(x1, x2, atol=1e-5, rtol=1e-5)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gelu_kernel(dtype):
    x = _rand((37, 53), 1, dtype, 3.0)
    for kind in ("erf", "tanh"):
        a, b = _both("gelu", x, kind)
        assert float((a.float() - b.float()).abs().max()) <= (1e-6 if dtype == torch.float32 else 2e-2)
    z = torch.tensor([1.0])
    assert abs(float(_both("gelu", z.cuda(), "erf")[0]) - 0.8413447) < 1e-6
    assert abs(float(_both("gelu", z.cuda(), "tanh")[0]) - 0.8411920) < 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("q_rank,kv_rank,rot_dim,pairs", [(20, 40, 8, 4), (80, 144, 24, 12), (33, 7, 10, 3)])
def test_latent_prepare_kernel(dtype, q_rank, kv_rank, rot_dim, pairs):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    T, page = 45, 8
    down = _rand((T, q_rank + kv_rank + rot_dim), 1, dtype, 2.0)
    qw, kw = _rand((q_rank,), 2, torch.bfloat16) + 1, _rand((kv_rank,), 3, torch.bfloat16) + 1
    inv_freq = (torch.rand(pairs, generator=torch.Generator().manual_seed(4)) + 0.01).cuda()
    # two sequences; the second starts far out, where a float32 angle has few digits left
    positions = torch.cat((torch.arange(30), torch.arange(100000, 100015))).int().cuda()
    seq = torch.cat((torch.zeros(30), torch.ones(15))).int().cuda()
    table = torch.full((2, 100015 // page + 3), -1, dtype=torch.int32)
    table[0, :4] = torch.tensor([5, 2, 7, 0])
    table[1, 100000 // page:100000 // page + 3] = torch.tensor([1, 6, 3])
    table[0, 1] = -1                                   # a page given back: its tokens are skipped
    table = table.cuda()
    c1 = torch.zeros((9, page, kv_rank + rot_dim), dtype=dtype).cuda()
    c2 = c1.clone()
    a = ops.latent_prepare(down, q_rank, kv_rank, rot_dim, qw, kw, 1e-5, inv_freq, 1.07, positions, seq, table, c1)
    b = torch_ops.latent_prepare(down, q_rank, kv_rank, rot_dim, qw, kw, 1e-5, inv_freq, 1.07, positions, seq, table, c2)
    tol = 2e-5 if dtype == torch.float32 else 4e-2
    assert float((a.float() - b.float()).abs().max()) <= tol * 4
    # the far positions' angles: float32 cos and sin of a float32 product, as the twin forms them
    assert float((c1.float() - c2.float()).abs().max()) <= tol * 8
    assert float(c1[8].abs().max()) == 0 and float(c1[2].abs().max()) == 0     # untouched pages
    assert ops.latent_prepare(down, q_rank, kv_rank, rot_dim, qw, kw, 1e-5, inv_freq, 1.0, positions, seq).shape == (T, q_rank)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,H,I,O", [(1, 3, 16, 40), (37, 5, 8, 24), (130, 2, 128, 300), (4, 16, 64, 512), (70, 3, 96, 20),
                                     (200, 2, 512, 128)])
def test_headwise_linear_kernel(dtype, T, H, I, O):
    from qwen3_from_scratch_amd import ops

    wide = _rand((T, H, I + 8), 1, dtype)          # rows that start at multiples of 16 bytes, as the model's do
    w = _rand((H, O, I), 2, dtype, I ** -0.5)
    out = torch.zeros((T, H, O + 3), dtype=dtype).cuda()
    ops.headwise_linear(wide[:, :, :I], w, out=out[:, :, :O])          # both seen through strides
    want = torch.einsum("thi,hoi->tho", wide[:, :, :I].double(), w.double())
    assert float((out[:, :, :O].double() - want).abs().max()) <= (1e-5 if dtype == torch.float32 else 3e-2)
    assert float(out[:, :, O:].abs().max()) == 0
    assert torch.equal(ops.headwise_linear(wide[:, :, :I].contiguous(), w), out[:, :, :O])
    odd = _rand((T, H, I + 3), 1, dtype)            # and rows that do not: the multiply-add kernel
    got = ops.headwise_linear(odd[:, :, 3:], w)
    want = torch.einsum("thi,hoi->tho", odd[:, :, 3:].double(), w.double())
    assert float((got.double() - want).abs().max()) <= (1e-5 if dtype == torch.float32 else 3e-2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rotate_heads_kernel(dtype):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    T, H, n = 33, 5, 12
    x = _rand((T, H, 20), 1, dtype)
    positions = (torch.arange(T) * 977).int().cuda()
    for pairs in (6, 4, 0):
        inv_freq = (torch.rand(pairs, generator=torch.Generator().manual_seed(2)) + 0.01).cuda()
        a = torch.zeros((T, H, n), dtype=dtype).cuda()
        b = a.clone()
        ops.rotate_heads(x[:, :, 8:], a, inv_freq, 1.1, positions)
        torch_ops.rotate_heads(x[:, :, 8:], b, inv_freq, 1.1, positions)
        assert float((a.float() - b.float()).abs().max()) <= (2e-5 if dtype == torch.float32 else 2e-2)
        if pairs < 6:
            assert torch.equal(a[:, :, 2 * pairs:], x[:, :, 8 + 2 * pairs:])


def _paged(rows_per_seq, page, Dk, dtype, seed):
    """Sequences' cached rows scattered over pages in a shuffled order; returns cache, table, rows."""
    blocks = [-(-n // page) for n in rows_per_seq]
    order = torch.randperm(sum(blocks) + 3, generator=torch.Generator().manual_seed(seed)).tolist()
    cache = torch.zeros((sum(blocks) + 3, page, Dk), dtype=dtype)
    table = torch.full((len(rows_per_seq), max(blocks)), -1, dtype=torch.int32)
    rows = []
    for b, n in enumerate(rows_per_seq):
        r = (torch.randn((n, Dk), generator=torch.Generator().manual_seed(seed + 1 + b))).to(dtype)
        rows.append(r)
        for j in range(blocks[b]):
            pg = order.pop()
            table[b, j] = pg
            part = r[j * page:(j + 1) * page]
            cache[pg, :part.shape[0]] = part
    return cache.cuda(), table.cuda(), rows


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("general", [False, True])
@pytest.mark.parametrize("H,Dk,Dv,page,window", [(3, 48, 40, 8, 19), (5, 160, 112, 16, 37), (5, 36, 24, 16, 0),
                                                 (16, 96, 64, 32, 70), (2, 200, 136, 8, 1), (4, 576, 512, 16, 100),
                                                 (8, 288, 256, 16, 0), (7, 64, 16, 8, 33)])
def test_latent_attention_kernel(dtype, H, Dk, Dv, page, window, general):
    """Prompts' portions beside single tokens, over scattered pages, against the twin; then
    queries made so that one key carries the whole softmax, that key just inside and just
    outside the window, at a page's first and last place, and far back without a window."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    kv = [150, 33, 1, 257, 64]
    q_lens = [37, 1, 1, 2, 64]
    cache, table, rows = _paged(kv, page, Dk, dtype, 11)
    cu = torch.tensor([0] + list(np.cumsum(q_lens)), dtype=torch.int32).cuda()
    kvl = torch.tensor(kv, dtype=torch.int32).cuda()
    q = _rand((sum(q_lens), H, Dk), 3, dtype, 1.5)
    scale = Dk ** -0.5
    if general and not (dtype == torch.bfloat16 and Dk % 32 == 0 and Dv % 16 == 0):
        pytest.skip("these sizes take the general kernel anyway")
    a = ops.latent_attention(q, cache, Dv, table, cu, kvl, max(q_lens), scale, window=window, general=general,
                             max_kv_len=max(kv))
    b = torch_ops.latent_attention(q, cache, Dv, table, cu, kvl, max(q_lens), scale, window=window)
    assert a.shape == (sum(q_lens), H, Dv)
    assert float((a.float() - b.float()).abs().max()) <= (2e-5 if dtype == torch.float32 else 3e-2)
    # one key stands out: the query is that key's row, scaled up
    seq, L = 3, kv[3]
    for back in sorted({0, 1, page - 1, page, window - 1, window, window + 1, L - 1} - {-1}):
        if back >= L:
            continue
        target = L - 1 - back
        peaked = q.clone()
        at = int(cu[seq]) + 1                           # the sequence's last token
        peaked[at] = (rows[seq][target] * 8.0).to(dtype).cuda()[None, :]
        got = ops.latent_attention(peaked, cache, Dv, table, cu, kvl, max(q_lens), 1.0, window=window,
                                   general=general)[at].float()
        visible = window == 0 or back < window
        want = rows[seq][target, :Dv].float().cuda()
        close = float((got - want[None, :]).abs().max()) <= 0.05
        assert close == visible, (back, visible)


@pytest.mark.gpu
@pytest.mark.parametrize("H,Dk,Dv,window", [(5, 160, 112, 0), (5, 160, 112, 300), (16, 576, 512, 700), (3, 64, 48, 0)])
def test_latent_attention_of_single_tokens_over_many_keys(H, Dk, Dv, window):
    """Steps of one token a sequence: the keys go over several blocks whose shares are merged; one
    sequence is a token long, one ends just behind a tile's edge."""
    import torch_ops
    from qwen3_from_scratch_amd import ops

    kv = [1000, 1, 513, 37, 2048]
    cache, table, rows = _paged(kv, 16, Dk, torch.bfloat16, 5)
    cu = torch.arange(len(kv) + 1, dtype=torch.int32).cuda()
    kvl = torch.tensor(kv, dtype=torch.int32).cuda()
    q = _rand((len(kv), H, Dk), 3, torch.bfloat16, 1.5)
    a = ops.latent_attention(q, cache, Dv, table, cu, kvl, 1, Dk ** -0.5, window=window, max_kv_len=max(kv))
    b = torch_ops.latent_attention(q, cache, Dv, table, cu, kvl, 1, Dk ** -0.5, window=window)
    assert ops._latent_splits(len(kv), len(kv), H, 1, max(kv), window) > 1
    assert float((a.float() - b.float()).abs().max()) <= 3e-2
    for back in (0, 31, 32, 500, window - 1, window, 2047):
        if back < 0:
            continue
        peaked = q.clone()
        peaked[4] = (rows[4][2047 - back] * 8.0).to(torch.bfloat16).cuda()[None, :]
        got = ops.latent_attention(peaked, cache, Dv, table, cu, kvl, 1, 1.0, window=window, max_kv_len=max(kv))[4].float()
        close = float((got - rows[4][2047 - back, :Dv].float().cuda()[None, :]).abs().max()) <= 0.05
        assert close == (window == 0 or back < window), back


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,width,E,top", [(1, 64, 9, 4), (77, 48, 5, 5), (300, 192, 70, 6), (9, 33, 3, 1)])
def test_router_kernel(dtype, T, width, E, top):
    h, router = _rand((T, width), 1, dtype), _rand((E, width), 2, dtype, 0.5)
    (chosen, weights), (chosen_t, weights_t) = _both("moe_route", h, router, top)
    s = torch.softmax(h.double() @ router.double().T, dim=-1)
    picked = torch.gather(s, 1, chosen.long())
    # the chosen ones are the largest, in falling order, each once
    assert bool((picked[:, :-1] >= picked[:, 1:] - 1e-6).all()) if top > 1 else True
    assert all(len(set(row)) == top for row in chosen.tolist())
    rest = s.clone().scatter_(1, chosen.long(), -1.0)
    assert bool((rest.max(dim=1).values <= picked[:, -1] + 1e-6).all())
    assert torch.allclose(weights.double(), picked / picked.sum(-1, keepdim=True), atol=2e-6)
    assert abs(float(weights.sum(-1).mean()) - 1.0) < 1e-5


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("T,width,ff,E,top,shared", [(1, 64, 32, 7, 3, True), (50, 48, 24, 5, 2, False),
                                                      (333, 128, 96, 6, 3, True), (17, 40, 20, 4, 4, True),
                                                      (5, 256, 64, 64, 1, False), (700, 96, 160, 3, 2, True),
                                                      (900, 64, 96, 2, 2, False), (800, 128, 192, 4, 2, True),
                                                      (300, 64, 64, 2, 2, False), (1000, 192, 320, 5, 3, True)])
def test_experts_kernels(dtype, T, width, ff, E, top, shared):
    import torch_ops
    from qwen3_from_scratch_amd import ops

    h = _rand((T, width), 1, dtype)
    up, down = _rand((E, ff, width), 2, dtype, width ** -0.5), _rand((E, width, ff), 3, dtype, ff ** -0.5)
    chosen, weights = torch_ops.moe_route(h, _rand((E, width), 4, dtype), top)
    if T > 20:
        chosen[:, 0] = 1                                # one expert takes a row of every token, others few or none
    extra = _rand((T, width), 5, dtype) if shared else None
    for act in ("erf", "tanh"):
        a = ops.moe_experts(h, chosen, weights, up, down, shared=extra, activation=act)
        b = torch_ops.moe_experts(h, chosen, weights, up, down, shared=extra, activation=act)
        assert float((a.float() - b.float()).abs().max()) <= (2e-5 if dtype == torch.float32 else 4e-2)
    again = ops.moe_experts(h, chosen, weights, up, down, shared=extra)
    assert torch.equal(again, ops.moe_experts(h, chosen, weights, up, down, shared=extra))   # whatever slots rows got


# ---- the model on the GPU ----

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_logits_under_every_cutting(folders, dtype):
    folder = folders[dtype]
    requests = _requests(folder, lengths=(70, 9, 141, 330, 25, 2, 1))
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16,
                             max_tokens=max_live_tokens(steps, page=16), max_requests=4)
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


@pytest.mark.gpu
def test_long_decoding_and_first_tokens(folders):
    """A request decoded token by token from its second token on, through graph replays, page
    ends and every window's edge, beside a request that is decoded from its very first."""
    for dtype in ("float32", "bfloat16"):
        folder = folders[dtype]
        vocab = load_model_config(folder).vocab
        requests = {"long": random_tokens(200, vocab, 7), "short": random_tokens(3, vocab, 8)}
        _, _, want = _truth(folder, requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=256, max_requests=2)
        steps = [([(rid, toks[:1], [0]) for rid, toks in requests.items()], [])]
        for i in range(1, 200):
            entries = [(rid, [toks[i]], [0]) for rid, toks in requests.items() if i < len(toks)]
            steps.append((entries, [rid for rid, toks in requests.items() if i == len(toks) - 1]))
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0


@pytest.mark.gpu
def test_greedy_generation_through_the_engine(folders):
    for dtype in ("float32", "bfloat16"):
        folder = folders[dtype]
        requests = _requests(folder)
        config, w, _ = _truth(folder, {})
        engine = SyncEngine(path=folder, dtype=dtype, device="cuda", max_len=256, block_size=16, num_blocks=30,
                            max_num_seqs=3, max_num_tokens=48, chunked_prefill_size=32)
        prompts = [toks[:n] for toks, n in zip(requests.values(), (60, 9, 41, 2))]
        got = engine.generate_ids(prompts, max_new_tokens=8, temperature=0.0, ignore_eos=True)
        for prompt, new in zip(prompts, got):
            logits = plain.logits_of_sequence(config, w, prompt + new)
            for i, token in enumerate(new):
                row = logits[len(prompt) + i - 1]
                slack = 0.0 if dtype == "float32" else 0.02 * float(row.max() - row.min())
                assert float(row[token]) >= float(row.max()) - slack - 1e-9
        assert engine.runner.manager.num_free() == 30


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program(folders, tmp_path, dtype):
    folder = folders[dtype]
    requests = _requests(folder)
    _, _, want = _truth(folder, requests)
    steps = trace_mixed(requests, seed=3)
    lines = [json.dumps({"step": i, "entries": [{"id": r, "tokens": t, "want": ws} for r, t, ws in entries],
                         "end": ends}) for i, (entries, ends) in enumerate(steps)]
    out = str(tmp_path / dtype)
    proc = subprocess.run(
        [sys.executable, os.path.join(ROOT, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out,
         "--max-tokens", str(max_live_tokens(steps, page=64))],
        input="\n".join(lines) + "\n", capture_output=True, text=True, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == ["done %d" % i for i in range(len(steps))]
    got, lengths = {}, {}
    for i, (entries, _) in enumerate(steps):
        wanted = [(r, lengths.get(r, 0) + p) for r, t, ws in entries for p in ws]
        for r, t, _ in entries:
            lengths[r] = lengths.get(r, 0) + len(t)
        if wanted:
            data = np.fromfile(os.path.join(out, "%d.f32" % i), dtype="<f4").reshape(len(wanted), -1)
            for key, row in zip(wanted, data):
                got[key] = torch.from_numpy(row.copy())
    assert _off(got, want, dtype) <= 1.0


def test_command_line_writes_a_folder_from_the_nested_config(tmp_path):
    """`--write_random` reads the architecture's name from the one string this config.json has."""
    from qwen3_from_scratch_amd.engine.cli import main

    source = tmp_path / "config.json"
    source.write_text(json.dumps(PLAIN))
    assert main(["--write_random", str(tmp_path / "m"), "--from_config", str(source), "--seed", "3"]) == 0
    assert load_model_config(str(tmp_path / "m")).to_dict() == PLAIN
    names = set(load_file(str(tmp_path / "m" / "model.safetensors")))
    assert "l1.mlp.e2.down" in names and "loop.step" not in names


@pytest.mark.gpu
def test_command_line_generates(tmp_path):
    folder = _write(tmp_path / "m", WIDE, peak=3.0)
    config, w, _ = _truth(folder, {})
    prompt = random_tokens(50, WIDE["vocab"], 12)
    proc = subprocess.run(
        [sys.executable, "-m", "qwen3_from_scratch_amd", "--path", folder, "--dtype", "float32", "--prompt_ids",
         ",".join(map(str, prompt)), "--max_new_tokens", "6", "--temperature", "0", "--ignore_eos", "--max_len", "128",
         "--block_size", "16", "--num_blocks", "16", "--max_num_seqs", "2"],
        capture_output=True, text=True, timeout=600, cwd=ROOT)
    assert proc.returncode == 0, proc.stderr[-2000:]
    got = [int(t) for t in proc.stdout.split()]
    seq = list(prompt)
    for _ in range(6):
        seq.append(int(torch.argmax(plain.logits_of_sequence(config, w, seq)[-1])))
    assert got == seq[len(prompt):]


def test_requests_share_a_prefix_where_no_layer_has_a_window(cpu_ops, tmp_path):
    """Without windows the latent rows of a shared beginning are pages like any other's: a second
    request takes them over, in every pass's plane, and generates what it would have alone."""
    data = copy.deepcopy(LOOPED)
    for layer in data["layers"]:
        layer["mixer"].pop("mask", None)
    folder = _write(tmp_path / "m", data, peak=3.0)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=128, block_size=8, num_blocks=40,
                        max_num_seqs=2, max_num_tokens=32, chunked_prefill_size=16, enable_prefix_cache=True)
    assert engine.runner.manager.prefix_cache
    stem = random_tokens(29, data["vocab"], 21)
    prompts = [stem + random_tokens(5, data["vocab"], 22), stem + random_tokens(9, data["vocab"], 23)]
    got = [engine.generate_ids([p], max_new_tokens=4, temperature=0.0, ignore_eos=True)[0] for p in prompts]
    assert engine.runner.manager.prefix_hits == 24            # three blocks of eight
    for prompt, new in zip(prompts, got):
        seq = list(prompt)
        for _ in range(4):
            seq.append(int(torch.argmax(plain.logits_of_sequence(config, w, seq)[-1])))
        assert new == seq[len(prompt):]
    # with a window anywhere the index stays off
    windowed = SyncEngine(path=_write(tmp_path / "w", LOOPED), dtype="float32", device="cpu", max_len=128, block_size=8,
                          num_blocks=40, max_num_seqs=2, enable_prefix_cache=True)
    assert not windowed.runner.manager.prefix_cache
