"""The Surasun architecture through the engine against tests/plain_surasun.py: each mixer alone in
a model of one layer, whole prompts against token-by-token decoding, portions down to two tokens,
mixed batches in which pages and state slots are used again, the residual behind every layer, long
decoding from the first token, and greedy generation through the engine, the command line and the
replay program. The configurations are made here; their sizes differ from layer to layer and avoid
values that hide a fault (one group, one norm part, equal key and value sizes, a rotation over the
whole head, as many key heads as query heads everywhere)."""

import copy
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch
from safetensors.torch import load_file, save_file

import plain_surasun as plain
from helpers import max_live_tokens, random_tokens, run_trace, trace_mixed, trace_portions, trace_tail_decoded, trace_whole
from qwen3_from_scratch_amd.config import load_model_config
from qwen3_from_scratch_amd.config.model_config import ConfigError
from qwen3_from_scratch_amd.config.surasun_config import SurasunConfig
from qwen3_from_scratch_amd.engine import StepEntry, SyncEngine, load_runner
from qwen3_from_scratch_amd.weights import write_random_model

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _mamba(heads, vdim, state, groups, conv, norm_groups):
    return {"heads": heads, "vdim": vdim, "state": state, "groups": groups, "conv": conv, "norm_groups": norm_groups}


def _unit(width, blocks, conv):
    return {"width": width, "blocks": blocks, "conv": conv}


def _sides(heads, kv_heads, dim, vdim, rot, cap, r_heads, r_dim, r_vdim, r_rot, decay, scales=(0.7, 1.3)):
    left = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": dim ** -0.5,
            "rot": {"dims": rot, "base": 5000.0}}
    if cap:
        left["softcap"] = cap
    right = {"heads": r_heads, "dim": r_dim, "vdim": r_vdim, "decay": decay}
    if r_rot:
        right["rot"] = {"dims": r_rot, "base": 300.0}
    return {"left": left, "right": right, "left_scale": scales[0], "right_scale": scales[1]}


def _layer(kind, mixer, ff=0):
    return {"type": kind, "mixer": mixer, "mlp": {"kind": "dense", "ff": ff} if ff else None}


# two streams; every kind of layer, with and without a feed-forward; groups, norm parts, key heads,
# rotations over part of a head, a side without a cap
MIXED = {"architecture": "Surasun", "vocab": 131, "width": 48, "norm": {"eps": 1e-5}, "residual_mult": 0.5, "streams": 2,
         "layers": [
             _layer("parallel", _sides(6, 2, 24, 16, 12, 30.0, 3, 16, 24, 8, [0.9, 0.97, 0.995]), ff=40),
             _layer("mamba2", _mamba(6, 8, 12, 3, 4, 2), ff=56),
             _layer("rglru", _unit(60, 3, 3)),
             _layer("parallel", _sides(2, 2, 8, 40, 8, 0.0, 2, 24, 8, 24, [0.5, 0.99], scales=(1.2, 0.4))),
             _layer("mamba2", _mamba(2, 24, 20, 1, 2, 3)),
         ]}
# one ordinary residual (no streams in the configuration), no multiplier
PLAIN = {"architecture": "Surasun", "vocab": 97, "width": 64, "norm": {"eps": 1e-6},
         "layers": [
             _layer("rglru", _unit(72, 1, 5), ff=48),
             _layer("mamba2", _mamba(4, 16, 16, 4, 3, 1)),
             _layer("parallel", _sides(4, 1, 16, 24, 6, 8.0, 1, 32, 16, 0, [0.98])),
         ]}
# four streams, sizes in steps of 64
WIDE = {"architecture": "Surasun", "vocab": 257, "width": 128, "norm": {"eps": 1e-5}, "residual_mult": 0.8, "streams": 4,
        "layers": [
            _layer("mamba2", _mamba(4, 64, 64, 2, 4, 2), ff=192),
            _layer("parallel", _sides(4, 2, 64, 128, 32, 20.0, 2, 128, 64, 64, [0.96, 0.999]), ff=128),
            _layer("rglru", _unit(256, 2, 4)),
        ]}
# one stream that is still a hyper-connection (its three numbers matter), odd sizes everywhere
ODD = {"architecture": "Surasun", "vocab": 53, "width": 40, "norm": {"eps": 1e-5}, "residual_mult": 1.5, "streams": 1,
       "layers": [
           _layer("parallel", _sides(3, 3, 10, 6, 4, 3.0, 1, 6, 5, 2, [0.9])),
           _layer("rglru", _unit(35, 5, 2), ff=18),
           _layer("mamba2", _mamba(3, 5, 7, 3, 5, 5)),
       ]}
# sizes at the kernels' ends: eight streams, eight taps, a state of 256, keys of 256 with values that are no
# multiple of a wavefront, thirty-two query heads on one key head, blocks and norm parts of one number, equal key and
# value sizes of 64 (the matrix-core attention kernels in bfloat16) with and without a cap
EDGES = {"architecture": "Surasun", "vocab": 70, "width": 64, "norm": {"eps": 1e-6}, "residual_mult": 0.25, "streams": 8,
         "layers": [
             _layer("mamba2", _mamba(2, 4, 256, 2, 8, 8)),
             _layer("parallel", _sides(32, 1, 8, 4, 8, 5.0, 1, 256, 300, 256, [0.99]), ff=24),
             _layer("rglru", _unit(24, 24, 8)),
             _layer("parallel", _sides(4, 2, 64, 64, 32, 12.0, 2, 8, 2, 4, [0.5, 0.9]), ff=24),
             _layer("parallel", _sides(2, 1, 64, 64, 64, 0.0, 1, 4, 4, 0, [0.7])),
             _layer("mamba2", _mamba(1, 70, 3, 1, 2, 1)),
         ]}
CONFIGS = {"mixed": MIXED, "plain": PLAIN, "wide": WIDE, "odd": ODD, "edges": EDGES}
# how the float32 folders are written: large weights and peaked queries; the configuration of the kernels' ends, whose
# long convolutions and wide states carry float32's own rounding furthest, with weights half as large
SHARP = {name: dict(peak=3.0) for name in CONFIGS}
SHARP["edges"] = dict(peak=2.0, std=0.1)
# one layer of each kind, the mixer alone
ALONE = {kind: {"architecture": "Surasun", "vocab": 61, "width": 32, "norm": {"eps": 1e-5}, "residual_mult": 0.3,
                "streams": 3, "layers": [_layer(kind, mixer)]}
         for kind, mixer in (("mamba2", _mamba(4, 8, 10, 2, 3, 2)), ("rglru", _unit(40, 4, 4)),
                             ("parallel", _sides(4, 2, 12, 20, 6, 10.0, 2, 12, 10, 4, [0.95, 0.99])))}


def _write(folder, data, seed=5, peak=None, std=0.2):
    """Random weights of the configuration, with the streams' tables near what a trained model has
    (a mix near the identity) and, with `peak`, query norms so large that a softmax stands on few keys."""
    folder = str(folder)
    write_random_model(folder, SurasunConfig.from_dict(data), seed=seed, std=std, norm_jitter=0.3)
    path = os.path.join(folder, "model.safetensors")
    tensors = load_file(path)
    g = torch.Generator().manual_seed(seed)
    for key in tensors:
        if key.endswith(".mix") and ".hc" in key:
            n = tensors[key].shape[0]
            tensors[key] = (torch.eye(n) + 0.3 * torch.randn(n, n, generator=g)).to(torch.bfloat16)
        if peak and key.endswith("q.norm"):
            tensors[key] = (tensors[key].float() * peak).to(torch.bfloat16)
        if key == "embed":
            tensors[key] = (tensors[key].float() * (0.2 / std)).to(torch.bfloat16)      # logits that span a few units
    save_file(tensors, path, metadata={"format": "pt"})
    return folder


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folder(request, tmp_path_factory):
    return _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], **SHARP[request.param])


@pytest.fixture(scope="module", params=sorted(CONFIGS))
def folders(request, tmp_path_factory):
    """{dtype: folder}. float32 gets large weights and peaked queries, where a key, a tap or a state
    left out stands far above float32's rounding. With those weights bfloat16's own rounding, at
    the places where the engine rounds, already moves a row by a twentieth of its spread or more
    (the recurrences carry it on), so bfloat16 gets weights under which that rounding stays at a
    third of the bound below."""
    return {"float32": _write(tmp_path_factory.mktemp(request.param), CONFIGS[request.param], **SHARP[request.param]),
            "bfloat16": _write(tmp_path_factory.mktemp(request.param + "_b"), CONFIGS[request.param], std=0.06)}


def _truth(folder, requests):
    with open(os.path.join(folder, "config.json")) as fh:
        config = json.load(fh)
    w = load_file(os.path.join(folder, "model.safetensors"))
    return config, w, {rid: plain.forward(config, w, toks) for rid, toks in requests.items()}


def _requests(folder, lengths=(70, 9, 41, 130, 25, 2, 1)):
    vocab = load_model_config(folder).vocab
    return {"s%d" % i: random_tokens(n, vocab, 260 + i) for i, n in enumerate(lengths)}


def _off(got, want, dtype):
    """The worst row: its difference (mean taken off, root mean square) over the spread of the true
    row, in units of what the dtype may be off by."""
    worst = 0.0
    for rid, logits in want.items():
        for p in range(logits.shape[0]):
            d = got[(rid, p)].double() - logits[p].double()
            err = float((d - d.mean()).pow(2).mean().sqrt() / logits[p].double().std())
            worst = max(worst, err / (5e-5 if dtype == "float32" else 5e-2))
    return worst


# ---- configuration, weights, cache ----

def test_config_is_read_by_its_own_keys_and_written_back(folder):
    config = load_model_config(folder)
    assert isinstance(config, SurasunConfig) and config.architecture == "Surasun"
    with open(os.path.join(folder, "config.json")) as fh:
        raw = json.load(fh)
    assert config.to_dict() == raw and [layer.type for layer in config.layers] == [e["type"] for e in raw["layers"]]
    assert config.streams == raw.get("streams", 0) and config.residual_mult == raw.get("residual_mult", 1.0)
    names = set(load_file(os.path.join(folder, "model.safetensors")))
    assert {"embed", "final.norm", "l0.norm1"} <= names and "head" not in names
    for i, entry in enumerate(raw["layers"]):
        assert ("l%d.norm2" % i in names) == ("l%d.mlp.gate" % i in names) == (entry["mlp"] is not None)
        assert ("l%d.hc1.mix" % i in names) == ("streams" in raw)
        assert ("l%d.hc2.in" % i in names) == ("streams" in raw and entry["mlp"] is not None)
        assert ("l%d.mix.left.q.b" % i in names) == ("l%d.mix.right.g" % i in names) == (entry["type"] == "parallel")
        assert ("l%d.mix.A_log" % i in names) == (entry["type"] == "mamba2")
        assert ("l%d.mix.ra.b" % i in names) == (entry["type"] == "rglru")


@pytest.mark.parametrize("change,word", [
    (lambda c: c["layers"][0].update(type="other"), "type"),
    (lambda c: c["layers"][1]["mixer"].pop("state"), "state"),
    (lambda c: c["layers"][1]["mixer"].update(groups=4), "groups"),
    (lambda c: c["layers"][2]["mixer"].update(blocks=7), "blocks"),
    (lambda c: c["layers"][0]["mlp"].update(kind="moe"), "kind"),
    (lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7), "even"),
    (lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4), "kv_heads"),
    (lambda c: c["layers"][0]["mixer"]["right"].update(decay=[0.5]), "decay"),
    (lambda c: c.pop("width"), "width"),
    (lambda c: c.update(streams=0), "streams"),
])
def test_config_errors_name_the_key(change, word):
    data = copy.deepcopy(MIXED)
    change(data)
    with pytest.raises(ConfigError, match=word):
        SurasunConfig.from_dict(data)


def test_cache_planes_hold_what_each_mixer_keeps(cpu_ops, tmp_path):
    """Every layer owns a plane: the recurrent mixers a state of their own size, the layer of two
    sides pages for the softmax side's keys and values and a state for the other side's."""
    runner = load_runner(_write(tmp_path / "m", MIXED), dtype="float32", device="cpu", page_size=8, max_tokens=128,
                         max_requests=3)
    needs = runner.model.plane_needs
    assert [bool(n.paged) for n in needs] == [True, False, False, True, False]
    assert [n.state_shape[0] for n in needs] == [3 * 16 * 24, 3 * (48 + 72) + 6 * 12 * 8, 2 * 60 + 60, 2 * 24 * 8,
                                                 1 * (48 + 40) + 2 * 20 * 24]
    assert [[t.name for t in n.paged] for n in needs if n.paged] == [["left.keys", "left.values"]] * 2
    assert len(runner.manager.groups) == 2 and len(runner.manager.state_groups) == 5
    assert not runner.manager.prefix_cache and runner.model.graph_safe()


# ---- each mixer alone, and the streams behind every layer ----

@pytest.mark.parametrize("kind", sorted(ALONE))
def test_one_mixer_alone_on_the_host(cpu_ops, tmp_path, kind):
    folder = _write(tmp_path / kind, ALONE[kind], seed=9, peak=2.0)
    requests = _requests(folder, lengths=(45, 3, 1, 20))
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=max_live_tokens(steps, page=8),
                             max_requests=4)
        assert _off(run_trace(runner, steps), want, "float32") <= 1.0, make.__name__


def _streams_behind(folder, tokens, device, dtype):
    runner = load_runner(folder, dtype=dtype, device=device, page_size=8, max_tokens=64, max_requests=1)
    seen = []

    def observe(i, x, pending):
        new = torch.einsum("st,nsw->ntw", pending.mix.double().cpu(), x.double().cpu())
        new = new + pending.write.double().cpu()[None, :, None] * pending.values.double().cpu()[:, None, :]
        seen.append(new.sum(dim=1))

    runner.model.observer = observe
    runner.step([StepEntry("r", tokens, [])])
    return seen


@pytest.mark.parametrize("name", ["mixed", "plain", "odd", "edges"])
def test_streams_behind_every_layer_on_the_host(cpu_ops, tmp_path, name):
    """The sum of the streams behind every layer, what the last sublayer still owes them included."""
    folder = _write(tmp_path / "m", CONFIGS[name])
    tokens = random_tokens(37, CONFIGS[name]["vocab"], 4)
    config, w, _ = _truth(folder, {})
    want = []
    plain.forward(config, w, tokens, want)
    seen = _streams_behind(folder, tokens, "cpu", "float32")
    assert len(seen) == len(want) == len(config["layers"])
    for got, truth in zip(seen, want):
        assert float((got - truth).abs().max()) <= 2e-5 * float(truth.abs().max())


def test_a_stream_table_that_is_ignored_shows(cpu_ops, tmp_path):
    """The three tables of a sublayer all matter: a model whose mix, read or write table is changed
    gives other logits, by far more than rounding (a block that used the ordinary residual instead
    would pass every comparison with weights that make the tables trivial)."""
    folder = _write(tmp_path / "m", MIXED)
    tokens = random_tokens(12, MIXED["vocab"], 3)
    config, w, _ = _truth(folder, {})
    base = plain.forward(config, w, tokens)
    for leaf in ("hc1.mix", "hc1.in", "hc1.out", "hc2.mix"):
        changed = dict(w)
        changed["l1." + leaf] = (w["l1." + leaf].float() * torch.tensor([1.5, 0.5])).to(torch.bfloat16)
        assert float((plain.forward(config, changed, tokens) - base).abs().max()) > 1e-2, leaf


# ---- the whole model ----

def test_logits_on_the_host_under_every_cutting(cpu_ops, folder):
    requests = _requests(folder)
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype="float32", device="cpu", page_size=8,
                             max_tokens=max_live_tokens(steps, page=8), max_requests=4)
        assert _off(run_trace(runner, steps), want, "float32") <= 1.0, make.__name__
        assert all(g.pool.num_free == g.pool.num_pages for g in runner.manager.groups)


def test_a_slot_that_is_used_again_starts_from_nothing(cpu_ops, tmp_path):
    """One state slot and a pool of a few pages: every request takes the slot and the pages the
    last one left, and must not see what that one kept there."""
    folder = _write(tmp_path / "m", MIXED)
    requests = _requests(folder, lengths=(33, 40, 5, 17))
    _, _, want = _truth(folder, requests)
    runner = load_runner(folder, dtype="float32", device="cpu", page_size=8, max_tokens=40, max_requests=1)
    got = run_trace(runner, trace_portions(requests, sizes=(7, 2, 13)))
    assert _off(got, want, "float32") <= 1.0
    assert runner.manager.slot("x") == 0 if runner.manager.has("x") else True


def test_greedy_generation_through_the_engine_on_the_host(cpu_ops, folder):
    requests = _requests(folder)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=256, block_size=8, num_blocks=60,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [toks[:n] for toks, n in zip(requests.values(), (30, 9, 41, 2))]
    got = engine.generate_ids(prompts, max_new_tokens=5, temperature=0.0, ignore_eos=True)
    for prompt, new in zip(prompts, got):
        assert new == plain.greedy(config, w, prompt, 5)
    assert engine.runner.manager.num_free() == 60


def test_a_preempted_request_builds_its_state_again_on_the_host(cpu_ops, tmp_path):
    """Too few pages for three requests at once: one is preempted, gives pages and state slot back, and
    later goes through its prompt and its generated tokens again from an empty state. What it generates
    is what it would have generated alone."""
    folder = _write(tmp_path / "m", MIXED, peak=3.0)
    config, w, _ = _truth(folder, {})
    engine = SyncEngine(path=folder, dtype="float32", device="cpu", max_len=128, block_size=8, num_blocks=12,
                        max_num_seqs=3, max_num_tokens=24, chunked_prefill_size=16)
    prompts = [random_tokens(n, MIXED["vocab"], 300 + n) for n in (30, 9, 41)]
    requests = [engine.add_request(p, engine.default_params(10, temperature=0.0, ignore_eos=True)) for p in prompts]
    steps = 0
    while engine.scheduler.has_work() and steps < 500:
        engine.step()
        engine.runner.manager.audit()
        steps += 1
    assert not engine.scheduler.has_work() and sum(r.preemptions for r in requests) >= 1
    for prompt, request in zip(prompts, requests):
        assert list(request.generated) == plain.greedy(config, w, prompt, 10)
    assert engine.runner.manager.num_free() == 12


def test_command_line_writes_a_folder_from_the_nested_config(tmp_path):
    from qwen3_from_scratch_amd.engine.cli import main

    source = tmp_path / "config.json"
    source.write_text(json.dumps(PLAIN))
    assert main(["--write_random", str(tmp_path / "m"), "--from_config", str(source), "--seed", "3"]) == 0
    assert load_model_config(str(tmp_path / "m")).to_dict() == PLAIN
    names = set(load_file(str(tmp_path / "m" / "model.safetensors")))
    assert "l2.mix.right.o" in names and "l0.hc1.mix" not in names


# ---- the model on the GPU ----

@pytest.mark.gpu
@pytest.mark.parametrize("kind", sorted(ALONE))
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_one_mixer_alone(tmp_path, kind, dtype):
    folder = _write(tmp_path / kind, ALONE[kind], seed=9, **(dict(peak=2.0) if dtype == "float32" else dict(std=0.06)))
    requests = _requests(folder, lengths=(45, 3, 1, 200))
    _, _, want = _truth(folder, requests)
    for make in (trace_whole, trace_tail_decoded, trace_portions, trace_mixed):
        steps = make(requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=max_live_tokens(steps, page=16),
                             max_requests=4)
        assert _off(run_trace(runner, steps), want, dtype) <= 1.0, make.__name__


@pytest.mark.gpu
def test_streams_behind_every_layer(tmp_path):
    folder = _write(tmp_path / "m", WIDE)
    tokens = random_tokens(50, WIDE["vocab"], 4)
    config, w, _ = _truth(folder, {})
    want = []
    plain.forward(config, w, tokens, want)
    for got, truth in zip(_streams_behind(folder, tokens, "cuda", "float32"), want):
        assert float((got - truth).abs().max()) <= 5e-5 * float(truth.abs().max())


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
    """A request decoded token by token from its second token on, through graph replays and page
    ends, beside a request that is decoded from its very first and one that joins later into a slot
    that was used before."""
    for dtype in ("float32", "bfloat16"):
        folder = folders[dtype]
        vocab = load_model_config(folder).vocab
        requests = {"long": random_tokens(200, vocab, 7), "short": random_tokens(3, vocab, 8),
                    "late": random_tokens(150, vocab, 9)}
        _, _, want = _truth(folder, requests)
        runner = load_runner(folder, dtype=dtype, device="cuda", page_size=16, max_tokens=416, max_requests=2)
        steps = []
        for i in range(200):
            entries = [(rid, [requests[rid][i]], [0]) for rid in ("long", "short") if i < len(requests[rid])]
            if i >= 50:
                entries.append(("late", [requests["late"][i - 50]], [0]))
            steps.append((entries, [rid for rid, _, _ in entries
                                    if (i - 50 if rid == "late" else i) == len(requests[rid]) - 1]))
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
            logits = plain.forward(config, w, prompt + new)
            for i, token in enumerate(new):
                row = logits[len(prompt) + i - 1]
                slack = 1e-4 if dtype == "float32" else 0.02 * float(row.max() - row.min())
                assert float(row[token]) >= float(row.max()) - slack
        assert engine.runner.manager.num_free() == 30


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_replay_program(tmp_path, dtype):
    folder = _write(tmp_path / "m", MIXED, **(dict(peak=3.0) if dtype == "float32" else dict(std=0.06)))
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
    assert [int(t) for t in proc.stdout.split()] == plain.greedy(config, w, prompt, 6)
