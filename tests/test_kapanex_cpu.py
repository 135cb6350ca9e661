"""Kapanex through the engine's own logic on the CPU (the kernel library replaced by the
plain-torch stand-in of tests/cpu_ops.py): configuration and weights, layers that run with
another layer's weights, window pages that are given back, per-request state in slots that
change hands, all ways of cutting the work, and greedy generation through the scheduler,
against the plain implementation."""
import json

import numpy as np
import pytest
import torch

import plain_kapanex
from cpu_ops import CpuOps
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
from kapanex_helpers import SMALL, make_weights, plain_greedy, plain_logits, write_folder
from tiny_llm_infer_amd.config import ConfigError, KapanexConfig
from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
from tiny_llm_infer_amd.engine.loading import load_model
from tiny_llm_infer_amd.engine.replay import Replayer
from tiny_llm_infer_amd.engine.runner import ModelRunner
from tiny_llm_infer_amd.registry import architecture_of
from tiny_llm_infer_amd.sampling.params import SamplingParams
from tiny_llm_infer_amd.weights.loader import WeightError

F64 = torch.float64


def _runner(folder, name, max_tokens, max_requests=4):
    model, _ = load_model(folder, "float32", "cpu", max_model_len=1024, ops=CpuOps())
    page = SMALL[name][1]
    return ModelRunner(model, model.env, page_size=page, num_pages=max_tokens // page,
                       max_requests=max_requests, max_batch_tokens=512)


def _replay(runner, steps):
    rp = Replayer(runner)
    return {st["step"]: rp.run_step(st) for st in steps}


def _requests(name, lengths, seed):
    vocab = SMALL[name][0]["vocab"]
    return {f"r{i}": random_prompt(vocab, n, seed + i) for i, n in enumerate(lengths)}


# ------------------------------------------------------------ configuration ---
def test_config_round_trip_registry_and_run_order():
    from tiny_llm_infer_amd.models.kapanex import kapanex_spec
    for name, (cfg, _, _) in SMALL.items():
        typed = KapanexConfig.from_dict(cfg)
        assert typed.to_dict() == cfg
        assert architecture_of(cfg).name == "Kapanex"
        spec = kapanex_spec(typed)
        own = [i for i, layer in enumerate(cfg["layers"]) if "weights_of" not in layer]
        assert len(spec.blocks) == len(own) and len(spec.schedule) == len(cfg["layers"])
        for i, (layer, call) in enumerate(zip(cfg["layers"], spec.schedule)):
            assert call.block == own.index(layer.get("weights_of", i))
            assert call.cache == (i if layer["type"] == "attention" else -1)      # a cache layer of its own


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("width"), "width"),
    (lambda c: c["layers"][0].update(type="conv"), "layer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"].pop("mask"), "size"),
    (lambda c: c["layers"][0]["mlp"].update(kind="dense"), "feed-forward kind"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(experts=7), "equal groups"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(keep=1), "cannot give"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][2].update(weights_of=1), "other sizes"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_config_errors(change, message):
    cfg = json.loads(json.dumps(SMALL["A"][0]))
    cfg["layers"][0]["mlp"]["router"]["top"] = 3            # (three experts need two groups of three)
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        KapanexConfig.from_dict(cfg)


def test_a_checkpoint_that_does_not_fit_is_refused(tmp_path):
    cfg, _, seed = SMALL["A"]
    w = make_weights(cfg, seed)
    del w["l0.mix.A_log"]
    w["l1.mlp.e2.up"] = w["l1.mlp.e2.up"][:-1]
    w["l2.norm1"] = torch.zeros(64, dtype=torch.bfloat16)           # layer 2 runs with the weights of layer 0
    folder = write_folder(str(tmp_path / "bad"), cfg, w)
    with pytest.raises(WeightError) as err:
        load_model(folder, "float32", "cpu", ops=CpuOps())
    assert err.value.missing == ["l0.mix.A_log"] and err.value.unexpected == ["l2.norm1"]
    assert [n for n, _, _ in err.value.wrong_shape] == ["l1.mlp.e2.up"]


def test_cache_layers_and_state_of_layers_that_share_weights(kapanex_folders):
    """Two attention layers with the same weights keep their keys apart (one group of cache layers, two
    layers in it); two delta layers with the same weights have a state each; the window gives pages back."""
    runner = _runner(kapanex_folders["A"], "A", 256)
    assert len(runner.cache.groups) == 1 and runner.cache.groups[0].cache_layers == [1, 3]
    assert runner.cache.groups[0].need.window == 20
    states = runner.states
    assert states[1] is None and states[3] is None
    assert states[0]["S"].shape == (5, 4, 16, 24) and states[0]["conv"].shape == (5, 3, 2 * 2 * 16 + 4 * 24)
    assert states[2]["S"].data_ptr() != states[0]["S"].data_ptr()
    runner.admit("a")
    toks = random_prompt(160, 100, 1)
    from tiny_llm_infer_amd.engine.runner import StepEntry
    runner.step([StepEntry("a", toks[:90], [])])
    held = [p for p in runner.cache.get("a").tables[0] if p >= 0]
    assert len(held) == 2                                         # positions 71..89 are all a query at 90 reads
    runner.release("a")


# ------------------------------------------------------------------ all the cuts ---
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(kapanex_folders, name):
    folder = kapanex_folders[name]
    reqs = _requests(name, [70, 45, 97, 33, 1, 58, 2], seed=5)
    want = plain_logits(folder, reqs)
    max_tokens = 256
    cuts = {
        "whole": trace_whole(reqs),
        "decode": trace_prefill_then_decode(reqs),
        "portions": trace_portions(reqs, seed=3),
        "mixed": trace_mixed(reqs, max_tokens=max_tokens, seed=9),
    }
    for cut, steps in cuts.items():
        runner = _runner(folder, name, max_tokens)
        got = collect(steps, _replay(runner, steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= 2e-5 * max(1.0, scale), f"{name}/{cut}/{rid}: error {err} at token {row}"
        runner.cache.check()
        assert not runner.cache.live()
        assert runner.cache.free_pages() == runner.cache.pages_per_group()


def test_token_by_token_equals_whole(kapanex_folders):
    """Every token decoded alone from position 0 (the state carries everything) against the whole prompt."""
    folder = kapanex_folders["A"]
    reqs = _requests("A", [60], seed=21)
    want = plain_logits(folder, reqs)
    steps = trace_prefill_then_decode(reqs, tail=59)
    runner = _runner(folder, "A", 64)
    got = collect(steps, _replay(runner, steps))
    err, row, scale = max_error(got["r0"], want["r0"])
    assert err <= 2e-5 * scale, (err, row)


def test_a_slot_that_changes_hands_carries_nothing_over(kapanex_folders):
    """One state slot and few pages, used by request after request: the second one's recurrent state and
    the kept rows of its convolution are those of a fresh sequence."""
    folder = kapanex_folders["C"]
    reqs = _requests("C", [37, 29, 41], seed=40)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, "C", 48, max_requests=1)
    steps = trace_portions(reqs, seed=1)
    got = collect(steps, _replay(runner, steps))
    for rid in reqs:
        err, row, scale = max_error(got[rid], want[rid])
        assert err <= 2e-5 * scale, (rid, err, row)
    assert runner.cache.pages_taken_total > runner.cache.num_pages


def test_unequal_requests_together_equal_each_alone(kapanex_folders):
    folder = kapanex_folders["R"]
    reqs = _requests("R", [3, 130, 34, 65], seed=60)
    alone = {}
    for rid, toks in reqs.items():
        runner = _runner(folder, "R", 256)
        alone[rid] = _replay(runner, trace_whole({rid: toks}))[0]
    runner = _runner(folder, "R", 512)
    step = {"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()],
            "end": list(reqs)}
    together = collect([step], _replay(runner, [step]))
    for rid in reqs:
        assert np.abs(together[rid] - alone[rid]).max() <= 1e-5


# ------------------------------------------------- generation through the scheduler ---
@pytest.mark.parametrize("name", ["A", "B"])
def test_greedy_generation_matches_plain(kapanex_folders, name):
    folder = kapanex_folders[name]
    vocab = SMALL[name][0]["vocab"]
    prompts = [random_prompt(vocab, n, 40 + n) for n in (5, 17, 33)]
    want = [plain_greedy(folder, p, 12) for p in prompts]
    args = dict(dtype="float32", device="cpu", max_model_len=128, page_size=SMALL[name][1], num_kv_blocks=64,
                max_num_seqs=4, max_num_batched_tokens=24, ops=CpuOps())
    eng = LLMEngine.from_folder(folder, **args)
    got = eng.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


# ------------------------------------------------------ the plain implementation itself ---
def test_plain_mechanisms_by_hand():
    """The plain implementation's own small facts, so that an oracle that is wrong in the same way as
    the engine does not go unnoticed."""
    x = torch.tensor([[1.0, 3.0, 5.0, 7.0]], dtype=F64)
    y = plain_kapanex.layer_norm(x, torch.tensor([1.0, 1.0, 2.0, 1.0], dtype=F64), 0.0)
    assert torch.allclose(y, torch.tensor([[-3.0, -1.0, 2.0, 3.0]], dtype=F64) / 5 ** 0.5)
    u = torch.tensor([[1.0], [2.0], [4.0]], dtype=F64)
    assert plain_kapanex.causal_conv(u, torch.tensor([[10.0, 1.0]], dtype=F64))[:, 0].tolist() == [1.0, 12.0, 24.0]
    # a window of 2: row 2 sees keys 1 and 2 only; equal scores, equal weights
    w = plain_kapanex.window_weights(torch.ones(3, 2, dtype=F64), torch.ones(3, 2, dtype=F64), 1.0, 2)
    assert w[2].tolist() == [0.0, 0.5, 0.5] and w[0].tolist() == [1.0, 0.0, 0.0]
    # a quarter turn of the pair (0, 2) at position 1 with frequency pi/2 (base chosen so); elements 1, 3 of a head of 4
    # belong to pair (1, 3) with a lower frequency, element 4 passes
    z = torch.zeros(2, 1, 5, dtype=F64)
    z[1, 0] = torch.tensor([1.0, 0.0, 0.0, 0.0, 9.0])
    r = plain_kapanex.rotate_part(z, 4, 1.0)                  # base 1: every frequency is 1
    assert torch.allclose(r[1, 0], torch.tensor([np.cos(1.0), 0.0, np.sin(1.0), 0.0, 9.0], dtype=F64))
    # the delta rule with beta 1 and no decay stores v under k and gives it back for q = k (unit keys)
    k = torch.tensor([[1.0, 0.0], [0.0, 1.0], [1.0, 0.0]], dtype=F64)
    v = torch.tensor([[2.0], [3.0], [5.0]], dtype=F64)
    o = plain_kapanex.delta_recurrence(k, k, v, torch.ones(3, dtype=F64), torch.ones(3, dtype=F64))
    assert o[:, 0].tolist() == [2.0, 3.0, 5.0]                # the third write replaces the first under the same key
    o = plain_kapanex.delta_recurrence(k, k, v, torch.full((3,), 0.5, dtype=F64), torch.full((3,), 0.5, dtype=F64))
    assert o[:, 0].tolist() == [1.0, 1.5, 0.5 * (5.0 - 0.25) + 0.25]
    # the router: groups of two, the best group by the sum of its two scores, then the best experts inside it
    z = torch.logit(torch.tensor([[0.9, 0.1, 0.6, 0.6, 0.2, 0.2]], dtype=F64))
    ids, wts = plain_kapanex.route(z, 2, 3, 1, 3.0)
    assert ids.tolist() == [[2, 3]] and torch.allclose(wts, torch.tensor([[1.5, 1.5]], dtype=F64))
    ids, wts = plain_kapanex.route(z, 2, 3, 2, 1.0)
    assert ids.tolist() == [[0, 2]] and torch.allclose(wts, torch.tensor([[0.6, 0.4]], dtype=F64))
