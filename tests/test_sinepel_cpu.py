"""Sinepel through the engine's own logic on the CPU (the kernel library replaced by the
plain-torch stand-in of tests/cpu_ops.py): configuration and weights, the cache manager's
blocks of positions, per-request state in slots that change hands, all ways of cutting the
work, and greedy generation through the scheduler, against the plain implementation."""
import json

import numpy as np
import pytest
import torch

import plain_sinepel
from cpu_ops import CpuOps
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
from sinepel_helpers import SMALL, make_weights, plain_greedy, plain_logits, write_folder
from tiny_llm_infer_amd.cache.manager import PAGE, CacheManager, CacheNeed, CacheRecord
from tiny_llm_infer_amd.config import ConfigError, SinepelConfig
from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
from tiny_llm_infer_amd.engine.loading import load_model
from tiny_llm_infer_amd.engine.replay import Replayer
from tiny_llm_infer_amd.engine.runner import ModelRunner
from tiny_llm_infer_amd.registry import architecture_of
from tiny_llm_infer_amd.sampling.params import SamplingParams
from tiny_llm_infer_amd.weights.loader import WeightError


def _runner(folder, name, max_tokens, max_requests=4):
    model, _ = load_model(folder, "float32", "cpu", ops=CpuOps())
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
def test_config_round_trip_and_registry():
    for name, (cfg, _, _) in SMALL.items():
        typed = SinepelConfig.from_dict(cfg)
        assert typed.to_dict() == cfg
        assert architecture_of(cfg).name == "Sinepel"
        assert len(typed.layers) == len(cfg["layers"]) and typed.streams == cfg["streams"]


@pytest.mark.parametrize("change, message", [
    (lambda c: c.pop("streams"), "streams"),
    (lambda c: c["layers"][0].update(type="recurrent"), "layer type"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][0]["mixer"].pop("mask"), "size"),
    (lambda c: c["layers"][0]["mlp"].update(kind="gated"), "feed-forward kind"),
    (lambda c: c["norm"].update(eps=0.0), "eps"),
])
def test_config_errors(change, message):
    cfg = json.loads(json.dumps(SMALL["P"][0]))
    change(cfg)
    with pytest.raises(ConfigError, match=message):
        SinepelConfig.from_dict(cfg)


def test_a_checkpoint_that_does_not_fit_is_refused(tmp_path):
    cfg, _, seed = SMALL["P"]
    w = make_weights(cfg, seed)
    del w["l0.hc1.mix"]
    w["l1.shift"] = w["l1.shift"][:-1]
    w["l1.mlp.up"] = torch.zeros(4, 4, dtype=torch.bfloat16)           # layer 1 has no feed-forward
    folder = write_folder(str(tmp_path / "bad"), cfg, w)
    with pytest.raises(WeightError) as err:
        load_model(folder, "float32", "cpu", ops=CpuOps())
    assert err.value.missing == ["l0.hc1.mix"] and err.value.unexpected == ["l1.mlp.up"]
    assert [n for n, _, _ in err.value.wrong_shape] == ["l1.shift"]


# ----------------------------------------------- blocks of positions in the cache ---
def test_pages_of_a_block_that_has_passed_are_given_back():
    need = CacheNeed((CacheRecord("k", (1, PAGE, 4)),), chunk=24)
    assert not need.keeps_all and need.reach == 24
    assert [need.first_read(p) for p in (0, 23, 24, 47, 48)] == [0, 0, 24, 24, 48]
    cm = CacheManager([need], page_size=8, num_pages=6, max_requests=2)
    cm.admit("a")
    held = []
    for total in (5, 23, 24, 25, 47, 48, 70, 72, 73):
        cm.reserve("a", total)
        cm.advance("a", total)
        cm.check()
        table = list(cm.get("a").tables[0])
        # the next row (position ``total``) reads from its block's first position on
        first = (total // 24 * 24) // 8
        assert all(p < 0 for p in table[:first]) and all(p >= 0 for p in table[first:])
        held.append(sum(p >= 0 for p in table))
    assert max(held) <= 3 and held[2] == 0 and held[5] == 0          # an edge of a block: nothing is kept
    cm.release("a")
    assert cm.free_pages() == [6]
    with pytest.raises(ValueError):
        CacheNeed((CacheRecord("k", (1, PAGE, 4)),), window=4, chunk=4)


# ------------------------------------------------------------------ all the cuts ---
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(sinepel_folders, name):
    folder = sinepel_folders[name]
    reqs = _requests(name, [70, 45, 97, 33, 1, 58], seed=5)
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


def test_token_by_token_equals_whole(sinepel_folders):
    """Every token decoded alone from position 0 (the state carries everything) against the whole prompt."""
    folder = sinepel_folders["P"]
    reqs = _requests("P", [60], seed=21)
    want = plain_logits(folder, reqs)
    steps = trace_prefill_then_decode(reqs, tail=59)
    runner = _runner(folder, "P", 64)
    got = collect(steps, _replay(runner, steps))
    err, row, scale = max_error(got["r0"], want["r0"])
    assert err <= 2e-5 * scale, (err, row)


def test_a_slot_that_changes_hands_carries_nothing_over(sinepel_folders):
    """One state slot and few pages, used by request after request: the second one's first rows
    (which read the kept rows of the shift and of the convolution) are those of a fresh sequence."""
    folder = sinepel_folders["Q"]
    reqs = _requests("Q", [37, 29, 41], seed=40)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, "Q", 48, max_requests=1)
    steps = trace_portions(reqs, seed=1)
    got = collect(steps, _replay(runner, steps))
    for rid in reqs:
        err, row, scale = max_error(got[rid], want[rid])
        assert err <= 2e-5 * scale, (rid, err, row)
    assert runner.cache.pages_taken_total > runner.cache.num_pages


def test_unequal_requests_together_equal_each_alone(sinepel_folders):
    folder = sinepel_folders["R"]
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
@pytest.mark.parametrize("name", ["P", "Q"])
def test_greedy_generation_matches_plain(sinepel_folders, name):
    folder = sinepel_folders[name]
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
    # so few pages that requests are preempted and computed again from their first token: the same tokens
    small = LLMEngine.from_folder(folder, **dict(args, num_kv_blocks=(3 if name == "P" else 7)))
    got = small.generate(prompts, SamplingParams(max_tokens=12, ignore_eos=True))
    assert [r.token_ids for r in got] == want
    if name == "Q":            # (its last layer keeps a whole request's keys; P gives its pages back block by block)
        assert small.scheduler.num_preemptions > 0


def test_plain_mechanisms_by_hand():
    """The plain implementation's own small facts, so that an oracle that is wrong in the same way as
    the engine does not go unnoticed."""
    h = torch.tensor([[1.0, 2.0], [3.0, 6.0], [5.0, 0.0]], dtype=torch.float64)
    out = plain_sinepel.token_shift(h, torch.tensor([0.5, 0.0], dtype=torch.float64))
    assert out.tolist() == [[0.5, 2.0], [2.0, 6.0], [4.0, 0.0]]
    u = torch.tensor([[1.0], [2.0], [4.0]], dtype=torch.float64)
    y = plain_sinepel.causal_conv(u, torch.tensor([[10.0, 1.0]], dtype=torch.float64))       # taps: older, newest
    assert y[:, 0].tolist() == [1.0, 12.0, 24.0]
    assert [plain_sinepel.chunk_visible(5, j, 4) for j in (3, 4, 5, 6)] == [False, True, True, False]
    x = torch.arange(12, dtype=torch.float64).reshape(2, 3, 2)
    mix = torch.tensor([[1.0, 2.0], [0.0, 1.0]], dtype=torch.float64)                          # [from, to]
    new = plain_sinepel.hyper_write(x, torch.zeros(3, 2, dtype=torch.float64), mix, torch.zeros(2, dtype=torch.float64))
    assert torch.equal(new[0], x[0]) and torch.equal(new[1], 2 * x[0] + x[1])
    w = plain_sinepel.attention_scores(torch.ones(3, 2, dtype=torch.float64), torch.ones(3, 2, dtype=torch.float64),
                                       1.0, 1.0, 1.0, 1.0, 8)
    # equal dot products: the weights fall with the distance as 1 / (1 + distance)
    assert torch.allclose(w[2], torch.tensor([1 / 3, 1 / 2, 1.0], dtype=torch.float64) / (1 / 3 + 1 / 2 + 1))
