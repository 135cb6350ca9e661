"""Kapanex on the GPU: each mechanism's kernels alone against the plain implementation's function
for it, then the model through the step function in every cut, in float32 and in bfloat16, keys at
the edges of the window and writes far back in the recurrent state, long decoding through recorded
launches, and greedy generation through the engine and the command line."""
import json
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

import plain_kapanex
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
from kapanex_helpers import (SMALL, _attention, _config, _delta, _layer, make_weights, plain_greedy, plain_logits,
                             rows_with_a_clear_choice, write_folder)

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {"float32": 2e-5, "bfloat16": 2.5e-2}       # of the largest logit; bfloat16: rounding of the small widths
# (configuration B: one expert of four a row, no shared one, heads of 16: nothing averages the rounding out)
TOL_OF = {("B", "bfloat16"): 6e-2}
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    return HipOps("cuda:0")


def _runner(folder, dtype, max_tokens, page, max_requests=4):
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    model, _ = load_model(folder, dtype, "cuda:0", max_model_len=2048)
    return ModelRunner(model, model.env, page_size=page, num_pages=max_tokens // page,
                       max_requests=max_requests, max_batch_tokens=1024)


def _replay(runner, steps):
    from tiny_llm_infer_amd.engine.replay import Replayer
    rp = Replayer(runner)
    return {st["step"]: rp.run_step(st) for st in steps}


def _requests(name, lengths, seed):
    vocab = SMALL[name][0]["vocab"]
    return {f"r{i}": random_prompt(vocab, n, seed + i) for i, n in enumerate(lengths)}


def _close(got, want, tol, what):
    got, want = got.detach().double().cpu(), want.double()
    err, scale = float((got - want).abs().max()), float(want.abs().max())
    assert err <= tol * max(scale, 1e-6), f"{what}: error {err:.3e}, scale {scale:.3e}"


def _view(starts, counts, slots):
    """A step of sequences that stand at ``starts`` and bring ``counts`` rows, as the step function packs it."""
    from tiny_llm_infer_amd.parts.base import StepView
    i32 = lambda v: torch.tensor([int(x) for x in v], dtype=torch.int32, device="cuda")
    row_start = [0] + list(np.cumsum(counts))
    pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
    sor = [i for i, c in enumerate(counts) for _ in range(c)]
    totals = [s + c for s, c in zip(starts, counts)]
    return StepView(num_rows=sum(counts), num_seqs=len(counts), token_ids=i32(pos), positions=i32(pos), seq_of_row=i32(sor),
                    row_start=i32(row_start), seq_start=i32(starts), seq_len=i32(totals), slots=i32(slots),
                    sample_rows=i32([0]), h_row_start=[int(r) for r in row_start], h_seq_start=list(starts),
                    h_seq_len=totals, h_slots=list(slots), max_rows_per_seq=max(counts), max_seq_len=max(totals),
                    reach=max(128, 1 << (max(totals) - 1).bit_length()))


# ----------------------------------------------------------------- layer norm ---
@pytest.mark.parametrize("n", [72, 50, 1024, 4100])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_layer_norm_of_the_residual_and_what_it_is_owed(ops, dtype, n):
    g = torch.Generator().manual_seed(n)
    dt, T = DTYPES[dtype], 7
    x = torch.randn(T, n, generator=g) * 3 + 1.5
    d1, d2 = torch.randn(T, n, generator=g).to(dt), torch.randn(T, n, generator=g).to(dt)
    w1, w2 = torch.randn(n, generator=g) + 1, torch.randn(n, generator=g) + 1
    tol = 2e-6 if dtype == "float32" else 6e-3
    for owed in ((), (d1,), (d1, d2)):
        total = x.double() + sum(d.double() for d in owed)
        resid = x.clone().cuda()
        a, b = ops.add_layernorm(resid, [d.cuda() for d in owed], (w1.cuda(), w2.cuda()), 1e-5, dt)
        _close(a, plain_kapanex.layer_norm(total, w1.double(), 1e-5), tol, "first norm")
        _close(b, plain_kapanex.layer_norm(total, w2.double(), 1e-5), tol, "second norm")
        _close(resid, total, 1e-6, "residual after the sum")
        resid = x.clone().cuda()
        rows = torch.tensor([5, 0, 6, 2], dtype=torch.int32).cuda()
        (a,) = ops.add_layernorm(resid, [d.cuda() for d in owed], (w2.cuda(),), 1e-5, dt, rows=rows, num_rows=3)
        _close(a, plain_kapanex.layer_norm(total, w2.double(), 1e-5)[[5, 0, 6]], tol, "rows of a list")
        assert torch.equal(resid.cpu(), x)


# ------------------------------------------------------------- the delta rule ---
def _plain_delta_core(raw, gates, conv, a_log, dt_bias, norm_w, eps, H, G, dk, dv, dt):
    """One whole sequence through the plain functions: raw [T, q | k | v | gate] as the projection stores it
    (rounded to the run's type), gates [T, b | a] float32 -> the gated, normed heads [T, H dv]."""
    T = raw.shape[0]
    x = raw.to(dt).double()
    qd, vd = G * dk, H * dv
    c = plain_kapanex.silu(plain_kapanex.causal_conv(x[:, :2 * qd + vd], conv.double()))
    q, k, v = c[:, :qd].view(T, G, dk), c[:, qd:2 * qd].view(T, G, dk), c[:, 2 * qd:].view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(gates[:, :H].double())
    decay = torch.exp(-torch.exp(a_log.double()) * torch.nn.functional.softplus(gates[:, H:].double() + dt_bias.double()))
    o = torch.stack([plain_kapanex.delta_recurrence(q[:, a // (H // G)], k[:, a // (H // G)], v[:, a], beta[:, a], decay[:, a])
                     for a in range(H)], dim=1)
    y = plain_kapanex.rms_unit(o, eps) * norm_w.double() * plain_kapanex.silu(x[:, 2 * qd + vd:].view(T, H, dv))
    return o.reshape(T, vd), y.reshape(T, vd)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("H, G, dk, dv, taps", [(4, 2, 16, 24, 4), (2, 2, 8, 8, 1), (3, 1, 40, 20, 2), (4, 2, 64, 64, 4),
                                                (2, 1, 128, 128, 3), (1, 1, 200, 72, 2)])
def test_delta_rule_kernels_in_portions_and_decoding(ops, dtype, H, G, dk, dv, taps):
    """Three sequences in slots that are used again, cut into portions of 1 to 40 rows that run side by side: the
    convolution's kept rows and the recurrent state carry each one on; a new sequence in an old slot starts clean."""
    g = torch.Generator().manual_seed(H * 100 + dk)
    dt = DTYPES[dtype]
    qd, vd = G * dk, H * dv
    C, ld = 2 * qd + vd, 2 * qd + 2 * vd
    conv = torch.randn(C, taps, generator=g) * 0.6
    a_log, dt_bias = torch.rand(H, generator=g) * 3 - 4, torch.randn(H, generator=g) * 0.5
    norm_w = torch.randn(dv, generator=g) * 0.1 + 1
    lengths = {"a": 61, "b": 9, "c": 47, "d": 30}
    raw = {k: torch.randn(n, ld, generator=g) for k, n in lengths.items()}
    gates = {k: torch.randn(n, 2 * H, generator=g) for k, n in lengths.items()}
    want = {k: _plain_delta_core(raw[k], gates[k], conv, a_log, dt_bias, norm_w, 1e-5, H, G, dk, dv, dt) for k in lengths}
    S = torch.full((3,) + tuple(ops.delta_state_shape(H, dk, dv)), 7.0, dtype=torch.float32, device="cuda")   # slots are never cleared
    kept = torch.full((3, max(taps - 1, 1), C), 5.0, dtype=dt, device="cuda") if taps > 1 else None
    slot = {"a": 0, "b": 1, "c": 2, "d": 1}                                       # d takes b's slot when b is done
    plan = [{"a": 3, "b": 9}, {"a": 1, "c": 2}, {"a": 40, "c": 1, "d": 1}, {"c": 1, "d": 2, "a": 2}, {"d": 27, "c": 43, "a": 15}]
    at = {k: 0 for k in lengths}
    got = {k: ([], []) for k in lengths}
    for portions in plan:
        keys = list(portions)
        view = _view([at[k] for k in keys], [portions[k] for k in keys], [slot[k] for k in keys])
        proj = torch.cat([raw[k][at[k]:at[k] + portions[k]] for k in keys]).to(dt).cuda()
        ba = torch.cat([gates[k][at[k]:at[k] + portions[k]] for k in keys]).cuda()
        turned = len(keys) % 2 == 1                       # b and a as [2 H, rows] in every other step
        o = ops.delta_rule(proj, ba.t().contiguous() if turned else ba, conv.t().contiguous().cuda(), a_log.cuda(),
                           dt_bias.cuda(), kept, S, view, H, G, dk, dv, taps, gates_transposed=turned)
        y = ops.gated_rmsnorm(o, proj, C, norm_w.cuda(), 1e-5, H, dv, dt)
        r = 0
        for k in keys:
            got[k][0].append(o[r:r + portions[k]].cpu())
            got[k][1].append(y[r:r + portions[k]].cpu())
            r += portions[k]
            at[k] += portions[k]
    assert at == lengths
    for k in lengths:
        _close(torch.cat(got[k][0]), want[k][0], 3e-5 if dtype == "float32" else 2e-2, f"{k}: heads' outputs")
        _close(torch.cat(got[k][1]), want[k][1], 3e-5 if dtype == "float32" else 2e-2, f"{k}: gated norm")


# ------------------------------------------------------------ routed experts ---
@pytest.mark.parametrize("E, top, groups, keep", [(6, 2, 3, 2), (4, 1, 1, 1), (8, 3, 8, 3), (16, 4, 4, 2), (64, 8, 8, 4), (5, 5, 1, 1)])
def test_router_choice_and_weights(ops, E, top, groups, keep):
    g = torch.Generator().manual_seed(E)
    z = torch.randn(37, E + 1, generator=g) * 2
    ids, wts, gate = ops.route_experts(z.cuda(), E, top, groups, keep, 2.5, True)
    want_ids, want_wts = plain_kapanex.route(z[:, :E].double(), top, groups, keep, 2.5)
    assert torch.equal(ids.cpu().long(), want_ids)
    _close(wts, want_wts, 1e-6, "weights")
    _close(gate, torch.sigmoid(z[:, E].double()), 1e-6, "shared gate")
    ids2, wts2, none = ops.route_experts(z[:, :E].contiguous().cuda(), E, top, groups, keep, 2.5, False)
    assert none is None and torch.equal(ids2, ids) and torch.equal(wts2, wts)
    ids3, wts3, gate3 = ops.route_experts(z.t().contiguous().cuda(), E, top, groups, keep, 2.5, True, transposed=True)
    assert torch.equal(ids3, ids) and torch.equal(wts3, wts) and torch.equal(gate3, gate)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("T, N, K", [(1, 9, 64), (5, 3, 100), (64, 17, 256), (300, 70, 128), (2048, 33, 512)])
def test_product_with_a_matrix_of_few_rows(ops, dtype, T, N, K):
    g = torch.Generator().manual_seed(T + N)
    x, w = torch.randn(T, K, generator=g).to(DTYPES[dtype]), torch.randn(N, K, generator=g).to(DTYPES[dtype])
    y, transposed = ops.small_product(x.cuda(), w.cuda())
    assert y.dtype == torch.float32 and transposed == (dtype == "bfloat16" and K % 8 == 0)
    _close(y.t() if transposed else y, x.double() @ w.double().t(), 2e-6, "product")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16-plain", "bfloat16-tiles-of-16", "bfloat16-tiles-of-64", "bfloat16-tiles-of-128"])
@pytest.mark.parametrize("T, E, top, n, ff", [(1, 4, 1, 48, 40), (5, 6, 2, 64, 32), (40, 8, 3, 100, 24), (300, 16, 4, 128, 64),
                                              (700, 8, 2, 256, 96), (130, 3, 3, 136, 200)])
def test_chosen_experts_applied_and_added(ops, dtype, T, E, top, n, ff):
    """The kernels that walk the pairs one by one (float32, and bfloat16 where the sizes are no multiples of 8 or
    they are asked for) and the ones that sort the pairs by expert and multiply tile by tile, in every tile size:
    some experts with no pair, some with fewer than a tile, rows whose experts share tiles with other rows."""
    g = torch.Generator().manual_seed(T)
    dtype, _, variant = dtype.partition("-")
    dt = DTYPES[dtype]
    x = torch.randn(T, n, generator=g).to(dt)
    w_gu = (torch.randn(E, 2 * ff, n, generator=g) * n ** -0.5).to(dt)
    w_down = (torch.randn(E, n, ff, generator=g) * ff ** -0.5).to(dt)
    ids = torch.stack([torch.randperm(E, generator=g)[:top] for _ in range(T)]).to(torch.int32)
    wts = torch.rand(T, top, generator=g) + 0.2
    shared, gate = torch.randn(T, n, generator=g).to(dt), torch.rand(T, generator=g)
    want = torch.zeros(T, n, dtype=F64)
    for t in range(T):
        for j in range(top):
            e = int(ids[t, j])
            want[t] += wts[t, j].double() * plain_kapanex.gated_ff(x[t].double(), w_gu[e, :ff].double(), w_gu[e, ff:].double(),
                                                                   w_down[e].double())
    packed = None if variant == "plain" else ops.pack_experts(w_gu.cuda(), w_down.cuda())
    assert (packed is not None) == (dtype == "bfloat16" and variant != "plain" and n % 8 == 0 and ff % 8 == 0)
    tol = 2e-5 if dtype == "float32" else 2e-2
    ops.moe_tile = int(variant.rsplit("-", 1)[1]) if variant.startswith("tiles") else 0
    try:
        rowmajor = (None, None) if packed is not None else (w_gu.cuda(), w_down.cuda())
        got = ops.apply_experts(x.cuda(), ids.cuda(), wts.cuda(), *rowmajor, packed, None, None)
        _close(got, want, tol, "experts")
        got = ops.apply_experts(x.cuda(), ids.cuda(), wts.cuda(), *rowmajor, packed, shared.cuda(), gate.cuda())
        _close(got, want + gate.double()[:, None] * shared.double(), tol, "experts and the shared one")
    finally:
        ops.moe_tile = 0


# ---------------------------------------------- keys at the window's edges, writes far back ---
def _needle_model(tmp_path, window, page):
    """One attention layer whose keys are its queries (same matrix, as many key heads as query heads), a large
    score scale and almost no rotation, so that a token's query finds the key of a like token among all others.
    Queries and keys read the first half of the width, values the second; tokens 88 and 89 have the same
    embedding but for the sign of its second half (whose mean is 0, so the layer norm's mean and variance agree):
    the query of 89 finds the key of 88, and the value found there is the opposite of its own."""
    cfg = _config(90, 32, [_layer("attention", _attention(2, 2, 16, 16, window, 2, scale=1.5), None)], emb_scale=3.0)
    w = {k: v.float() for k, v in make_weights(cfg, 4).items()}
    w["l0.mix.q"][:, 16:] = 0.0
    w["l0.mix.k"] = w["l0.mix.q"].clone()
    w["l0.mix.v"][:, :16] = 0.0
    e = w["embed"][89].to(torch.bfloat16).float()
    e[16:] = torch.tensor([1.0, -1.0] * 8) * e[16:].abs().to(torch.bfloat16).float().mean().to(torch.bfloat16).float()
    w["embed"][89] = e
    w["embed"][88] = torch.cat([e[:16], -e[16:]])
    return cfg, write_folder(str(tmp_path / f"needle{window}"), cfg, {k: v.to(torch.bfloat16) for k, v in w.items()})


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("window, page", [(24, 16), (16, 16), (33, 8)])
def test_one_key_that_stands_out_just_inside_and_just_outside_the_window(tmp_path, dtype, window, page):
    """The token that the last query looks for stands window - 1 positions back (seen) or window positions back
    (not seen); the last token runs in a whole prompt, at the end of a portion of two, and decoded alone."""
    cfg, folder = _needle_model(tmp_path, window, page)
    w = plain_kapanex.read_model(folder)[1]
    n, needle = 3 * window + 5, 89
    logits = {}
    for back in (window - 1, window):
        toks = [t % 88 for t in random_prompt(88, n, 6)]              # neither id is in any of the other places
        toks[n - 1 - back], toks[n - 1] = 88, needle
        want = plain_kapanex.forward(cfg, w, toks)[-1].numpy()
        logits[back] = want
        for tail in (0, 1, 2):                                          # whole; the last token alone; a portion of two
            runner = _runner(folder, dtype, 256, page)
            runner.admit("x")
            from tiny_llm_infer_amd.engine.runner import StepEntry
            if tail:
                runner.step([StepEntry("x", toks[:n - tail], [])])
                got = runner.step([StepEntry("x", toks[n - tail:], [tail - 1])])
            else:
                got = runner.step([StepEntry("x", toks, [n - 1])])
            err = np.abs(got[0].double().cpu().numpy() - want).max()
            assert err <= TOL[dtype] * np.abs(want).max(), (back, tail, err)
    # the test would not see a window that is one off if the needle did not matter
    assert np.abs(logits[window - 1] - logits[window]).max() > 0.04 * np.abs(logits[window]).max()


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_write_hundreds_of_tokens_back_still_counts(tmp_path, dtype):
    """Decays near 1: the recurrent state remembers the whole sequence, so a state that is lost or mixed up at a
    portion's start, or in long decoding, shows in the last logits."""
    cfg = _config(120, 64, [_layer("delta", _delta(4, 2, 16, 32, 3), None), _layer("delta", _delta(2, 1, 32, 16, 2), None)])
    folder = write_folder(str(tmp_path / "memory"), cfg, make_weights(cfg, 8, long_memory=True))
    reqs = {"r0": random_prompt(120, 420, 1), "r1": random_prompt(120, 150, 2)}
    want = plain_logits(folder, reqs)
    w = plain_kapanex.read_model(folder)[1]
    other = list(reqs["r0"])
    other[5] = (other[5] + 1) % 120
    moved = plain_kapanex.forward(cfg, w, other)[-1].numpy()
    assert np.abs(moved - want["r0"][-1]).max() > 1e-3 * np.abs(want["r0"]).max()      # 50 times the float32 bound
    for steps in (trace_prefill_then_decode(reqs, tail=100), trace_portions(reqs, seed=2), trace_mixed(reqs, 640, seed=3)):
        got = collect(steps, _replay(_runner(folder, dtype, 640, 16), steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= TOL[dtype] * scale, (rid, err, row)


# ------------------------------------------------------------- the model, every cut ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(kapanex_folders, kapanex_clear_folders, name, dtype):
    """float32: weights that are random throughout.  bfloat16: weights whose routers have no close calls, which
    rounding would turn (the routers' choice among groups is then left to float32)."""
    folder = (kapanex_clear_folders if dtype == "bfloat16" else kapanex_folders)[name]
    reqs = _requests(name, [70, 45, 197, 33, 1, 58, 2, 3], seed=5)
    want = plain_logits(folder, reqs)
    clear = {rid: len(t) for rid, t in reqs.items()}
    if dtype == "bfloat16":
        assert rows_with_a_clear_choice(folder, reqs, margin=0.1) == clear
    max_tokens = 384
    cuts = {
        "whole": trace_whole(reqs),
        "decode": trace_prefill_then_decode(reqs),
        "portions": trace_portions(reqs, seed=3),
        "mixed": trace_mixed(reqs, max_tokens=max_tokens, seed=9),
    }
    for cut, steps in cuts.items():
        runner = _runner(folder, dtype, max_tokens, SMALL[name][1])
        got = collect(steps, _replay(runner, steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= TOL_OF.get((name, dtype), TOL[dtype]) * scale, \
                f"{name}/{dtype}/{cut}/{rid}: error {err:.3e} at token {row} (scale {scale:.3e})"
        runner.cache.check()
        assert not runner.cache.live() and runner.cache.free_pages() == runner.cache.pages_per_group()
        if cut == "mixed":
            assert runner.cache.pages_taken_total > runner.cache.num_pages


def test_unequal_requests_together_equal_each_alone(kapanex_folders):
    """float32: a request's logits in a batch of unequal requests are those it has alone, to rounding."""
    folder = kapanex_folders["R"]
    reqs = _requests("R", [3, 130, 34, 65], seed=60)
    alone = {rid: _replay(_runner(folder, "float32", 256, 32), trace_whole({rid: toks}))[0] for rid, toks in reqs.items()}
    step = {"step": 0, "entries": [{"id": r, "tokens": t, "want": list(range(len(t)))} for r, t in reqs.items()], "end": list(reqs)}
    together = collect([step], _replay(_runner(folder, "float32", 512, 32), [step]))
    for rid in reqs:
        assert np.abs(together[rid] - alone[rid]).max() <= 2e-5 * np.abs(alone[rid]).max()


def test_long_decoding_through_recorded_launches(kapanex_clear_folders):
    """150 tokens decoded one by one for three requests at once (bfloat16: the steps are replayed from
    recordings), the window passing over decoded tokens and its pages given back on the way."""
    folder = kapanex_clear_folders["R"]
    reqs = _requests("R", [160, 171, 183], seed=77)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, "bfloat16", 768, 32)
    steps = [{"step": 0, "entries": [{"id": r, "tokens": t[:len(t) - 150], "want": []} for r, t in reqs.items()], "end": []}]
    for j in range(150):
        steps.append({"step": j + 1, "entries": [{"id": r, "tokens": [t[len(t) - 150 + j]], "want": [0]} for r, t in reqs.items()],
                      "end": list(reqs) if j == 149 else []})
    got = collect(steps, _replay(runner, steps))
    assert runner.graph_replays > 100
    for rid, toks in reqs.items():
        err, row, scale = max_error(got[rid], want[rid][len(toks) - 150:])
        assert err <= TOL["bfloat16"] * scale, (rid, err, row)


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_greedy_generation_through_the_engine(kapanex_folders, kapanex_clear_folders, dtype):
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = (kapanex_clear_folders if dtype == "bfloat16" else kapanex_folders)["A"]
    prompts = [random_prompt(160, n, 90 + n) for n in (4, 19, 30, 41)]
    eng = LLMEngine.from_folder(folder, dtype=dtype, max_model_len=128, page_size=16, num_kv_blocks=32, max_num_seqs=3,
                                max_num_batched_tokens=32)
    got = eng.generate(prompts, SamplingParams(max_tokens=10, ignore_eos=True))
    if dtype == "float32":
        assert [r.token_ids for r in got] == [plain_greedy(folder, p, 10) for p in prompts]
    else:
        # rounding may turn a close call: every token must be the plain implementation's choice or within
        # the rounding error of it, given the tokens before
        cfg, w = plain_kapanex.read_model(folder)
        for p, r in zip(prompts, got):
            logits = plain_kapanex.forward(cfg, w, p + r.token_ids)[len(p) - 1:-1]
            for z, t in zip(logits, r.token_ids):
                assert float(z.max() - z[t]) <= 2 * TOL["bfloat16"] * float(z.abs().max())
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


# ------------------------------------------------------------------ the command line ---
def test_the_programs_take_a_kapanex_folder(kapanex_folders, tmp_path):
    """bin/trace_run replays a mixed trace, model_main --infer generates greedily, and a model of random
    weights made from a config.json alone loads and generates."""
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = kapanex_folders["C"], SMALL["C"][0]["vocab"]
    reqs = _requests("C", [40, 9, 77, 23, 52], seed=12)
    want = plain_logits(folder, reqs)
    steps = trace_mixed(reqs, max_tokens=192, seed=4)
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", "float32",
                           "--out", str(tmp_path / "out"), "--max-tokens", "192"],
                          input="".join(json.dumps(s) + "\n" for s in steps), text=True, stdout=subprocess.PIPE,
                          stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert proc.stdout.split("\n")[:-1] == [f"done {s['step']}" for s in steps]
    outputs = {s["step"]: np.fromfile(tmp_path / "out" / f"{s['step']}.f32", dtype="<f4").reshape(-1, vocab)
               for s in steps if sum(len(e["want"]) for e in s["entries"])}
    got = collect(steps, outputs)
    for rid in reqs:
        err, row, scale = max_error(got[rid], want[rid])
        assert err <= TOL["float32"] * scale, (rid, err, row)
    prompt = random_prompt(vocab, 21, 3)
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "model_main"), "--infer", "--model", folder, "--dtype",
                           "float32", "--prompt-ids", ",".join(map(str, prompt)), "--max-new-tokens", "8", "--ignore-eos",
                           "--max-seq-len", "64", "--num-kv-blocks", "16"],
                          text=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert [int(t) for t in proc.stdout.split()] == plain_greedy(folder, prompt, 8)
    cfg_file = tmp_path / "config.json"
    cfg_file.write_text(json.dumps(SMALL["R"][0]))
    proc = subprocess.run([sys.executable, os.path.join(root, "bin", "model_main"), "--infer", "--config", str(cfg_file),
                           "--random-weights", "--seed", "5", "--prompt-ids", "1,2,3,4,5", "--max-new-tokens", "6",
                           "--ignore-eos", "--max-seq-len", "64", "--num-kv-blocks", "16"],
                          text=True, stdout=subprocess.PIPE, stderr=subprocess.PIPE, timeout=600)
    assert proc.returncode == 0, proc.stderr[-2000:]
    assert len(proc.stdout.split()) == 6
