"""Sinepel on the GPU: each mechanism's kernels alone against the plain implementation's function
for it, then the model through the step function in every cut, in float32 and in bfloat16, long
decoding through recorded launches, and greedy generation through the engine."""
import numpy as np
import pytest
import torch

import plain_sinepel
from helpers import collect, max_error, random_prompt, trace_mixed, trace_portions, trace_prefill_then_decode, trace_whole
from sinepel_helpers import SMALL, plain_greedy, plain_logits

pytestmark = pytest.mark.gpu
F64 = torch.float64
TOL = {"float32": 2e-5, "bfloat16": 2.5e-2}       # of the largest logit; bfloat16: rounding of the small widths
DTYPES = {"float32": torch.float32, "bfloat16": torch.bfloat16}


@pytest.fixture(scope="module")
def ops():
    from tiny_llm_infer_amd.kernels.ops import HipOps
    return HipOps("cuda:0")


def _runner(folder, name, dtype, max_tokens, max_requests=4, page=None):
    from tiny_llm_infer_amd.engine.loading import load_model
    from tiny_llm_infer_amd.engine.runner import ModelRunner
    model, _ = load_model(folder, dtype, "cuda:0")
    page = page or SMALL[name][1]
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


# ----------------------------------------------------------------- small kernels ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_embedding_activation_softcap(ops, dtype):
    g = torch.Generator().manual_seed(1)
    dt = DTYPES[dtype]
    table, pos = torch.randn(50, 24, generator=g).to(dt), torch.randn(30, 24, generator=g).to(dt)
    ids, where = [3, 49, 0, 7, 7], [0, 29, 5, 1, 2]
    got = ops.embed(table.cuda(), torch.tensor(ids, dtype=torch.int32).cuda(), 5, scale=1.75,
                    positions=torch.tensor(where, dtype=torch.int32).cuda(), pos_table=pos.cuda())
    want = table.double()[ids] * 1.75 + pos.double()[where]
    _close(got, want, 1e-6, "embedding")
    got = ops.embed(table.cuda(), torch.tensor(ids, dtype=torch.int32).cuda(), 5, scale=0.5)
    _close(got, table.double()[ids] * 0.5, 1e-6, "embedding without positions")
    x = (torch.randn(7, 40, generator=g) * 3).to(dt)
    z = x.double()
    for name, want in (("relu2", torch.relu(z) ** 2), ("relu", torch.relu(z)), ("silu", z * torch.sigmoid(z)),
                       ("gelu_tanh", 0.5 * z * (1 + torch.tanh((2 / torch.pi) ** 0.5 * (z + 0.044715 * z ** 3))))):
        _close(ops.activation(x.cuda(), name), want, 1e-6 if dtype == "float32" else 5e-3, name)
    z = torch.randn(3, 33, generator=g) * 20
    _close(ops.softcap(z.clone().cuda(), 7.5), plain_sinepel.soft_cap(z.double(), 7.5), 1e-6, "soft cap")


@pytest.mark.parametrize("streams", [1, 2, 3, 5])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_streams_read_norm_write(ops, streams, dtype):
    """The streams take a sublayer's output, are read and normed: against hyper_write, hyper_read, rms_norm."""
    from tiny_llm_infer_amd.parts.hyper import StreamDelta
    g = torch.Generator().manual_seed(streams)
    T, n, S = 9, 72, streams
    x = torch.randn(T, S, n, generator=g)
    y = torch.randn(T, n, generator=g).to(DTYPES[dtype])
    mix, out_w, in_w = torch.randn(S, S, generator=g), torch.randn(S, generator=g), torch.randn(S, generator=g)
    weight = torch.randn(n, generator=g) + 1
    xs = x.double().permute(1, 0, 2)                                           # [S, T, n] as the plain functions take it
    new = plain_sinepel.hyper_write(xs, y.double(), mix.double(), out_w.double())
    want = plain_sinepel.rms_norm(plain_sinepel.hyper_read(new, in_w.double()), weight.double(), 1e-5)
    resid = x.clone().cuda()
    got = ops.streams_norm(resid, StreamDelta(y.cuda(), mix.cuda(), out_w.cuda()), in_w.cuda(), weight.cuda(), 1e-5,
                           torch.float32)
    _close(got, want, 2e-5, "normed rows")
    _close(resid, new.permute(1, 0, 2), 2e-6, "streams after the write")
    # nothing owed: the streams stay, and so they do with a list of rows
    resid2 = x.clone().cuda()
    got = ops.streams_norm(resid2, None, in_w.cuda(), weight.cuda(), 1e-5, torch.float32)
    _close(got, plain_sinepel.rms_norm(plain_sinepel.hyper_read(xs, in_w.double()), weight.double(), 1e-5), 2e-5, "no write")
    assert torch.equal(resid2.cpu(), x)
    rows = torch.tensor([4, 0, 8], dtype=torch.int32).cuda()
    got = ops.streams_norm(resid2, StreamDelta(y.cuda(), mix.cuda(), out_w.cuda()), in_w.cuda(), weight.cuda(), 1e-5,
                           torch.float32, rows=rows, num_rows=3)
    _close(got, want[[4, 0, 8]], 2e-5, "rows of a list")
    assert torch.equal(resid2.cpu(), x)
    _close(ops.streams_open(x[:, 0].contiguous().cuda(), S), x[:, :1].expand(T, S, n), 0.0, "opening the streams")
    if dtype == "bfloat16":
        # the owed rows as float32 partial sums of a product whose k range was split: added and rounded by the kernel
        from tiny_llm_infer_amd.kernels.ops import DeferredSum
        pieces = torch.randn(3, T, n, generator=g)
        y3 = (pieces[0] + pieces[1] + pieces[2]).to(torch.bfloat16)
        new3 = plain_sinepel.hyper_write(xs, y3.double(), mix.double(), out_w.double())
        resid3 = x.clone().cuda()
        got = ops.streams_norm(resid3, StreamDelta(DeferredSum(pieces.cuda(), torch.bfloat16), mix.cuda(), out_w.cuda()),
                               in_w.cuda(), weight.cuda(), 1e-5, torch.float32)
        _close(got, plain_sinepel.rms_norm(plain_sinepel.hyper_read(new3, in_w.double()), weight.double(), 1e-5), 2e-5, "partial sums")
        _close(resid3, new3.permute(1, 0, 2), 2e-6, "streams after partial sums")


class _Bench:
    """One attention layer's cache, state and packed steps, made by the engine's own cache manager and
    step packing, for calling the mixer's kernels directly."""

    def __init__(self, dtype, heads, kv_heads, dim, taps, mask, page=8, pages=24, slots=3):
        from tiny_llm_infer_amd.cache.manager import CacheManager
        from tiny_llm_infer_amd.config.base import PartSpec
        from tiny_llm_infer_amd.parts.base import build_part
        self.dt = DTYPES[dtype]
        names = {r: r for r in ("q", "q_bias", "q_conv", "k", "k_bias", "k_conv", "o", "temp", "r1", "r2")}
        self.mixer = build_part("mixer", PartSpec("conv_key_attention", dict(
            hidden_size=8, num_heads=heads, num_kv_heads=kv_heads, head_dim=dim, scale=1.0, conv_taps=taps, mask=mask), names))
        self.cm = CacheManager([self.mixer.cache_need()], page, pages, slots)
        self.page, self.C = page, (heads + kv_heads) * dim
        self.k = torch.zeros(1, pages + 1, kv_heads, page, dim, dtype=self.dt, device="cuda")
        need = self.mixer.state_need()
        self.state = None if need is None else torch.zeros((slots + 1,) + need.shape, dtype=self.dt, device="cuda")
        self.args = (heads, kv_heads, dim, taps)

    def step(self, ops, portions, qk, bias, conv, scale, temp, penalty, mask):
        """portions: {request: number of rows}; qk: the rows' raw projections in that order."""
        from tiny_llm_infer_amd.parts.base import GroupView, LayerCache, StepView
        keys = list(portions)
        for key in keys:
            if key not in self.cm:
                self.cm.admit(key)
            self.cm.reserve(key, self.cm.get(key).num_tokens + portions[key])
        rcs = [self.cm.get(k) for k in keys]
        starts, counts = [rc.num_tokens for rc in rcs], [portions[k] for k in keys]
        width = max(4, max(len(rc.tables[0]) for rc in rcs))
        tables = torch.full((len(keys), width), -1, dtype=torch.int32)
        for i, rc in enumerate(rcs):
            tables[i, :len(rc.tables[0])] = torch.tensor(list(rc.tables[0]), dtype=torch.int32)
        row_start = [0] + list(np.cumsum(counts))
        i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")
        pos = [s + j for s, c in zip(starts, counts) for j in range(c)]
        sor = [i for i, c in enumerate(counts) for _ in range(c)]
        totals = [s + c for s, c in zip(starts, counts)]
        group = GroupView({"k": self.k}, tables.cuda(), width, self.page, None)
        view = StepView(num_rows=sum(counts), num_seqs=len(keys), token_ids=i32(pos), positions=i32(pos),
                        seq_of_row=i32(sor), row_start=i32([int(r) for r in row_start]), seq_start=i32(starts),
                        seq_len=i32(totals), slots=i32([rc.slot for rc in rcs]), sample_rows=i32([0]),
                        h_row_start=[int(r) for r in row_start], h_seq_start=starts, h_seq_len=totals,
                        h_slots=[rc.slot for rc in rcs], max_rows_per_seq=max(counts), max_seq_len=max(totals),
                        reach=max(128, 1 << (max(totals) - 1).bit_length()), groups=[group])
        out = ops.conv_key_attention(qk.to(self.dt).cuda(), bias.cuda(), conv.t().contiguous().cuda(), self.state, view,
                                     LayerCache(group, 0, True), *self.args, scale, temp, penalty, mask)
        for key in keys:
            self.cm.advance(key, self.cm.get(key).num_tokens + portions[key])
        return out


def _plain_mixer_core(raw, bias, conv, heads, kv_heads, dim, scale, temp, r1, r2, size, dt):
    """The plain functions on one whole sequence's raw projections [T, C]: bias, convolution, attention with
    the keys as values.  Rounded where the engine stores (q and the cached keys) so that bfloat16 compares."""
    u = raw.to(dt).double() + bias.double()
    y = plain_sinepel.causal_conv(u, conv.double()).to(dt).double()
    q, k = y[:, :heads * dim], y[:, heads * dim:]
    out = torch.zeros(raw.shape[0], heads * dim, dtype=F64)
    for a in range(heads):
        g = a // (heads // kv_heads)
        w = plain_sinepel.attention_scores(q[:, a * dim:(a + 1) * dim], k[:, g * dim:(g + 1) * dim], scale,
                                           float(temp[a]), float(r1[a]), float(r2[a]), size)
        out[:, a * dim:(a + 1) * dim] = w @ k[:, g * dim:(g + 1) * dim]
    return out


@pytest.mark.parametrize("dtype", ["float32", "bfloat16", "bfloat16-tiles-of-32"])
@pytest.mark.parametrize("heads, kv_heads, dim, taps, size, page", [
    (4, 2, 16, 3, 24, 8), (3, 3, 8, 1, 7, 4), (2, 1, 64, 4, 32, 16), (8, 2, 32, 2, 80, 8), (1, 1, 48, 5, 16, 8), (4, 4, 128, 2, 64, 16)])
def test_mixer_kernels_in_portions_and_decoding(ops, dtype, heads, kv_heads, dim, taps, size, page):
    if dtype.endswith("32") and dtype != "float32":
        dtype = "bfloat16"
        ops.attention_tile_rows = 32
    try:
        _mixer_kernels_in_portions_and_decoding(ops, dtype, heads, kv_heads, dim, taps, size, page)
    finally:
        ops.attention_tile_rows = 16


def _mixer_kernels_in_portions_and_decoding(ops, dtype, heads, kv_heads, dim, taps, size, page):
    """Convolution (with the kept rows), keys into pages, attention inside blocks of positions: two sequences
    in unequal portions, then token by token, against the plain functions on the whole sequences."""
    g = torch.Generator().manual_seed(dim + taps)
    C = (heads + kv_heads) * dim
    lens = {"a": 2 * size + 9, "b": size + 3}
    raw = {k: torch.randn(n, C, generator=g) for k, n in lens.items()}
    bias, conv = torch.randn(C, generator=g) * 0.3, torch.randn(C, taps, generator=g) * 0.6
    temp, r1, r2 = torch.rand(heads, generator=g) + 0.5, torch.rand(heads, generator=g) + 0.2, torch.rand(heads, generator=g) * 2
    scale = dim ** -0.5
    bench = _Bench(dtype, heads, kv_heads, dim, taps, ("chunk", size), page=page, pages=(sum(lens.values()) // page + 4))
    got = {k: [] for k in lens}
    at = {k: 0 for k in lens}
    plan = [{"a": 5, "b": 2}, {"a": size - 3}, {"b": size - 1, "a": 2}, {"a": 1, "b": 1}, {"a": 1}, {"a": size + 3, "b": 1}]
    while any(at[k] < lens[k] for k in lens):
        portions = plan.pop(0) if plan else {k: 1 for k in lens if at[k] < lens[k]}
        portions = {k: min(n, lens[k] - at[k]) for k, n in portions.items() if at[k] < lens[k]}
        qk = torch.cat([raw[k][at[k]:at[k] + n] for k, n in portions.items()])
        out = bench.step(ops, portions, qk, bias, conv, scale, temp.cuda(), (r1.cuda(), r2.cuda()), ("chunk", size))
        r = 0
        for k, n in portions.items():
            got[k].append(out[r:r + n].double().cpu())
            r += n
            at[k] += n
    for k in lens:
        want = _plain_mixer_core(raw[k], bias, conv, heads, kv_heads, dim, scale, temp, r1, r2, size, DTYPES[dtype])
        _close(torch.cat(got[k]), want, 2e-5 if dtype == "float32" else 2e-2, f"sequence {k}")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("dim, size, decode", [(16, 24, False), (16, 24, True), (64, 32, False), (64, 32, True), (32, 200, True)])
def test_one_key_that_stands_out_at_the_edges_of_a_block(ops, dtype, dim, size, decode):
    """A key just outside the row's block of positions is scaled so that it would take all the weight if it
    were seen; one just inside (the block's first position, far from the row) so that it does take it."""
    g = torch.Generator().manual_seed(size)
    n = 2 * size + 2 if size < 100 else size + 40
    raw = torch.randn(n, 2 * dim, generator=g) * 0.3
    direction = torch.randn(dim, generator=g)
    direction /= direction.norm()
    rows = [size, 2 * size - 1] if size < 100 else [size - 1, size + 30]
    for r in rows:
        raw[r, :dim] = direction * 6                                 # the queries that are looked at
    start = rows[-1] // size * size
    raw[start, dim:] = direction * 12                                # just inside the last row's block
    raw[start - 1, dim:] = direction * 40                            # just outside it
    bias, conv = torch.zeros(2 * dim), torch.ones(2 * dim, 1)
    temp, r1, r2 = torch.ones(1), torch.full((1,), 0.3), torch.full((1,), 1.0)
    bench = _Bench(dtype, 1, 1, dim, 1, ("chunk", size), page=8, pages=n // 8 + 3)
    args = (bias, conv, 1.0, temp.cuda(), (r1.cuda(), r2.cuda()), ("chunk", size))
    if decode:
        head = rows[0] - 3
        outs = [bench.step(ops, {"a": head}, raw[:head], *args)] + [bench.step(ops, {"a": 1}, raw[i:i + 1], *args) for i in range(head, n)]
        out = torch.cat(outs)
    else:
        out = bench.step(ops, {"a": n}, raw, *args)
    want = _plain_mixer_core(raw, bias, conv, 1, 1, dim, 1.0, temp, r1, r2, size, DTYPES[dtype])
    _close(out[rows], want[rows], 2e-5 if dtype == "float32" else 2e-2, "rows at the edges")
    last = out[rows[-1]].double().cpu()
    inside = raw[start, dim:].to(DTYPES[dtype]).double()
    assert (last - inside).abs().max() <= 0.05 * inside.abs().max(), "the block's first key does not take the weight"


def test_token_shift_keeps_each_sequences_last_row(ops):
    from tiny_llm_infer_amd.parts.base import StepView
    g = torch.Generator().manual_seed(9)
    n, lens = 40, {0: 7, 2: 3}                                       # slot -> rows
    h = {s: torch.randn(c + 2, n, generator=g) for s, c in lens.items()}
    mu = torch.rand(n, generator=g)
    kept = torch.full((4, n), 99.0).cuda()                          # (what an earlier request left in the slots)
    i32 = lambda v: torch.tensor(v, dtype=torch.int32, device="cuda")

    def view(counts, starts):
        rs = [0] + list(np.cumsum(counts))
        return StepView(num_rows=sum(counts), num_seqs=2, token_ids=i32([0]), positions=i32([0]),
                        seq_of_row=i32([i for i, c in enumerate(counts) for _ in range(c)]), row_start=i32([int(r) for r in rs]),
                        seq_start=i32(starts), seq_len=i32([0, 0]), slots=i32(list(lens)), sample_rows=i32([0]),
                        h_row_start=[int(r) for r in rs], h_seq_start=starts, h_seq_len=[0, 0], h_slots=list(lens),
                        max_rows_per_seq=max(counts))
    first = torch.cat([h[0][:7], h[2][:3]])
    out1 = ops.token_shift(first.cuda(), mu.cuda(), kept, view([7, 3], [0, 0]), torch.float32)
    second = torch.cat([h[0][7:], h[2][3:]])
    out2 = ops.token_shift(second.cuda(), mu.cuda(), kept, view([2, 2], [7, 3]), torch.float32)
    for i, s in enumerate(lens):
        want = plain_sinepel.token_shift(h[s].double(), mu.double())
        got = torch.cat([out1[[0, 7][i]:[7, 10][i]], out2[2 * i:2 * i + 2]])
        _close(got, want, 1e-6, f"slot {s}")
    assert torch.equal(kept[1].cpu(), torch.full((n,), 99.0))


# ------------------------------------------------------------- the model, every cut ---
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("name", list(SMALL))
def test_all_cuts_match_plain(sinepel_folders, name, dtype):
    folder = sinepel_folders[name]
    reqs = _requests(name, [70, 45, 197, 33, 1, 58], seed=5)
    want = plain_logits(folder, reqs)
    max_tokens = 384
    cuts = {
        "whole": trace_whole(reqs),
        "decode": trace_prefill_then_decode(reqs),
        "portions": trace_portions(reqs, seed=3),
        "mixed": trace_mixed(reqs, max_tokens=max_tokens, seed=9),
    }
    for cut, steps in cuts.items():
        runner = _runner(folder, name, dtype, max_tokens)
        got = collect(steps, _replay(runner, steps))
        for rid in reqs:
            err, row, scale = max_error(got[rid], want[rid])
            assert err <= TOL[dtype] * scale, f"{name}/{dtype}/{cut}/{rid}: error {err:.3e} at token {row} (scale {scale:.3e})"
        runner.cache.check()
        assert not runner.cache.live() and runner.cache.free_pages() == runner.cache.pages_per_group()
        if cut == "mixed":
            assert runner.cache.pages_taken_total > runner.cache.num_pages


def test_long_decoding_through_recorded_launches(sinepel_folders):
    """150 tokens decoded one by one for three requests at once (bfloat16: the steps are replayed from
    recordings), over several blocks of positions and pages that are given back on the way."""
    folder = sinepel_folders["R"]
    reqs = _requests("R", [160, 171, 183], seed=77)
    want = plain_logits(folder, reqs)
    runner = _runner(folder, "R", "bfloat16", 768)
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
def test_greedy_generation_through_the_engine(sinepel_folders, dtype):
    from tiny_llm_infer_amd.engine.llm_engine import LLMEngine
    from tiny_llm_infer_amd.sampling.params import SamplingParams
    folder = sinepel_folders["P"]
    prompts = [random_prompt(200, n, 90 + n) for n in (4, 19, 30, 41)]
    eng = LLMEngine.from_folder(folder, dtype=dtype, max_model_len=128, page_size=16, num_kv_blocks=32, max_num_seqs=3,
                                max_num_batched_tokens=32)
    got = eng.generate(prompts, SamplingParams(max_tokens=10, ignore_eos=True))
    if dtype == "float32":
        assert [r.token_ids for r in got] == [plain_greedy(folder, p, 10) for p in prompts]
    else:
        # rounding may turn a close call: every token must be the plain implementation's choice or within
        # the rounding error of it, given the tokens before
        cfg, w = plain_sinepel.read_model(folder)
        for p, r in zip(prompts, got):
            logits = plain_sinepel.forward(cfg, w, p + r.token_ids)[len(p) - 1:-1]
            for z, t in zip(logits, r.token_ids):
                assert float(z.max() - z[t]) <= 2 * TOL["bfloat16"] * float(z.abs().max())
    eng.runner.cache.check()
    assert eng.runner.cache.free_pages() == eng.runner.cache.pages_per_group()


# ------------------------------------------------------------------ the command line ---
def test_the_programs_take_a_sinepel_folder(sinepel_folders, tmp_path):
    """bin/trace_run replays a mixed trace, model_main --infer generates greedily, and a model of random
    weights made from a config.json alone (what bench.py --designs runs) loads and generates."""
    import json
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder, vocab = sinepel_folders["Q"], SMALL["Q"][0]["vocab"]
    reqs = _requests("Q", [40, 9, 77, 23, 52], seed=12)
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
