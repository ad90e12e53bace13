"""The Natilix family inside the engine (registry, loader, scheduler, paged KV + state slots,
kernels) against the plain oracle of ``natilix_oracle``: whole prompts, token-by-token
decoding, portions down to two tokens, mixed batches against each request alone, blocks and
slots that are used again, long decoding, first tokens, other sizes, greedy generation through
``LLMEngine.generate``.  Every test runs on the CPU (fp32); the ``gpu`` variants run the HIP
kernels in float32 and bfloat16."""
import pytest
import torch

import natilix_fixtures as fx
from natilix_oracle import Oracle

from minivllm_amd.engine.llm_engine import LLMEngine
from minivllm_amd.models.registry import config_from_path
from minivllm_amd.sampling_parameters import SamplingParams

CASES = [pytest.param("cpu", "float32", id="cpu-fp32"),
         pytest.param("cuda", "float32", id="gpu-fp32", marks=pytest.mark.gpu),
         pytest.param("cuda", "bfloat16", id="gpu-bf16", marks=pytest.mark.gpu)]


def make_engine(tmp_path, c, w, device, dtype, blocks=24, block_size=8, seqs=3, score=True, **kw):
    folder = fx.save_checkpoint(str(tmp_path / "ckpt"), c, w)
    mc = config_from_path(folder)
    mc.max_position = blocks * block_size
    cfg = dict(model=mc, checkpoint_path=folder, dtype=dtype, device=device,
               block_size=block_size, max_cached_blocks=blocks, max_num_sequences=seqs,
               max_model_length=blocks * block_size,
               max_num_batched_tokens=blocks * block_size, eos=-1, score_only=score,
               graph_batch_sizes=[1, 2, seqs], tuned_gemms=False)
    cfg.update(kw)
    return LLMEngine(cfg)


def tokens(n, vocab, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, vocab, (n,), generator=g).tolist()


def close(got, want, dtype):
    """Error measure of a logit row: spread of the difference over the vocabulary, relative
    to the spread of the logits themselves."""
    if isinstance(want, Expected):
        n = want.logits.shape[0] if dtype == "float32" else want.sure
        got, want = got[:n], want.logits[:n]
        if n == 0:
            return
    d = got.double() - want.double()
    d = d - d.mean(-1, keepdim=True)
    e = d.pow(2).mean(-1).sqrt() / want.double().std(-1)
    # float32 pins the computation; bfloat16 runs the same kernel templates with 16-bit loads
    # and stores, so there the bound is what rounding does to these small, high-gain models
    # (a peaked softmax or a routing weight amplifies single roundings): typical rows tight,
    # the worst row loose
    lim = 2e-4 if dtype == "float32" else 0.25
    assert float(e.max()) < lim, f"logits differ: {float(e.max()):.3g} (limit {lim})"
    if dtype != "float32":
        assert float(e.median()) < 0.04, f"typical row differs: {float(e.median()):.3g}"


def run_schedule(eng, reqs, schedule):
    """``schedule``: list of steps, each a list of (name, count).  Returns name -> [len, V]."""
    at = {k: 0 for k in reqs}
    got = {k: [] for k in reqs}
    for step in schedule:
        entries, end = [], []
        for name, n in step:
            lo = at[name]
            entries.append({"id": name, "tokens": reqs[name][lo:lo + n], "want": list(range(n))})
            at[name] = lo + n
            if at[name] == len(reqs[name]):
                end.append(name)
        out = eng.score_step(entries, end)
        for name, _ in step:
            got[name].append(out[name])
    return {k: torch.cat(v) for k, v in got.items() if v}


class Expected:
    """The oracle's logits for a token list, and the first token at which one of its routing
    decisions is a close call (16-bit rounding may decide it the other way, and the recurrent
    state then carries the difference on): bfloat16 runs are compared up to there."""

    def __init__(self, c, w, toks):
        o = Oracle(c, w)
        self.logits = o.feed(toks).float()
        close_calls = [t for t, m in enumerate(o.margin) if m < 0.08]
        self.sure = close_calls[0] if close_calls else len(toks)
        self.trace = o.trace


def oracle_logits(c, w, toks):
    return Expected(c, w, toks)


@pytest.mark.parametrize("device,dtype", CASES)
def test_whole_prompt_and_every_layer(tmp_path, device, dtype):
    c, w = fx.default_config(), fx.weights(fx.default_config(), 1)
    toks = tokens(37, c["vocab"], 2)
    eng = make_engine(tmp_path, c, w, device, dtype)
    seen = []
    eng.model_runner.model.model.layer_hook = lambda i, x: seen.append(x.detach().float().cpu().clone())
    got = run_schedule(eng, {"a": toks}, [[("a", len(toks))]])["a"]
    want = oracle_logits(c, w, toks)
    close(got, want, dtype)
    assert len(seen) == len(c["layers"])
    n = len(toks) if dtype == "float32" else want.sure
    assert n >= 10, "the fixture's routing is a close call too early for a 16-bit comparison"
    for x, ref in zip(seen, want.trace):
        lim = 1e-4 if dtype == "float32" else 0.15
        assert float((x[:n] - ref.float()[:n]).abs().max()) < lim * float(ref.abs().max())
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_token_by_token_equals_prefill(tmp_path, device, dtype):
    c, w = fx.default_config(), fx.weights(fx.default_config(), 3)
    toks = tokens(29, c["vocab"], 4)
    eng = make_engine(tmp_path, c, w, device, dtype)
    want = oracle_logits(c, w, toks)
    got = run_schedule(eng, {"a": toks}, [[("a", 1)] for _ in toks])["a"]     # first tokens, then decode
    close(got, want, dtype)
    got = run_schedule(eng, {"b": toks}, [[("b", 20)]] + [[("b", 1)]] * 9)["b"]
    close(got, want, dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
@pytest.mark.parametrize("cuts", [[2, 2, 3, 1, 9, 8, 2, 16, 2, 5], [7, 43], [1, 2, 47], [25, 25]])
def test_portions_cut_anywhere(tmp_path, device, dtype, cuts):
    c, w = fx.default_config(), fx.weights(fx.default_config(), 5)
    toks = tokens(sum(cuts), c["vocab"], 6)
    eng = make_engine(tmp_path, c, w, device, dtype)
    got = run_schedule(eng, {"a": toks}, [[("a", n)] for n in cuts])["a"]
    close(got, oracle_logits(c, w, toks), dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_mixed_batches_equal_each_request_alone(tmp_path, device, dtype):
    c, w = fx.default_config(), fx.weights(fx.default_config(), 7)
    reqs = {"a": tokens(41, c["vocab"], 8), "b": tokens(5, c["vocab"], 9), "c": tokens(23, c["vocab"], 10),
            "d": tokens(1, c["vocab"], 11), "e": tokens(18, c["vocab"], 12)}
    sched = [[("a", 9), ("b", 2)],
             [("a", 1), ("b", 1), ("c", 17)],              # a one-token portion next to a prompt
             [("b", 1), ("c", 1)],                         # decode step of two; a sits out
             [("a", 20), ("b", 1), ("c", 1)],              # b ends: its slot and blocks return
             [("a", 1), ("c", 1), ("d", 1)],               # d takes b's slot, first token alone
             [("e", 3), ("a", 1), ("c", 1)],
             [("e", 15), ("a", 9), ("c", 2)]]
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=14, seqs=3)
    got = run_schedule(eng, reqs, sched)
    for k, toks in reqs.items():
        close(got[k], oracle_logits(c, w, toks), dtype)
    bm = eng.scheduler.block_manager
    assert bm.num_free_blocks == bm.num_blocks and eng.scheduler.state_pool.num_free == 3
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_pool_and_slots_used_again(tmp_path, device, dtype):
    """Two slots, a KV pool of just over one request: every later request runs on blocks and a
    slot that an earlier one has left dirty."""
    c, w = fx.default_config(), fx.weights(fx.default_config(), 13)
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=9, seqs=2)
    for i, n in enumerate([60, 33, 64, 9, 2]):
        toks = tokens(n, c["vocab"], 20 + i)
        cut = max(1, n // 3)
        got = run_schedule(eng, {"r": toks}, [[("r", cut)], [("r", n - cut)]] if n > 1 else [[("r", 1)]])["r"]
        close(got, oracle_logits(c, w, toks), dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_long_decoding_over_many_blocks(tmp_path, device, dtype):
    c = fx.config([(fx.attention(heads=2, kv_heads=2, dim=8, vdim=8, rot_dims=8, original=16), None),
                   (fx.delta(heads=1, kv_heads=1, dim=16, vdim=4, conv=4), fx.moe(experts=4, top=4, groups=2, keep=2))],
                  width=24, vocab=61, bigram=None)
    w = fx.weights(c, 14)
    toks = tokens(150, c["vocab"], 15)
    eng = make_engine(tmp_path, c, w, device, dtype, blocks=40, block_size=4)
    got = run_schedule(eng, {"a": toks}, [[("a", 3)]] + [[("a", 1)]] * 147)["a"]
    close(got, oracle_logits(c, w, toks), dtype)
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_sizes_that_happen_to_be_one_or_equal(tmp_path, device, dtype):
    """One head, one expert group, top = every expert, taps = 1, heads == kv heads, rotation on
    the whole head, a single layer of each kind."""
    for layers in ([(fx.attention(heads=1, kv_heads=1, dim=8, vdim=8, rot_dims=8, v_mix=False),
                     fx.moe(experts=2, top=2, groups=1, keep=1))],
                   [(fx.delta(heads=1, kv_heads=1, dim=8, vdim=8, conv=1), None)],
                   [(fx.delta(heads=6, kv_heads=3, dim=4, vdim=36, conv=6), fx.moe(experts=8, top=3, groups=4, keep=2)),
                    (fx.attention(heads=8, kv_heads=1, dim=6, vdim=70, rot_dims=2), None)]):
        c = fx.config(layers, width=16, vocab=50)
        w = fx.weights(c, 16)
        toks = tokens(21, c["vocab"], 17)
        eng = make_engine(tmp_path, c, w, device, dtype)
        got = run_schedule(eng, {"a": toks}, [[("a", 2)], [("a", 12)]] + [[("a", 1)]] * 7)["a"]
        close(got, oracle_logits(c, w, toks), dtype)
        eng.exit()


@pytest.mark.parametrize("device,dtype", CASES)
def test_greedy_generation_through_the_scheduler(tmp_path, device, dtype):
    c, w = fx.default_config(), fx.weights(fx.default_config(), 18)
    prompts = [tokens(n, c["vocab"], 30 + n) for n in (11, 3, 26, 1)]
    eng = make_engine(tmp_path, c, w, device, dtype, score=False, seqs=3, blocks=30,
                      max_num_batched_tokens=32)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=10, ignore_eos=True))
    for p, gen in zip(prompts, out["token_ids"]):
        orc = Oracle(c, w)
        lg = orc.feed(p)[-1]
        for t in gen:
            top2 = lg.topk(2).values
            if dtype == "bfloat16" and float(top2[0] - top2[1]) < 0.15:
                break                      # a near tie: 16-bit rounding may pick either
            assert int(lg.argmax()) == t
            lg = orc.feed([t])[-1]
    eng.exit()


@pytest.mark.parametrize("device,dtype", CASES[:2])
def test_generation_survives_preemption_and_mixed_steps(tmp_path, device, dtype):
    """A KV pool too small for all requests at once (sequences are preempted and prefetched
    again from position 0: their state slot and blocks have been used by others meanwhile) and
    running sequences riding along with prefill steps: greedy tokens still equal the oracle's."""
    c, w = fx.default_config(), fx.weights(fx.default_config(), 19)
    prompts = [tokens(n, c["vocab"], 60 + n) for n in (21, 17, 9, 30)]
    eng = make_engine(tmp_path, c, w, device, dtype, score=False, seqs=3, blocks=11, block_size=8,
                      max_num_batched_tokens=24, enable_mixed_batches=True)
    out = eng.generate(prompts, SamplingParams(temperature=0.0, max_tokens=14, ignore_eos=True))
    assert eng.scheduler.num_preemptions > 0 and eng.scheduler.num_mixed_steps > 0
    for p, gen in zip(prompts, out["token_ids"]):
        orc = Oracle(c, w)
        lg = orc.feed(p)[-1]
        for t in gen:
            assert int(lg.argmax()) == t
            lg = orc.feed([t])[-1]
    assert eng.scheduler.state_pool.num_free == 3
    eng.exit()
