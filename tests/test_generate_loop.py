"""The generation loop's decisions, against a fake backend (no GPU): stop tokens are not
emitted, shorter sequences end earlier and give their slot back at once, batches follow one
another, lengths and the context bound finish a request."""
from typing import List

import pytest

from agave_amd.engine.generate import GenerationStats, generate
from agave_amd.sampling import SamplingParams


class FakeBackend:
    """Next token = (last token fed + 1) % 50; records what it was asked."""

    def __init__(self, max_slots=3, max_context=64):
        self.max_slots, self.max_context = max_slots, max_context
        self.free = list(range(max_slots))
        self.length = {}
        self.steps: List[dict] = []
        self.max_live = 0

    def alloc_slot(self):
        s = self.free.pop(0)
        self.length[s] = 0
        self.max_live = max(self.max_live, len(self.length))
        return s

    def free_slot(self, s):
        assert s in self.length, "slot freed twice"
        del self.length[s]
        self.free.append(s)

    def step_sample(self, slots, tokens, rows):
        assert len(slots) == len(tokens) == len(rows) and len(set(slots)) == len(slots)
        for s, t in zip(slots, tokens):
            assert s in self.length and len(t) >= 1
            self.length[s] += len(t)
            assert self.length[s] <= self.max_context
        self.steps.append({"slots": list(slots), "n": [len(t) for t in tokens], "u": [r.u for r in rows],
                           "gen": [list(r.generated) for r in rows]})
        return [(t[-1] + 1) % 50 for t in tokens]


def test_stop_token_is_not_emitted_and_short_sequences_leave():
    be = FakeBackend()
    prompts = [[10, 11], [40], [5]]
    res = generate(be, prompts, SamplingParams(max_tokens=8), eos_ids=[13, 44])
    assert [r.tokens for r in res] == [[12], [41, 42, 43], [6, 7, 8, 9, 10, 11, 12]]
    assert [r.finish_reason for r in res] == ["stop", "stop", "stop"]
    assert be.steps[0]["n"] == [2, 1, 1]                       # unequal prompts in one step
    assert [len(s["slots"]) for s in be.steps] == [3, 3, 2, 2, 1, 1, 1, 1]   # the batch shrinks
    assert be.length == {} and sorted(be.free) == [0, 1, 2]


def test_max_tokens_and_context():
    be = FakeBackend(max_context=6)
    res = generate(be, [[1, 2, 3], [1, 2, 3, 4, 5, 6, 7]], SamplingParams(max_tokens=3, ignore_eos=True), eos_ids=[5])
    assert res[0].tokens == [4, 5, 6] and res[0].finish_reason == "length"      # eos ignored
    assert res[1].tokens == [] and res[1].finish_reason == "context"            # the prompt does not fit
    res = generate(be, [[1, 2, 3, 4]], SamplingParams(max_tokens=50))
    # 4 prompt positions + tokens fed back must stay within 6 positions
    assert res[0].finish_reason == "context" and res[0].tokens == [5, 6, 7]
    with pytest.raises(ValueError, match="empty"):
        generate(be, [[]])


def test_batches_follow_one_another_and_reuse_slots():
    be = FakeBackend(max_slots=2)
    stats = GenerationStats()
    res = generate(be, [[i] for i in range(5)], SamplingParams(max_tokens=2), stats=stats)
    assert [r.tokens for r in res] == [[i + 1, i + 2] for i in range(5)]
    assert stats.batches == 3 and be.max_live == 2
    assert stats.tokens == 10 and stats.prefill_tokens == 5 and stats.decode_tokens == 5
    assert [r.request for r in res] == list(range(5))


def test_per_request_streams_do_not_depend_on_batch_mates():
    p = SamplingParams(max_tokens=4, temperature=0.8, seed=3)
    a = FakeBackend(max_slots=3)
    generate(a, [[1], [2], [3]], p)
    b = FakeBackend(max_slots=1)
    generate(b, [[1], [2], [3]], p)
    ua = [[s["u"][s["slots"].index(sl)] for s in a.steps if sl in s["slots"]] for sl in (0, 1, 2)]
    ub = [[s["u"][0] for s in b.steps[i * 4:(i + 1) * 4]] for i in range(3)]
    assert ua == ub and len(set(ua[0])) == 4 and ua[0] != ua[1]
    c = FakeBackend(max_slots=3)
    generate(c, [[1], [2], [3]], SamplingParams(max_tokens=4, temperature=0.8, seed=4))
    assert c.steps[0]["u"] != a.steps[0]["u"]


def test_repeat_penalty_sees_generated_ids_only_after_the_first_token():
    be = FakeBackend(max_slots=1)
    generate(be, [[7, 8]], SamplingParams(max_tokens=3, repeat_penalty=1.3))
    assert [s["gen"][0] for s in be.steps] == [[], [9], [9, 10]]


def test_sampling_params_are_checked():
    for bad in (dict(max_tokens=0), dict(temperature=-1), dict(top_p=0.0), dict(top_p=1.5), dict(top_k=-1),
                dict(repeat_penalty=0)):
        with pytest.raises(ValueError):
            SamplingParams(**bad)


class AheadBackend(FakeBackend):
    """The same model with ``launch_step`` / ``finish_step``: a launched step's tokens may come from
    what the step before it sampled (``carry``), which the backend keeps as the device would."""

    def __init__(self, *a, **kw):
        super().__init__(*a, **kw)
        self.sampled: List[int] = []
        self.in_flight = 0
        self.max_in_flight = 0
        self.busy = set()                # slots of launched, unfinished steps

    def free_slot(self, s):
        assert s not in self.busy, "slot freed while a launched step still uses it"
        super().free_slot(s)

    def launch_step(self, slots, tokens, rows, carry=None):
        if carry is not None:
            assert tokens is None and len(carry) == len(slots)
            tokens = [[self.sampled[k]] for k in carry]
        self.sampled = self.step_sample(slots, tokens, rows)
        self.in_flight += 1
        self.max_in_flight = max(self.max_in_flight, self.in_flight)
        self.busy |= set(slots)
        return (list(self.sampled), list(slots))

    def finish_step(self, handle):
        toks, slots = handle
        self.in_flight -= 1
        self.busy -= set(slots)
        return toks


@pytest.mark.parametrize("prompts,params,eos", [
    ([[10, 11], [40], [5]], SamplingParams(max_tokens=8), [13, 44]),
    ([[1, 2, 3], [9], [30, 31]], SamplingParams(max_tokens=3, ignore_eos=True), [5]),
    ([[i] for i in range(7)], SamplingParams(max_tokens=5), [4, 9]),
    ([[1, 2, 3, 4], [2]], SamplingParams(max_tokens=50), []),
    ([[3]], SamplingParams(max_tokens=1), []),
])
def test_one_step_ahead_gives_the_same_results_and_loses_no_slot(prompts, params, eos):
    plain, ahead = FakeBackend(max_slots=3, max_context=9), AheadBackend(max_slots=3, max_context=9)
    sa, sb = GenerationStats(), GenerationStats()
    a = generate(plain, prompts, params, eos_ids=eos, stats=sa)
    b = generate(ahead, prompts, params, eos_ids=eos, stats=sb)
    assert [(r.tokens, r.finish_reason) for r in a] == [(r.tokens, r.finish_reason) for r in b]
    assert (sa.tokens, sa.prefill_tokens, sa.decode_tokens, sa.batches) == (sb.tokens, sb.prefill_tokens, sb.decode_tokens, sb.batches)
    assert ahead.length == {} and sorted(ahead.free) == [0, 1, 2] and ahead.in_flight == 0
    assert ahead.max_in_flight <= 2
    if len(prompts) > 1 or params.max_tokens > 1:
        assert ahead.max_in_flight == 2                         # it does run ahead


def test_one_step_ahead_keeps_each_request_stream_of_draws():
    p = SamplingParams(max_tokens=4, temperature=0.8, seed=3)
    a, b = FakeBackend(max_slots=3), AheadBackend(max_slots=3)
    generate(a, [[1], [2], [3]], p, eos_ids=[4])                # request 1 stops early: one step too many
    generate(b, [[1], [2], [3]], p, eos_ids=[4])
    for sl in (0, 1, 2):
        ua = [s["u"][s["slots"].index(sl)] for s in a.steps if sl in s["slots"]]
        ub = [s["u"][s["slots"].index(sl)] for s in b.steps if sl in s["slots"]]
        assert ub[:len(ua)] == ua and len(ub) - len(ua) in (0, 1)


def test_repeat_penalty_is_not_run_ahead():
    be = AheadBackend(max_slots=1)
    generate(be, [[7, 8]], SamplingParams(max_tokens=3, repeat_penalty=1.3))
    assert be.max_in_flight == 0 and [s["gen"][0] for s in be.steps] == [[], [9], [9, 10]]


def test_the_sampler_is_told_what_the_rows_need():
    """Which of the sampler's kernels a batch needs is decided on the host, from the rows'
    options, exactly as a row decides for itself on the device."""
    from agave_amd.ops import sampling as S

    class Row:
        def __init__(self, temperature, top_k=0, top_p=1.0):
            self.temperature, self.top_k, self.top_p = temperature, top_k, top_p
    vocab = 5000
    assert S.kinds_of([Row(0.0), Row(0.0, 40, 0.5)], vocab) == 0                    # greedy rows need neither
    assert S.kinds_of([Row(0.0), Row(0.7)], vocab) == S.KIND_TEMPERATURE
    assert S.kinds_of([Row(0.7, top_k=vocab)], vocab) == S.KIND_TEMPERATURE          # top-k of the whole row is none
    assert S.kinds_of([Row(0.7, top_p=1.0), Row(0.7, top_k=0)], vocab) == S.KIND_TEMPERATURE
    assert S.kinds_of([Row(0.7, top_k=3)], vocab) == S.KIND_ALL
    assert S.kinds_of([Row(0.0), Row(1.2, top_p=0.9)], vocab) == S.KIND_ALL


def test_command_line_options_follow_the_reference():
    """src/main.zig:325-382: names, short forms and defaults of the options this library has."""
    from agave_amd.cli import build_parser, parse_ids
    ap = build_parser()
    a = ap.parse_args(["m"])
    assert (a.max_tokens, a.temperature, a.top_p, a.top_k, a.repeat_penalty, a.seed) == (512, 0.0, 1.0, 0, 1.0, None)
    assert a.ctx_size is None and a.backend == "auto" and not (a.json or a.quiet or a.verbose or a.debug or a.profile)
    a = ap.parse_args(["m", "2 17 5", "-n", "9", "-t", "0.8", "--top-p", "0.9", "--top-k", "40", "--repeat-penalty", "1.1",
                       "--seed", "3", "--ctx-size", "0", "--prefill-batch-size", "512", "--json", "--model-info", "-q", "-V",
                       "-d", "--profile", "--backend", "rocm"])
    assert (a.max_tokens, a.temperature, a.top_p, a.top_k, a.repeat_penalty, a.seed) == (9, 0.8, 0.9, 40, 1.1, 3)
    assert a.ctx_size == 0 and a.prefill_batch_size == 512 and a.json and a.model_info and a.quiet and a.verbose
    assert a.debug and a.profile and a.backend == "rocm" and a.prompt == "2 17 5"
    assert parse_ids("2, 17  5") == [2, 17, 5]
    with pytest.raises(SystemExit):
        parse_ids("hello")


@pytest.mark.parametrize("backend_cls", [FakeBackend, AheadBackend])
def test_a_cancelled_call_returns_what_it_has_and_loses_no_slot(backend_cls):
    """The reference's cancel flag (src/models/gemma3.zig:141, 342), looked at between steps: requests
    that had ended keep their reason, the others and those still queued end as "cancelled"."""
    class Cancellable(backend_cls):
        def __init__(self, after, *a, **kw):
            super().__init__(*a, **kw)
            self.after, self.flag, self.cleared = after, False, 0

        def cancel_requested(self):
            return self.flag

        def clear_cancel(self):
            self.flag = False
            self.cleared += 1

        def step_sample(self, slots, tokens, rows):
            out = super().step_sample(slots, tokens, rows)
            if len(self.steps) == self.after:
                self.flag = True                      # as if another thread had called cancel() during this step
            return out

    # a request to cancel that arrives before the call's first step ends it there, and is used up by it
    be = Cancellable(10 ** 9, max_slots=2, max_context=64)
    be.flag = True
    res = generate(be, [[10], [20], [30]], SamplingParams(max_tokens=5), eos_ids=[])
    assert [r.finish_reason for r in res] == ["cancelled"] * 3 and all(r.tokens == [] for r in res)
    assert be.steps == [] and sorted(be.free) == [0, 1] and be.cleared == 1 and not be.flag
    res = generate(be, [[10]], SamplingParams(max_tokens=2), eos_ids=[])
    assert res[0].finish_reason == "length" and be.cleared == 1           # nothing to clear in a call that ran through

    be = Cancellable(4, max_slots=2, max_context=64)
    res = generate(be, [[10], [20], [30]], [SamplingParams(max_tokens=2), SamplingParams(max_tokens=30),
                                            SamplingParams(max_tokens=30)], eos_ids=[])
    assert be.cleared == 1
    assert res[0].finish_reason == "length" and res[0].tokens == [11, 12]
    assert res[1].finish_reason == "cancelled" and res[1].tokens[:3] == [21, 22, 23] and len(res[1].tokens) in (4, 5)
    assert res[2].finish_reason == "cancelled" and res[2].tokens == []         # never started
    assert be.length == {} and sorted(be.free) == [0, 1] and len(be.steps) <= 5
    # without a cancel the same call runs to its end
    be = Cancellable(10 ** 9, max_slots=2, max_context=64)
    res = generate(be, [[10], [20]], SamplingParams(max_tokens=6), eos_ids=[])
    assert [r.finish_reason for r in res] == ["length", "length"]


def test_log_probabilities_go_to_the_requests_that_ask():
    class WithLogprobs(FakeBackend):
        def step_sample(self, slots, tokens, rows):
            out = super().step_sample(slots, tokens, rows)
            self.last_logprobs = [-(t + 1) / 10 for t in out] if any(r.logprob for r in rows) else None
            return out

    be = WithLogprobs()
    res = generate(be, [[10], [20]], [SamplingParams(max_tokens=3, logprobs=True), SamplingParams(max_tokens=3)], eos_ids=[13])
    assert res[0].tokens == [11, 12] and res[0].finish_reason == "stop"            # 13 stops it and is not emitted
    assert res[0].logprobs == [-1.2, -1.3] and res[1].logprobs == [] and res[1].tokens == [21, 22, 23]


def test_replay_cuts_requests_into_the_steps_of_each_mode():
    """The step records that bin/trace_run makes from whole requests: every position is fed once,
    in order, and its logits are found where the plan says; batches end their requests as their
    tokens run out and never hold more than the plan's count of tokens."""
    from agave_amd.engine.replay import plan_steps, tokens_held
    reqs = [{"id": "a", "tokens": list(range(100, 140)), "prompt": 10, "batch": 0},
            {"id": "b", "tokens": list(range(200, 203)), "prompt": 3, "batch": 0},
            {"id": "c", "tokens": list(range(300, 370)), "batch": 1}]
    for mode in ("whole", "tail32", "batched"):
        records, where = plan_steps(mode, reqs)
        fed = {r["id"]: [] for r in reqs}
        live, ended = set(), set()
        for i, rec in enumerate(records):
            assert rec["step"] == i
            sizes = {len(e["tokens"]) for e in rec["entries"]}
            starts = [e["id"] not in live for e in rec["entries"]]
            assert all(starts) or (not any(starts) and sizes == {1})      # all start, or all go on by one token
            row = 0
            for e in rec["entries"]:
                assert e["id"] not in ended and e["want"] == list(range(len(e["tokens"])))
                for k, t in enumerate(e["tokens"]):
                    assert where[e["id"]][len(fed[e["id"]])] == (i, row + k)
                    fed[e["id"]].append(t)
                row += len(e["tokens"])
                live.add(e["id"])
            for rid in rec["end"]:
                live.discard(rid)
                ended.add(rid)
        assert fed == {r["id"]: r["tokens"] for r in reqs} and not live
        if mode == "whole":
            assert [len(r["entries"]) for r in records] == [1, 1, 1] and tokens_held(records) == 128
        if mode == "tail32":
            assert len(records) == (1 + 32) + (1 + 2) + (1 + 32)
        if mode == "batched":
            assert [e["id"] for e in records[0]["entries"]] == ["a", "b"] and records[0]["end"] == ["b"]
            assert len(records) == (1 + 30) + (1 + 32) and tokens_held(records) == 128
    with pytest.raises(ValueError, match="unknown mode"):
        plan_steps("sideways", reqs)
    with pytest.raises(ValueError, match="must differ"):
        plan_steps("whole", [reqs[0], reqs[0]])
