"""The scheduler's decisions, with a fake engine that scripts logits and records what ran
(the reference tests its scheduler the same way: src/engine.rs:3158-3599)."""
import pytest
import torch

from macllm_infer_amd.cache import CacheExhausted
from macllm_infer_amd.engine.scheduler import EngineConfig, QueueFull, Scheduler
from macllm_infer_amd.sampling import GREEDY, SamplingParams


class FakeCache:
    def __init__(self, engine):
        self.engine = engine

    def can_ever_fit(self, tokens):
        return tokens <= self.engine.capacity


class FakeEngine:
    """Next token = (last token of the lane + 1) % vocab; counts pages of ``page`` tokens."""
    vocab_size = 50
    max_context = 200

    def __init__(self, capacity=10_000, page=4):
        self.capacity, self.page = capacity, page
        self.lengths = {}
        self.calls = []
        self.cache = FakeCache(self)

    def add_request(self, request):
        assert request not in self.lengths
        self.lengths[request] = 0

    def finish(self, request):
        del self.lengths[request]

    def pages(self, lengths):
        return sum(-(-length // self.page) for length in lengths)

    def step(self, lanes):
        grown = dict(self.lengths)
        for lane in lanes:
            grown[lane.request] += len(lane.tokens)
        if self.pages(grown.values()) * self.page > self.capacity:
            raise CacheExhausted("pages", 1, 0, self.capacity // self.page)
        self.calls.append([(lane.request, list(lane.tokens), self.lengths[lane.request], list(lane.want))
                           for lane in lanes])
        self.lengths = grown
        rows = []
        for lane in lanes:
            for place in lane.want:
                row = torch.zeros(self.vocab_size)
                row[(lane.tokens[place] + 1) % self.vocab_size] = 5.0
                rows.append(row)
        return torch.stack(rows) if rows else torch.zeros(0, self.vocab_size)


class ArgmaxSampler:
    def sample(self, logits, rows):
        assert logits.shape[0] == len(rows)
        return torch.argmax(logits, dim=-1).tolist()


def run(prompts, params=GREEDY, config=None, engine=None, stop=()):
    engine = engine or FakeEngine()
    scheduler = Scheduler(engine, ArgmaxSampler(), config or EngineConfig(), stop)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, params if isinstance(params, SamplingParams) else params[index])
    finished = scheduler.run()
    return engine, scheduler, finished


def test_prompt_is_cut_into_portions_and_only_the_last_is_sampled():
    params = SamplingParams(max_new_tokens=3, temperature=0.0)
    engine, _, finished = run([[1, 2, 3, 4, 5, 6, 7]], params,
                              EngineConfig(scheduler_token_budget=3, prefill_token_quantum=3))
    portions = [call[0] for call in engine.calls]
    assert [(p[1], p[2], p[3]) for p in portions[:3]] == [([1, 2, 3], 0, []), ([4, 5, 6], 3, []), ([7], 6, [0])]
    assert [(p[1], p[2]) for p in portions[3:]] == [([8], 7), ([9], 8)]          # decoded tokens, one each
    assert finished[0].generated == [8, 9, 10] and finished[0].finish_reason == "length"
    assert engine.lengths == {}                                                    # everything given back


def test_token_budget_and_round_robin():
    """Budget 4, quantum 3: requests not reached keep their place and go first next round
    (src/engine.rs:4968)."""
    params = SamplingParams(max_new_tokens=2, temperature=0.0)
    engine, _, finished = run([[1, 2, 3, 4, 5], [10, 11, 12, 13, 14], [20]], params,
                              EngineConfig(scheduler_token_budget=4, prefill_token_quantum=3))
    for call in engine.calls:
        assert sum(len(tokens) for _, tokens, _, _ in call) <= 4
    first = [(request, tokens) for request, tokens, _, _ in engine.calls[0]]
    assert first == [(0, [1, 2, 3]), (1, [10])]
    second = [(request, tokens) for request, tokens, _, _ in engine.calls[1]]
    assert second[0] == (2, [20])                       # the unvisited request is first in line
    assert {k: v.generated for k, v in finished.items()} == {0: [6, 7], 1: [15, 16], 2: [21, 22]}


def test_mixed_rows_stay_aligned():
    """Portions of prompts beside decoded tokens: logits row i belongs to the i-th sampled lane
    (src/engine.rs:4701)."""
    params = [SamplingParams(max_new_tokens=4, temperature=0.0), SamplingParams(max_new_tokens=2, temperature=0.0)]
    engine, _, finished = run([[5], [30, 31, 32, 33, 34, 35]], params,
                              EngineConfig(scheduler_token_budget=4, prefill_token_quantum=3))
    assert finished[0].generated == [6, 7, 8, 9] and finished[1].generated == [36, 37]
    mixed = [call for call in engine.calls if len(call) == 2 and {len(call[0][1]), len(call[1][1])} == {1, 3}]
    assert mixed, "a decode token ran beside a prompt portion"


def test_admission_limits_and_rejections():
    engine = FakeEngine(capacity=40)
    params = SamplingParams(max_new_tokens=4, temperature=0.0)
    scheduler = Scheduler(engine, ArgmaxSampler(), EngineConfig(max_active_sequences=2, queue_capacity=5))
    scheduler.submit("empty", [], params)
    scheduler.submit("vocab", [1, 50], params)
    scheduler.submit("context", list(range(10)) * 20, params)
    scheduler.submit("capacity", list(range(40)), params)
    scheduler.submit("ok1", [1, 2], params)
    with pytest.raises(QueueFull):
        scheduler.submit("late", [1], params)
    scheduler.step()
    scheduler.submit("ok2", [3], params)
    scheduler.submit("ok3", [4], params)
    finished = scheduler.run()
    assert finished["empty"].finish_reason == "rejected: prompt must contain at least one token"
    assert "vocabulary" in finished["vocab"].finish_reason and "context" in finished["context"].finish_reason
    assert "cache capacity" in finished["capacity"].finish_reason
    assert all(len(call) <= 2 for call in engine.calls)            # never more than two live
    assert finished["ok3"].generated == [5, 6, 7, 8]


def test_stop_token_is_not_emitted_and_ignore_eos():
    _, _, finished = run([[1]], SamplingParams(max_new_tokens=8, temperature=0.0), stop=(4,))
    assert finished[0].generated == [2, 3] and finished[0].finish_reason == "stop"
    _, _, finished = run([[1]], SamplingParams(max_new_tokens=5, temperature=0.0, ignore_eos=True), stop=(4,))
    assert finished[0].generated == [2, 3, 4, 5, 6] and finished[0].finish_reason == "length"
    _, _, finished = run([[1]], SamplingParams(max_new_tokens=5, temperature=0.0, stop_token_ids=(3,)))
    assert finished[0].generated == [2] and finished[0].finish_reason == "stop"


def test_page_pressure_drops_the_last_lane_for_a_round():
    """Pages for 6 tokens (3 pages of 2): three 2-token prompts fill them; decoding then needs
    a fourth page... the round shrinks until it fits (src/engine.rs:4845)."""
    engine = FakeEngine(capacity=12, page=4)
    params = SamplingParams(max_new_tokens=1, temperature=0.0)
    _, scheduler, finished = run([[1, 2, 3, 4], [5, 6, 7, 8], [9, 10, 11, 12], [13, 14, 15, 16]], params,
                                 engine=engine)
    assert all(request.finish_reason == "length" for request in finished.values())
    assert len(engine.calls[0]) == 3                                  # the fourth lane waited
    assert [request for request, _, _, _ in engine.calls[1]] == [3]


def test_irreducible_pressure_fails_only_that_request():
    """Two requests whose growth cannot both fit: the one whose single lane cannot be reserved
    fails with resource_exhausted and frees its pages; the other completes
    (src/engine.rs:4898)."""
    engine = FakeEngine(capacity=16, page=4)
    params = SamplingParams(max_new_tokens=6, temperature=0.0)
    _, _, finished = run([[1, 2, 3, 4, 5, 6, 7], [20, 21, 22, 23, 24, 25, 26]], params, engine=engine)
    reasons = sorted(request.finish_reason for request in finished.values())
    assert reasons == ["length", "resource_exhausted"]
    done = [request for request in finished.values() if request.finish_reason == "length"][0]
    assert len(done.generated) == 6
    assert engine.lengths == {}


def test_scheduler_settings_are_checked():
    with pytest.raises(ValueError):
        EngineConfig(prefill_token_quantum=10, scheduler_token_budget=5)
    with pytest.raises(ValueError):
        SamplingParams(top_p=0.0)
    with pytest.raises(ValueError):
        SamplingParams(temperature=-1.0)
    with pytest.raises(ValueError):
        SamplingParams(repetition_penalty=0.0)
    defaults = SamplingParams()                # the reference's defaults, src/sampling.rs:23-33
    assert (defaults.temperature, defaults.top_k, defaults.top_p, defaults.repetition_penalty, defaults.seed,
            defaults.max_new_tokens) == (0.7, 20, 0.8, 1.1, 42, 128)


def test_cancelled_requests_never_start_or_stop_before_their_next_token():
    """A request cancelled while it waits holds nothing and never runs; one cancelled while it
    decodes ends before its next token is emitted and gives back what it holds; the others go on
    (src/engine.rs:1668-1672, src/generation.rs:1217-1220)."""
    engine = FakeEngine()
    params = SamplingParams(max_new_tokens=6, temperature=0.0)

    def on_token(request, token):
        if request.request_id == 0 and len(request.generated) == 2:
            request.cancel()

    scheduler = Scheduler(engine, ArgmaxSampler(), EngineConfig(max_active_sequences=2), (), on_token)
    for index, prompt in enumerate([[1, 2, 3], [10, 11], [20, 21]]):
        scheduler.submit(index, prompt, params)
    assert scheduler.cancel(2) and not scheduler.cancel("nobody")
    finished = scheduler.run()
    assert finished[2].finish_reason == "cancelled" and finished[2].generated == []
    assert all(request != 2 for call in engine.calls for request, _, _, _ in call)
    assert finished[0].finish_reason == "cancelled" and finished[0].generated == [4, 5]     # the third was not emitted
    assert finished[1].finish_reason == "length" and finished[1].generated == [12, 13, 14, 15, 16, 17]
    assert engine.lengths == {}


def test_a_request_cancelled_between_rounds_is_finished_before_the_next():
    engine = FakeEngine()
    scheduler = Scheduler(engine, ArgmaxSampler(), EngineConfig(scheduler_token_budget=2, prefill_token_quantum=2))
    scheduler.submit("a", [1, 2, 3, 4, 5, 6], SamplingParams(max_new_tokens=4, temperature=0.0))
    scheduler.step()
    assert engine.lengths == {"a": 2}
    assert scheduler.cancel("a")
    done = scheduler.step()
    assert [request.finish_reason for request in done] == ["cancelled"] and engine.lengths == {} and len(engine.calls) == 1


def test_the_callers_own_stop_condition_ends_a_request_after_the_token():
    """``on_token`` returning False is the caller's stop sequence: the token stays emitted and the
    reason is "stop" (src/generation.rs:1244-1254)."""
    engine = FakeEngine()
    scheduler = Scheduler(engine, ArgmaxSampler(), EngineConfig(), (), lambda request, token: token != 7)
    scheduler.submit("a", [4], SamplingParams(max_new_tokens=10, temperature=0.0))
    finished = scheduler.run()
    assert finished["a"].generated == [5, 6, 7] and finished["a"].finish_reason == "stop"


def test_a_portion_that_does_not_end_its_prompt_is_cut_to_the_size_the_engine_prefers():
    """An engine whose steps run best at certain sizes says so; the scheduler then cuts a portion that would be
    cut anyway a few tokens shorter, never one that ends its prompt, never below one token, and the tokens it
    left come with the next portion."""
    class Sized(FakeEngine):
        max_context = 400

        def step_token_target(self, lanes, tokens):
            return tokens - tokens % 16 if tokens - tokens % 16 > lanes else tokens      # multiples of 16

    engine = Sized()
    prompt = [index % 50 for index in range(100)]
    params = SamplingParams(max_new_tokens=3, temperature=0.0)
    config = EngineConfig(max_active_sequences=2, scheduler_token_budget=45, prefill_token_quantum=40)
    engine, scheduler, finished = run([[7, 8, 9], prompt], params, config, engine)
    steps = [[(request, len(tokens)) for request, tokens, _, _ in call] for call in engine.calls]
    # the first round: the short prompt whole (it ends: untouched) beside 40 of the long one: 43 tokens -> 32
    assert steps[0] == [(0, 3), (1, 29)]
    # the second round: a decoded token beside a portion of 40: 41 -> 32
    assert steps[1] == [(0, 1), (1, 31)]
    # the third round: the last 40 tokens end the prompt: not cut, although 41 is no preferred size
    assert steps[2] == [(0, 1), (1, 40)] and engine.calls[2][1][3] == [39]
    assert sum(count for step in steps[:3] for request, count in step if request == 1) == 100
    assert finished[1].generated == [(prompt[-1] + 1) % 50, (prompt[-1] + 2) % 50, (prompt[-1] + 3) % 50]
    assert finished[0].generated == [10, 11, 12]


class AheadEngine(FakeEngine):
    """A fake engine whose lanes may take their token from the device (``Lane.feed``)."""
    feeds_tokens = True

    def step(self, lanes):
        for lane in lanes:
            if lane.feed is not None:
                source, row = lane.feed
                lane.tokens = [int(source[row])]
        return super().step(lanes)


class AsyncArgmaxSampler(ArgmaxSampler):
    """Leaves its tokens "on the device": the scheduler then queues a round before it has read the one before."""
    class Handle:
        def __init__(self, tokens):
            self.device = tokens

        def wait(self):
            return self.device.tolist()

    def sample_async(self, logits, rows):
        assert logits.shape[0] == len(rows)
        return self.Handle(torch.argmax(logits, dim=-1).to(torch.int32))


@pytest.mark.parametrize("prompts, stopper", [([[1, 2, 3], [11, 12, 13]], 0), ([[11, 12, 13], [1, 2, 3]], 1)])
@pytest.mark.parametrize("ahead", [True, False])
def test_a_stop_token_on_its_way_while_a_single_lane_finds_no_pages(prompts, stopper, ahead):
    """Two pages of four tokens, two requests of three prompt tokens: the round in which both want a second page
    shrinks to the first request's lane, which alone does not fit either.  The round before is then still on its way,
    and its token for the request that counts 4, 5 is that request's stop token.  Whether the lane without pages
    belongs to the request that stops (it must end once, with "stop") or to the other one (which fits as soon as the
    stopped request's page is back, and must not fail with resource_exhausted), the outcome is the one of a scheduler
    that waits for every round's tokens."""
    engine = AheadEngine(capacity=8, page=4)
    scheduler = Scheduler(engine, AsyncArgmaxSampler(), EngineConfig(), (5,))
    assert scheduler.ahead
    scheduler.ahead = ahead
    params = SamplingParams(max_new_tokens=6, temperature=0.0)
    for index, prompt in enumerate(prompts):
        scheduler.submit(index, prompt, params)
    finished = scheduler.run()
    other = 1 - stopper
    assert finished[stopper].finish_reason == "stop" and finished[stopper].generated == [4]
    assert finished[other].finish_reason == "length" and finished[other].generated == [14, 15, 16, 17, 18, 19]
    assert engine.lengths == {} and not scheduler.active


def test_a_single_lane_without_pages_and_nothing_on_its_way_fails_alone_a_round_ahead():
    """The same pressure with no stop token anywhere: nothing that is on its way can free a page, so the request
    whose lane cannot grow fails with resource_exhausted, once, and the other runs to its length."""
    engine = AheadEngine(capacity=8, page=4)
    scheduler = Scheduler(engine, AsyncArgmaxSampler(), EngineConfig())
    params = SamplingParams(max_new_tokens=6, temperature=0.0)
    for index, prompt in enumerate([[1, 2, 3], [11, 12, 13]]):
        scheduler.submit(index, prompt, params)
    finished = scheduler.run()
    assert sorted(request.finish_reason for request in finished.values()) == ["length", "resource_exhausted"]
    assert engine.lengths == {} and not scheduler.active


class ConstrainedSampler(AsyncArgmaxSampler):
    """The best allowed token of every row (what the sampler's mask and argmax make of a row)."""
    def _masked(self, logits, rows):
        logits = logits.clone()
        for index, row in enumerate(rows):
            if row.allowed is not None:
                kept = torch.full_like(logits[index], float("-inf"))
                kept[list(row.allowed)] = logits[index, list(row.allowed)]
                logits[index] = kept
        return logits

    def sample(self, logits, rows):
        return super().sample(self._masked(logits, rows), rows)

    def sample_async(self, logits, rows):
        return super().sample_async(self._masked(logits, rows), rows)


@pytest.mark.parametrize("ahead", [True, False])
def test_a_constraint_that_follows_the_generated_tokens_is_asked_with_all_of_them(ahead):
    """The fake model wants last + 1; request 0 may only take last + 2 (of what it generated last, or 20 to begin
    with), request 1 only tokens of a fixed list, request 2 anything, and request 3's constraint allows nothing
    after two tokens.  A round ahead, the scheduler reads the round on its way before it asks request 0's
    constraint; the outcome is that of the scheduler that waits, and request 3 fails alone."""
    engine = AheadEngine()
    scheduler = Scheduler(engine, ConstrainedSampler(), EngineConfig(), ())
    scheduler.ahead = ahead
    asked = []

    def plus_two(generated):
        asked.append(list(generated))
        return [(generated[-1] + 2) % 50] if generated else [20]

    common = dict(max_new_tokens=5, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    scheduler.submit(0, [1, 2, 3], SamplingParams(allowed_token_ids=plus_two, **common))
    scheduler.submit(1, [7, 8], SamplingParams(allowed_token_ids=(30, 31, 40), **common))
    scheduler.submit(2, [11, 12, 13, 14], SamplingParams(**common))
    scheduler.submit(3, [5], SamplingParams(allowed_token_ids=lambda generated: [9] if len(generated) < 2 else [], **common))
    finished = scheduler.run()
    assert finished[0].generated == [20, 22, 24, 26, 28] and finished[0].finish_reason == "length"
    assert asked == [[], [20], [20, 22], [20, 22, 24], [20, 22, 24, 26]]      # every call saw every token before it
    assert set(finished[1].generated) <= {30, 31, 40} and len(finished[1].generated) == 5
    assert finished[2].generated == [15, 16, 17, 18, 19]
    assert finished[3].generated == [9, 9] and finished[3].finish_reason.startswith("failed")
    assert "rejected every token" in finished[3].finish_reason
    assert not engine.lengths                                                 # everything was given back
    # the constrained request's lanes carried the tokens it generated, never one still on its way
    lanes_of_0 = [tokens for call in engine.calls for request, tokens, _, _ in call if request == 0]
    assert lanes_of_0 == [[1, 2, 3], [20], [22], [24], [26]]


def test_a_constraint_beyond_the_vocabulary_ends_its_request_alone():
    """A fixed list that names a token the model does not have is refused at admission; a list that comes to name one
    later ends its request there; the request beside them runs to its length."""
    engine = AheadEngine()
    scheduler = Scheduler(engine, ConstrainedSampler(), EngineConfig(), ())
    common = dict(max_new_tokens=4, temperature=0.0, top_k=0, top_p=1.0, repetition_penalty=1.0)
    scheduler.submit(0, [1, 2], SamplingParams(allowed_token_ids=(3, 50), **common))                  # the vocabulary is 0 .. 49
    scheduler.submit(1, [4, 5], SamplingParams(allowed_token_ids=lambda generated: [7] if len(generated) < 2 else [77], **common))
    scheduler.submit(2, [9], SamplingParams(**common))
    finished = scheduler.run()
    assert finished[0].finish_reason.startswith("rejected") and "allowed_token_ids" in finished[0].finish_reason
    assert finished[0].generated == []
    assert finished[1].generated == [7, 7] and "outside the model vocabulary" in finished[1].finish_reason
    assert finished[2].generated == [10, 11, 12, 13] and finished[2].finish_reason == "length"
    assert not engine.lengths


def test_allowed_token_ids_are_checked_where_they_are_given():
    with pytest.raises(ValueError, match="at least one token"):
        SamplingParams(allowed_token_ids=())
    with pytest.raises(ValueError, match="at least one token"):
        SamplingParams(allowed_token_ids=(3, -1))
    params = SamplingParams(allowed_token_ids=[4, 2])
    assert params.allowed_token_ids == (4, 2) and params.allowed_after([1, 2]) == (4, 2) and not params.constrained_by_history
    follows = SamplingParams(allowed_token_ids=lambda generated: None if not generated else [generated[-1]])
    assert follows.constrained_by_history and follows.allowed_after([]) is None and follows.allowed_after([3, 8]) == (8,)
