"""The rollout runner and coordinator over a scripted engine (host logic; scenarios follow the reference's
tests/test_rollout.py:100-121, 241-508, 510-560 and 692-700, with a queue-backed stand-in for its environments)."""
import asyncio
from collections import deque
from dataclasses import dataclass
from types import SimpleNamespace

import pytest

from climbing_gym_amd.rollout import (DirectHarness, Harness, HarnessRequest, HarnessState, RolloutConfig, RolloutCoordinator,
                                      RolloutCoordinatorConfig, RolloutRunner, RolloutRunnerConfig, build_trajectory_turn)
from climbing_gym_amd.types import GenerationOutput, GenerationResult


@dataclass
class Plan:
    text: str
    delay: float = 0.0


class ScriptedEngine:
    """Answers requests with the next plan of a list; an aborted request gives its plan back."""

    def __init__(self, plans):
        self.plans, self.held = deque(plans), {}
        self.calls, self.aborted = [], []
        self.synced, self.parked = [], []

    async def generate(self, prompt, *, sampling=None, request_id=None):
        plan = self.plans.popleft()
        self.held[request_id] = plan
        self.calls.append((str(prompt), sampling, request_id))
        if plan.delay:
            await asyncio.sleep(plan.delay)
        self.held.pop(request_id, None)
        out = GenerationOutput(index=0, text=plan.text, token_ids=(21, 22), completion_logprobs=(-0.1, -0.2),
                               finish_reason="stop", stop_reason=None)
        return GenerationResult(request_id=request_id, prompt=str(prompt), prompt_token_ids=(11, 12), outputs=(out,),
                                finished=True, raw_output=plan)

    async def abort_async(self, request_id):
        self.aborted.append(request_id)
        plan = self.held.pop(request_id, None)
        if plan is not None:
            self.plans.appendleft(plan)

    def sync_from_model(self, model, *, drain_timeout=300):
        self.synced.append((model, drain_timeout))
        return "version-1"

    def sleep(self, *, level=1, mode="abort"):
        self.parked.append((level, mode))


class Rows:
    def __init__(self, examples):
        self.examples, self.is_empty = examples, not examples

    def __len__(self):
        return len(self.examples)


class QueueEnv:
    """Prompts with an expected answer; reward 1 when the response ends with it."""

    def __init__(self, rows, *, queued=True):
        self.rows = [SimpleNamespace(prompt=q, target=a, dataset_index=i) for i, (q, a) in enumerate(rows)]
        self.queue = deque(self.rows if queued else ())
        self.cursor = len(self.rows) if queued else 0
        self.seen_turn_counts = []

    @property
    def pending_example_count(self):
        return len(self.queue)

    def next_example(self):
        return self.queue.popleft() if self.queue else None

    def next_batch(self, count):
        taken = tuple(self.rows[self.cursor:self.cursor + count])
        self.cursor += len(taken)
        return Rows(taken)

    def enqueue_examples(self, examples):
        self.queue.extend(examples)

    def evaluate_response(self, example, response, *, turn_count, turn_metadata):
        self.seen_turn_counts.append(turn_count)
        return SimpleNamespace(reward=SimpleNamespace(reward=1.0 if response.strip().endswith(example.target) else 0.0))


class TwoStepHarness(DirectHarness):
    """Keeps asking while the completion says 'more' (at most `limit` turns)."""
    tag = "two-step"

    def __init__(self, limit=2):
        self.limit = limit

    def next_request(self, example, state):
        if state.finished:
            return None
        history = "".join(turn.response for turn in state.turns)
        return HarnessRequest(prompt=example.prompt + history)

    def apply_result(self, example, state, result):
        text = result.text
        state.turns.append(build_trajectory_turn(turn_index=len(state.turns) + 1, prompt=result.prompt, response=text,
                                                 result=result, metadata={"harness": self.tag}))
        if "more" not in text or len(state.turns) >= self.limit:
            state.final_response, state.finished = text, True
            state.terminal_reason = "answered" if "more" not in text else "max_turns"


def collect(runner, env, engine, harness=None, **request):
    return asyncio.run(runner.collect(env=env, engine=engine, harness=harness or DirectHarness(),
                                      rollout_config=RolloutConfig(**request)))


def test_direct_harness_is_a_harness_and_gives_a_single_turn():
    assert isinstance(DirectHarness(), Harness)
    env = QueueEnv([("2 + 2?", "4")])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1))
    engine = ScriptedEngine([Plan("work, so 4")])
    (only,) = collect(runner, env, engine, num_rollouts=1)
    assert only.terminal_reason == "single_turn" and only.finished and only.evaluation.reward.reward == 1.0
    assert only.group_id == 0 and only.rollout_index == 0 and only.metadata == {"harness": "direct"}
    (turn,) = only.turns
    assert turn.prompt_token_ids == (11, 12) and turn.completion_token_ids == (21, 22)
    assert turn.completion_logprobs == (-0.1, -0.2) and turn.finish_reason == "stop"
    assert turn.metadata == {"harness": "direct", "completion_token_count": 2}
    prompt, sampling, request_id = engine.calls[0]
    assert prompt == "2 + 2?" and sampling is None and request_id.startswith("rollout-0-0-")
    assert runner.last_stats == {"effective_group_target": 1.0, "selected_group_count": 1.0, "effective_group_count": 1.0,
                                 "sampled_group_count": 1.0, "dropped_zero_std_group_count": 0.0,
                                 "carried_in_unfinished_group_count": 0.0, "carried_out_unfinished_group_count": 0.0,
                                 "requests_issued": 1.0, "requests_completed": 1.0, "aborted_request_count": 0.0}


def test_groups_of_equal_rewards_are_replaced_until_one_differs():
    env = QueueEnv([("q0", "1"), ("q1", "1")])
    engine = ScriptedEngine([Plan("1"), Plan("1"), Plan("1"), Plan("2")])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1, max_inflight_requests=2))
    found = collect(runner, env, engine, num_rollouts=2)
    assert [t.evaluation.reward.reward for t in found] == [1.0, 0.0]
    assert [t.rollout_index for t in found] == [0, 1] and {t.group_id for t in found} == {1}
    stats = runner.last_stats
    assert (stats["sampled_group_count"], stats["dropped_zero_std_group_count"], stats["effective_group_count"]) == (2.0, 1.0, 1.0)


def test_a_finished_flat_group_is_not_replayed_by_the_next_call():
    env = QueueEnv([("q0", "1")])
    engine = ScriptedEngine([Plan("1"), Plan("1")])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1, max_inflight_requests=2))
    assert collect(runner, env, engine, num_rollouts=2) == []
    assert collect(runner, env, engine, num_rollouts=2) == []
    assert runner.last_stats["sampled_group_count"] == 0.0 and runner.last_stats["carried_in_unfinished_group_count"] == 0.0


def test_without_dynamic_sampling_flat_groups_are_kept():
    env = QueueEnv([("q0", "1")])
    engine = ScriptedEngine([Plan("1"), Plan("1")])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1, max_inflight_requests=2, use_dynamic_sampling=False))
    found = collect(runner, env, engine, num_rollouts=2)
    assert [t.evaluation.reward.reward for t in found] == [1.0, 1.0]
    stats = runner.last_stats
    assert (stats["selected_group_count"], stats["effective_group_count"], stats["dropped_zero_std_group_count"]) == (1.0, 0.0, 0.0)


def test_unfinished_groups_continue_in_the_next_call():
    env = QueueEnv([("q0", "1"), ("q1", "1")])
    engine = ScriptedEngine([Plan("1"), Plan(" more "), Plan("1")])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1, max_inflight_requests=2))
    harness = TwoStepHarness()
    first = collect(runner, env, engine, harness, num_rollouts=1)
    carried = runner.last_stats["carried_out_unfinished_group_count"]
    second = collect(runner, env, engine, harness, num_rollouts=1)
    assert len(first) == 1 and carried == 1.0
    assert len(second) == 1 and len(second[0].turns) == 2 and second[0].terminal_reason == "answered"
    assert engine.calls[2][0] == "q1 more "                       # the second turn saw the first turn's text
    assert runner.last_stats["sampled_group_count"] == 0.0 and runner.last_stats["carried_in_unfinished_group_count"] == 1.0
    assert env.seen_turn_counts == [1, 2]


def test_requests_still_in_flight_are_aborted_once_the_target_is_met():
    env = QueueEnv([("q0", "1"), ("q1", "1")])
    engine = ScriptedEngine([Plan("1"), Plan("1", delay=0.2)])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1, max_inflight_requests=2))
    found = collect(runner, env, engine, num_rollouts=1)
    assert len(found) == 1 and len(engine.aborted) == 1 and engine.aborted[0].startswith("rollout-1-0-")
    assert runner.last_stats["aborted_request_count"] == 1.0 and runner.last_stats["carried_out_unfinished_group_count"] == 1.0
    assert list(engine.plans) == [Plan("1", delay=0.2)]            # the aborted request's plan went back


def test_in_flight_requests_never_exceed_the_limit_and_groups_go_in_order():
    env = QueueEnv([(f"q{i}", "1") for i in range(6)])
    peak = 0

    class Counting(ScriptedEngine):
        async def generate(self, prompt, **kw):
            nonlocal peak
            peak = max(peak, len(self.held) + 1)
            return await super().generate(prompt, **kw)

    engine = Counting([Plan("1", delay=0.01) for _ in range(6)])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=6, max_inflight_requests=3))
    found = collect(runner, env, engine, num_rollouts=1)
    assert peak == 3 and sorted(t.group_id for t in found) == list(range(6))     # groups come back as they finish
    assert [call[0] for call in engine.calls] == [f"q{i}" for i in range(6)]


def test_the_request_budget_ends_rollouts_that_have_turns_and_drops_the_others():
    env = QueueEnv([("q0", "1"), ("q1", "1")])
    engine = ScriptedEngine([Plan(" more "), Plan(" more "), Plan("unused")])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=2, max_inflight_requests=1))
    found = collect(runner, env, engine, TwoStepHarness(limit=3), num_rollouts=1, max_total_requests=2)
    # one in flight at a time, in group order: both requests go to the first group, which then ends as it is
    assert len(found) == 1 and found[0].terminal_reason == "budget_exhausted" and len(found[0].turns) == 2
    assert found[0].final_response == " more " and runner.last_stats["requests_issued"] == 2.0
    assert len(engine.plans) == 1


def test_a_stalled_engine_raises():
    env = QueueEnv([("q0", "1")])
    engine = ScriptedEngine([Plan("1", delay=0.3)])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=1, stall_timeout_seconds=0.01, progress_log_interval_seconds=0.0))
    with pytest.raises(RuntimeError, match="stalled waiting for completions"):
        collect(runner, env, engine, num_rollouts=1)


def test_a_harness_without_a_request_for_an_unfinished_rollout_is_an_error():
    class Silent(DirectHarness):
        def next_request(self, example, state):
            return None
    with pytest.raises(RuntimeError, match="no request for an unfinished state"):
        collect(RolloutRunner(), QueueEnv([("q0", "1")]), ScriptedEngine([]), Silent(), num_rollouts=1)


def test_several_completions_per_request_are_refused():
    env = QueueEnv([("q0", "1")])
    with pytest.raises(ValueError, match="sampling.n == 1"):
        collect(RolloutRunner(), env, ScriptedEngine([]), num_rollouts=1, sampling=SimpleNamespace(n=2))

    class Greedy(DirectHarness):   # a request's own sampling is checked too
        def next_request(self, example, state):
            return HarnessRequest(prompt=example.prompt, sampling=SimpleNamespace(n=3))
    with pytest.raises(ValueError, match="sampling.n == 1"):
        collect(RolloutRunner(), QueueEnv([("q0", "1")]), ScriptedEngine([]), Greedy(), num_rollouts=1)


def test_the_empty_queue_is_refilled_from_the_dataset():
    env = QueueEnv([(f"q{i}", "1") for i in range(3)], queued=False)
    engine = ScriptedEngine([Plan("1") for _ in range(3)])
    runner = RolloutRunner(RolloutRunnerConfig(effective_batch_size=3, max_inflight_requests=2))
    found = collect(runner, env, engine, num_rollouts=1)
    assert sorted(t.example.dataset_index for t in found) == [0, 1, 2] and env.cursor == 3


@pytest.mark.parametrize("kwargs,message", [
    ({"effective_batch_size": 0}, "effective_batch_size must be > 0"),
    ({"max_inflight_requests": 0}, "max_inflight_requests must be > 0"),
    ({"reward_std_epsilon": -1.0}, "reward_std_epsilon must be >= 0"),
    ({"stall_timeout_seconds": -1.0}, "stall_timeout_seconds must be >= 0"),
    ({"progress_log_interval_seconds": -1.0}, "progress_log_interval_seconds must be >= 0"),
])
def test_runner_settings_are_validated(kwargs, message):
    with pytest.raises(ValueError, match=message):
        RolloutRunnerConfig(**kwargs)
    with pytest.raises(ValueError, match="num_rollouts must be > 0"):
        RolloutConfig(num_rollouts=0)
    with pytest.raises(ValueError, match="max_total_requests must be > 0"):
        RolloutConfig(num_rollouts=1, max_total_requests=0)


def test_coordinator_collects_parks_and_syncs_weights():
    env = QueueEnv([(f"q{i}", "1") for i in range(4)], queued=False)
    engine = ScriptedEngine([Plan("1"), Plan("1", delay=0.02), Plan("1"), Plan("1"), Plan("1")])
    settings = RolloutRunnerConfig(effective_batch_size=4, max_inflight_requests=2, use_dynamic_sampling=False)
    coordinator = RolloutCoordinator(engine=engine, env=env, harness=DirectHarness(),
                                     config=RolloutCoordinatorConfig(num_rollouts=1, batch_size=4, runner_config=settings))
    batch = coordinator.collect()
    assert sorted(batch.indices) == [0, 1, 2, 3] and len(batch.trajectories) == 4
    assert len(engine.calls) == 4                                  # no prefetch past the four groups needed
    assert batch.stats["sampled_group_count"] == 4.0 and batch.stats["aborted_request_count"] == 0.0
    assert engine.parked == [(1, "abort")]
    assert coordinator.sync_weights("policy", drain_timeout=7) == "version-1" and engine.synced == [("policy", 7)]
    with pytest.raises(TypeError, match="sync_from_model"):
        RolloutCoordinator(engine=object(), env=env, harness=DirectHarness(),
                           config=RolloutCoordinatorConfig(num_rollouts=1)).sync_weights("policy")


def test_coordinator_without_prompts_raises_and_refuses_a_running_loop():
    coordinator = RolloutCoordinator(engine=ScriptedEngine([]), env=QueueEnv([], queued=False), harness=DirectHarness(),
                                     config=RolloutCoordinatorConfig(num_rollouts=1))
    with pytest.raises(RuntimeError, match="could not build a prompt batch"):
        coordinator.collect()

    async def inside():
        with pytest.raises(RuntimeError, match="active event loop"):
            coordinator.collect()
    asyncio.run(inside())
