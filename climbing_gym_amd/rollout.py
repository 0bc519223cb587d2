"""Rollout collection over the async engine: the trainers' side of `generate` / `abort`.

A collection keeps a bounded number of single-output requests in flight against an engine with the adapter's
interface (`await engine.generate(prompt, sampling=, request_id=)`, `abort_async` or `abort`), lets a harness turn
completions into (possibly multi-turn) trajectories, scores finished prompt groups through the environment and returns
`effective_batch_size` groups whose rewards differ (with dynamic sampling, groups of identical rewards are replaced).

Behaviour follows rollout/runner.py:90-489 (limits 97-135, issue order 307-340, request ids and the single-output rule
272-305 and 84-87, group scoring 186-246, budget exhaustion 248-262, stall and heartbeat 360-395, abort of the surplus
342-358, carry-over of unfinished groups and the statistics 413-432, the loop 437-489), rollout/config.py:9-42,
rollout/contracts.py:11-92, rollout/harnesses/direct.py:9-42 and rollout/coordinator.py:13-180.  The environment is
duck-typed (envs/contracts.py: `next_example`, `pending_example_count`, `next_batch`, `enqueue_examples`,
`evaluate_response(...).reward.reward`); environments themselves are not part of this package.
"""
from __future__ import annotations

import asyncio
import inspect
import logging
import uuid
from dataclasses import dataclass, field
from statistics import pstdev
from typing import Any, Mapping, Optional, Protocol, runtime_checkable

from .types import BehaviorTopK
from ._checks import reject

log = logging.getLogger(__name__)


# ------------------------------------------------------------------------------------------------ settings
@dataclass(frozen=True)
class RolloutConfig:
    """What to ask for: rollouts per prompt, default sampling, an optional cap on engine requests (config.py:9-20)."""
    num_rollouts: int
    sampling: Any = None
    max_total_requests: Optional[int] = None

    def __post_init__(self):
        reject(self.num_rollouts <= 0, "num_rollouts must be > 0")
        reject(self.max_total_requests is not None and self.max_total_requests <= 0,
               "max_total_requests must be > 0 when provided")


@dataclass(frozen=True)
class RolloutRunnerConfig:
    """How to run it (config.py:23-42)."""
    effective_batch_size: int = 1
    max_inflight_requests: Optional[int] = None
    reward_std_epsilon: float = 1e-8
    use_dynamic_sampling: bool = True
    stall_timeout_seconds: float = 120.0
    progress_log_interval_seconds: float = 15.0

    def __post_init__(self):
        reject(self.effective_batch_size <= 0, "effective_batch_size must be > 0")
        reject(self.max_inflight_requests is not None and self.max_inflight_requests <= 0,
               "max_inflight_requests must be > 0 when provided")
        for name in ("reward_std_epsilon", "stall_timeout_seconds", "progress_log_interval_seconds"):
            reject(getattr(self, name) < 0, f"{name} must be >= 0")


# ------------------------------------------------------------------------------------------------ records
@dataclass(frozen=True)
class HarnessRequest:
    prompt: Any
    sampling: Any = None


@dataclass(frozen=True)
class TrajectoryTurn:
    turn_index: int
    prompt: str
    response: str
    prompt_token_ids: tuple
    completion_token_ids: tuple
    completion_logprobs: Optional[tuple]
    finish_reason: Optional[str]
    stop_reason: Optional[str]
    metadata: Mapping[str, Any] = field(default_factory=dict)
    behavior_topk: Optional[BehaviorTopK] = None


@dataclass(frozen=True)
class Trajectory:
    group_id: int
    rollout_index: int
    example: Any
    turns: tuple
    final_response: str
    finished: bool
    terminal_reason: str
    evaluation: Any
    metadata: Mapping[str, Any] = field(default_factory=dict)


@dataclass
class HarnessState:
    rollout_index: int
    turns: list = field(default_factory=list)
    finished: bool = False
    final_response: str = ""
    terminal_reason: str = ""
    metadata: dict = field(default_factory=dict)


def build_trajectory_turn(*, turn_index: int, prompt: str, response: str, result: Any, metadata: Mapping[str, Any]) -> TrajectoryTurn:
    """One engine result as a turn: ids and logprobs of its first output (contracts.py:53-77)."""
    outputs = getattr(result, "outputs", ()) or ()
    first = outputs[0] if outputs else None
    logprobs = getattr(first, "completion_logprobs", None)
    return TrajectoryTurn(
        turn_index=turn_index, prompt=str(prompt), response=str(response),
        prompt_token_ids=tuple(getattr(result, "prompt_token_ids", ()) or ()),
        completion_token_ids=tuple(getattr(first, "token_ids", ()) or ()),
        completion_logprobs=None if logprobs is None else tuple(logprobs or ()),
        finish_reason=None if first is None else first.finish_reason,
        stop_reason=None if first is None else first.stop_reason,
        metadata=dict(metadata), behavior_topk=getattr(first, "behavior_topk", None))


@runtime_checkable
class Harness(Protocol):
    def create_state(self, example, rollout_index: int) -> HarnessState: ...
    def next_request(self, example, state: HarnessState) -> Optional[HarnessRequest]: ...
    def apply_result(self, example, state: HarnessState, result) -> None: ...
    def force_finish(self, state: HarnessState, reason: str) -> None: ...


class DirectHarness:
    """One request per rollout: the example's prompt as it is, the completion as the answer (harnesses/direct.py)."""
    tag = "direct"

    def create_state(self, example, rollout_index: int) -> HarnessState:
        return HarnessState(rollout_index=int(rollout_index), metadata={"harness": self.tag})

    def next_request(self, example, state: HarnessState) -> Optional[HarnessRequest]:
        asked = state.finished or bool(state.turns)
        return None if asked else HarnessRequest(prompt=str(example.prompt))

    def apply_result(self, example, state: HarnessState, result) -> None:
        meta = {"harness": self.tag, "completion_token_count": len(result.outputs[0].token_ids)}
        turn = build_trajectory_turn(turn_index=1, prompt=str(getattr(result, "prompt", "")),
                                     response=str(getattr(result, "text", "")), result=result, metadata=meta)
        state.turns.append(turn)
        state.final_response, state.finished, state.terminal_reason = turn.response, True, "single_turn"

    def force_finish(self, state: HarnessState, reason: str) -> None:
        if state.finished:
            return
        if state.turns and not state.final_response:
            state.final_response = state.turns[-1].response
        state.finished, state.terminal_reason = True, str(reason)


# ------------------------------------------------------------------------------------------------ the runner
def require_single_output(sampling) -> None:
    """Every engine request yields one completion: a sampling object with n other than 1 is refused (runner.py:72-87)."""
    count = getattr(sampling, "n", None) if sampling is not None else None
    try:
        count = None if count is None else int(count)
    except (TypeError, ValueError):
        count = None
    reject(count not in (None, 1), "RolloutRunner requires sampling.n == 1 for each engine request.")


@dataclass
class _Lane:
    """One rollout of a prompt group."""
    index: int
    state: HarnessState
    request_id: Optional[str] = None
    dropped: bool = False

    @property
    def idle(self) -> bool:   # may be given a request
        return not (self.dropped or self.state.finished or self.request_id is not None)


@dataclass(eq=False)
class _Group:
    ident: int
    example: Any
    lanes: list

    def in_flight(self) -> int:
        return sum(lane.request_id is not None for lane in self.lanes)

    def complete(self) -> bool:
        return all(lane.dropped or lane.state.finished for lane in self.lanes)


class _Collection:
    """State and steps of one `collect` call."""

    def __init__(self, runner: "RolloutRunner", env, engine, harness, request: RolloutConfig):
        cfg = runner.runner_config
        self.runner, self.env, self.engine, self.harness, self.request = runner, env, engine, harness, request
        self.loop = asyncio.get_running_loop()
        self.groups: list = runner._take_unfinished()
        self.carried_in = len(self.groups)
        self.target = int(cfg.effective_batch_size)
        self.per_group = int(request.num_rollouts)
        self.max_requests = (max(1, self.target * self.per_group) if cfg.max_inflight_requests is None
                             else int(cfg.max_inflight_requests))
        self.max_groups = max(1, self.max_requests // self.per_group)
        self.chosen: list = []            # lists of trajectories, one per selected group
        self.flying: dict = {}            # task -> (request id, group, lane)
        self.effective = self.sampled = self.dropped_flat = self.issued = self.completed = self.aborted = 0
        self.progress_at = self.logged_at = self.loop.time()

    # -- limits
    def budget_left(self) -> bool:
        cap = self.request.max_total_requests
        return cap is None or self.issued < int(cap)

    def satisfied(self) -> bool:
        return len(self.chosen) >= self.target

    def summary(self) -> str:
        return (f"selected={len(self.chosen)}/{self.target} pending={len(self.flying)} active_groups={len(self.groups)} "
                f"sampled_groups={self.sampled} carried_in={self.carried_in} requests_issued={self.issued} "
                f"requests_completed={self.completed}")

    # -- new prompt groups
    def _draw_example(self):
        example = self.env.next_example()
        if example is not None:
            return example
        # the queue is dry: pull enough rows from the dataset to fill the active groups (at least one)
        want = max(1, max(1, self.max_groups) - int(self.env.pending_example_count))
        try:
            rows = self.env.next_batch(want)
        except RuntimeError:
            return None
        if rows.is_empty:
            return None
        self.env.enqueue_examples(rows.examples)
        return self.env.next_example()

    def _open_group(self) -> bool:
        example = self._draw_example()
        if example is None:
            return False
        self.sampled += 1
        ident = self.runner._new_group_id()
        lanes = [_Lane(i, self.harness.create_state(example, i)) for i in range(self.per_group)]
        self.groups.append(_Group(ident, example, lanes))
        return True

    # -- requests
    def _send(self, group: _Group, lane: _Lane) -> bool:
        ask = self.harness.next_request(group.example, lane.state)
        if ask is None:
            if lane.state.finished:
                return False
            raise RuntimeError("Harness returned no request for an unfinished state.")
        sampling = self.request.sampling if ask.sampling is None else ask.sampling
        require_single_output(sampling)
        request_id = f"rollout-{group.ident}-{lane.index}-{uuid.uuid4().hex}"
        lane.request_id = request_id
        task = asyncio.create_task(self.engine.generate(ask.prompt, sampling=sampling, request_id=request_id))
        self.flying[task] = (request_id, group, lane)
        self.issued += 1
        return True

    def _send_one_from_open_groups(self) -> bool:
        for group in list(self.groups):
            if group.in_flight() >= self.per_group:
                continue
            for lane in group.lanes:
                if lane.idle and self._send(group, lane):
                    return True
        return False

    def fill(self) -> None:
        """Issue requests until the in-flight limit, the request budget or the supply of prompts stops it: open groups
        first, in order; a new group only while there is room for one and (without dynamic sampling) need of one."""
        while len(self.flying) < self.max_requests and self.budget_left():
            if self._send_one_from_open_groups():
                continue
            if len(self.groups) >= self.max_groups:
                return
            if not self.runner.runner_config.use_dynamic_sampling and len(self.chosen) + len(self.groups) >= self.target:
                return
            if not self._open_group():
                return

    # -- finished groups
    def _score(self, group: _Group) -> list:
        scored = []
        for lane in sorted(group.lanes, key=lambda item: item.index):
            turns = tuple(lane.state.turns)
            if lane.dropped or not turns:
                continue
            answer = str(lane.state.final_response or turns[-1].response)
            verdict = self.env.evaluate_response(group.example, answer, turn_count=len(turns),
                                                 turn_metadata=tuple(dict(turn.metadata) for turn in turns))
            scored.append(Trajectory(group_id=group.ident, rollout_index=lane.index, example=group.example, turns=turns,
                                     final_response=answer, finished=bool(lane.state.finished),
                                     terminal_reason=str(lane.state.terminal_reason), evaluation=verdict,
                                     metadata=dict(lane.state.metadata)))
        return scored

    def _rewards_differ(self, scored: list) -> bool:
        if self.per_group < 2:
            return True
        rewards = [float(item.evaluation.reward.reward) for item in scored]
        return len(rewards) >= 2 and float(pstdev(rewards)) > float(self.runner.runner_config.reward_std_epsilon)

    def retire(self, group: _Group) -> None:
        if group in self.groups:
            self.groups.remove(group)
        scored = self._score(group)
        if not scored:
            return
        useful = self._rewards_differ(scored)
        if useful:
            self.effective += 1
        elif self.runner.runner_config.use_dynamic_sampling:
            self.dropped_flat += 1
            return
        if not self.satisfied():
            self.chosen.append(scored)

    def close_out_budget(self) -> None:
        """No request may be issued any more: rollouts that have turns end as they are, those without are dropped."""
        for group in list(self.groups):
            for lane in group.lanes:
                if not lane.idle:
                    continue
                if lane.state.turns:
                    self.harness.force_finish(lane.state, "budget_exhausted")
                else:
                    lane.dropped = True
            if group.complete():
                self.retire(group)

    # -- waiting
    def wait_limit(self) -> Optional[float]:
        cfg = self.runner.runner_config
        limit = cfg.progress_log_interval_seconds if cfg.progress_log_interval_seconds > 0.0 else None
        if cfg.stall_timeout_seconds > 0.0:
            left = cfg.stall_timeout_seconds - (self.loop.time() - self.progress_at)
            reject(left <= 0.0, f"Rollout runner stalled before wait: {self.summary()}", RuntimeError)
            limit = left if limit is None else min(limit, left)
        return limit

    def nothing_arrived(self) -> None:
        cfg = self.runner.runner_config
        now = self.loop.time()
        if cfg.progress_log_interval_seconds > 0.0 and now - self.logged_at >= cfg.progress_log_interval_seconds:
            log.info("Rollout runner heartbeat: %s", self.summary())
            self.logged_at = now
        reject(cfg.stall_timeout_seconds > 0.0 and now - self.progress_at >= cfg.stall_timeout_seconds,
               f"Rollout runner stalled waiting for completions: {self.summary()}", RuntimeError)

    def absorb(self, done) -> None:
        for task in done:
            _, group, lane = self.flying.pop(task)
            lane.request_id = None
            result = task.result()
            self.completed += 1
            self.progress_at = self.loop.time()
            self.harness.apply_result(group.example, lane.state, result)
            if group.complete():
                self.retire(group)

    async def abort_rest(self) -> None:
        stop = getattr(self.engine, "abort_async", None) or getattr(self.engine, "abort", None)
        tasks = []
        for task, (request_id, _, lane) in list(self.flying.items()):
            if stop is not None:
                outcome = stop(request_id)
                if inspect.isawaitable(outcome):
                    await outcome
            self.aborted += 1
            lane.request_id = None
            del self.flying[task]
            if not task.done():
                task.cancel()
            tasks.append(task)
        if tasks:
            await asyncio.gather(*tasks, return_exceptions=True)

    def statistics(self, unfinished: list) -> dict:
        return {"effective_group_target": float(self.target), "selected_group_count": float(len(self.chosen)),
                "effective_group_count": float(self.effective), "sampled_group_count": float(self.sampled),
                "dropped_zero_std_group_count": float(self.dropped_flat),
                "carried_in_unfinished_group_count": float(self.carried_in),
                "carried_out_unfinished_group_count": float(len(unfinished)), "requests_issued": float(self.issued),
                "requests_completed": float(self.completed), "aborted_request_count": float(self.aborted)}


class RolloutRunner:
    """`await runner.collect(env=, engine=, harness=, rollout_config=)` -> trajectories of the selected groups, group by
    group, rollouts in index order.  Groups still unfinished when the target is met are kept for the next call;
    `last_stats` describes the last call (runner.py:420-432)."""

    def __init__(self, runner_config: RolloutRunnerConfig = RolloutRunnerConfig()):
        self.runner_config = runner_config
        self.last_stats: dict = {}
        self._unfinished: list = []
        self._group_ids = 0

    def _take_unfinished(self) -> list:
        groups, self._unfinished = list(self._unfinished), []
        return groups

    def _new_group_id(self) -> int:
        self._group_ids += 1
        return self._group_ids - 1

    async def collect(self, *, env, engine, harness, rollout_config: RolloutConfig) -> list:
        require_single_output(rollout_config.sampling)
        run = _Collection(self, env, engine, harness, rollout_config)
        log.info("Rollout runner start: %s", run.summary())
        while not run.satisfied():
            run.fill()
            if run.satisfied():
                break
            if not run.flying:
                if not run.budget_left():
                    run.close_out_budget()
                break
            done, _ = await asyncio.wait(set(run.flying), return_when=asyncio.FIRST_COMPLETED, timeout=run.wait_limit())
            if done:
                run.absorb(done)
            else:
                run.nothing_arrived()
        if run.flying and run.satisfied():
            await run.abort_rest()
        if not run.flying and not run.budget_left():
            run.close_out_budget()
        self._unfinished = [group for group in run.groups if not group.complete()]
        self.last_stats = run.statistics(self._unfinished)
        log.info("Rollout runner complete: %s", run.summary())
        return [trajectory for group in run.chosen for trajectory in group]


# ------------------------------------------------------------------------------------------------ the coordinator
@dataclass(frozen=True)
class TrajectoryBatch:
    indices: tuple
    trajectories: tuple
    stats: dict


@dataclass(frozen=True)
class RolloutCoordinatorConfig:
    num_rollouts: int
    sampling: Any = None
    max_total_requests: Optional[int] = None
    batch_size: int = 1
    engine_sleep_level: int = 1
    engine_sleep_mode: str = "abort"
    runner_config: Optional[RolloutRunnerConfig] = None


class RolloutCoordinator:
    """Synchronous front of the runner for a training loop: tops up the environment's prompt queue, collects one batch,
    parks the engine, and pushes new policy weights into it (coordinator.py:82-180)."""

    def __init__(self, *, engine, env, harness, config: RolloutCoordinatorConfig, rollout_runner: Optional[RolloutRunner] = None):
        self.engine, self.env, self.harness, self.config = engine, env, harness, config
        self.rollout_config = RolloutConfig(num_rollouts=int(config.num_rollouts), sampling=config.sampling,
                                            max_total_requests=config.max_total_requests)
        settings = config.runner_config or RolloutRunnerConfig(effective_batch_size=int(config.batch_size))
        self.rollout_runner = rollout_runner or RolloutRunner(settings)

    @property
    def last_stats(self) -> dict:
        return dict(getattr(self.rollout_runner, "last_stats", {}))

    def sync_weights(self, model, *, drain_timeout: int = 300):
        """New policy weights into the engine in place: `sync_from_model(model)`, else `sync()` (coordinator.py:13-27)."""
        push = getattr(self.engine, "sync_from_model", None)
        if callable(push):
            return push(model, drain_timeout=drain_timeout)
        push = getattr(self.engine, "sync", None)
        if callable(push):
            return push(drain_timeout=drain_timeout)
        raise TypeError("Rollout engine must provide sync_from_model(model, ...) or sync(...).")

    def park(self) -> None:
        rest = getattr(self.engine, "sleep", None)
        if callable(rest):
            rest(level=self.config.engine_sleep_level, mode=self.config.engine_sleep_mode)

    def _top_up(self) -> int:
        missing = max(0, int(self.config.batch_size)) - int(self.env.pending_example_count)
        if missing <= 0:
            return 0
        rows = self.env.next_batch(missing)
        if rows.is_empty:
            return 0
        self.env.enqueue_examples(rows.examples)
        return len(rows)

    async def collect_async(self) -> TrajectoryBatch:
        waiting, loaded = int(self.env.pending_example_count), self._top_up()
        try:
            found = tuple(await self.rollout_runner.collect(env=self.env, engine=self.engine, harness=self.harness,
                                                            rollout_config=self.rollout_config))
        finally:
            self.park()
        stats = self.last_stats
        nothing_to_do = (not found and waiting <= 0 and loaded <= 0 and stats.get("sampled_group_count", 0.0) <= 0.0
                         and stats.get("carried_in_unfinished_group_count", 0.0) <= 0.0)
        reject(nothing_to_do, "RolloutCoordinator could not build a prompt batch from the provided rows.", RuntimeError)
        indices = []
        for item in found:   # dataset rows behind the batch, each once, in order of appearance
            row = getattr(item.example, "dataset_index", None)
            if row is not None and int(row) not in indices:
                indices.append(int(row))
        return TrajectoryBatch(indices=tuple(indices), trajectories=found, stats=stats)

    def collect(self) -> TrajectoryBatch:
        try:
            asyncio.get_running_loop()
        except RuntimeError:
            return asyncio.run(self.collect_async())
        raise RuntimeError("RolloutCoordinator.collect() cannot be called from an active event loop; "
                           "use `await rollout_coordinator.collect_async()` instead.")
