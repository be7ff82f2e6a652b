"""The scheduler's ragged mode without a GPU: steps that mix portions of prompts with decoded tokens, blocks that
grow with the sequence, recurrent-state slots that are handed on, preemption by recomputation, replayed plans."""
import pytest

from splitwise_amd.config import CacheConfig, SchedulerConfig
from splitwise_amd.core.scheduler import Scheduler
from splitwise_amd.sampling_params import SamplingParams
from splitwise_amd.sequence import Logprob, Sequence, SequenceGroup, SequenceStatus


def make(num_blocks=16, max_seqs=3, budget=32, block_size=4, max_len=1000):
    sc = SchedulerConfig(budget, max_seqs, max_len, ragged_steps=True)
    cc = CacheConfig(block_size, 0.9, 0)
    cc.num_gpu_blocks, cc.num_cpu_blocks = num_blocks, 0
    return Scheduler(sc, cc)


def add(sched, rid, n, seq_id, t=0.0, max_tokens=4):
    seq = Sequence(seq_id, None, list(range(n)), sched.cache_config.block_size)
    group = SequenceGroup(rid, [seq], SamplingParams(temperature=0.0, max_tokens=max_tokens), t)
    sched.add_seq_group(group)
    return group, seq


def finish_step(sched, token=7):
    """What the engine does after a step: advance, append the sampled token."""
    for group, seq, n, sampled in sched.last_ragged:
        seq.num_computed_tokens += n
        if sampled:
            seq.append_token_id(token, {token: Logprob(0.0)})


def by_id(metas):
    return {m.request_id: m for m in metas}


def test_prompts_are_cut_to_the_budget_and_decode_beside_portions():
    sched = make(budget=10)
    _, a = add(sched, "a", 23, 0, t=0.0)
    _, b = add(sched, "b", 3, 1, t=1.0)
    metas, outs = sched.schedule()
    m = by_id(metas)
    assert m["a"].token_chunk == {0: 10} and m["a"].num_computed == {0: 0} and not m["a"].do_sample
    assert "b" not in m and outs.num_batched_tokens == 10          # the budget is spent
    finish_step(sched)
    metas, _ = sched.schedule()
    m = by_id(metas)
    assert m["a"].token_chunk == {0: 10} and m["a"].num_computed == {0: 10}
    finish_step(sched)
    metas, _ = sched.schedule()                                       # a's last 3, then b whole
    m = by_id(metas)
    assert m["a"].token_chunk == {0: 3} and m["a"].do_sample
    assert m["b"].token_chunk == {1: 3} and m["b"].do_sample and m["b"].num_computed == {1: 0}
    finish_step(sched)
    assert a.get_len() == 24 and b.get_len() == 4
    metas, outs = sched.schedule()                                    # both decode now
    m = by_id(metas)
    assert m["a"].token_chunk == {0: 1} and m["a"].num_computed == {0: 23} and not m["a"].is_prompt
    assert m["b"].token_chunk == {1: 1} and not outs.prompt_run
    # blocks cover every token, the newest included
    assert len(m["a"].block_tables[0]) == 6 and len(m["b"].block_tables[1]) == 1


def test_state_slots_are_reused_and_limit_admission():
    sched = make(max_seqs=2, budget=64)
    ga, a = add(sched, "a", 5, 0, t=0.0)
    gb, b = add(sched, "b", 5, 1, t=1.0)
    gc, c = add(sched, "c", 5, 2, t=2.0)
    metas, _ = sched.schedule()
    m = by_id(metas)
    assert set(m) == {"a", "b"}
    assert {m["a"].state_slots[0], m["b"].state_slots[1]} == {0, 1}
    finish_step(sched)
    slot_a = m["a"].state_slots[0]
    a.status = SequenceStatus.FINISHED_STOPPED
    sched.free_seq(a)
    sched.free_finished_seq_groups()
    metas, _ = sched.schedule()
    m = by_id(metas)
    assert set(m) == {"b", "c"} and m["c"].state_slots[2] == slot_a     # the freed slot goes out next
    assert sched.state_slots.num_free() == 0


def test_out_of_blocks_preempts_the_youngest_and_recomputes_it():
    sched = make(num_blocks=4, budget=64, block_size=4)
    _, a = add(sched, "a", 7, 0, t=0.0, max_tokens=50)
    _, b = add(sched, "b", 7, 1, t=1.0, max_tokens=50)
    sched.schedule()
    finish_step(sched)                                                # both 8 tokens: 2 blocks each, pool full
    metas, _ = sched.schedule()
    assert set(by_id(metas)) == {"a", "b"}
    finish_step(sched)                                                # 9 tokens each: a third block is needed
    metas, _ = sched.schedule()
    m = by_id(metas)
    assert set(m) == {"a"} and b.status == SequenceStatus.WAITING and b.num_computed_tokens == 0
    assert sched.num_preemptions == 1 and sched.state_slots.num_free() == 2
    assert len(m["a"].block_tables[0]) == 3
    finish_step(sched)
    a.status = SequenceStatus.FINISHED_STOPPED
    sched.free_seq(a)
    sched.free_finished_seq_groups()
    metas, _ = sched.schedule()                                       # b again, from its first token, outputs kept
    m = by_id(metas)
    assert m["b"].num_computed == {1: 0} and m["b"].token_chunk == {1: b.get_len()} and m["b"].do_sample


def test_a_plan_runs_exactly_what_it_names_and_samples_nothing():
    sched = make(num_blocks=6, max_seqs=2, budget=8, block_size=4)
    _, a = add(sched, "a", 6, 0)
    _, b = add(sched, "b", 2, 1)
    metas, outs = sched.schedule_ragged({"a": 5, "b": 2}, {"a": [0, 4]})
    m = by_id(metas)
    assert m["a"].token_chunk == {0: 5} and m["a"].logits_at == [0, 4] and not m["a"].do_sample
    assert m["b"].token_chunk == {1: 2} and not m["b"].do_sample and m["b"].logits_at is None
    finish_step(sched)
    a.data.prompt_token_ids.extend(range(9))                           # the prompt grows by 9: 15 tokens, 4 blocks
    metas, _ = sched.schedule_ragged({"a": 10})                       # b sits this step out
    m = by_id(metas)
    assert set(m) == {"a"} and m["a"].num_computed == {0: 5} and len(m["a"].block_tables[0]) == 4
    finish_step(sched)
    with pytest.raises(ValueError):
        sched.schedule_ragged({"a": 1})                               # nothing is left of a
    with pytest.raises(KeyError):
        sched.schedule_ragged({"zz": 1})
    sched.abort_seq_group(["a", "b"])
    assert sched.block_manager.get_num_free_gpu_blocks() == 6 and sched.state_slots.num_free() == 2
    _, c = add(sched, "c", 30, 2)
    with pytest.raises(RuntimeError):
        sched.schedule_ragged({"c": 30})                              # 8 blocks asked of a pool of 6


def test_too_long_prompts_are_ignored():
    sched = make(num_blocks=4, block_size=4)
    g, _ = add(sched, "a", 40, 0)
    metas, outs = sched.schedule()
    assert not metas and outs.ignored_seq_groups == [g]


def test_trace_replay_refuses_models_without_ragged_steps(tmp_path):
    """Exit code 3, at the start, for an architecture whose steps are not ragged."""
    from splitwise_amd.entrypoints import trace_replay
    assert trace_replay.main(["--model", "llama-tiny", "--dtype", "bfloat16", "--out", str(tmp_path), "--max-tokens", "64"]) == 3
