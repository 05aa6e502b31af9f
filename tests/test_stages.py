"""Policy stages (join / swap) against answers worked out by hand from the
reference's statements (deserve_worker/engine/pipeline/stage/swap.py:24-107,
join.py:28-221).  Page size 16 throughout; pages(n) = ceil(n / 16)."""
import pytest
import torch

from deserve_amd.engine.pipeline.processor import StepRequest
from deserve_amd.engine.pipeline.stage.join import (DecodeFirstAgggregatedJoinStage,
                                                    PrefillFirstAgggregatedJoinStage,
                                                    VanillaJoinStage)
from deserve_amd.engine.pipeline.stage.swap import SwapStage
from deserve_amd.task import SamplingParams, TaskData, TaskManager

SP = SamplingParams()


def toks(n, base=0):
    return torch.arange(base, base + n, dtype=torch.int32)


def manager(**tasks):
    """name=(start_pos, seqlen, initial_seqlen)"""
    m = TaskManager(1024, 16)
    for name, (start, seqlen, initial) in tasks.items():
        m.add(TaskData(name, start, 0, seqlen, initial, SP))
    return m


def decode_request(ids, mb=0):
    r = StepRequest.empty(mb, torch.int32, "cpu")
    for i, t in enumerate(ids):
        r.append_exec(t, toks(1, 100 + i), None)
    return r


# ------------------------------------------------------------------ swap stage
def swap_fixture():
    m = manager(A=(0, 0, 100), B=(0, 0, 20), C=(33, 1, 8), D=(16, 1, 8))
    sus_p = {"A": toks(40), "B": toks(10)}
    sus_d = {"C": toks(1), "D": toks(1)}
    off_p, off_d = {}, {}
    return SwapStage(m, sus_p, sus_d, off_p, off_d), sus_p, sus_d, off_p, off_d


def test_swap_deficit_evicts_longest_waiting_prefills_first():
    st, sus_p, sus_d, off_p, off_d = swap_fixture()
    rest, r = st.process(-8, StepRequest.empty(0, torch.int32, "cpu"))
    # A frees ceil(100/16) = 7 -> -1; B frees ceil(20/16) = 2 -> +1
    assert rest == 1 and r.offload_task_ids == ["A", "B"]
    assert sus_p == {} and set(off_p) == {"A", "B"} and set(sus_d) == {"C", "D"} and off_d == {}


def test_swap_deficit_goes_on_to_waiting_decodes():
    st, sus_p, sus_d, off_p, off_d = swap_fixture()
    rest, r = st.process(-10, StepRequest.empty(0, torch.int32, "cpu"))
    # A +7, B +2 -> -1; decodes tie on length, the later one goes first: D holds ceil(16/16) = 1
    assert rest == 0 and r.offload_task_ids == ["A", "B", "D"]
    assert set(sus_d) == {"C"} and set(off_d) == {"D"}


def test_swap_deficit_cuts_the_tail_of_the_running_batch():
    m = manager(E1=(16, 1, 8), E2=(32, 1, 8), E3=(48, 1, 8))
    off_d = {}
    st = SwapStage(m, {}, {}, {}, off_d)
    r = decode_request(["E1", "E2", "E3"])
    rest, r = st.process(-3, r)
    # dropping E3 frees its 3 pages and the 1 its next token would need
    assert rest == 1 and r.exec_task_ids == ["E1", "E2"] and r.offload_task_ids == ["E3"]
    assert r.xs.tolist() == [100, 101] and off_d["E3"].tolist() == [102]
    assert r.exec_seqlens == [1, 1]
    with pytest.raises(RuntimeError, match="Unable to fetch enough pages"):
        st.process(-100, decode_request(["E1", "E2"]))


def test_swap_surplus_reloads_in_order_and_stops_at_the_first_misfit():
    def fixture():
        m = manager(P1=(0, 0, 64), P2=(0, 0, 10), Q=(40, 1, 8))
        sus_p, sus_d = {}, {}
        off_p, off_d = {"P1": toks(30), "P2": toks(5)}, {"Q": toks(1)}
        return SwapStage(m, sus_p, sus_d, off_p, off_d), sus_p, sus_d, off_p, off_d

    st, sus_p, sus_d, off_p, off_d = fixture()
    rest, r = st.process(6, StepRequest.empty(0, torch.int32, "cpu"))
    # P1 needs 4 -> 2, P2 needs 1 -> 1, Q needs ceil(40/16) = 3 > 1
    assert rest == 1 and r.reload_task_ids == ["P1", "P2"]
    assert set(sus_p) == {"P1", "P2"} and off_p == {} and set(off_d) == {"Q"}

    st, sus_p, sus_d, off_p, off_d = fixture()
    rest, r = st.process(3, StepRequest.empty(0, torch.int32, "cpu"))
    # P1 does not fit, which also ends the prefill pass (P2 is not tried); Q fits exactly
    assert rest == 0 and r.reload_task_ids == ["Q"] and set(off_p) == {"P1", "P2"} and set(sus_d) == {"Q"}

    st, *_ = fixture()
    rest, r = st.process(0, StepRequest.empty(0, torch.int32, "cpu"))
    assert rest == 0 and r.reload_task_ids == [] and r.offload_task_ids == []


# ------------------------------------------------------------------ join stages
def test_decode_first_tops_up_with_prefill_chunks():
    m = manager(d1=(16, 1, 8), d2=(5, 1, 3), sp1=(4, 0, 7), g1=(0, 0, 4), g2=(0, 0, 6))
    pending = {"g2": (toks(6), SP), "g1": (toks(4, 50), SP)}
    sus_p, sus_d = {"sp1": toks(3, 20)}, {}
    st = DecodeFirstAgggregatedJoinStage(m, pending, sus_p, sus_d, 8)
    rest, r = st.process(10, decode_request(["d1", "d2"]))
    # d1's next token opens a page (-1); sp1's 3 tokens ride along; g1 is the shorter new
    # prompt: 1 page, 3 of its 4 tokens fit the batch of 8, the last one waits
    assert rest == 8
    assert r.exec_task_ids == ["d1", "d2", "sp1", "g1"] and r.exec_seqlens == [1, 1, 3, 3]
    assert r.xs.tolist() == [100, 101, 20, 21, 22, 50, 51, 52]
    assert r.init_tasks == {"g1": (4, SP)} and set(pending) == {"g2"}
    assert sus_p["g1"].tolist() == [53] and "sp1" not in sus_p


def test_decode_first_without_budget_only_adds_decodes_that_fit():
    m = manager(d1=(16, 1, 8), w1=(32, 1, 8), w2=(7, 1, 3), g1=(0, 0, 4))
    pending = {"g1": (toks(4), SP)}
    sus_d = {"w1": toks(1, 7), "w2": toks(1, 8)}
    st = DecodeFirstAgggregatedJoinStage(m, pending, {}, sus_d, 8)
    rest, r = st.process(1, decode_request(["d1"]))
    # d1 takes the only page; no prefill (budget 0); w1 would need a page, w2 (7 -> 8) does not
    assert rest == 0 and r.exec_task_ids == ["d1", "w2"] and set(sus_d) == {"w1"} and set(pending) == {"g1"}


def test_prefill_first_switches_the_batch_and_parks_the_decodes():
    m = manager(d1=(16, 1, 8), d2=(5, 1, 3), g1=(0, 0, 4))
    pending, sus_p, sus_d = {"g1": (toks(4, 50), SP)}, {}, {}
    st = PrefillFirstAgggregatedJoinStage(m, pending, sus_p, sus_d, 8)
    req = decode_request(["d1", "d2"])
    req.cancel_task_ids = ["gone"]
    rest, r = st.process(10, req)
    # g1: 1 page; the parked decodes rejoin behind it while there is room: d1 +1 page, d2 none
    assert rest == 8 and r.exec_task_ids == ["g1", "d1", "d2"] and r.exec_seqlens == [4, 1, 1]
    assert r.xs.tolist() == [50, 51, 52, 53, 100, 101] and r.cancel_task_ids == ["gone"]
    assert sus_d == {} and pending == {}

    pending = {"g1": (toks(4, 50), SP)}
    st = PrefillFirstAgggregatedJoinStage(m, pending, {}, {}, 8)
    rest, r = st.process(0, decode_request(["d1", "d2"]))
    # the prompt does not fit: the decodes go on and overdraw the budget by d1's page
    assert rest == -1 and r.exec_task_ids == ["d1", "d2"] and set(pending) == {"g1"}


def test_prefill_first_splits_a_long_prompt():
    m = manager(g1=(0, 0, 20))
    pending, sus_p = {"g1": (toks(20), SP)}, {}
    st = PrefillFirstAgggregatedJoinStage(m, pending, sus_p, {}, 8)
    rest, r = st.process(5, StepRequest.empty(1, torch.int32, "cpu"))
    assert rest == 3 and r.exec_task_ids == ["g1"] and r.exec_seqlens == [8] and r.init_tasks == {"g1": (20, SP)}
    assert sus_p["g1"].tolist() == list(range(8, 20)) and r.microbatch_id == 1
    # next round: the remainder continues without new page accounting
    m.get("g1").start_pos, m.get("g1").seqlen = 8, 0
    rest, r = st.process(3, StepRequest.empty(1, torch.int32, "cpu"))
    assert rest == 3 and r.exec_seqlens == [8] and sus_p["g1"].tolist() == [16, 17, 18, 19] and r.init_tasks == {}


def test_vanilla_runs_one_whole_prompt_or_else_the_decodes():
    m = manager(d1=(16, 1, 8), w1=(3, 1, 2), g1=(0, 0, 40), g2=(0, 0, 2))
    pending, sus_d = {"g1": (toks(40), SP), "g2": (toks(2, 60), SP)}, {"w1": toks(1, 9)}
    st = VanillaJoinStage(m, pending, sus_d)
    rest, r = st.process(2, decode_request(["d1"]))
    # shortest prompt first: g2 (1 page); d1 steps aside
    assert rest == 1 and r.exec_task_ids == ["g2"] and r.xs.tolist() == [60, 61] and r.init_tasks == {"g2": (2, SP)}
    assert set(sus_d) == {"w1", "d1"} and set(pending) == {"g1"}
    rest, r = st.process(2, StepRequest.empty(0, torch.int32, "cpu"))
    # g1 needs 3 pages > 2: decodes instead, in arrival order; d1 opens a page
    assert rest == 1 and r.exec_task_ids == ["w1", "d1"] and sus_d == {}


def test_step_request_helpers():
    r = StepRequest.empty(2, torch.int32, "cpu")
    assert r.is_empty() and r.get_bsz() == 0
    r.append_exec("a", toks(3), (3, SP))
    r.append_exec("b", toks(1, 9), None)
    assert r.xs.tolist() == [0, 1, 2, 9] and r.exec_seqlens == [3, 1] and not r.is_empty()
    r.offload_task_ids.append("x")
    r.refresh()
    assert r.exec_seqlens == [1, 1] and r.init_tasks == {} and r.offload_task_ids == []
    with pytest.raises(AssertionError):
        r.append_exec("c", toks(0), None)
