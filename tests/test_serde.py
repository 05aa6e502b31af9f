"""Stage-hop wire format: framing, the safetensors container against the safetensors
package (both directions), the empty-tensor quirk, and what the metadata loader refuses."""
import json
import pickle
import struct
import sys
import types

import pytest
import torch

from deserve_amd import serde
from deserve_amd.engine.pipeline.processor import StepRequest
from deserve_amd.task import SamplingParams

safetensors_torch = pytest.importorskip("safetensors.torch")


def _tensors():
    g = torch.Generator().manual_seed(3)
    return {
        "xs": torch.randn((5, 32, 128), generator=g).to(torch.bfloat16),
        "ids": torch.arange(7, dtype=torch.int64),
        "mask": torch.tensor([True, False, True]),
        "h": torch.randn((2, 3), generator=g).to(torch.float16),
        "f": torch.randn((4,), generator=g),
        "b": torch.arange(5, dtype=torch.uint8),
    }


def _same(a, b):
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a.view(torch.uint8) if a.dtype != torch.bool else a,
                                                                     b.view(torch.uint8) if b.dtype != torch.bool else b)


def test_known_answer_bytes_of_a_small_message():
    """Every byte of a one-tensor message, written out by hand."""
    meta = {"group_id": 1}
    t = torch.tensor([1.0, -2.0], dtype=torch.float32)
    msg = serde.dumps({"x": t}, meta)
    pick = pickle.dumps(meta)
    header = b'{"x":{"dtype":"F32","shape":[2],"data_offsets":[0,8]}}'
    header += b" " * (-len(header) % 8)
    want = (len(pick).to_bytes(4, "big") + pick + struct.pack("<Q", len(header)) + header
            + struct.pack("<ff", 1.0, -2.0))
    assert msg == want


def test_container_is_read_by_the_safetensors_package_and_reads_what_it_writes():
    tensors = _tensors()
    ours = serde.save_container(tensors)
    theirs = safetensors_torch.load(ours)
    assert set(theirs) == set(tensors) and all(_same(theirs[k], tensors[k]) for k in tensors)
    back = serde.load_container(safetensors_torch.save(tensors))
    assert set(back) == set(tensors) and all(_same(back[k], tensors[k]) for k in tensors)
    # with a metadata entry in the header, as the package writes when asked to
    back = serde.load_container(safetensors_torch.save(tensors, metadata={"who": "test"}))
    assert set(back) == set(tensors)
    # every tensor starts on a multiple of its element size
    n = struct.unpack("<Q", ours[:8])[0]
    assert n % 8 == 0
    for name, info in json.loads(ours[8: 8 + n]).items():
        assert info["data_offsets"][0] % tensors[name].element_size() == 0


def test_message_round_trip_with_the_reference_framing_and_the_empty_tensor_quirk():
    tensors = _tensors()
    tensors["nothing"] = torch.empty((0,), dtype=torch.bfloat16)
    meta = {"group_id": 3, "exec_task_ids": ["a", "b"], "exec_seqlens": [1, 512],
            "init_tasks": {"b": (512, SamplingParams(temperature=0.5, max_new_tokens=9))}}
    msg = serde.dumps(tensors, meta)
    n = int.from_bytes(msg[:4], "big")
    assert pickle.loads(msg[4: 4 + n]) == meta                      # the reference's own reader of the metadata
    raw = safetensors_torch.load(msg[4 + n:])                        # ... and of the tensors
    assert "#nothing" in raw and raw["#nothing"].shape == (1,) and raw["#nothing"].dtype == torch.bfloat16
    got, got_meta = serde.loads(msg)
    assert got_meta == meta and set(got) == set(tensors)
    assert got["nothing"].shape == (0,) and got["nothing"].dtype == torch.bfloat16
    assert all(_same(got[k], tensors[k]) for k in tensors)
    # a message framed the way the reference frames it, container written by the package
    ref_msg = n.to_bytes(4, "big") + msg[4: 4 + n] + safetensors_torch.save(
        {("#" + k if v.numel() == 0 else k): (torch.ones((1,), dtype=v.dtype) if v.numel() == 0 else v)
         for k, v in tensors.items()})
    got2, meta2 = serde.loads(ref_msg)
    assert meta2 == meta and all(_same(got2[k], tensors[k]) for k in tensors)


def test_step_request_crosses_the_hop_unchanged():
    req = StepRequest.empty(2, torch.bfloat16, device="cpu")
    req.append_exec("t0", torch.ones((1, 4096), dtype=torch.bfloat16))
    req.append_exec("t1", torch.zeros((3, 4096), dtype=torch.bfloat16), init_info=(3, SamplingParams(top_p=0.9)))
    req.cancel_task_ids, req.offload_task_ids, req.reload_task_ids = ["c"], ["o"], ["r"]
    back = StepRequest.from_safetensors(*serde.loads(serde.dumps(*req.into_safetensors())))
    assert back.microbatch_id == 2 and back.exec_task_ids == ["t0", "t1"] and back.exec_seqlens == [1, 3]
    assert (back.cancel_task_ids, back.offload_task_ids, back.reload_task_ids) == (["c"], ["o"], ["r"])
    assert back.init_tasks == {"t1": (3, SamplingParams(top_p=0.9))} and torch.equal(back.xs, req.xs)
    assert back.get_tensors_size() == 4 * 4096 * 2
    empty = StepRequest.from_safetensors(*serde.loads(serde.dumps(*StepRequest.empty(0, torch.float16, "cpu").into_safetensors())))
    assert empty.is_empty() and empty.xs.dtype == torch.float16


def test_pydantic_sampling_params_of_a_reference_peer_are_mapped():
    """A peer running the reference pickles its pydantic SamplingParams under
    deserve_worker.task; the loader maps it onto this package's class."""
    pydantic = pytest.importorskip("pydantic")
    mod = types.ModuleType("deserve_worker.task")

    class SamplingParams_(pydantic.BaseModel):
        temperature: float = 0.0
        top_p: float = 1.0
        max_seq_len: int = 4096
        max_new_tokens: int = 4096
        dump_probs_num: int = 0

    SamplingParams_.__name__ = SamplingParams_.__qualname__ = "SamplingParams"
    SamplingParams_.__module__ = "deserve_worker.task"
    mod.SamplingParams = SamplingParams_
    parent = types.ModuleType("deserve_worker")
    saved = {k: sys.modules.get(k) for k in ("deserve_worker", "deserve_worker.task")}
    sys.modules["deserve_worker"], sys.modules["deserve_worker.task"] = parent, mod
    try:
        pick = pickle.dumps({"init_tasks": {"t": (7, SamplingParams_(temperature=0.25, max_new_tokens=11))}})
    finally:
        for k, v in saved.items():
            if v is None:
                sys.modules.pop(k, None)
            else:
                sys.modules[k] = v
    msg = len(pick).to_bytes(4, "big") + pick + serde.save_container({"xs": torch.zeros(1)})
    _, meta = serde.loads(msg)
    assert meta["init_tasks"]["t"] == (7, SamplingParams(temperature=0.25, max_new_tokens=11))


def test_loader_refuses_foreign_classes_and_broken_frames():
    class Evil:
        def __reduce__(self):
            return (print, ("executed",))

    pick = pickle.dumps({"x": Evil()})
    msg = len(pick).to_bytes(4, "big") + pick + serde.save_container({"xs": torch.zeros(1)})
    with pytest.raises(pickle.UnpicklingError):
        serde.loads(msg)
    good = serde.dumps({"xs": torch.zeros(3)}, {"a": 1})
    with pytest.raises(ValueError):
        serde.loads(good[:3])
    with pytest.raises(ValueError):
        serde.loads((1 << 20).to_bytes(4, "big") + good[4:])
    with pytest.raises(ValueError):
        serde.load_container(good[4 + int.from_bytes(good[:4], "big"):][:-4])     # data cut short
    with pytest.raises(ValueError):
        serde.save_container({"c": torch.zeros(2, dtype=torch.complex64)})
