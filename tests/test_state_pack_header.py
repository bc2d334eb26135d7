"""The packed-state header is JSON: ordinary training states are rebuilt without unpickling
anything; only leaves JSON cannot express are pickled, and only accepted when allowed."""

import collections
import io
import json
import math
import pickle
from datetime import timedelta

import pytest
import torch

from torchft_amd import CheckpointServer, state_pack


def _roundtrip(state, allow_pickle=True):
    plan = state_pack.plan_pack(state)
    assert not plan.tensors  # CPU-only states: everything travels in the header
    meta = state_pack.parse_header(plan.header(), allow_pickle)
    return state_pack._fill(meta["skeleton"], [])


def test_training_state_shapes_survive_without_pickle(monkeypatch):
    state = {
        "user": {
            "optim": {
                "state": {0: {"step": torch.tensor(7.0), "big": 2 ** 70}, 1: {"step": torch.tensor(8.0)}},
                "param_groups": [{"lr": 4e-4, "betas": (0.9, 0.95), "params": [0, 1], "nesterov": False,
                                  "foreach": None, "inf": math.inf}],
            },
            "od": collections.OrderedDict([("b", 1), ("a", (1, (2, 3)))]),
            "tuple_key": {(1, 2): "x", 3: "y", "__tft__": "a key that looks like a tag"},
            "empty": torch.empty(0, 3, dtype=torch.bfloat16),
            "half": torch.arange(6, dtype=torch.float16).view(2, 3),
            "flags": torch.tensor([True, False]),
        },
        "torchft": {"step": 20, "batches_committed": 40},
    }
    monkeypatch.setattr(pickle, "loads", lambda *_a, **_k: pytest.fail("unpickled"))
    monkeypatch.setattr(pickle, "dumps", lambda *_a, **_k: pytest.fail("pickled"))
    out = _roundtrip(state, allow_pickle=False)
    assert out["torchft"] == state["torchft"]
    assert out["user"]["optim"]["param_groups"] == state["user"]["optim"]["param_groups"]
    assert isinstance(out["user"]["optim"]["param_groups"][0]["betas"], tuple)
    assert list(out["user"]["optim"]["state"].keys()) == [0, 1]
    assert out["user"]["optim"]["state"][0]["big"] == 2 ** 70
    assert torch.equal(out["user"]["optim"]["state"][1]["step"], torch.tensor(8.0))
    assert type(out["user"]["od"]) is collections.OrderedDict and list(out["user"]["od"]) == ["b", "a"]
    assert out["user"]["od"]["a"] == (1, (2, 3))
    assert out["user"]["tuple_key"] == state["user"]["tuple_key"]
    assert out["user"]["empty"].shape == (0, 3) and out["user"]["empty"].dtype == torch.bfloat16
    assert torch.equal(out["user"]["half"], state["user"]["half"])
    assert torch.equal(out["user"]["flags"], state["user"]["flags"])
    json.loads(state_pack.plan_pack(state).header())  # it really is JSON


class _Scheduler:
    def __init__(self, gamma):
        self.gamma = gamma

    def __eq__(self, other):
        return isinstance(other, _Scheduler) and other.gamma == self.gamma


def test_non_json_leaves_need_allow_pickle():
    state = {"sched": _Scheduler(0.5), "n": 1}
    assert _roundtrip(state, allow_pickle=True) == state
    with pytest.raises(ValueError, match="allow_pickle=True"):
        _roundtrip(state, allow_pickle=False)
    # over the transport: the default mirrors the reference (accepts), a strict server refuses
    server = CheckpointServer(timeout=timedelta(seconds=10))
    strict = CheckpointServer(timeout=timedelta(seconds=10), allow_pickle=False)
    server.send_checkpoint([], 3, state, timedelta(seconds=10))
    assert server.recv_checkpoint(0, server.metadata(), 3, timedelta(seconds=10)) == state
    with pytest.raises(ValueError, match="allow_pickle=True"):
        strict.recv_checkpoint(0, server.metadata(), 3, timedelta(seconds=10))
    server.shutdown()
    strict.shutdown()


def test_malformed_headers_are_rejected():
    good = state_pack.plan_pack({"a": 1}).header()
    assert state_pack.header_total_bytes(good) == 0
    for bad in (b"\x80\x04garbage", b"[]", b'{"skeleton":1}', b'{"total_bytes":-1}'):
        with pytest.raises(ValueError):
            state_pack.parse_header(bad)
    doc = json.loads(good)
    doc["entries"] = [[0, 8, "torch.float32", [4], False, False]]  # 16 bytes claimed as 8
    doc["total_bytes"] = 256
    with pytest.raises(ValueError, match="disagree"):
        state_pack.parse_header(json.dumps(doc).encode())
    doc["entries"] = [[512, 16, "torch.float32", [4], False, False]]
    with pytest.raises(ValueError, match="outside the payload"):
        state_pack.parse_header(json.dumps(doc).encode())
    doc["entries"] = []
    doc["skeleton"] = {"__tft__": "mystery"}
    with pytest.raises(ValueError, match="unknown node kind"):
        state_pack.parse_header(json.dumps(doc).encode())
    with pytest.raises(ValueError, match="bad magic"):
        state_pack.read_packed(io.BytesIO(b"12345678" + b"\0" * 16), None)


def test_peer_supplied_sizes_are_bounded_before_anything_is_allocated():
    """The header length and the payload size come from the peer: an oversized header length is
    refused before that many bytes are read, and the entries are validated against the
    announced payload size before a staging buffer of that size would be allocated."""
    import struct

    huge = state_pack.MAGIC + struct.pack("<Q", state_pack.MAX_HEADER_BYTES + 1)
    with pytest.raises(ValueError, match="refused"):
        state_pack.read_header(io.BytesIO(huge))
    with pytest.raises(EOFError):
        state_pack.read_header(io.BytesIO(state_pack.MAGIC + struct.pack("<Q", 100) + b"{}"))
    with pytest.raises(EOFError):
        state_pack.read_header(io.BytesIO(state_pack.MAGIC + b"\1\2"))
    # an entry outside the payload: refused by read_packed before the device is touched
    doc = {"skeleton": None, "entries": [[1 << 40, 16, "torch.float32", [4], False, False]],
           "total_bytes": 1 << 20}
    header = json.dumps(doc).encode()
    wire = state_pack.MAGIC + struct.pack("<Q", len(header)) + header
    with pytest.raises(ValueError, match="outside the payload"):
        state_pack.read_packed(io.BytesIO(wire), None)
    # validation without decoding the skeleton never unpickles
    doc = {"skeleton": {"__tft__": "pickle", "type": "x", "data": "AAAA"}, "entries": [], "total_bytes": 0}
    meta = state_pack.parse_header(json.dumps(doc).encode(), allow_pickle=False, decode_skeleton=False)
    assert meta["skeleton"] is None and meta["total_bytes"] == 0


def test_split_range_covers_the_payload_on_aligned_boundaries():
    for total in (0, 1, 255, 256, 257, 10_000, (1 << 30) + 123):
        for parts in (1, 2, 3, 4, 7):
            ranges = [state_pack.split_range(total, p, parts) for p in range(parts)]
            assert ranges[0][0] == 0 and ranges[-1][1] == total
            for (lo, hi), (lo2, _) in zip(ranges, ranges[1:]):
                assert lo <= hi == lo2
            assert all(lo % 256 == 0 for lo, hi in ranges if hi > lo)
    with pytest.raises(ValueError):
        state_pack.split_range(10, 2, 2)
