"""The messages a worker hands to the tensor-parallel coordinator when a save or a load has finished, as plain Python.

Field names, field order and the JSON a message turns into follow
kv_cache_manager/py_connector/common/tp_coordinator.py:14-70 (SendBlockFinishedEvent, LoadBlockFinishedEvent,
CoordinateMessage, CoordinateMsgSerializer). The reference serialises the dataclasses with orjson; `dumps` here gives
the same JSON object (dataclass fields in declaration order, nested) from the standard library, so a
TpCoordinatorServer decodes either. The transport (ZMQ push/pull) is not part of this package: DataTransferManager
only needs an object with `send(bytes)`.
"""
import dataclasses
import json
import time
from dataclasses import dataclass, field
from typing import List, Union


@dataclass
class SendBlockFinishedEvent:
    request_id: str
    tp_rank: int
    write_session_id: str
    is_success_list: List[bool] = field(default_factory=list)
    remote_uris: List[str] = field(default_factory=list)
    type: str = "SendBlockFinishedEvent"


@dataclass
class LoadBlockFinishedEvent:
    request_id: str
    tp_rank: int
    epoch: int
    failed_block_idxs: List[int] = field(default_factory=list)
    type: str = "LoadBlockFinishedEvent"


CoordinateEventUnion = Union[SendBlockFinishedEvent, LoadBlockFinishedEvent]


@dataclass
class CoordinateMessage:
    send_time: float
    content: CoordinateEventUnion
    create_time: float = field(default_factory=time.time)


msg_type_mapping = {
    "SendBlockFinishedEvent": SendBlockFinishedEvent,
    "LoadBlockFinishedEvent": LoadBlockFinishedEvent,
}


class CoordinateMsgSerializer:
    @staticmethod
    def dumps(obj: CoordinateMessage) -> bytes:
        return json.dumps(dataclasses.asdict(obj), separators=(",", ":")).encode()

    @staticmethod
    def loads(input_bytes: bytes) -> CoordinateMessage:
        msg = json.loads(input_bytes)
        content = msg_type_mapping[msg["content"]["type"]](**msg["content"])
        return CoordinateMessage(send_time=msg["send_time"], create_time=msg["create_time"], content=content)
