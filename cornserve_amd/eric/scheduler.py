"""Batching of embedding requests in front of the encoder (the policy of eric/engine/scheduler.py:133-190 and the batch
records of eric/schema.py:20-37,62-75,140-215, without the tracing spans and the msgpack transport, which belong to
the engine around the path).

Policy, as observed from outside: items are served in arrival order; one batch takes the waiting items at the head of
the line that share the first one's modality and adapter, up to `max_batch_size` items, and a request is reported
finished when its last item is.  Two additions for the kernels behind `Worker.execute_model`:

* `max_batch_patches` bounds a batch by its total patch count: throughput is flat from about 8192 patches up (every
  GEMM launch then fills the 256 compute units for at least one full round) while activation memory and latency keep
  growing with the batch; a batch always takes at least one item;
* items handed out by `schedule()` are IN FLIGHT until `process_batch_result` reports them, and a second
  `schedule()` before that skips them: the caller can take batch k+1 (and start its upload, `Worker.upload`) while
  batch k is still running.

The book-keeping is one flat line of item slots (arrival order) plus a count of unfinished items per request.
"""

from __future__ import annotations

from collections import deque
from collections.abc import Callable
from enum import Enum
from dataclasses import dataclass, field

import torch

from cornserve_amd.eric.api import Modality
from cornserve_amd.eric.worker import WorkerBatch


@dataclass
class ProcessedEmbeddingData:
    """One modality item of a request, after preprocessing (reference: schema.py:20-37)."""

    id: str
    modality: Modality
    model_id: str
    data: dict[str, torch.Tensor]
    receiver_sidecar_ranks: list[list[int]] | None = None


@dataclass
class EngineEnqueueRequest:
    """A request as the engine queues it (reference: schema.py:62-75)."""

    request_id: str
    data: list[ProcessedEmbeddingData]


@dataclass
class SchedulerBatch(WorkerBatch):
    """Items that run in one forward pass (reference: schema.py:140-215)."""

    def to_worker_batch(self) -> WorkerBatch:
        """The same batch as a plain WorkerBatch.  Everything travels, including the upload event of a batch whose
        host tensors `Worker.upload` has already sent ahead (without it the compute stream would not wait for the
        copies).  `Worker.execute_model` and `Worker.upload` also take the SchedulerBatch itself."""
        return WorkerBatch(modality=self.modality, adapter_name=self.adapter_name, request_ids=self.request_ids,
                           data_ids=self.data_ids, chunk_ids=self.chunk_ids, num_chunks=self.num_chunks,
                           receiver_ranks=self.receiver_ranks, data=self.data, _dump_prefix=self._dump_prefix,
                           _uploaded=self._uploaded)

    def add_data(self, request_id: str, data: list[ProcessedEmbeddingData], chunk_ids: list[int],
                 num_chunks: list[int]) -> None:
        if not len(data) == len(chunk_ids) == len(num_chunks):
            raise ValueError("data, chunk_ids and num_chunks must have one entry per item")
        for item, chunk_id, num_chunk in zip(data, chunk_ids, num_chunks):
            if self.modality != item.modality:
                raise ValueError(f"Cannot batch different modalities together: {self.modality} != {item.modality} "
                                 f"(Data ID: {item.id})")
            self.request_ids.append(request_id)
            self.data_ids.append(item.id)
            self.chunk_ids.append(chunk_id)
            self.num_chunks.append(num_chunk)
            self.receiver_ranks.append(item.receiver_sidecar_ranks)
            for key, value in item.data.items():
                self.data.setdefault(key, []).append(value)
        for key, values in self.data.items():
            assert len(values) == len(self.data_ids), f"Data length mismatch for key {key}: {len(values)} != {len(self.data_ids)}"


def patch_count(item: ProcessedEmbeddingData) -> int:
    """Rows the encoder will process for one item: the product of a `*_grid_thw` entry where the processor gives one
    (Qwen family), else tiles x (side / 14)^2 for [tiles, 3, S, S] pixels (SigLIP towers), else the first axis."""
    for key, value in item.data.items():
        if key.endswith("grid_thw"):
            return int(torch.as_tensor(value).reshape(-1, 3).prod(dim=1).sum())
    for key, value in item.data.items():
        if key.startswith("pixel_values") and value.dim() == 4:
            return int(value.shape[0]) * (int(value.shape[2]) // 14) * (int(value.shape[3]) // 14)
    first = next(iter(item.data.values()))
    return int(first.shape[0]) if first.dim() else 1


class _State(Enum):
    WAITING = 0
    IN_FLIGHT = 1


@dataclass
class _Slot:
    request_id: str
    item: ProcessedEmbeddingData
    state: _State = _State.WAITING


class Scheduler:
    """Arrival-order batching with a patch budget and in-flight tracking (policy of scheduler.py:133-190)."""

    def __init__(self, max_batch_size: int | None = None, max_batch_patches: int | None = None,
                 count_patches: Callable[[ProcessedEmbeddingData], int] = patch_count) -> None:
        if max_batch_patches is not None and max_batch_patches < 1:
            raise ValueError("max_batch_patches must be positive")
        if max_batch_size is not None and max_batch_size < 1:
            raise ValueError("max_batch_size must be positive")
        self.max_batch_size = max_batch_size
        self.max_batch_patches = max_batch_patches
        self.count_patches = count_patches
        self._line: deque[_Slot] = deque()            # unfinished items, arrival order
        self._open: dict[str, int] = {}               # request id -> items not yet reported done
        self._slot_of: dict[tuple[str, str], _Slot] = {}

    # ------------------------------------------------------------------ intake
    def enqueue(self, request: EngineEnqueueRequest) -> None:
        if request.request_id in self._open:
            raise ValueError(f"request {request.request_id} is already queued")
        if not request.data:
            raise ValueError(f"request {request.request_id} has no data")
        seen = set()
        for item in request.data:
            if item.id in seen:
                raise ValueError(f"request {request.request_id} lists data id {item.id} twice")
            seen.add(item.id)
        self._open[request.request_id] = len(request.data)
        for item in request.data:
            slot = _Slot(request.request_id, item)
            self._line.append(slot)
            self._slot_of[(request.request_id, item.id)] = slot

    def has_waiting_requests(self) -> bool:
        """Requests that are not finished yet (waiting or in flight), as the reference's method counts them.  A loop that
        calls `schedule()` again before `process_batch_result()` (upload-ahead) must gate on `has_schedulable_items()`
        instead: with every item in flight this stays True and `schedule()` has nothing to return (it raises)."""
        return bool(self._open)

    def has_schedulable_items(self) -> bool:
        """Items that a `schedule()` call could take right now (everything else is in flight)."""
        return any(slot.state is _State.WAITING for slot in self._line)

    # ------------------------------------------------------------------ batching
    def schedule(self) -> SchedulerBatch:
        """The next batch; its items are in flight until `process_batch_result` names them."""
        batch: SchedulerBatch | None = None
        patches = 0
        for slot in self._line:
            if slot.state is not _State.WAITING:
                continue
            item = slot.item
            if batch is None:
                batch = SchedulerBatch(modality=item.modality, adapter_name=item.model_id)
            elif item.modality != batch.modality or item.model_id != batch.adapter_name:
                break                                   # the line is served in order: no overtaking
            if self.max_batch_patches is not None:
                n = self.count_patches(item)
                if len(batch) > 0 and patches + n > self.max_batch_patches:
                    break
                patches += n
            batch.add_data(request_id=slot.request_id, data=[item], chunk_ids=[0], num_chunks=[1])
            slot.state = _State.IN_FLIGHT
            if self.max_batch_size is not None and len(batch) == self.max_batch_size:
                break
        if batch is None:
            raise RuntimeError("nothing to schedule: the queue is empty or every item is in flight")
        return batch

    def process_batch_result(self, request_ids: list[str], data_ids: list[str]) -> list[str]:
        """Report items as done.  Returns the requests whose last item this was, in the order given."""
        if len(request_ids) != len(data_ids):
            raise ValueError("request_ids and data_ids must have one entry per item")
        # every pair is checked before any state changes: a bad pair leaves the bookkeeping as it was
        keys = list(zip(request_ids, data_ids))
        if len(set(keys)) != len(keys):
            raise KeyError("an item is reported twice in one call")
        for key in keys:
            if key not in self._slot_of:
                raise KeyError(f"item {key[1]} of request {key[0]} is not queued (reported twice?)")
        finished: list[str] = []
        for key in keys:
            slot = self._slot_of.pop(key)
            slot.state = None                          # finished: dropped from the line below
            self._open[key[0]] -= 1
            if self._open[key[0]] == 0:
                del self._open[key[0]]
                finished.append(key[0])
        while self._line and self._line[0].state is None:
            self._line.popleft()
        if len(self._line) > 4 * len(self._slot_of) + 16:   # finished items stuck behind an unfinished head
            self._line = deque(slot for slot in self._line if slot.state is not None)
        return finished
