"""Batching of embedding requests in front of the encoder (reference: eric/engine/scheduler.py:22-190 and the batch
records of eric/schema.py:20-37,62-75,140-215, without the tracing spans and the msgpack transport, which belong to
the engine around the path).

Same policy as the reference: the queue is served in arrival order, and one batch takes the waiting items at its head
that share the first item's modality and adapter, up to `max_batch_size` items.  One addition for the kernels behind
`Worker.execute_model`: `max_batch_patches` bounds the batch by its total patch count, because their throughput is
flat from about 8192 patches up (every GEMM launch then fills the 256 compute units for at least one full round) while
activation memory and latency keep growing with the batch; a batch always takes at least one item.
"""

from __future__ import annotations

from collections import defaultdict
from collections.abc import Callable, Generator
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
        return WorkerBatch(modality=self.modality, adapter_name=self.adapter_name, request_ids=self.request_ids,
                           data_ids=self.data_ids, chunk_ids=self.chunk_ids, num_chunks=self.num_chunks,
                           receiver_ranks=self.receiver_ranks, data=self.data, _dump_prefix=self._dump_prefix)

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


class RequestQueue:
    """Requests in arrival order with a done flag per item (reference: scheduler.py:22-130)."""

    def __init__(self) -> None:
        self.request_id_to_request: dict[str, EngineEnqueueRequest] = {}
        self.request_id_to_data_done: dict[str, dict[str, bool]] = defaultdict(dict)

    def __len__(self) -> int:
        return len(self.request_id_to_request)

    def enqueue(self, request: EngineEnqueueRequest) -> None:
        self.request_id_to_request[request.request_id] = request
        for data in request.data:
            self.request_id_to_data_done[request.request_id][data.id] = False

    def mark_done(self, request_ids: list[str], data_ids: list[str]) -> list[str]:
        """Flag the items as done; returns (and forgets) the requests whose items are all done."""
        assert len(request_ids) == len(data_ids)
        for request_id, data_id in zip(request_ids, data_ids):
            self.request_id_to_data_done[request_id][data_id] = True
        finished = []
        for request_id in dict.fromkeys(request_ids):
            if all(self.request_id_to_data_done[request_id].values()):
                finished.append(request_id)
                del self.request_id_to_request[request_id]
                del self.request_id_to_data_done[request_id]
        return finished

    def is_done(self, request_id: str, data_id: str | None = None) -> bool:
        if request_id not in self.request_id_to_request:
            return True
        if data_id is None:
            return False
        return self.request_id_to_data_done[request_id][data_id]

    def peek_request(self) -> EngineEnqueueRequest:
        assert self.request_id_to_request, "Queue is empty"
        return next(iter(self.request_id_to_request.values()))

    def peek_data(self) -> ProcessedEmbeddingData:
        request = self.peek_request()
        assert request.data, "Request has no data"
        for data in request.data:
            if not self.is_done(request.request_id, data.id):
                return data
        raise ValueError("No waiting data in a waiting request")

    def iter_waiting(self, modality: Modality, model_id: str, max_items: int | None = None,
                     ) -> Generator[tuple[EngineEnqueueRequest, ProcessedEmbeddingData], None, None]:
        """Waiting items from the head of the queue until the modality or the adapter changes."""
        count = 0
        for request in self.request_id_to_request.values():
            for data in request.data:
                if self.is_done(request.request_id, data.id):
                    continue
                if data.modality != modality or data.model_id != model_id:
                    return
                yield request, data
                count += 1
                if count == max_items:
                    return


class Scheduler:
    """Reference: scheduler.py:133-190."""

    def __init__(self, max_batch_size: int | None = None, max_batch_patches: int | None = None,
                 count_patches: Callable[[ProcessedEmbeddingData], int] = patch_count) -> None:
        if max_batch_patches is not None and max_batch_patches < 1:
            raise ValueError("max_batch_patches must be positive")
        self.max_batch_size = max_batch_size
        self.max_batch_patches = max_batch_patches
        self.count_patches = count_patches
        self.queue = RequestQueue()

    def enqueue(self, request: EngineEnqueueRequest) -> None:
        self.queue.enqueue(request)

    def has_waiting_requests(self) -> bool:
        return len(self.queue) > 0

    def schedule(self) -> SchedulerBatch:
        """The next batch; only called while requests are waiting."""
        head = self.queue.peek_data()
        batch = SchedulerBatch(modality=head.modality, adapter_name=head.model_id)
        patches = 0
        for req, data in self.queue.iter_waiting(modality=head.modality, model_id=head.model_id,
                                                 max_items=self.max_batch_size):
            if self.max_batch_patches is not None:
                n = self.count_patches(data)
                if len(batch) > 0 and patches + n > self.max_batch_patches:
                    break
                patches += n
            batch.add_data(request_id=req.request_id, data=[data], chunk_ids=[0], num_chunks=[1])
        assert batch.request_ids, "Batch should not be empty"
        return batch

    def process_batch_result(self, request_ids: list[str], data_ids: list[str]) -> list[str]:
        """Returns the requests that are completely done."""
        return self.queue.mark_done(request_ids, data_ids)
