"""The step after the forward pass: handing a batch's embeddings to the sidecar.

Mirrors what the reference's worker does around the model call (eric/executor/worker.py:279-344, without the
tracing spans): run `model(modality, adapter_name, data)`, then for every item whose `receiver_ranks` entry is not
None call `sidecar.send(data=embedding, id=data_id, chunk_id=..., num_chunks=..., dst_sidecar_ranks=...)`.  The
embeddings this build's encoders return are contiguous device tensors (row slices of one output buffer), which is
what the reference's sender needs to export them by IPC handle (sidecar/api.py:236-243).

`MockSidecar` implements the reference client's file-based test mode (sidecar/api.py:41-59,176-188): with
CORNSERVE_MOCK_SIDECAR=1 and CORNSERVE_MOCK_SIDECAR_MAPPING='{"<id>-<chunk>": "<path>", ...}' every tensor is
saved with torch.save to the mapped path (other values as JSON), so the encoders can be exercised by the
reference's executor test harness without a running sidecar.

`Worker.upload` is this build's addition on the inbound side: it starts the host-to-device copy of a batch's
pixel tensors (floating point or uint8) on a side stream through pinned staging buffers, so that the copy of batch k+1 runs while the encoder works
on batch k; `execute_model` then makes the compute stream wait for that copy only.

`Worker.download` is the outbound counterpart for the copy the reference's sidecar SERVER performs after it has opened
the IPC handle: device-to-host into its shared-memory slot on a stream of its own (services/sidecar/sender.py:498-529,
`buffer.data.copy_(data, non_blocking=True)` under `torch.cuda.stream(stream)`).  Here the copy of batch k's
embeddings goes into pinned host memory on a side stream while batch k+1 computes.  The embeddings themselves stay
exportable the way the reference's client exports them (`reduce_tensor`, sidecar/serde.py:89-95): contiguous row
slices of one allocation of torch's caching allocator.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any

import torch

from cornserve_amd.eric.api import Modality


@dataclass
class WorkerBatch:
    """Same fields as the reference's WorkerBatch (eric/schema.py:101-137), minus the tracing carriers."""

    modality: Modality
    adapter_name: str
    request_ids: list[str] = field(default_factory=list)
    data_ids: list[str] = field(default_factory=list)
    chunk_ids: list[int] = field(default_factory=list)
    num_chunks: list[int] = field(default_factory=list)
    receiver_ranks: list[list[list[int]] | None] = field(default_factory=list)
    data: dict[str, list[torch.Tensor]] = field(default_factory=dict)
    _dump_prefix: str | None = None
    _uploaded: Any = None   # event recorded after the batch's host-to-device copies (set by Worker.upload)

    def __len__(self) -> int:
        return len(self.data_ids)


def mock_sidecar_enabled() -> bool:
    return os.environ.get("CORNSERVE_MOCK_SIDECAR", "0").lower() in ("1", "true")


class MockSidecar:
    """The reference client's mocking branch of `Sidecar.send` as a stand-alone object."""

    def __init__(self, mapping: dict[str, str | Path] | None = None) -> None:
        if mapping is None:
            raw = os.environ.get("CORNSERVE_MOCK_SIDECAR_MAPPING", "")
            mapping = json.loads(raw) if raw else {}
        self.mapping = {k: Path(v) for k, v in mapping.items()}

    def send(self, data: Any, id: str, dst_sidecar_ranks: list[list[int]], chunk_id: int = 0, num_chunks: int = 1,
             stream: bool = False) -> None:
        key = f"{id}-{chunk_id}"
        if key not in self.mapping:
            raise ValueError(f"Mocking sidecar but key {key} not in mapping")
        path = self.mapping[key]
        if isinstance(data, torch.Tensor):
            torch.save(data, path)
        else:
            path.write_text(json.dumps(data))


class Download:
    """Embeddings on their way to pinned host memory (see Worker.download)."""

    def __init__(self, host: list[torch.Tensor], done: "torch.cuda.Event") -> None:
        self._host, self._done = host, done
        self._consumed = False

    def ready(self) -> bool:
        return self._done.query()

    def wait(self) -> list[torch.Tensor]:
        """Block until the copies have landed and return the host tensors.  They are views of one pinned buffer of the
        worker's ring and stay valid until that buffer's turn comes again, i.e. for `download_slots` - 1 further
        `Worker.download` calls (one, with the default two buffers); a consumer that keeps them longer must copy
        them, or the worker must be built with a deeper ring.  Waiting marks the buffer as handed over: a download that
        is neither waited on nor released blocks the reuse of its buffer (`Worker.download` raises)."""
        self._done.synchronize()
        self._consumed = True
        return self._host

    def release(self) -> None:
        """Give the buffer back without reading it (the copy, if still running, is waited for first)."""
        self._done.synchronize()
        self._consumed = True
        self._host = []


class Worker:
    """Runs batches through one encoder and forwards the embeddings (reference: Worker.execute_model)."""

    def __init__(self, model, sender_sidecar_client=None, download_slots: int = 2) -> None:
        """`download_slots`: depth of the ring of pinned host buffers `download` cycles through (at least 2: one being
        filled while the previous one is read)."""
        if download_slots < 2:
            raise ValueError("download_slots must be at least 2")
        self.model = model
        if sender_sidecar_client is None and mock_sidecar_enabled():
            sender_sidecar_client = MockSidecar()
        self.sender_sidecar_client = sender_sidecar_client
        self._copy_stream: torch.cuda.Stream | None = None
        self._d2h_stream: torch.cuda.Stream | None = None
        self._d2h_slots: list[torch.Tensor | None] = [None] * download_slots   # pinned buffers, used in turn
        self._d2h_owner: list[Download | None] = [None] * download_slots       # the download each one was last lent to
        self._d2h_turn = 0

    def download(self, embeddings: list[torch.Tensor]) -> Download:
        """Start copying a batch's embeddings to pinned host memory on a side stream (default priority) and return at
        once: the copy waits for the kernels that produce the embeddings (an event on the compute stream) and runs
        while the next batch computes.  The pinned buffers of the ring are used in turn and grown on demand, so the
        steady state allocates nothing.  A buffer is only lent again once the download it was last lent to has been
        waited on or released; otherwise the consumer would read the next batch's bytes in the previous batch's views
        without any error, so this raises RuntimeError instead (wait on downloads in order, or deepen the ring)."""
        device = self.model.device
        if device.type != "cuda":
            raise RuntimeError("download needs the model on a GPU")
        if self._d2h_stream is None:
            self._d2h_stream = torch.cuda.Stream(device=device)
        for e in embeddings:
            if not (isinstance(e, torch.Tensor) and e.is_cuda and e.is_contiguous()):
                raise ValueError("download takes contiguous device tensors")
        sizes = [(e.numel() * e.element_size() + 255) // 256 * 256 for e in embeddings]
        total = max(sum(sizes), 256)
        turn = self._d2h_turn
        owner = self._d2h_owner[turn]
        if owner is not None and not owner._consumed:
            raise RuntimeError(f"download ring overrun: the download started {len(self._d2h_slots)} calls ago has been "
                               "neither waited on nor released, and its pinned buffer is due for reuse")
        self._d2h_turn = (turn + 1) % len(self._d2h_slots)
        slot = self._d2h_slots[turn]
        if slot is None or slot.numel() < total:
            slot = self._d2h_slots[turn] = torch.empty((total,), dtype=torch.uint8, pin_memory=True)
        compute = torch.cuda.current_stream(device)
        produced = torch.cuda.Event()
        produced.record(compute)
        host, offset = [], 0
        with torch.cuda.stream(self._d2h_stream):
            self._d2h_stream.wait_event(produced)
            for e, size in zip(embeddings, sizes):
                dst = slot[offset : offset + e.numel() * e.element_size()].view(e.dtype).view(e.shape)
                dst.copy_(e, non_blocking=True)
                e.record_stream(self._d2h_stream)
                host.append(dst)
                offset += size
            done = torch.cuda.Event()
            done.record(self._d2h_stream)
        started = self._d2h_owner[turn] = Download(host, done)
        return started

    def upload(self, batch: WorkerBatch) -> WorkerBatch:
        """Start copying the batch's host tensors to the model's device and return at once.  Every host tensor is
        staged in pinned memory (a copy from pageable memory would block the host until it is done) and copied on
        a side stream of default priority; an event recorded behind the copies travels with the batch, and
        `execute_model` makes the compute stream wait for it.  Call it for batch k+1 before `execute_model(batch k)`
        returns control to the device queue, and the copy overlaps the encoder's work.  Device tensors pass through."""
        device = self.model.device
        if device.type != "cuda":
            raise RuntimeError("upload needs the model on a GPU")
        if self._copy_stream is None:
            self._copy_stream = torch.cuda.Stream(device=device)
        staged: dict[str, list[torch.Tensor]] = {}
        with torch.cuda.stream(self._copy_stream):
            for key, tensors in batch.data.items():
                out = []
                for t in tensors:
                    if (isinstance(t, torch.Tensor) and t.device.type == "cpu" and t.numel() > 0
                            and (t.is_floating_point() or t.dtype == torch.uint8)):
                        # floating-point tensors are converted to the model's dtype on the way into the staging buffer
                        # (the rounding the device cast would apply, on half the bytes); uint8 frames stay bytes
                        staged_dtype = self.model.dtype if t.is_floating_point() else t.dtype
                        pinned = torch.empty(t.shape, dtype=staged_dtype, pin_memory=True)
                        pinned.copy_(t)
                        out.append(pinned.to(device, non_blocking=True))
                    else:
                        out.append(t)   # integer tensors (grids, crop counts) stay on the host, where they are read
                staged[key] = out
            done = torch.cuda.Event()
            done.record(self._copy_stream)
        batch.data = staged
        batch._uploaded = done
        return batch

    @torch.inference_mode()
    def execute_model(self, batch: WorkerBatch) -> list[torch.Tensor]:
        n = len(batch)
        if not (len(batch.chunk_ids) == len(batch.num_chunks) == len(batch.receiver_ranks) == n):
            raise ValueError("data_ids, chunk_ids, num_chunks and receiver_ranks must have one entry per item")
        if batch._uploaded is not None:
            compute = torch.cuda.current_stream(self.model.device)
            compute.wait_event(batch._uploaded)
            for tensors in batch.data.values():   # the copies were allocated on the side stream
                for t in tensors:
                    if isinstance(t, torch.Tensor) and t.is_cuda:
                        t.record_stream(compute)
        output = self.model(modality=batch.modality, adapter_name=batch.adapter_name, batch=batch.data)
        if len(output) != n:
            raise RuntimeError(f"the model returned {len(output)} embeddings for {n} items")
        if self.sender_sidecar_client is not None:
            for i in range(n):
                dst = batch.receiver_ranks[i]
                if dst is None:
                    continue
                emb = output[i]
                if not emb.is_contiguous():   # the reference's sender would copy: keep that cost visible here
                    raise RuntimeError("embeddings handed to the sidecar must be contiguous")
                self.sender_sidecar_client.send(data=emb, id=batch.data_ids[i], chunk_id=batch.chunk_ids[i],
                                                num_chunks=batch.num_chunks[i], dst_sidecar_ranks=dst)
        if batch._dump_prefix is not None:
            torch.save([o.cpu() for o in output], batch._dump_prefix + "-tp1.pt")
        return output
